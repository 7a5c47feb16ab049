// RMSNorm and AdaLN for any row width: cols a multiple of one 16-byte access
// (8 two-byte or 4 four-byte elements), up to 1024 accesses per row (8192 / 4096
// columns), for bf16, fp16 and fp32.  The widths and types the tuned kernels in
// rmsnorm.hip / adaln.hip are not built for land here, so that smaller models
// (other hidden sizes and head dimensions) still run fused.
//
// Same arithmetic and rounding points as the tuned kernels, same row -> lane
// geometry, but the width is a run-time argument: a row is laid over a padded
// geometry of LANES x CHUNKS accesses (the smallest instantiated one that holds
// it) and every lane knows which of its accesses fall inside the row.  Accesses
// outside read zeros and write nothing.  The parameter-gradient reduction is
// the same fixed-order two-stage scheme, so results are bit-identical from run
// to run.
#include <hip/hip_runtime.h>

#include "norm_device.h"
#include "norm_host.h"

// Stores of dx / out: 1 = write-through at device scope (RowWriter<1>), 0 = plain streaming store.
// Measured both ways per width: backward gains up to 7 % with write-through for rows of up to six
// accesses per lane (512 columns 212 -> 197 us, 1024 196 -> 186 us, 1536 184 -> 182 us) and loses 3-4 %
// at eight and twelve (4096, 6144 columns), so the wide geometries keep the plain store.
#ifndef TTN_ANY_FWD_STORE
#define TTN_ANY_FWD_STORE 0
#endif
#ifndef TTN_ANY_BWD_STORE
#define TTN_ANY_BWD_STORE 1
#endif

namespace ttn {

template <typename T, int LANES_, int CHUNKS_>
struct PadGeom {
    static constexpr int VEC = Elem<T>::VEC;
    static constexpr int LANES = LANES_;
    static constexpr int CHUNKS = CHUNKS_;
    static constexpr int RPW = kWaveSize / LANES;
    static_assert(LANES >= kMinRowLanes, "the host's row-stride cap assumes at most kMaxRowsPerWave rows per wavefront");
    static_assert(LANES == 8 || LANES == 16 || LANES == 32 || LANES == 64, "row must fill an aligned lane group");
    static_assert(LANES == 64 || CHUNKS == 1, "only full wavefronts take several accesses per lane");
};

// Which of this lane's accesses lie inside a row of `pieces` 16-byte pieces.
template <typename G>
struct LaneMask {
    bool in[G::CHUNKS];
    __device__ __forceinline__ LaneMask(int l, int pieces) {
#pragma unroll
        for (int k = 0; k < G::CHUNKS; ++k) in[k] = k * G::LANES + l < pieces;
    }
};

template <typename G>
__device__ __forceinline__ void load_row(u32x4 (&dst)[G::CHUNKS], const void *row_base, int l, bool ok,
                                         const LaneMask<G> &m) {
    const u32x4 *p = reinterpret_cast<const u32x4 *>(row_base) + l;
#pragma unroll
    for (int k = 0; k < G::CHUNKS; ++k) dst[k] = (ok && m.in[k]) ? load16_stream(p + k * G::LANES) : u32x4{0, 0, 0, 0};
}

template <typename G>
__device__ __forceinline__ void load_param(u32x4 (&dst)[G::CHUNKS], const void *base, int l, const LaneMask<G> &m) {
    const u32x4 *p = reinterpret_cast<const u32x4 *>(base) + l;
#pragma unroll
    for (int k = 0; k < G::CHUNKS; ++k) dst[k] = m.in[k] ? load16(p + k * G::LANES) : u32x4{0, 0, 0, 0};
}

// Workgroup-level flush of per-lane column sums: rows of a wavefront folded by
// shuffles, wavefronts added into LDS in wavefront order, one fp32 row of
// NSETS*C partial sums written out.  lds holds NSETS*C floats.
template <typename G, int NSETS>
__device__ __forceinline__ void flush_partials_anywidth(float (&acc)[NSETS][G::CHUNKS][G::VEC],
                                                        float *__restrict__ partial_row, float *lds, int C,
                                                        const LaneMask<G> &m) {
    constexpr int VEC = G::VEC, LANES = G::LANES, CHUNKS = G::CHUNKS;
    const int lane = threadIdx.x & 63;
    const int sub = lane / LANES;
    const int l = lane % LANES;
    const int wave = wave_id_in_block();
#pragma unroll
    for (int s = 0; s < NSETS; ++s)
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[s][k][j] = fold_rows_of_wave<LANES>(acc[s][k][j]);
    for (int wv = 0; wv < kRowWaves; ++wv) {
        if (wave == wv && sub == 0) {
#pragma unroll
            for (int s = 0; s < NSETS; ++s)
#pragma unroll
                for (int k = 0; k < CHUNKS; ++k) {
                    if (!m.in[k]) continue;
                    float *p = lds + s * C + (k * LANES + l) * VEC;
#pragma unroll
                    for (int j = 0; j < VEC; ++j) p[j] = (wv == 0) ? acc[s][k][j] : p[j] + acc[s][k][j];
                }
        }
        __syncthreads();
    }
    for (int i = threadIdx.x; i < NSETS * C; i += kRowThreads) partial_row[i] = lds[i];
}

// ------------------------------------------------------------------ RMSNorm

template <typename T, int LANES, int CHUNKS, typename Map>
__global__ __launch_bounds__(kRowThreads) void anywidth_rmsnorm_fwd_kernel(
    T *__restrict__ out, float *__restrict__ rstd, const T *__restrict__ x, const T *__restrict__ w,
    const Map map, int C, float eps) {
    using G = PadGeom<T, LANES, CHUNKS>;
    using E = Elem<T>;
    constexpr int VEC = G::VEC, RPW = G::RPW;
    const int lane = threadIdx.x & 63;
    const int sub = lane / LANES;
    const int l = lane % LANES;
    const int wave = wave_id_in_block();
    const LaneMask<G> m(l, C / VEC);

    u32x4 wr[CHUNKS];
    load_param<G>(wr, w, l, m);

    const int64_t groups = map.template groups<RPW>();
    const int64_t stride = (int64_t)gridDim.x * kRowWaves;
    for (int64_t grp = (int64_t)blockIdx.x * kRowWaves + wave; grp < groups; grp += stride) {
        keep_packed(wr);
        const RowAddr at = map.template locate<RPW>(grp, sub, C);
        const int64_t row = at.row;
        const bool ok = at.ok;
        u32x4 xr[CHUNKS];
        load_row<G>(xr, x + at.xoff, l, ok, m);

        float ss = 0.0f;
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            float v[VEC];
            E::unpack(xr[k], v);
#pragma unroll
            for (int j = 0; j < VEC; ++j) ss = fmaf(v[j], v[j], ss);
        }
        ss = group_sum<LANES>(ss);
        const float r = 1.0f / sqrtf(ss / (float)C + eps);
        if (ok && l == 0) rstd[row] = r;

        // the wavefront's rows are consecutive in out: base = its first row
        const RowWriter<TTN_ANY_FWD_STORE> wo(out + map.template locate<RPW>(grp, 0, C).row * C,
                                              (uint32_t)(sub * C * (int)sizeof(T)) + l * 16);
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            float v[VEC], wv[VEC];
            E::unpack(xr[k], v);
            E::unpack(wr[k], wv);
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] *= r;
            E::round(v);  // y = normalised row in the element type
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] *= wv[j];
            if (ok && m.in[k]) wo.put(k * LANES, E::pack(v));
        }
    }
}

template <typename T, int LANES, int CHUNKS, typename Map>
__global__ __launch_bounds__(kRowThreads) void anywidth_rmsnorm_bwd_kernel(
    T *__restrict__ dx, float *__restrict__ partial, const T *__restrict__ g, const T *__restrict__ x,
    const T *__restrict__ w, const float *__restrict__ rstd, const Map map, int C) {
    using G = PadGeom<T, LANES, CHUNKS>;
    using E = Elem<T>;
    constexpr int VEC = G::VEC, RPW = G::RPW;
    extern __shared__ float lds[];
    const int lane = threadIdx.x & 63;
    const int sub = lane / LANES;
    const int l = lane % LANES;
    const int wave = wave_id_in_block();
    const LaneMask<G> m(l, C / VEC);

    u32x4 wr[CHUNKS];
    load_param<G>(wr, w, l, m);
    float acc[1][CHUNKS][VEC];
#pragma unroll
    for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[0][k][j] = 0.0f;

    const int64_t groups = map.template groups<RPW>();
    const int64_t stride = (int64_t)gridDim.x * kRowWaves;
    for (int64_t grp = (int64_t)blockIdx.x * kRowWaves + wave; grp < groups; grp += stride) {
        keep_packed(wr);
        const RowAddr at = map.template locate<RPW>(grp, sub, C);
        const int64_t row = at.row;
        const bool ok = at.ok;
        u32x4 gr[CHUNKS], xr[CHUNKS];
        load_row<G>(gr, g + row * C, l, ok, m);
        load_row<G>(xr, x + at.xoff, l, ok, m);
        const float r = ok ? rstd[row] : 0.0f;

        // pass 1: gy = rnd(g*w) kept packed; row dot  sum_c gy * x
        u32x4 gyp[CHUNKS];
        float dot = 0.0f;
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            float gv[VEC], wv[VEC], xv[VEC];
            E::unpack(gr[k], gv);
            E::unpack(wr[k], wv);
#pragma unroll
            for (int j = 0; j < VEC; ++j) gv[j] *= wv[j];
            gyp[k] = E::pack(gv);
            E::unpack(gyp[k], gv);
            E::unpack(xr[k], xv);
#pragma unroll
            for (int j = 0; j < VEC; ++j) dot = fmaf(gv[j], xv[j], dot);
        }
        dot = group_sum<LANES>(dot);
        // dx = r*(gy - xhat * mean_c(gy*xhat)) = gy*r + x*coef
        const float coef = -((dot / (float)C) * r * r * r);
        // the second pass unpacks the row again rather than holding pass 1's fp32 copies live
        keep_packed(gr);
        keep_packed(xr);
        keep_packed(gyp);

        // dx goes through its own strides: base = the wavefront's first row, the lane adds its row's distance
        const int64_t doff0 = map.template locate<RPW>(grp, 0, C).doff;
        const RowWriter<(TTN_ANY_BWD_STORE && CHUNKS <= 6)> wd(
            dx + doff0, (uint32_t)((at.doff - doff0) * (int64_t)sizeof(T)) + l * 16);
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            float gv[VEC], gy[VEC], xv[VEC], o[VEC], y[VEC];
            E::unpack(gr[k], gv);
            E::unpack(gyp[k], gy);
            E::unpack(xr[k], xv);
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                o[j] = fmaf(xv[j], coef, gy[j] * r);
                y[j] = xv[j] * r;
            }
            if (ok && m.in[k]) wd.put(k * LANES, E::pack(o));
            E::round(y);  // y = normalised row in the element type
#pragma unroll
            for (int j = 0; j < VEC; ++j) y[j] *= gv[j];
            E::round(y);  // g*y materialised in the element type before the column sum
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[0][k][j] += y[j];
        }
    }
    flush_partials_anywidth<G, 1>(acc, partial + (int64_t)blockIdx.x * C, lds, C, m);
}

// -------------------------------------------------------------------- AdaLN

// GATED = true: the normalised row is first formed as h2 = rnd(x + rnd(attn * gate[b])) (the gated residual
// update that precedes the norm in the transformer blocks) and written out too.
template <typename T, int LANES, int CHUNKS, bool GATED>
__global__ __launch_bounds__(kRowThreads) void anywidth_adaln_fwd_kernel(
    T *__restrict__ out, float *__restrict__ mean, float *__restrict__ rstd, const T *__restrict__ x,
    const T *__restrict__ scale, const T *__restrict__ shift, T *__restrict__ h2_out, const T *__restrict__ attn,
    const T *__restrict__ gate, int64_t rows_per_sample, const SampleLayout lay, int blocks_per_sample, int C,
    float eps) {
    using G = PadGeom<T, LANES, CHUNKS>;
    using E = Elem<T>;
    constexpr int VEC = G::VEC, RPW = G::RPW;
    const int lane = threadIdx.x & 63;
    const int sub = lane / LANES;
    const int l = lane % LANES;
    const int wave = wave_id_in_block();
    const int64_t b = blockIdx.x / blocks_per_sample;  // sample this workgroup serves
    const int slot = blockIdx.x % blocks_per_sample;
    const LaneMask<G> m(l, C / VEC);

    u32x4 tr[CHUNKS], hr[CHUNKS];
    [[maybe_unused]] u32x4 qr[GATED ? CHUNKS : 1];
    load_param<G>(tr, scale + b * C, l, m);
    load_param<G>(hr, shift + b * C, l, m);
    if constexpr (GATED) load_param<G>(qr, gate + b * C, l, m);
#pragma unroll
    for (int k = 0; k < CHUNKS; ++k) {  // t = rnd(1 + scale)
        float v[VEC];
        E::unpack(tr[k], v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = 1.0f + v[j];
        tr[k] = E::pack(v);
    }

    const int64_t groups = (rows_per_sample + RPW - 1) / RPW;
    const int64_t stride = (int64_t)blocks_per_sample * kRowWaves;
    for (int64_t grp = (int64_t)slot * kRowWaves + wave; grp < groups; grp += stride) {
        keep_packed(tr);
        keep_packed(hr);
        if constexpr (GATED) keep_packed(qr);
        const int64_t rs = grp * RPW + sub;
        const bool ok = rs < rows_per_sample;
        const int64_t row = lay.row(b, rs);
        const int64_t first = lay.row(b, grp * RPW) * C;  // the wavefront's first row: base of what it writes
        const uint32_t lane_bytes = (uint32_t)(sub * lay.row_stride * C * (int64_t)sizeof(T)) + l * 16;
        u32x4 xr[CHUNKS];
        load_row<G>(xr, x + row * C, l, ok, m);
        if constexpr (GATED) {
            u32x4 ar[CHUNKS];
            load_row<G>(ar, attn + row * C, l, ok, m);
            const RowWriter<TTN_ANY_FWD_STORE> wh(h2_out + first, lane_bytes);
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k) {
                float hv[VEC], av[VEC], gv[VEC];
                E::unpack(xr[k], hv);
                E::unpack(ar[k], av);
                E::unpack(qr[k], gv);
#pragma unroll
                for (int j = 0; j < VEC; ++j) av[j] *= gv[j];
                E::round(av);  // attn * gate materialised in the element type
#pragma unroll
                for (int j = 0; j < VEC; ++j) hv[j] += av[j];
                xr[k] = E::pack(hv);  // h2: the new residual stream, and the row that is normalised
                if (ok && m.in[k]) wh.put(k * LANES, xr[k]);
            }
        }

        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            float v[VEC];
            E::unpack(xr[k], v);
#pragma unroll
            for (int j = 0; j < VEC; ++j) s += v[j];
        }
        const float mu = group_sum<LANES>(s) / (float)C;
        float q = 0.0f;
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            float v[VEC];
            E::unpack(xr[k], v);
            if (m.in[k]) {  // padding must not count as (0 - mu)^2
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const float d = v[j] - mu;
                    q = fmaf(d, d, q);
                }
            }
        }
        const float r = 1.0f / sqrtf(group_sum<LANES>(q) / (float)C + eps);
        if (ok && l == 0) {
            mean[row] = mu;
            rstd[row] = r;
        }

        const float nmr = -(mu * r);
        const RowWriter<TTN_ANY_FWD_STORE> wo(out + first, lane_bytes);
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            float v[VEC], tv[VEC], hv[VEC];
            E::unpack(xr[k], v);
            E::unpack(tr[k], tv);
            E::unpack(hr[k], hv);
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] = centred<T>(v[j], mu, r, nmr);
            E::round(v);  // xn
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] *= tv[j];
            E::round(v);  // xn * (1 + scale)
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] += hv[j];
            if (ok && m.in[k]) wo.put(k * LANES, E::pack(v));
        }
    }
}

// GATED: x is the saved h2; dx = dh = rnd(rnd(dx of the norm) + e) with e the gradient arriving at h2 from
// its other use (may be null), da = rnd(dh * gate[b]) is written too and dgate[b] += rnd(dh * attn) is a
// third set of column sums.  RES: dx = rnd(rnd(dx of the norm) + e), e the gradient the input receives
// from its other consumer.  (Same forms as the tuned kernels.)
template <typename T, int LANES, int CHUNKS, bool GATED, bool RES>
__global__ __launch_bounds__(kRowThreads) void anywidth_adaln_bwd_kernel(
    T *__restrict__ dx, float *__restrict__ partial, const T *__restrict__ g, const T *__restrict__ x,
    const T *__restrict__ scale, const float *__restrict__ mean, const float *__restrict__ rstd,
    T *__restrict__ da, const T *__restrict__ e, const T *__restrict__ attn, const T *__restrict__ gate,
    int64_t rows_per_sample, const SampleLayout lay, int blocks_per_sample, int C) {
    static_assert(!(GATED && RES), "the gated form handles e itself");
    static_assert(!(GATED || RES) || CHUNKS <= 6, "the gated and residual forms are built for rows of up to six accesses per lane");
    constexpr int NSETS = GATED ? 3 : 2;
    using G = PadGeom<T, LANES, CHUNKS>;
    using E = Elem<T>;
    constexpr int VEC = G::VEC, RPW = G::RPW;
    // the widest rows have no registers left for the modulation row: it is staged in LDS, in the
    // area the final flush uses afterwards
    constexpr bool kParamInRegs = CHUNKS <= 8;
    // ... nor for gx = rnd(g*t) between the two passes: it is formed again (same rounding, same value)
    constexpr bool kKeepGx = CHUNKS * VEC <= 64;
    extern __shared__ float lds[];
    const int lane = threadIdx.x & 63;
    const int sub = lane / LANES;
    const int l = lane % LANES;
    const int wave = wave_id_in_block();
    const int64_t b = blockIdx.x / blocks_per_sample;
    const int slot = blockIdx.x % blocks_per_sample;
    const LaneMask<G> m(l, C / VEC);

    auto one_plus = [](const u32x4 &raw) -> u32x4 {  // t = rnd(1 + scale)
        float v[VEC];
        E::unpack(raw, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = 1.0f + v[j];
        return E::pack(v);
    };
    u32x4 tr[kParamInRegs ? CHUNKS : 1];
    [[maybe_unused]] u32x4 qr[GATED ? CHUNKS : 1];
    u32x4 *lds_t = reinterpret_cast<u32x4 *>(lds);  // shares the flush area: dead before the flush starts
    if constexpr (kParamInRegs) {
        load_param<G>(tr, scale + b * C, l, m);
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) tr[k] = one_plus(tr[k]);
    } else {
        for (int i = threadIdx.x; i < C / VEC; i += kRowThreads)
            lds_t[i] = one_plus(load16(reinterpret_cast<const u32x4 *>(scale + b * C) + i));
        __syncthreads();
    }
    if constexpr (GATED) load_param<G>(qr, gate + b * C, l, m);

    float acc[NSETS][CHUNKS][VEC];  // [0] = dscale, [1] = dshift, [2] = dgate
#pragma unroll
    for (int s = 0; s < NSETS; ++s)
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[s][k][j] = 0.0f;

    const int64_t groups = (rows_per_sample + RPW - 1) / RPW;
    const int64_t stride = (int64_t)blocks_per_sample * kRowWaves;
    for (int64_t grp = (int64_t)slot * kRowWaves + wave; grp < groups; grp += stride) {
        if constexpr (kParamInRegs) keep_packed(tr);
        if constexpr (GATED) keep_packed(qr);
        const int64_t rs = grp * RPW + sub;
        const bool ok = rs < rows_per_sample;
        const int64_t row = lay.row(b, rs);
        const int64_t first = lay.row(b, grp * RPW) * C;
        const uint32_t lane_bytes = (uint32_t)(sub * lay.row_stride * C * (int64_t)sizeof(T)) + l * 16;
        u32x4 gr[CHUNKS], xr[CHUNKS];
        [[maybe_unused]] u32x4 er[(GATED || RES) ? CHUNKS : 1], ar[GATED ? CHUNKS : 1];
        load_row<G>(gr, g + row * C, l, ok, m);
        load_row<G>(xr, x + row * C, l, ok, m);
        if constexpr (GATED || RES) load_row<G>(er, e + row * C, l, ok && e != nullptr, m);
        if constexpr (GATED) load_row<G>(ar, attn + row * C, l, ok, m);
        const float r = ok ? rstd[row] : 0.0f;
        const float mu = ok ? mean[row] : 0.0f;
        const float nmr = -(mu * r);  // xhat = x*r + nmr

        auto gx_of = [&](int k) -> u32x4 {  // rnd(g * t) for access k, in the element type
            float gv[VEC], tv[VEC];
            E::unpack(gr[k], gv);
            if constexpr (kParamInRegs)
                E::unpack(tr[k], tv);
            else
                E::unpack(m.in[k] ? lds_t[k * LANES + l] : u32x4{0, 0, 0, 0}, tv);
#pragma unroll
            for (int j = 0; j < VEC; ++j) gv[j] *= tv[j];
            return E::pack(gv);
        };
        // pass 1: gx = rnd(g*t); s1 = sum_c gx; s2 = sum_c gx * xhat
        u32x4 gxp[kKeepGx ? CHUNKS : 1];
        float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            const u32x4 gxk = gx_of(k);
            if constexpr (kKeepGx) gxp[k] = gxk;
            // padding: g = 0 there, so gx = 0 and neither sum sees xhat = nmr
            if constexpr (kHasDot2<T>) {
                // straight from the packed pairs; s2 holds sum_c gx * x here, turned into sum_c gx * xhat below
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    s1 = dot2<T>(gxk[i], kOnesPair<T>, s1);
                    s2 = dot2<T>(gxk[i], xr[k][i], s2);
                }
            } else {
                float gv[VEC], xv[VEC];
                E::unpack(gxk, gv);
                E::unpack(xr[k], xv);
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    s1 += gv[j];
                    s2 = fmaf(gv[j], centred<T>(xv[j], mu, r, nmr), s2);
                }
            }
        }
        s1 = group_sum<LANES>(s1);
        s2 = group_sum<LANES>(s2);
        if constexpr (kHasDot2<T>) s2 = r * (s2 - mu * s1);
        const float m1 = s1 / (float)C, m2 = s2 / (float)C;
        // dx = r*(gx - m1 - xhat*m2) = r*gx + x*K1 + K0
        const float k1 = -(r * m2), k0 = -(r * m1);
        const float K1 = k1 * r;
        const float K0 = fmaf(k1, nmr, k0);
        // the second pass unpacks the row again rather than holding pass 1's fp32 copies live
        keep_packed(gr);
        keep_packed(xr);
        if constexpr (kKeepGx) keep_packed(gxp);

        constexpr int kDxStore = (TTN_ANY_BWD_STORE && CHUNKS <= 6 && !GATED);
        const RowWriter<kDxStore> wd(dx + first, lane_bytes);
        const RowWriter<0> wa(GATED ? da + first : nullptr, lane_bytes);
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            float gv[VEC], gx[VEC], xv[VEC], o[VEC], xn[VEC];
            E::unpack(gr[k], gv);
            if constexpr (kKeepGx)
                E::unpack(gxp[k], gx);
            else
                E::unpack(gx_of(k), gx);
            E::unpack(xr[k], xv);
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                o[j] = fmaf(r, gx[j], fmaf(xv[j], K1, K0));
                xn[j] = centred<T>(xv[j], mu, r, nmr);
                acc[1][k][j] += gv[j];
            }
            if constexpr (GATED || RES) {
                float ev[VEC];
                E::round(o);  // the norm's dx, materialised in the element type
                E::unpack(er[k], ev);
#pragma unroll
                for (int j = 0; j < VEC; ++j) o[j] += ev[j];
            }
            const u32x4 dxp = E::pack(o);
            if (ok && m.in[k]) wd.put(k * LANES, dxp);
            if constexpr (GATED) {
                float av[VEC], qv[VEC];
                E::unpack(dxp, o);  // dh as stored
                E::unpack(ar[k], av);
                E::unpack(qr[k], qv);
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    qv[j] *= o[j];
                    av[j] *= o[j];
                }
                if (ok && m.in[k]) wa.put(k * LANES, E::pack(qv));
                E::round(av);  // dh*attn materialised in the element type before the column sum
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc[2][k][j] += av[j];
            }
            E::round(xn);  // the normalised row in the element type
#pragma unroll
            for (int j = 0; j < VEC; ++j) xn[j] *= gv[j];
            E::round(xn);  // g*xn materialised in the element type before the column sum
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[0][k][j] += xn[j];
        }
    }
    if constexpr (!kParamInRegs) __syncthreads();  // every wavefront is done reading lds_t
    flush_partials_anywidth<G, NSETS>(acc, partial + (int64_t)blockIdx.x * (NSETS * C), lds, C, m);
}

// ---------------------------------------------------------------- dispatch

constexpr int kMaxPieces = 1024;  // 16-byte accesses per row: 64 lanes x 16

bool anywidth_supported(int64_t cols, int dtype) {
    if (dtype != TT_NORM_BF16 && dtype != TT_NORM_F32 && dtype != TT_NORM_F16) return false;
    const int vec = 16 / (int)elem_bytes(dtype);
    return cols > 0 && cols % vec == 0 && cols / vec <= kMaxPieces;
}

// The smallest instantiated geometry that holds `pieces` accesses.
struct GeomChoice {
    int lanes, chunks;
};
static GeomChoice choose_geometry(int pieces) {
    if (pieces <= 8) return {8, 1};
    if (pieces <= 16) return {16, 1};
    if (pieces <= 32) return {32, 1};
    const int need = (pieces + 63) / 64;
    for (int c : {1, 2, 3, 4, 6, 8, 12, 16})
        if (need <= c) return {64, c};
    return {0, 0};
}

// Calls F<T, LANES, CHUNKS>::run(args...) for the run-time (dtype, geometry).
#define TTN_ANYWIDTH_GEOMS(X, T) \
    X(T, 8, 1) X(T, 16, 1) X(T, 32, 1) X(T, 64, 1) X(T, 64, 2) X(T, 64, 3) X(T, 64, 4) X(T, 64, 6) X(T, 64, 8) X(T, 64, 12) X(T, 64, 16)

template <template <typename, int, int> class F, typename... Args>
static int dispatch(int dtype, GeomChoice gc, Args... args) {
#define TTN_TRY(T, L, K) \
    if (gc.lanes == L && gc.chunks == K) return F<T, L, K>::run(args...);
    if (dtype == TT_NORM_BF16) {
        TTN_ANYWIDTH_GEOMS(TTN_TRY, bf16_t)
    } else if (dtype == TT_NORM_F16) {
        TTN_ANYWIDTH_GEOMS(TTN_TRY, f16_t)
    } else {
        TTN_ANYWIDTH_GEOMS(TTN_TRY, float)
    }
#undef TTN_TRY
    return fail(TT_NORM_EUNSUPPORTED, "no kernel geometry for %d lanes x %d accesses", gc.lanes, gc.chunks);
}

// Launch policy.  Forward: narrow rows (one access per lane) use a persistent grid of 16 workgroups
// per compute unit, wider rows one row per wavefront.  Backward is persistent (column sums live in
// registers); the grid shrinks as rows widen so that each compute unit keeps about the same number
// of bytes in flight.
constexpr int kOneShotAny = 1 << 20;
static int fwd_blocks_per_cu(int chunks) { return chunks == 1 ? 16 : kOneShotAny; }
static int bwd_blocks_per_cu(int chunks) { return chunks >= 6 ? 1 : (chunks >= 3 ? 2 : (chunks == 2 ? 3 : 6)); }

static GeomChoice geometry_for(int64_t cols, int dtype) {
    return choose_geometry((int)(cols / (16 / (int)elem_bytes(dtype))));
}

// Grid for (batch, rows_per_sample) under geometry gc; status != OK on failure.
static int plan_for(RowPlan *plan, int64_t batch, int64_t rows_per_sample, GeomChoice gc, bool backward) {
    int st = TT_NORM_OK;
    const int cus = current_device_cus(&st);
    if (st != TT_NORM_OK) return st;
    *plan = make_row_plan(batch, rows_per_sample, kWaveSize / gc.lanes,
                          backward ? bwd_blocks_per_cu(gc.chunks) : fwd_blocks_per_cu(gc.chunks), cus);
    if (plan->blocks > 0x7fffffffLL) return fail(TT_NORM_EINVAL, "grid too large");
    return TT_NORM_OK;
}

template <typename Map>
struct RmsOn {  // the RMSNorm kernels over one kind of row map
    template <typename T, int LANES, int CHUNKS>
    struct Fwd {
        static int run(const RowPlan &p, void *out, float *rstd, const void *x, const void *w, const Map &map, int C,
                       double eps, hipStream_t stream) {
            RowKernelProfile prof(stream);
            anywidth_rmsnorm_fwd_kernel<T, LANES, CHUNKS, Map><<<dim3((unsigned)p.blocks), dim3(kRowThreads), 0, stream>>>(
                (T *)out, rstd, (const T *)x, (const T *)w, map, C, (float)eps);
            return TT_NORM_OK;
        }
    };
    template <typename T, int LANES, int CHUNKS>
    struct Bwd {
        static int run(const RowPlan &p, void *dx, void *ws, const void *g, const void *x, const void *w,
                       const float *rstd, const Map &map, int C, hipStream_t stream) {
            RowKernelProfile prof(stream);
            anywidth_rmsnorm_bwd_kernel<T, LANES, CHUNKS, Map>
                <<<dim3((unsigned)p.blocks), dim3(kRowThreads), (size_t)C * sizeof(float), stream>>>(
                    (T *)dx, (float *)ws, (const T *)g, (const T *)x, (const T *)w, rstd, map, C);
            return TT_NORM_OK;
        }
    };
};

struct AdalnExtra {  // operands of the gated / residual forms (null otherwise)
    void *h2_or_da;   // forward: h2 out; backward: dattn out
    const void *e;    // backward: the other gradient (dh2 or dres), may be null for the gated form
    const void *attn;
    const void *gate;
};

template <bool GATED, bool RES>
struct AdalnOn {
    template <typename T, int LANES, int CHUNKS>
    struct Fwd {
        static int run(const RowPlan &p, void *out, float *mean, float *rstd, const void *x, const void *scale,
                       const void *shift, const AdalnExtra &ex, int64_t rows_per_sample, SampleLayout lay, int C,
                       double eps, hipStream_t stream) {
            if constexpr (GATED && CHUNKS > 6) {
                return fail(TT_NORM_EUNSUPPORTED, "gated residual + AdaLN: rows of more than six 16-byte accesses per lane");
            } else {
                RowKernelProfile prof(stream);
                anywidth_adaln_fwd_kernel<T, LANES, CHUNKS, GATED><<<dim3((unsigned)p.blocks), dim3(kRowThreads), 0, stream>>>(
                    (T *)out, mean, rstd, (const T *)x, (const T *)scale, (const T *)shift, (T *)ex.h2_or_da,
                    (const T *)ex.attn, (const T *)ex.gate, rows_per_sample, lay, p.blocks_per_sample, C, (float)eps);
                return TT_NORM_OK;
            }
        }
    };
    template <typename T, int LANES, int CHUNKS>
    struct Bwd {
        static int run(const RowPlan &p, void *dx, void *ws, const void *g, const void *x, const void *scale,
                       const float *mean, const float *rstd, const AdalnExtra &ex, int64_t rows_per_sample,
                       SampleLayout lay, int C, hipStream_t stream) {
            if constexpr ((GATED || RES) && CHUNKS > 6) {
                return fail(TT_NORM_EUNSUPPORTED, "gated / residual AdaLN backward: rows of more than six 16-byte accesses per lane");
            } else {
                constexpr int NSETS = GATED ? 3 : 2;
                RowKernelProfile prof(stream);
                anywidth_adaln_bwd_kernel<T, LANES, CHUNKS, GATED, RES>
                    <<<dim3((unsigned)p.blocks), dim3(kRowThreads), (size_t)NSETS * C * sizeof(float), stream>>>(
                        (T *)dx, (float *)ws, (const T *)g, (const T *)x, (const T *)scale, mean, rstd,
                        (T *)ex.h2_or_da, (const T *)ex.e, (const T *)ex.attn, (const T *)ex.gate, rows_per_sample,
                        lay, p.blocks_per_sample, C);
                return TT_NORM_OK;
            }
        }
    };
};

template <typename Map>
static int rmsnorm_forward_on(void *out, float *rstd, const void *x, const void *w, const Map &map, int64_t rows,
                              int64_t cols, double eps, int dtype, hipStream_t stream) {
    if (rows == 0) return TT_NORM_OK;
    const GeomChoice gc = geometry_for(cols, dtype);
    RowPlan p;
    int st = plan_for(&p, 1, rows, gc, false);
    if (st != TT_NORM_OK) return st;
    st = dispatch<RmsOn<Map>::template Fwd>(dtype, gc, p, out, rstd, x, w, map, (int)cols, eps, stream);
    return st != TT_NORM_OK ? st : check_launch("rmsnorm forward launch");
}

int anywidth_rmsnorm_forward(void *out, float *rstd, const void *x, const void *w, int64_t rows, int64_t cols,
                             double eps, int dtype, hipStream_t stream) {
    if (TTN_WIDE_ROWS && widerow_takes(cols, dtype)) return widerow_rmsnorm_forward(out, rstd, x, w, rows, cols, eps, dtype, stream);
    return rmsnorm_forward_on(out, rstd, x, w, DenseRows{rows}, rows, cols, eps, dtype, stream);
}

int anywidth_rmsnorm_forward_strided(void *out, float *rstd, const void *x, const void *w, const Strided3Rows &map,
                                     int64_t cols, double eps, int dtype, hipStream_t stream) {
    return rmsnorm_forward_on(out, rstd, x, w, map, map.n0 * map.n1 * map.n2, cols, eps, dtype, stream);
}

static size_t backward_scratch(int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype, int nsets) {
    if (batch <= 0 || rows_per_sample <= 0 || !anywidth_supported(cols, dtype)) return 0;
    RowPlan p;
    if (plan_for(&p, batch, rows_per_sample, geometry_for(cols, dtype), true) != TT_NORM_OK) return 0;
    size_t need = (size_t)p.blocks * nsets * cols * sizeof(float);
    if (TTN_WIDE_ROWS && widerow_takes(cols, dtype)) {  // dense rows take the other kernels, strided views these
        const size_t wide = widerow_backward_workspace_bytes(batch, rows_per_sample, cols, dtype, nsets);
        if (wide == 0) return 0;
        if (wide > need) need = wide;
    }
    return need;
}

size_t anywidth_rmsnorm_backward_workspace_bytes(int64_t rows, int64_t cols, int dtype) {
    return backward_scratch(1, rows, cols, dtype, 1);
}

template <typename Map>
static int rmsnorm_backward_on(void *dx, void *dw, const void *g, const void *x, const void *w, const float *rstd,
                               const Map &map, int64_t rows, int64_t cols, int dtype, void *ws, size_t ws_bytes,
                               hipStream_t stream) {
    if (rows == 0) return launch_colreduce(dw, nullptr, nullptr, nullptr, 1, 0, cols, cols, dtype, stream);
    const GeomChoice gc = geometry_for(cols, dtype);
    RowPlan p;
    int st = plan_for(&p, 1, rows, gc, true);
    if (st != TT_NORM_OK) return st;
    const size_t need = (size_t)p.blocks * cols * sizeof(float);
    if (!ws || ws_bytes < need)
        return fail(TT_NORM_EWORKSPACE, "rmsnorm backward: workspace %zu B < required %zu B", ws_bytes, need);
    if (!aligned16(ws)) return fail(TT_NORM_EALIGN, "rmsnorm backward: workspace %p not 16-byte aligned", ws);
    st = dispatch<RmsOn<Map>::template Bwd>(dtype, gc, p, dx, ws, g, x, w, rstd, map, (int)cols, stream);
    if (st != TT_NORM_OK) return st;
    st = check_launch("rmsnorm backward launch");
    if (st != TT_NORM_OK) return st;
    return launch_colreduce(dw, nullptr, nullptr, (const float *)ws, 1, p.blocks_per_sample, cols, cols, dtype,
                            stream);
}

int anywidth_rmsnorm_backward(void *dx, void *dw, const void *g, const void *x, const void *w,
                              const float *rstd, int64_t rows, int64_t cols, int dtype, void *ws,
                              size_t ws_bytes, hipStream_t stream) {
    if (TTN_WIDE_ROWS && widerow_takes(cols, dtype))
        return widerow_rmsnorm_backward(dx, dw, g, x, w, rstd, rows, cols, dtype, ws, ws_bytes, stream);
    return rmsnorm_backward_on(dx, dw, g, x, w, rstd, DenseRows{rows}, rows, cols, dtype, ws, ws_bytes, stream);
}

int anywidth_rmsnorm_backward_strided(void *dx, void *dw, const void *g, const void *x, const void *w,
                                      const float *rstd, const Strided3Rows &map, int64_t cols, int dtype,
                                      void *ws, size_t ws_bytes, hipStream_t stream) {
    return rmsnorm_backward_on(dx, dw, g, x, w, rstd, map, map.n0 * map.n1 * map.n2, cols, dtype, ws, ws_bytes,
                               stream);
}

static SampleLayout layout_of(int64_t batch, int64_t rows_per_sample, bool seq_first) {
    return seq_first ? SampleLayout{1, batch} : SampleLayout{rows_per_sample, 1};
}

bool anywidth_wide_forms_supported(int64_t cols, int dtype) {
    if (!anywidth_supported(cols, dtype)) return false;
    // rows of up to six accesses per lane here; wider dense rows on the wide-row kernels
    return geometry_for(cols, dtype).chunks <= 6 || (TTN_WIDE_ROWS && widerow_takes(cols, dtype));
}

template <bool GATED>
static int adaln_forward_any(void *out, float *mean, float *rstd, const void *x, const void *scale,
                             const void *shift, const AdalnExtra &ex, int64_t batch, int64_t rows_per_sample,
                             int64_t cols, double eps, int dtype, bool seq_first, hipStream_t stream) {
    if (rows_per_sample == 0) return TT_NORM_OK;
    const GeomChoice gc = geometry_for(cols, dtype);
    RowPlan p;
    int st = plan_for(&p, batch, rows_per_sample, gc, false);
    if (st != TT_NORM_OK) return st;
    st = dispatch<AdalnOn<GATED, false>::template Fwd>(dtype, gc, p, out, mean, rstd, x, scale, shift, ex, rows_per_sample,
                                                       layout_of(batch, rows_per_sample, seq_first), (int)cols, eps,
                                                       stream);
    return st != TT_NORM_OK ? st : check_launch("adaln forward launch");
}

int anywidth_adaln_forward(void *out, float *mean, float *rstd, const void *x, const void *scale,
                           const void *shift, int64_t batch, int64_t rows_per_sample, int64_t cols, double eps,
                           int dtype, hipStream_t stream, bool seq_first) {
    if (TTN_WIDE_ROWS && widerow_takes(cols, dtype))
        return widerow_adaln_forward(out, mean, rstd, x, scale, shift, batch, rows_per_sample, cols, eps, dtype, seq_first,
                                     stream);
    return adaln_forward_any<false>(out, mean, rstd, x, scale, shift, AdalnExtra{nullptr, nullptr, nullptr, nullptr},
                                    batch, rows_per_sample, cols, eps, dtype, seq_first, stream);
}

int anywidth_gated_adaln_forward(void *h2, void *out, float *mean, float *rstd, const void *h, const void *attn,
                                 const void *gate, const void *scale, const void *shift, int64_t batch,
                                 int64_t rows_per_sample, int64_t cols, double eps, int dtype, hipStream_t stream) {
    if (TTN_WIDE_ROWS && widerow_takes(cols, dtype))
        return widerow_gated_adaln_forward(h2, out, mean, rstd, h, attn, gate, scale, shift, batch, rows_per_sample, cols,
                                           eps, dtype, stream);
    return adaln_forward_any<true>(out, mean, rstd, h, scale, shift, AdalnExtra{h2, nullptr, attn, gate}, batch,
                                   rows_per_sample, cols, eps, dtype, false, stream);
}

size_t anywidth_adaln_backward_workspace_bytes(int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype) {
    return backward_scratch(batch, rows_per_sample, cols, dtype, 2);
}

template <bool GATED, bool RES>
static int adaln_backward_any(void *dx, void *dscale, void *dshift, void *dgate, const void *g, const void *x,
                              const void *scale, const float *mean, const float *rstd, const AdalnExtra &ex,
                              int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype, void *ws,
                              size_t ws_bytes, bool seq_first, hipStream_t stream) {
    constexpr int NSETS = GATED ? 3 : 2;
    if (rows_per_sample == 0)
        return launch_colreduce(dscale, dshift, dgate, nullptr, batch, 0, cols, NSETS * cols, dtype, stream);
    const GeomChoice gc = geometry_for(cols, dtype);
    RowPlan p;
    int st = plan_for(&p, batch, rows_per_sample, gc, true);
    if (st != TT_NORM_OK) return st;
    const size_t need = (size_t)p.blocks * NSETS * cols * sizeof(float);
    if (!ws || ws_bytes < need)
        return fail(TT_NORM_EWORKSPACE, "adaln backward: workspace %zu B < required %zu B", ws_bytes, need);
    if (!aligned16(ws)) return fail(TT_NORM_EALIGN, "adaln backward: workspace %p not 16-byte aligned", ws);
    st = dispatch<AdalnOn<GATED, RES>::template Bwd>(dtype, gc, p, dx, ws, g, x, scale, mean, rstd, ex, rows_per_sample,
                                                     layout_of(batch, rows_per_sample, seq_first), (int)cols, stream);
    if (st != TT_NORM_OK) return st;
    st = check_launch("adaln backward launch");
    if (st != TT_NORM_OK) return st;
    return launch_colreduce(dscale, dshift, dgate, (const float *)ws, batch, p.blocks_per_sample, cols, NSETS * cols,
                            dtype, stream);
}

int anywidth_adaln_backward(void *dx, void *dscale, void *dshift, const void *g, const void *x,
                            const void *scale, const float *mean, const float *rstd, int64_t batch,
                            int64_t rows_per_sample, int64_t cols, int dtype, void *ws, size_t ws_bytes,
                            hipStream_t stream, bool seq_first) {
    if (TTN_WIDE_ROWS && widerow_takes(cols, dtype))
        return widerow_adaln_backward(dx, dscale, dshift, g, x, scale, mean, rstd, batch, rows_per_sample, cols, dtype, ws,
                                      ws_bytes, seq_first, stream);
    return adaln_backward_any<false, false>(dx, dscale, dshift, nullptr, g, x, scale, mean, rstd,
                                            AdalnExtra{nullptr, nullptr, nullptr, nullptr}, batch, rows_per_sample, cols,
                                            dtype, ws, ws_bytes, seq_first, stream);
}

int anywidth_adaln_backward_residual(void *dx, void *dscale, void *dshift, const void *g, const void *dres,
                                     const void *x, const void *scale, const float *mean, const float *rstd,
                                     int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype, void *ws,
                                     size_t ws_bytes, hipStream_t stream) {
    if (TTN_WIDE_ROWS && widerow_takes(cols, dtype))
        return widerow_adaln_backward_residual(dx, dscale, dshift, g, dres, x, scale, mean, rstd, batch, rows_per_sample,
                                               cols, dtype, ws, ws_bytes, stream);
    return adaln_backward_any<false, true>(dx, dscale, dshift, nullptr, g, x, scale, mean, rstd,
                                           AdalnExtra{nullptr, dres, nullptr, nullptr}, batch, rows_per_sample, cols, dtype,
                                           ws, ws_bytes, false, stream);
}

size_t anywidth_gated_adaln_backward_workspace_bytes(int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype) {
    return backward_scratch(batch, rows_per_sample, cols, dtype, 3);
}

int anywidth_gated_adaln_backward(void *dh, void *dattn, void *dgate, void *dscale, void *dshift, const void *g,
                                  const void *dh2, const void *h2, const void *attn, const void *gate,
                                  const void *scale, const float *mean, const float *rstd, int64_t batch,
                                  int64_t rows_per_sample, int64_t cols, int dtype, void *ws, size_t ws_bytes,
                                  hipStream_t stream) {
    if (TTN_WIDE_ROWS && widerow_takes(cols, dtype))
        return widerow_gated_adaln_backward(dh, dattn, dgate, dscale, dshift, g, dh2, h2, attn, gate, scale, mean, rstd,
                                            batch, rows_per_sample, cols, dtype, ws, ws_bytes, stream);
    return adaln_backward_any<true, false>(dh, dscale, dshift, dgate, g, h2, scale, mean, rstd,
                                           AdalnExtra{dattn, dh2, attn, gate}, batch, rows_per_sample, cols, dtype, ws,
                                           ws_bytes, false, stream);
}

}  // namespace ttn
