// RMSNorm and AdaLN for WIDE rows: more than 384 16-byte pieces per row (above 3072 two-byte / 1536
// four-byte columns, up to 1024 pieces), dense rows only (contiguous, or sample-major / sequence-first AdaLN).
// One wavefront per row would have to hold 8 to 16 accesses per lane and tensor, which leaves a compute unit
// with too few wavefronts to keep its share of the memory system busy; here the four wavefronts of a
// workgroup share a row instead: wavefront w owns the contiguous slice of ppw = ceil(pieces / 4) pieces that
// starts at piece w * ppw (CH = 2, 3 or 4 accesses per lane, the last one partly filled when ppw is not a
// multiple of 64, so the four wavefronts always carry equal shares), the row statistics are exchanged through
// LDS with one barrier per row, and a lane still owns fixed columns, so the parameter-gradient sums stay in
// registers and every wavefront writes its own slice of the workgroup's partial row (no cross-wavefront
// addition at all).
//
// Grids (measured at 4096, 5120 and 8192 two-byte columns, 730 MB per tensor): RMSNorm forward one-shot (one
// row per workgroup); AdaLN forward in short-lived workgroups of four rows each, which amortise the set-up of
// the modulation row (kept as fp32 values) and still retire and get replaced as the grid drains; both request
// the next row before the current row's output pass.  Backward persistent, two workgroups per compute unit that
// overlap each other (no request ahead inside a wavefront), write-through stores.  The gated residual and residual forms
// (GATED / RES, as in adaln.hip) use the same grids as the plain form, so that the column sums are added in the
// same order and a fused call is bit-identical to its parts.  Dense fp32 rows of 3072 columns (768 pieces) take
// their backward here too: a wavefront that owns such a row has registers for one row buffer only.
//
// Same arithmetic and rounding points as the kernels in rmsnorm.hip / adaln.hip / anywidth.hip; the
// variance of AdaLN is formed per wavefront about the wavefront's own mean and merged
// (sum_w [M2_w + n_w (m_w - mu)^2], exact up to the rounding of m_w), which needs one exchange instead of two.
#include <hip/hip_runtime.h>

#include "norm_device.h"
#include "norm_host.h"

// Workgroups per compute unit of the persistent grids (forward, backward).
#ifndef TTN_WIDE_FWD_BLOCKS_PER_CU
#define TTN_WIDE_FWD_BLOCKS_PER_CU 4
#endif
#ifndef TTN_WIDE_BWD_BLOCKS_PER_CU
#define TTN_WIDE_BWD_BLOCKS_PER_CU 2
#endif
// Forward grids: rows per workgroup (1 = one-shot grid, N = short-lived workgroups of N rows each, 0 = persistent
// grid of TTN_WIDE_FWD_BLOCKS_PER_CU resident workgroups per compute unit).
#ifndef TTN_WIDE_RMS_FWD_ROWS_PER_BLOCK
#define TTN_WIDE_RMS_FWD_ROWS_PER_BLOCK 1
#endif
#ifndef TTN_WIDE_ADALN_FWD_ROWS_PER_BLOCK
#define TTN_WIDE_ADALN_FWD_ROWS_PER_BLOCK 4
#endif
// Stores: 1 = write-through at device scope (RowWriter<1>), 0 = plain streaming store.
#ifndef TTN_WIDE_FWD_STORE
#define TTN_WIDE_FWD_STORE 0
#endif
#ifndef TTN_WIDE_BWD_STORE
#define TTN_WIDE_BWD_STORE 1
#endif
// Forward: 1 = the next row is requested before the current row's output pass.
#ifndef TTN_WIDE_FWD_PREFETCH
#define TTN_WIDE_FWD_PREFETCH 1
#endif
// AdaLN forward, 2-byte rows: 1 = rnd(1 + scale) and shift stay resident as fp32 values (unpacked once per workgroup),
// 0 = they stay packed and are unpacked for every row.
#ifndef TTN_WIDE_FWD_PARAMS_F32
#define TTN_WIDE_FWD_PARAMS_F32 1
#endif
// Backward: 1 = the next row's g and x are requested between the two passes of the current row; 0 = a row is
// requested when the one before it is done (the two workgroups of a compute unit overlap each other instead:
// 347 / 372 us against 380 / 385 us for RMSNorm / AdaLN backward at 89 100 x 4096 two-byte columns, and one
// workgroup per compute unit without the request ahead is far slower, 504 / 560 us).
#ifndef TTN_WIDE_BWD_PREFETCH
#define TTN_WIDE_BWD_PREFETCH 0
#endif

namespace ttn {

#ifndef TTN_GATED_3072_WIDE
#define TTN_GATED_3072_WIDE 0
#endif
// Measurement builds: 1 = the dense backward at 3072 two-byte columns on these kernels instead of the tuned ones.
#ifndef TTN_16BIT_3072_BWD_WIDE
#define TTN_16BIT_3072_BWD_WIDE 0
#endif
// narrower rows belong to the one-wavefront-per-row kernels
constexpr int kWidePiecesMin = (TTN_GATED_3072_WIDE || TTN_16BIT_3072_BWD_WIDE) ? 384 : 385;

// Which of this lane's CH accesses lie inside a row of `pieces` 16-byte pieces, for wavefront `wave`.
template <int CH>
struct WideMask {
    bool in[CH];
    __device__ __forceinline__ WideMask(int wave, int lane, int pieces, int ppw) {
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            const int at = k * kWaveSize + lane;  // piece inside the wavefront's slice
            in[k] = at < ppw && wave * ppw + at < pieces;
        }
    }
};

template <int CH>
__device__ __forceinline__ void wide_load(u32x4 (&dst)[CH], const u32x4 *p, bool ok, const WideMask<CH> &m) {
#pragma unroll
    for (int k = 0; k < CH; ++k) dst[k] = (ok && m.in[k]) ? load16_stream(p + k * kWaveSize) : u32x4{0, 0, 0, 0};
}

__device__ __forceinline__ float uniform(float v) {
    return as_f32((uint32_t)__builtin_amdgcn_readfirstlane((int)as_u32(v)));
}

// Every wavefront deposits N wave-uniform values; after one barrier all of them can be read back as
// slot[w * N + n].  Callers alternate between two slots from row to row, so a wavefront that runs ahead
// into the next row writes the other slot while the slower ones still read this one.
template <int N>
__device__ __forceinline__ void wide_exchange(const float (&v)[N], float *slot, int wave, int lane) {
    if (lane == 0) {
#pragma unroll
        for (int n = 0; n < N; ++n) slot[wave * N + n] = v[n];
    }
    __syncthreads();
}

// sum over the four wavefronts of value n, in wavefront order
template <int N>
__device__ __forceinline__ float wide_total(const float *slot, int n) {
    return uniform(((slot[n] + slot[N + n]) + slot[2 * N + n]) + slot[3 * N + n]);
}

// ------------------------------------------------------------------ RMSNorm

template <typename T, int CH>
__global__ __launch_bounds__(kRowThreads) void wide_rmsnorm_fwd_kernel(T *__restrict__ out, float *__restrict__ rstd,
                                                                       const T *__restrict__ x, const T *__restrict__ w,
                                                                       int64_t rows, int C, int ppw, float eps) {
    using E = Elem<T>;
    constexpr int VEC = E::VEC;
    __shared__ float xch[2][kRowWaves];
    const int lane = threadIdx.x & 63;
    const int wave = wave_id_in_block();
    const WideMask<CH> m(wave, lane, C / VEC, ppw);
    const int64_t slice = (int64_t)wave * ppw * VEC;  // first column of this wavefront's slice

    u32x4 wr[CH];
#pragma unroll
    for (int k = 0; k < CH; ++k)
        wr[k] = m.in[k] ? load16(reinterpret_cast<const u32x4 *>(w + slice) + k * kWaveSize + lane) : u32x4{0, 0, 0, 0};

    int parity = 0;
    u32x4 xr[CH];
    if ((int64_t)blockIdx.x < rows)
        wide_load<CH>(xr, reinterpret_cast<const u32x4 *>(x + (int64_t)blockIdx.x * C + slice) + lane, true, m);
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x, parity ^= 1) {
        keep_packed(wr);
#if !TTN_WIDE_FWD_PREFETCH
        if (row != (int64_t)blockIdx.x) wide_load<CH>(xr, reinterpret_cast<const u32x4 *>(x + row * C + slice) + lane, true, m);
#endif
        float ss = 0.0f;
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            float v[VEC];
            E::unpack(xr[k], v);
#pragma unroll
            for (int j = 0; j < VEC; ++j) ss = fmaf(v[j], v[j], ss);
        }
        const float part[1] = {group_sum<kWaveSize>(ss)};
        wide_exchange<1>(part, xch[parity], wave, lane);
#if TTN_WIDE_FWD_PREFETCH
        u32x4 xn[CH];
        const int64_t next = row + gridDim.x;
        wide_load<CH>(xn, reinterpret_cast<const u32x4 *>(x + next * C + slice) + lane, next < rows, m);
#endif
        const float r = 1.0f / sqrtf(wide_total<1>(xch[parity], 0) / (float)C + eps);
        if (wave == 0 && lane == 0) rstd[row] = r;

        const RowWriter<TTN_WIDE_FWD_STORE> wo(out + row * C + slice, lane * 16);
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            float v[VEC], wv[VEC];
            E::unpack(xr[k], v);
            E::unpack(wr[k], wv);
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] *= r;
            E::round(v);  // y = normalised row in the element type
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] *= wv[j];
            if (m.in[k]) wo.put(k * kWaveSize, E::pack(v));
        }
#if TTN_WIDE_FWD_PREFETCH
#pragma unroll
        for (int k = 0; k < CH; ++k) xr[k] = xn[k];
#endif
    }
}

// The resident second factor of gy = rnd(g * w) / gx = rnd(g * t): masked pairs (or packed halves) for
// 2-byte rows, fp32 values for 4-byte rows.
template <typename T, int CH>
struct WideParam {
    using E = Elem<T>;
    using Factor = PairFactor<std::conditional_t<kHasDot2<T>, T, bf16_t>>;
    Factor f[kHasDot2<T> ? CH : 1];
    float v[kHasDot2<T> ? 1 : CH][E::VEC];
    __device__ __forceinline__ void set(int k, const u32x4 &packed) {
        if constexpr (kHasDot2<T>)
            f[k].set(packed);
        else
            E::unpack(packed, v[k]);
    }
    // rnd(g * param) for access k, in the element type
    __device__ __forceinline__ u32x4 times(int k, const u32x4 &g) const {
        if constexpr (kHasDot2<T>) {
            return rounded_products<T>(g, f[k]);
        } else {
            float gv[E::VEC];
            E::unpack(g, gv);
#pragma unroll
            for (int j = 0; j < E::VEC; ++j) gv[j] *= v[k][j];
            return E::pack(gv);
        }
    }
};

// acc += rnd(g * rnd(n)) per column, n the eight (four) fp32 values of the normalised row for this access
template <typename T>
__device__ __forceinline__ void add_rounded_products(float (&acc)[Elem<T>::VEC], const u32x4 &g,
                                                     float (&n)[Elem<T>::VEC], uint32_t one_lo, uint32_t one_hi) {
    using E = Elem<T>;
    if constexpr (kHasDot2<T>) {
        PairFactor<T> nf;
        nf.set_rounded(n);
        const u32x4 pp = rounded_products<T>(g, nf);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc[2 * i] = dot2<T>(pp[i], one_lo, acc[2 * i]);
            acc[2 * i + 1] = dot2<T>(pp[i], one_hi, acc[2 * i + 1]);
        }
    } else {
        float gv[E::VEC];
        E::unpack(g, gv);
        E::round(n);
#pragma unroll
        for (int j = 0; j < E::VEC; ++j) n[j] *= gv[j];
        E::round(n);
#pragma unroll
        for (int j = 0; j < E::VEC; ++j) acc[j] += n[j];
    }
}

// acc += g per column
template <typename T>
__device__ __forceinline__ void add_elements(float (&acc)[Elem<T>::VEC], const u32x4 &g, uint32_t one_lo, uint32_t one_hi) {
    using E = Elem<T>;
    if constexpr (kHasDot2<T>) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc[2 * i] = dot2<T>(g[i], one_lo, acc[2 * i]);
            acc[2 * i + 1] = dot2<T>(g[i], one_hi, acc[2 * i + 1]);
        }
    } else {
        float gv[E::VEC];
        E::unpack(g, gv);
#pragma unroll
        for (int j = 0; j < E::VEC; ++j) acc[j] += gv[j];
    }
}

// This wavefront's column sums into its slice of the workgroup's partial row (NSETS sets of C columns).
template <typename T, int CH, int NSETS>
__device__ __forceinline__ void wide_store_partials(float (&acc)[NSETS][CH][Elem<T>::VEC], float *partial_row, int C,
                                                    int64_t slice, int lane, const WideMask<CH> &m) {
    constexpr int VEC = Elem<T>::VEC;
#pragma unroll
    for (int s = 0; s < NSETS; ++s)
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            if (!m.in[k]) continue;
            float *p = partial_row + (int64_t)s * C + slice + (k * kWaveSize + lane) * VEC;
#pragma unroll
            for (int q = 0; q < VEC / 4; ++q) {
                // copies the compiler cannot see through, so that the 16-byte store does not pin the accumulators to
                // groups of four consecutive registers for the whole kernel (see flush_column_partials)
                float a0 = acc[s][k][4 * q], a1 = acc[s][k][4 * q + 1], a2 = acc[s][k][4 * q + 2], a3 = acc[s][k][4 * q + 3];
                asm volatile("" : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3));
                *reinterpret_cast<u32x4 *>(p + 4 * q) = u32x4{as_u32(a0), as_u32(a1), as_u32(a2), as_u32(a3)};
            }
        }
}

template <typename T, int CH>
__global__ __launch_bounds__(kRowThreads) void wide_rmsnorm_bwd_kernel(T *__restrict__ dx, float *__restrict__ partial,
                                                                       const T *__restrict__ g, const T *__restrict__ x,
                                                                       const T *__restrict__ w,
                                                                       const float *__restrict__ rstd, int64_t rows, int C, int ppw) {
    using E = Elem<T>;
    constexpr int VEC = E::VEC;
    __shared__ float xch[2][kRowWaves];
    const int lane = threadIdx.x & 63;
    const int wave = wave_id_in_block();
    const WideMask<CH> m(wave, lane, C / VEC, ppw);
    const int64_t slice = (int64_t)wave * ppw * VEC;
    const uint32_t one_lo = opaque_const(kOneLo<std::conditional_t<kHasDot2<T>, T, bf16_t>>);
    const uint32_t one_hi = opaque_const(kOneHi<std::conditional_t<kHasDot2<T>, T, bf16_t>>);

    WideParam<T, CH> wp;
#pragma unroll
    for (int k = 0; k < CH; ++k)
        wp.set(k, m.in[k] ? load16(reinterpret_cast<const u32x4 *>(w + slice) + k * kWaveSize + lane) : u32x4{0, 0, 0, 0});
    float acc[1][CH][VEC];
#pragma unroll
    for (int k = 0; k < CH; ++k)
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[0][k][j] = 0.0f;

    struct Row {
        u32x4 g[CH], x[CH];
        float r;
    };
    auto fetch = [&](Row &b, int64_t row) {
        const bool ok = row < rows;
        wide_load<CH>(b.g, reinterpret_cast<const u32x4 *>(g + row * C + slice) + lane, ok, m);
        wide_load<CH>(b.x, reinterpret_cast<const u32x4 *>(x + row * C + slice) + lane, ok, m);
        b.r = ok ? rstd[wave_uniform(row)] : 0.0f;
    };
    int parity = 0;
    auto process = [&](Row &b, int64_t row, auto &&between_passes) {
        const float r = b.r;
        // pass 1: gy = rnd(g*w) kept packed; this wavefront's share of sum_c gy * x
        u32x4 gyp[CH];
        float dot = 0.0f;
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            gyp[k] = wp.times(k, b.g[k]);
            if constexpr (kHasDot2<T>) {
#pragma unroll
                for (int i = 0; i < 4; ++i) dot = dot2<T>(gyp[k][i], b.x[k][i], dot);
            } else {
                float gy[VEC], xv[VEC];
                E::unpack(gyp[k], gy);
                E::unpack(b.x[k], xv);
#pragma unroll
                for (int j = 0; j < VEC; ++j) dot = fmaf(gy[j], xv[j], dot);
            }
        }
        const float part[1] = {group_sum<kWaveSize>(dot)};
        wide_exchange<1>(part, xch[parity], wave, lane);
        between_passes();
        const float coef = -((wide_total<1>(xch[parity], 0) / (float)C) * r * r * r);
        parity ^= 1;

        const RowWriter<TTN_WIDE_BWD_STORE> wd(dx + row * C + slice, lane * 16);
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            float gy[VEC], xv[VEC], o[VEC], y[VEC];
            E::unpack(gyp[k], gy);
            E::unpack(b.x[k], xv);
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                o[j] = fmaf(xv[j], coef, gy[j] * r);
                y[j] = xv[j] * r;
            }
            if (m.in[k]) wd.put(k * kWaveSize, E::pack(o));
            add_rounded_products<T>(acc[0][k], b.g[k], y, one_lo, one_hi);  // dw += rnd(g * rnd(y))
        }
    };

    const int64_t stride = gridDim.x;
    int64_t row = blockIdx.x;
    if (row < rows) {
#if TTN_WIDE_BWD_PREFETCH
        Row b0, b1;
        fetch(b0, row);
        for (;;) {
            process(b0, row, [&] { fetch(b1, row + stride); });
            row += stride;
            if (row >= rows) break;
            process(b1, row, [&] { fetch(b0, row + stride); });
            row += stride;
            if (row >= rows) break;
        }
#else
        for (; row < rows; row += stride) {
            Row b0;
            fetch(b0, row);
            process(b0, row, [] {});
        }
#endif
    }
    wide_store_partials<T, CH, 1>(acc, partial + (int64_t)blockIdx.x * C, C, slice, lane, m);
}

// -------------------------------------------------------------------- AdaLN

// GATED: the row that is normalised is h2 = rnd(x + rnd(attn * gate[b])), which is written out too (the gated
// residual update in front of the norm; same form as the kernels of adaln.hip / anywidth.hip).
template <typename T, int CH, bool GATED>
__global__ __launch_bounds__(kRowThreads) void wide_adaln_fwd_kernel(T *__restrict__ out, float *__restrict__ mean,
                                                                     float *__restrict__ rstd, const T *__restrict__ x,
                                                                     const T *__restrict__ scale,
                                                                     const T *__restrict__ shift, T *__restrict__ h2_out,
                                                                     const T *__restrict__ attn, const T *__restrict__ gate,
                                                                     int64_t rows_per_sample,
                                                                     const SampleLayout lay, int blocks_per_sample, int C,
                                                                     int ppw, float eps) {
    using E = Elem<T>;
    constexpr int VEC = E::VEC;
    __shared__ float xch[2][kRowWaves * 2];
    const int lane = threadIdx.x & 63;
    const int wave = wave_id_in_block();
    const int64_t b = blockIdx.x / blocks_per_sample;
    const int slot = blockIdx.x % blocks_per_sample;
    const WideMask<CH> m(wave, lane, C / VEC, ppw);
    const int64_t slice = (int64_t)wave * ppw * VEC;
    // columns of the row inside wavefront i's slice
    auto cols_of = [&](int i) { return max(0, min(ppw * VEC, C - i * ppw * VEC)); };
    float inv_n[kRowWaves];  // 1 / columns of each wavefront's slice (0 for an empty slice)
#pragma unroll
    for (int i = 0; i < kRowWaves; ++i) inv_n[i] = cols_of(i) > 0 ? 1.0f / (float)cols_of(i) : 0.0f;
    const float inv_n_mine = cols_of(wave) > 0 ? 1.0f / (float)cols_of(wave) : 0.0f;  // the same bits as inv_n[wave]
    const float inv_c = 1.0f / (float)C;

    // rnd(1 + scale) and shift of this wavefront's columns: packed as they arrive, or (2-byte rows) as fp32 values
    constexpr bool kParamsF32 = TTN_WIDE_FWD_PARAMS_F32 && sizeof(T) == 2;
    u32x4 tr[kParamsF32 ? 1 : CH], hr[kParamsF32 ? 1 : CH];
    float tf[kParamsF32 ? CH : 1][VEC], hf[kParamsF32 ? CH : 1][VEC];
#pragma unroll
    for (int k = 0; k < CH; ++k) {
        const u32x4 zero{0, 0, 0, 0};
        const u32x4 tp = m.in[k] ? load16(reinterpret_cast<const u32x4 *>(scale + b * C + slice) + k * kWaveSize + lane) : zero;
        const u32x4 hp = m.in[k] ? load16(reinterpret_cast<const u32x4 *>(shift + b * C + slice) + k * kWaveSize + lane) : zero;
        float v[VEC];
        E::unpack(tp, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = 1.0f + v[j];
        if constexpr (kParamsF32) {
            E::round(v);  // t = rnd(1 + scale)
#pragma unroll
            for (int j = 0; j < VEC; ++j) tf[k][j] = v[j];
            E::unpack(hp, hf[k]);
        } else {
            tr[k] = E::pack(v);  // t = rnd(1 + scale)
            hr[k] = hp;
        }
    }

    [[maybe_unused]] u32x4 qr[GATED ? CH : 1];  // gate[b], packed
    if constexpr (GATED) {
#pragma unroll
        for (int k = 0; k < CH; ++k)
            qr[k] = m.in[k] ? load16(reinterpret_cast<const u32x4 *>(gate + b * C + slice) + k * kWaveSize + lane)
                            : u32x4{0, 0, 0, 0};
    }

    int parity = 0;
    u32x4 xr[CH];
    [[maybe_unused]] u32x4 ar[GATED ? CH : 1];
    if (slot < rows_per_sample) {
        wide_load<CH>(xr, reinterpret_cast<const u32x4 *>(x + lay.row(b, slot) * C + slice) + lane, true, m);
        if constexpr (GATED)
            wide_load<CH>(ar, reinterpret_cast<const u32x4 *>(attn + lay.row(b, slot) * C + slice) + lane, true, m);
    }
    for (int64_t rs = slot; rs < rows_per_sample; rs += blocks_per_sample, parity ^= 1) {
        if constexpr (!kParamsF32) {
            keep_packed(tr);
            keep_packed(hr);
        }
        if constexpr (GATED) keep_packed(qr);
        const int64_t row = lay.row(b, rs);
#if !TTN_WIDE_FWD_PREFETCH
        if (rs != slot) {
            wide_load<CH>(xr, reinterpret_cast<const u32x4 *>(x + row * C + slice) + lane, true, m);
            if constexpr (GATED) wide_load<CH>(ar, reinterpret_cast<const u32x4 *>(attn + row * C + slice) + lane, true, m);
        }
#endif
        if constexpr (GATED) {
            const RowWriter<0> wh(h2_out + row * C + slice, lane * 16);
#pragma unroll
            for (int k = 0; k < CH; ++k) {
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
                if (m.in[k]) wh.put(k * kWaveSize, xr[k]);
            }
        }
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            if constexpr (kHasDot2<T>) {
#pragma unroll
                for (int i = 0; i < 4; ++i) s = dot2<T>(xr[k][i], kOnesPair<T>, s);
            } else {
                float v[VEC];
                E::unpack(xr[k], v);
#pragma unroll
                for (int j = 0; j < VEC; ++j) s += v[j];
            }
        }
        s = group_sum<kWaveSize>(s);
        const float m_mine = s * inv_n_mine;  // the centre of this wavefront's squares; any value near its mean serves
        float q = 0.0f;
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            float v[VEC];
            E::unpack(xr[k], v);
            if (m.in[k]) {  // padding must not count as (0 - mean)^2
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const float d = v[j] - m_mine;
                    q = fmaf(d, d, q);
                }
            }
        }
        const float part[2] = {s, group_sum<kWaveSize>(q)};
        wide_exchange<2>(part, xch[parity], wave, lane);
#if TTN_WIDE_FWD_PREFETCH
        u32x4 xn[CH];
        const int64_t rs_next = rs + blocks_per_sample;
        const bool more = rs_next < rows_per_sample;
        wide_load<CH>(xn, reinterpret_cast<const u32x4 *>(x + lay.row(b, more ? rs_next : rs) * C + slice) + lane, more, m);
        [[maybe_unused]] u32x4 an[GATED ? CH : 1];
        if constexpr (GATED)
            wide_load<CH>(an, reinterpret_cast<const u32x4 *>(attn + lay.row(b, more ? rs_next : rs) * C + slice) + lane, more, m);
#endif
        const float *sl = xch[parity];
        const float mu = wide_total<2>(sl, 0) / (float)C;
        float m2 = 0.0f;
#pragma unroll
        for (int i = 0; i < kRowWaves; ++i) {  // merge of the per-wavefront sums of squares about their own centres
            const float d = sl[2 * i] * inv_n[i] - mu;  // an empty slice contributes q = 0 and n = 0
            m2 += sl[2 * i + 1] + (float)cols_of(i) * d * d;
        }
        const float r = 1.0f / sqrtf(uniform(m2) * inv_c + eps);
        if (wave == 0 && lane == 0) {
            mean[row] = mu;
            rstd[row] = r;
        }

        const float nmr = -(mu * r);
        const RowWriter<TTN_WIDE_FWD_STORE> wo(out + row * C + slice, lane * 16);
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            float v[VEC], tv[VEC], hv[VEC];
            E::unpack(xr[k], v);
            if constexpr (kParamsF32) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    tv[j] = tf[k][j];
                    hv[j] = hf[k][j];
                }
            } else {
                E::unpack(tr[k], tv);
                E::unpack(hr[k], hv);
            }
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] = centred<T>(v[j], mu, r, nmr);
            E::round(v);  // xn
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] *= tv[j];
            E::round(v);  // xn * (1 + scale)
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] += hv[j];
            if (m.in[k]) wo.put(k * kWaveSize, E::pack(v));
        }
#if TTN_WIDE_FWD_PREFETCH
#pragma unroll
        for (int k = 0; k < CH; ++k) xr[k] = xn[k];
        if constexpr (GATED) {
#pragma unroll
            for (int k = 0; k < CH; ++k) ar[k] = an[k];
        }
#endif
    }
}

// GATED: x is the saved h2; dx = dh = rnd(rnd(dx of the norm) + e) with e the gradient arriving at h2 from its other
// use (may be null), da = rnd(dh * gate[b]) is written too and dgate[b] += rnd(dh * attn) is a third set of column
// sums.  RES: dx = rnd(rnd(dx of the norm) + e), e the gradient the input receives from its other consumer.
template <typename T, int CH, bool GATED, bool RES>
__global__ __launch_bounds__(kRowThreads) void wide_adaln_bwd_kernel(T *__restrict__ dx, float *__restrict__ partial,
                                                                     const T *__restrict__ g, const T *__restrict__ x,
                                                                     const T *__restrict__ scale,
                                                                     const float *__restrict__ mean,
                                                                     const float *__restrict__ rstd, T *__restrict__ da,
                                                                     const T *__restrict__ e, const T *__restrict__ attn,
                                                                     const T *__restrict__ gate, int64_t rows_per_sample,
                                                                     const SampleLayout lay, int blocks_per_sample, int C,
                                                                     int ppw) {
    static_assert(!(GATED && RES), "the gated form handles e itself");
    constexpr int NSETS = GATED ? 3 : 2;
    using E = Elem<T>;
    constexpr int VEC = E::VEC;
    __shared__ float xch[2][kRowWaves * 2];
    const int lane = threadIdx.x & 63;
    const int wave = wave_id_in_block();
    const int64_t smp = blockIdx.x / blocks_per_sample;
    const int slot = blockIdx.x % blocks_per_sample;
    const WideMask<CH> m(wave, lane, C / VEC, ppw);
    const int64_t slice = (int64_t)wave * ppw * VEC;
    const uint32_t one_lo = opaque_const(kOneLo<std::conditional_t<kHasDot2<T>, T, bf16_t>>);
    const uint32_t one_hi = opaque_const(kOneHi<std::conditional_t<kHasDot2<T>, T, bf16_t>>);

    WideParam<T, CH> tp;  // t = rnd(1 + scale[sample])
#pragma unroll
    for (int k = 0; k < CH; ++k) {
        float v[VEC];
        E::unpack(m.in[k] ? load16(reinterpret_cast<const u32x4 *>(scale + smp * C + slice) + k * kWaveSize + lane)
                          : u32x4{0, 0, 0, 0}, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = 1.0f + v[j];
        tp.set(k, E::pack(v));
    }
    [[maybe_unused]] u32x4 qr[GATED ? CH : 1];  // gate[sample], packed
    if constexpr (GATED) {
#pragma unroll
        for (int k = 0; k < CH; ++k)
            qr[k] = m.in[k] ? load16(reinterpret_cast<const u32x4 *>(gate + smp * C + slice) + k * kWaveSize + lane)
                            : u32x4{0, 0, 0, 0};
    }
    float acc[NSETS][CH][VEC];  // [0] = dscale, [1] = dshift, [2] = dgate
#pragma unroll
    for (int s = 0; s < NSETS; ++s)
#pragma unroll
        for (int k = 0; k < CH; ++k)
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[s][k][j] = 0.0f;

    struct Row {
        u32x4 g[CH], x[CH];
        u32x4 e[(GATED || RES) ? CH : 1], a[GATED ? CH : 1];
        float r, mu;
        int64_t row;
    };
    auto fetch = [&](Row &b, int64_t rs) {
        const bool ok = rs < rows_per_sample;
        b.row = lay.row(smp, ok ? rs : 0);
        wide_load<CH>(b.g, reinterpret_cast<const u32x4 *>(g + b.row * C + slice) + lane, ok, m);
        wide_load<CH>(b.x, reinterpret_cast<const u32x4 *>(x + b.row * C + slice) + lane, ok, m);
        if constexpr (GATED || RES)
            wide_load<CH>(b.e, reinterpret_cast<const u32x4 *>(e + b.row * C + slice) + lane, ok && e != nullptr, m);
        if constexpr (GATED) wide_load<CH>(b.a, reinterpret_cast<const u32x4 *>(attn + b.row * C + slice) + lane, ok, m);
        const int64_t srow = wave_uniform(b.row);
        b.r = ok ? rstd[srow] : 0.0f;
        b.mu = ok ? mean[srow] : 0.0f;
    };
    int parity = 0;
    auto process = [&](Row &b, auto &&between_passes) {
        const float r = b.r, mu = b.mu;
        const float nmr = -(mu * r);  // xhat = x*r + nmr
        // pass 1: gx = rnd(g*t) kept packed; this wavefront's share of sum_c gx and sum_c gx * x (2-byte) / gx * xhat
        u32x4 gxp[CH];
        float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            gxp[k] = tp.times(k, b.g[k]);
            if constexpr (kHasDot2<T>) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    s1 = dot2<T>(gxp[k][i], kOnesPair<T>, s1);
                    s2 = dot2<T>(gxp[k][i], b.x[k][i], s2);
                }
            } else {
                float gx[VEC], xv[VEC];
                E::unpack(gxp[k], gx);
                E::unpack(b.x[k], xv);
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    s1 += gx[j];
                    s2 = fmaf(gx[j], centred<T>(xv[j], mu, r, nmr), s2);  // padding: gx = 0 there
                }
            }
        }
        const float part[2] = {group_sum<kWaveSize>(s1), group_sum<kWaveSize>(s2)};
        wide_exchange<2>(part, xch[parity], wave, lane);
        between_passes();
        s1 = wide_total<2>(xch[parity], 0);
        s2 = wide_total<2>(xch[parity], 1);
        parity ^= 1;
        if constexpr (kHasDot2<T>) s2 = r * (s2 - mu * s1);
        const float m1 = s1 / (float)C, m2 = s2 / (float)C;
        // dx = r*(gx - m1 - xhat*m2) = r*gx + x*K1 + K0
        const float k1 = -(r * m2), k0 = -(r * m1);
        const float K1 = k1 * r;
        const float K0 = fmaf(k1, nmr, k0);

        const RowWriter<GATED ? 0 : TTN_WIDE_BWD_STORE> wd(dx + b.row * C + slice, lane * 16);
        const RowWriter<0> wa(GATED ? da + b.row * C + slice : nullptr, lane * 16);
        if constexpr (GATED) keep_packed(qr);
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            float gx[VEC], xv[VEC], o[VEC], xn[VEC];
            E::unpack(gxp[k], gx);
            E::unpack(b.x[k], xv);
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                o[j] = fmaf(r, gx[j], fmaf(xv[j], K1, K0));
                xn[j] = centred<T>(xv[j], mu, r, nmr);
            }
            if constexpr (GATED || RES) {
                float ev[VEC];
                E::round(o);  // the norm's dx, materialised in the element type
                E::unpack(b.e[k], ev);
#pragma unroll
                for (int j = 0; j < VEC; ++j) o[j] += ev[j];
            }
            const u32x4 dxp = E::pack(o);
            if (m.in[k]) wd.put(k * kWaveSize, dxp);
            if constexpr (GATED) {
                float av[VEC], qv[VEC];
                E::unpack(dxp, o);  // dh as stored
                E::unpack(b.a[k], av);
                E::unpack(qr[k], qv);
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    qv[j] *= o[j];
                    av[j] *= o[j];
                }
                if (m.in[k]) wa.put(k * kWaveSize, E::pack(qv));
                E::round(av);  // dh*attn materialised in the element type before the column sum
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc[2][k][j] += av[j];
            }
            add_elements<T>(acc[1][k], b.g[k], one_lo, one_hi);                // dshift += g (padding: g = 0)
            add_rounded_products<T>(acc[0][k], b.g[k], xn, one_lo, one_hi);    // dscale += rnd(g * rnd(xhat))
        }
    };

    const int64_t stride = blocks_per_sample;
    int64_t rs = slot;
    if (rs < rows_per_sample) {
#if TTN_WIDE_BWD_PREFETCH
        Row b0, b1;
        fetch(b0, rs);
        for (;;) {
            process(b0, [&] { fetch(b1, rs + stride); });
            rs += stride;
            if (rs >= rows_per_sample) break;
            process(b1, [&] { fetch(b0, rs + stride); });
            rs += stride;
            if (rs >= rows_per_sample) break;
        }
#else
        for (; rs < rows_per_sample; rs += stride) {
            Row b0;
            fetch(b0, rs);
            process(b0, [] {});
        }
#endif
    }
    wide_store_partials<T, CH, NSETS>(acc, partial + (int64_t)blockIdx.x * (NSETS * C), C, slice, lane, m);
}

// ------------------------------------------------------------------ host side

bool widerow_takes(int64_t cols, int dtype) {
    if (!anywidth_supported(cols, dtype)) return false;
    return cols / (16 / (int64_t)elem_bytes(dtype)) >= kWidePiecesMin;
}

#ifndef TTN_F32_3072_BWD_WIDE
#define TTN_F32_3072_BWD_WIDE 1
#endif
bool gated_forward_on_wide_rows(int64_t cols, int dtype) {
    return TTN_GATED_3072_WIDE && TTN_WIDE_ROWS && dtype != TT_NORM_F32 && cols == 3072;
}
bool dense_backward_on_wide_rows(int64_t cols, int dtype) {
    if (TTN_16BIT_3072_BWD_WIDE && TTN_WIDE_ROWS && dtype != TT_NORM_F32 && cols == 3072) return true;
    return TTN_F32_3072_BWD_WIDE && TTN_WIDE_ROWS && dtype == TT_NORM_F32 && cols == 3072;
}

// pieces per wavefront (a quarter of the row, rounded up) and the accesses per lane that takes
static int wide_pieces_per_wave(int64_t cols, int dtype) {
    const int64_t pieces = cols / (16 / (int64_t)elem_bytes(dtype));
    return (int)((pieces + kRowWaves - 1) / kRowWaves);
}
static int wide_chunks(int64_t cols, int dtype) {
    return (wide_pieces_per_wave(cols, dtype) + kWaveSize - 1) / kWaveSize;  // 2, 3 or 4 for 385..1024 pieces
}

// Workgroups of `kernel` that one compute unit holds at a time (asked of the runtime once per kernel): a
// persistent grid must not be larger than what is resident, or its surplus workgroups run as a second round.
template <typename K>
static int resident_blocks_per_cu(K kernel, int wanted) {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, kRowThreads, 0) != hipSuccess || n < 1) {
        (void)hipGetLastError();
        return wanted;
    }
    return n < wanted ? n : wanted;
}

// One row per workgroup and step: `per_cu` workgroups per compute unit, split evenly over the samples.
// With rows_per_block > 0 the grid is sized by the rows instead: workgroups of that many rows each, which retire
// and are replaced as the grid drains.
static int wide_plan(RowPlan *p, int64_t batch, int64_t rows_per_sample, int per_cu, int rows_per_block = 0) {
    int st = TT_NORM_OK;
    const int cus = current_device_cus(&st);
    if (st != TT_NORM_OK) return st;
    int64_t budget = ((int64_t)cus * per_cu) / batch;
    if (rows_per_block > 0) budget = (rows_per_sample + rows_per_block - 1) / rows_per_block;
    if (budget < 1) budget = 1;
    const int64_t bps = rows_per_sample < budget ? (rows_per_sample > 0 ? rows_per_sample : 1) : budget;
    p->rows_per_wave = 1;
    p->blocks_per_sample = (int)bps;
    p->blocks = batch * bps;
    if (p->blocks > 0x7fffffffLL) return fail(TT_NORM_EINVAL, "grid too large");
    return TT_NORM_OK;
}

size_t widerow_backward_workspace_bytes(int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype, int nsets) {
    if (batch <= 0 || rows_per_sample <= 0 || !widerow_takes(cols, dtype)) return 0;
    RowPlan p;
    if (wide_plan(&p, batch, rows_per_sample, TTN_WIDE_BWD_BLOCKS_PER_CU) != TT_NORM_OK) return 0;
    return (size_t)p.blocks * nsets * cols * sizeof(float);
}

#define TTN_WIDE_DISPATCH(dtype, ch, CALL)                                    \
    do {                                                                      \
        if ((dtype) == TT_NORM_BF16) {                                        \
            if ((ch) == 2) { CALL(bf16_t, 2); } else if ((ch) == 3) { CALL(bf16_t, 3); } else { CALL(bf16_t, 4); } \
        } else if ((dtype) == TT_NORM_F16) {                                  \
            if ((ch) == 2) { CALL(f16_t, 2); } else if ((ch) == 3) { CALL(f16_t, 3); } else { CALL(f16_t, 4); }    \
        } else {                                                              \
            if ((ch) == 2) { CALL(float, 2); } else if ((ch) == 3) { CALL(float, 3); } else { CALL(float, 4); }    \
        }                                                                     \
    } while (0)

int widerow_rmsnorm_forward(void *out, float *rstd, const void *x, const void *w, int64_t rows, int64_t cols,
                            double eps, int dtype, hipStream_t stream) {
    if (rows == 0) return TT_NORM_OK;
    RowPlan p;
    int st = TT_NORM_OK;
    const int ch = wide_chunks(cols, dtype), ppw = wide_pieces_per_wave(cols, dtype);
    {
        RowKernelProfile prof(stream);
#define CALL(T, CH)                                                                                         \
    do {                                                                                                    \
        static const int per_cu = resident_blocks_per_cu(wide_rmsnorm_fwd_kernel<T, CH>, TTN_WIDE_FWD_BLOCKS_PER_CU); \
        st = wide_plan(&p, 1, rows, per_cu, TTN_WIDE_RMS_FWD_ROWS_PER_BLOCK);                               \
        if (st != TT_NORM_OK) return st;                                                                    \
        wide_rmsnorm_fwd_kernel<T, CH><<<dim3((unsigned)p.blocks), dim3(kRowThreads), 0, stream>>>(         \
            (T *)out, rstd, (const T *)x, (const T *)w, rows, (int)cols, ppw, (float)eps);                  \
    } while (0)
        TTN_WIDE_DISPATCH(dtype, ch, CALL);
#undef CALL
    }
    return check_launch("rmsnorm forward launch (wide rows)");
}

int widerow_rmsnorm_backward(void *dx, void *dw, const void *g, const void *x, const void *w, const float *rstd,
                             int64_t rows, int64_t cols, int dtype, void *ws, size_t ws_bytes, hipStream_t stream) {
    if (rows == 0) return launch_colreduce(dw, nullptr, nullptr, nullptr, 1, 0, cols, cols, dtype, stream);
    RowPlan p;
    int st = wide_plan(&p, 1, rows, TTN_WIDE_BWD_BLOCKS_PER_CU);
    if (st != TT_NORM_OK) return st;
    const size_t need = (size_t)p.blocks * cols * sizeof(float);
    if (!ws || ws_bytes < need)
        return fail(TT_NORM_EWORKSPACE, "rmsnorm backward: workspace %zu B < required %zu B", ws_bytes, need);
    if (!aligned16(ws)) return fail(TT_NORM_EALIGN, "rmsnorm backward: workspace %p not 16-byte aligned", ws);
    const int ch = wide_chunks(cols, dtype), ppw = wide_pieces_per_wave(cols, dtype);
    {
        RowKernelProfile prof(stream);
#define CALL(T, CH)                                                                                         \
    wide_rmsnorm_bwd_kernel<T, CH><<<dim3((unsigned)p.blocks), dim3(kRowThreads), 0, stream>>>(             \
        (T *)dx, (float *)ws, (const T *)g, (const T *)x, (const T *)w, rstd, rows, (int)cols, ppw)
        TTN_WIDE_DISPATCH(dtype, ch, CALL);
#undef CALL
    }
    st = check_launch("rmsnorm backward launch (wide rows)");
    if (st != TT_NORM_OK) return st;
    return launch_colreduce(dw, nullptr, nullptr, (const float *)ws, 1, p.blocks_per_sample, cols, cols, dtype, stream);
}

struct WideExtra {  // operands of the gated / residual forms (null otherwise)
    void *h2_or_da;    // forward: h2 out; backward: da out
    const void *e;     // backward: the gradient arriving at h2 / at the input from its other use
    const void *attn;
    const void *gate;
};

template <bool GATED>
static int wide_adaln_forward_t(void *out, float *mean, float *rstd, const void *x, const void *scale,
                                const void *shift, const WideExtra &ex, int64_t batch, int64_t rows_per_sample,
                                int64_t cols, double eps, int dtype, bool seq_first, hipStream_t stream) {
    if (rows_per_sample == 0) return TT_NORM_OK;
    RowPlan p;
    int st = TT_NORM_OK;
    const SampleLayout lay = seq_first ? SampleLayout{1, batch} : SampleLayout{rows_per_sample, 1};
    const int ch = wide_chunks(cols, dtype), ppw = wide_pieces_per_wave(cols, dtype);
    {
        RowKernelProfile prof(stream);
#define CALL(T, CH)                                                                                         \
    do {                                                                                                    \
        static const int per_cu =                                                                           \
            resident_blocks_per_cu(wide_adaln_fwd_kernel<T, CH, GATED>, TTN_WIDE_FWD_BLOCKS_PER_CU);        \
        st = wide_plan(&p, batch, rows_per_sample, per_cu, TTN_WIDE_ADALN_FWD_ROWS_PER_BLOCK);              \
        if (st != TT_NORM_OK) return st;                                                                    \
        wide_adaln_fwd_kernel<T, CH, GATED><<<dim3((unsigned)p.blocks), dim3(kRowThreads), 0, stream>>>(    \
            (T *)out, mean, rstd, (const T *)x, (const T *)scale, (const T *)shift, (T *)ex.h2_or_da,       \
            (const T *)ex.attn, (const T *)ex.gate, rows_per_sample, lay, p.blocks_per_sample, (int)cols,   \
            ppw, (float)eps);                                                                               \
    } while (0)
        TTN_WIDE_DISPATCH(dtype, ch, CALL);
#undef CALL
    }
    return check_launch("adaln forward launch (wide rows)");
}

int widerow_adaln_forward(void *out, float *mean, float *rstd, const void *x, const void *scale, const void *shift,
                          int64_t batch, int64_t rows_per_sample, int64_t cols, double eps, int dtype, bool seq_first,
                          hipStream_t stream) {
    return wide_adaln_forward_t<false>(out, mean, rstd, x, scale, shift, WideExtra{nullptr, nullptr, nullptr, nullptr},
                                       batch, rows_per_sample, cols, eps, dtype, seq_first, stream);
}

int widerow_gated_adaln_forward(void *h2, void *out, float *mean, float *rstd, const void *h, const void *attn,
                                const void *gate, const void *scale, const void *shift, int64_t batch,
                                int64_t rows_per_sample, int64_t cols, double eps, int dtype, hipStream_t stream) {
    return wide_adaln_forward_t<true>(out, mean, rstd, h, scale, shift, WideExtra{h2, nullptr, attn, gate}, batch,
                                      rows_per_sample, cols, eps, dtype, false, stream);
}

template <bool GATED, bool RES>
static int wide_adaln_backward_t(void *dx, void *dscale, void *dshift, void *dgate, const void *g, const void *x,
                                 const void *scale, const float *mean, const float *rstd, const WideExtra &ex,
                                 int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype, void *ws,
                                 size_t ws_bytes, bool seq_first, hipStream_t stream) {
    constexpr int NSETS = GATED ? 3 : 2;
    if (rows_per_sample == 0)
        return launch_colreduce(dscale, dshift, dgate, nullptr, batch, 0, cols, NSETS * cols, dtype, stream);
    RowPlan p;
    int st = TT_NORM_OK;
    const SampleLayout lay = seq_first ? SampleLayout{1, batch} : SampleLayout{rows_per_sample, 1};
    const int ch = wide_chunks(cols, dtype), ppw = wide_pieces_per_wave(cols, dtype);
    {
        RowKernelProfile prof(stream);
        // The same grid for the plain, gated and residual forms of a shape, so that their column sums are added in
        // the same order and the fused forms stay bit-identical to their parts; an instantiation whose registers
        // leave room for one workgroup per compute unit only (gated, four accesses per lane) runs its grid in two
        // rounds.
#define CALL(T, CH)                                                                                         \
    do {                                                                                                    \
        st = wide_plan(&p, batch, rows_per_sample, TTN_WIDE_BWD_BLOCKS_PER_CU);                             \
        if (st != TT_NORM_OK) return st;                                                                    \
        const size_t need = (size_t)p.blocks * NSETS * cols * sizeof(float);                                \
        if (!ws || ws_bytes < need)                                                                         \
            return fail(TT_NORM_EWORKSPACE, "adaln backward: workspace %zu B < required %zu B", ws_bytes, need); \
        if (!aligned16(ws)) return fail(TT_NORM_EALIGN, "adaln backward: workspace %p not 16-byte aligned", ws); \
        wide_adaln_bwd_kernel<T, CH, GATED, RES><<<dim3((unsigned)p.blocks), dim3(kRowThreads), 0, stream>>>( \
            (T *)dx, (float *)ws, (const T *)g, (const T *)x, (const T *)scale, mean, rstd, (T *)ex.h2_or_da, \
            (const T *)ex.e, (const T *)ex.attn, (const T *)ex.gate, rows_per_sample, lay, p.blocks_per_sample, \
            (int)cols, ppw);                                                                                \
    } while (0)
        TTN_WIDE_DISPATCH(dtype, ch, CALL);
#undef CALL
    }
    st = check_launch("adaln backward launch (wide rows)");
    if (st != TT_NORM_OK) return st;
    return launch_colreduce(dscale, dshift, dgate, (const float *)ws, batch, p.blocks_per_sample, cols, NSETS * cols,
                            dtype, stream);
}

int widerow_adaln_backward(void *dx, void *dscale, void *dshift, const void *g, const void *x, const void *scale,
                           const float *mean, const float *rstd, int64_t batch, int64_t rows_per_sample, int64_t cols,
                           int dtype, void *ws, size_t ws_bytes, bool seq_first, hipStream_t stream) {
    return wide_adaln_backward_t<false, false>(dx, dscale, dshift, nullptr, g, x, scale, mean, rstd,
                                               WideExtra{nullptr, nullptr, nullptr, nullptr}, batch, rows_per_sample,
                                               cols, dtype, ws, ws_bytes, seq_first, stream);
}

int widerow_adaln_backward_residual(void *dx, void *dscale, void *dshift, const void *g, const void *dres,
                                    const void *x, const void *scale, const float *mean, const float *rstd,
                                    int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype, void *ws,
                                    size_t ws_bytes, hipStream_t stream) {
    return wide_adaln_backward_t<false, true>(dx, dscale, dshift, nullptr, g, x, scale, mean, rstd,
                                              WideExtra{nullptr, dres, nullptr, nullptr}, batch, rows_per_sample, cols,
                                              dtype, ws, ws_bytes, false, stream);
}

int widerow_gated_adaln_backward(void *dh, void *dattn, void *dgate, void *dscale, void *dshift, const void *g,
                                 const void *dh2, const void *h2, const void *attn, const void *gate,
                                 const void *scale, const float *mean, const float *rstd, int64_t batch,
                                 int64_t rows_per_sample, int64_t cols, int dtype, void *ws, size_t ws_bytes,
                                 hipStream_t stream) {
    return wide_adaln_backward_t<true, false>(dh, dscale, dshift, dgate, g, h2, scale, mean, rstd,
                                              WideExtra{dattn, dh2, attn, gate}, batch, rows_per_sample, cols, dtype, ws,
                                              ws_bytes, false, stream);
}

}  // namespace ttn
