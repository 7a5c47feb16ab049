// Fused AdaLayerNorm for gfx950: LayerNorm without affine, then per-sample
// modulation  out = LN(x) * (1 + scale[b]) + shift[b];  forward, and a
// single-pass backward producing dx plus per-workgroup partial column sums
// for dscale and dshift.
//
// Math (rounding points follow the eager graph of
// teletron/models/dit/dit_fusedlayers.py:198,223; "rnd" = round to the element
// type, identity for fp32):
//   forward   mu = mean_c(x); r = 1/sqrt(mean_c((x-mu)^2) + eps)
//             xn = rnd((x-mu)*r); t = rnd(1+scale[b]); out = rnd(rnd(xn*t) + shift[b])
//   backward  gx = rnd(g*t); xhat = (x-mu)*r
//             dx = rnd(r*(gx - mean_c(gx) - xhat*mean_c(gx*xhat)))
//             dshift[b,c] = sum_s g;  dscale[b,c] = sum_s rnd(g * rnd(xhat))
// The variance is taken about the mean over the row held in registers (two
// passes over registers, one over memory).  HBM traffic per row: forward reads
// x and writes out (+8 B of statistics); backward reads g and x, writes dx.
#include <atomic>

#include "norm_device.h"
#include "norm_host.h"

// Backward pipeline shape at 3072 columns (measured back-to-back at 118 800 rows, with
// write-through stores): two row buffers, the next row requested half-way through the current
// one: 359 us; plain loop with one row buffer 373 us; next row requested a full row ahead 384 us.
#ifndef TTN_ADALN_BWD_ROW_BUFFERS
#define TTN_ADALN_BWD_ROW_BUFFERS 2
#endif
// Gated backward, 2-byte rows: when attn and e (the gradient arriving at h2) are fetched.
//   0: with g and x, one row at a time
//   1: at the start of a row's processing (they are needed in its second pass only), while g and x of
//      the NEXT row are requested between the two passes (two g/x buffers)
//   2: in the second pass, where they are used
#ifndef TTN_GATED_OPERANDS
#define TTN_GATED_OPERANDS 1
#endif
#ifndef TTN_ADALN_BWD_PREFETCH_MID
#define TTN_ADALN_BWD_PREFETCH_MID 1
#endif
// Stores of dx / out: 1 = write-through at device scope (RowWriter<1>), 0 = plain streaming store.
// Backward (2 reads + 1 write): 379 -> 358 us with write-through; the gated backward (4 reads + 2 writes)
// and the forward kernels measure the same either way and stay plain.
#ifndef TTN_ADALN_FWD_STORE
#define TTN_ADALN_FWD_STORE 0
#endif
#ifndef TTN_ADALN_BWD_STORE
#define TTN_ADALN_BWD_STORE 1
#endif
// Dynamic LDS requested by the forward launch (0: none).  Only a throttle on how many
// one-shot workgroups a compute unit holds at once; the kernel does not touch it.
// AdaLN forward spends longer in the ALU per row than RMSNorm forward and wants all the
// wavefronts its registers and its staged parameters allow (six workgroups per compute unit for
// 2-byte rows: 236 us at 118 800 rows against 238 with four and 280 with three).  The gated form
// moves twice the bytes per row (2 reads + 2 writes) and streams best with three workgroups per
// compute unit (12 KiB on top of its 30 KiB: 482 vs 509 us between backward launches).  4-byte rows
// carry twice the bytes per wavefront: 40 KiB on top of the staged modulation rows leaves two
// workgroups per compute unit (232 vs 244 us at 59 400 rows).
#ifndef TTN_ADALN_FWD_DYN_LDS
#define TTN_ADALN_FWD_DYN_LDS (C >= 1024 ? (sizeof(T) == 4 ? 40960 : (GATED ? 12288 : 0)) : 0)
#endif
// Backward row fetch: all of g's accesses, then all of x's (two contiguous 6 KiB runs per
// wavefront at 3072 columns) rather than alternating 1 KiB pieces; worth ~0.7 %.
#ifndef TTN_BWD_LOAD_RUNS
#define TTN_BWD_LOAD_RUNS 1
#endif
// 1: a row's first pass waits for the stores of the row before it (see kDrainStores in the kernel)
#ifndef TTN_BWD_DRAIN_STORES
#define TTN_BWD_DRAIN_STORES 1
#endif
#ifndef TTN_BWD_WAVES_PER_SIMD
#define TTN_BWD_WAVES_PER_SIMD 1
#endif
// Backward arithmetic on 2-byte rows taken from the packed pairs (bit 0: gx = rnd(g*t) as one packed
// dot product per element against masked parameter pairs instead of unpack + multiply; bit 1: the
// column sums dshift += g and dscale += rnd(g*rnd(xhat)) as packed dot products against (1,0) / (0,1),
// so g is never unpacked).  A product of two bf16 or fp16 values is exact in fp32, so every rounding
// point stays where it was.
#ifndef TTN_BWD_PACKED_MATH
#define TTN_BWD_PACKED_MATH 3
#endif
// Cache-policy bits of the backward kernels' row loads at 3072 columns (sc0 = 1, nt = 2, sc1 = 16) issued as
// buffer loads over a per-row base in scalar registers; -1 = plain global loads with the non-temporal hint.
// 19 (system scope + non-temporal: the row passes through no cache on its way in) measures 0.4-0.5 % faster over
// the whole cfg4 step than -1 on every box tried (five pairs of runs on two boxes), 0 (cached loads) 4-5 % slower.
#ifndef TTN_BWD_LOAD_POLICY
#define TTN_BWD_LOAD_POLICY 19
#endif
// Measurement only (results are wrong): rows are read and written modulo this count, so that the working set of
// a full-size launch stays in the L2 (1024) or the last-level cache; 0 = off.
#ifndef TTN_BWD_ROW_WRAP
#define TTN_BWD_ROW_WRAP 0
#endif
// Share of the compute units the persistent backward grids at 3072 columns cover, in per cent.
#ifndef TTN_BWD_GRID_PERCENT
#define TTN_BWD_GRID_PERCENT 100
#endif

namespace ttn {

// Loads this sample's modulation row and returns t = rnd(1 + scale) packed in
// the element type.
template <typename T, int C>
__device__ __forceinline__ void load_one_plus_scale(u32x4 *tr, const T *__restrict__ scale_row, int l) {
    using G = RowGeom<T, C>;
    using E = Elem<T>;
#pragma unroll
    for (int k = 0; k < G::CHUNKS; ++k) {
        float v[G::VEC];
        E::unpack(load16(reinterpret_cast<const u32x4 *>(scale_row) + k * G::LANES + l), v);
#pragma unroll
        for (int j = 0; j < G::VEC; ++j) v[j] = 1.0f + v[j];
        tr[k] = E::pack(v);
    }
}

// GATED = true: the normalised tensor is first formed as h2 = rnd(x + rnd(attn * gate[b])) (the
// gated residual update that precedes the norm in the transformer blocks) and written out too.
template <typename T, int C, bool WRITE_XNORM, bool GATED>
__global__ __launch_bounds__(kRowThreads) TTN_MIN_WAVES_PER_SIMD(sizeof(T) == 2 ? (GATED ? 3 : 4) : 2) void adaln_fwd_kernel(
    T *__restrict__ out, T *__restrict__ xnorm, float *__restrict__ mean, float *__restrict__ rstd,
    const T *__restrict__ x, const T *__restrict__ scale, const T *__restrict__ shift,
    T *__restrict__ h2_out, const T *__restrict__ attn, const T *__restrict__ gate,
    int64_t rows_per_sample, const SampleLayout lay, int blocks_per_sample, float eps) {
    using G = RowGeom<T, C>;
    using E = Elem<T>;
    constexpr int VEC = G::VEC, LANES = G::LANES, CHUNKS = G::CHUNKS, RPW = G::RPW;
    const int lane = threadIdx.x & 63;
    const int sub = lane / LANES;
    const int l = lane % LANES;
    const int wave = wave_id_in_block();
    const int64_t b = blockIdx.x / blocks_per_sample;
    const int slot = blockIdx.x % blocks_per_sample;
    wave_clock_mark(kClockAdalnFwd, 0);

    // This sample's modulation row, staged once per workgroup through LDS AS FP32: each thread forms
    // t = rnd(1 + scale) for its share of the 16-byte pieces and stores t and shift unpacked, four
    // floats per 16-byte slot in VEC/4 planes (plane p of piece i = elements 4p..4p+3, so a wavefront's
    // 16-byte reads of one plane are contiguous).  The last pass then takes its parameters with LDS
    // reads instead of unpacking them in the ALU: at 3072 two-byte columns that is 96 of ~800 VALU
    // instructions per row, and this kernel is the one closest to being ALU-bound when the part
    // runs at reduced clocks.  (One-shot wavefronts reading the row themselves would each repeat 12
    // loads and ~120 VALU instructions per 6 KiB of useful traffic.)
    constexpr int kPieces = C / VEC;  // 16-byte pieces per parameter row
    constexpr int kPlanes = VEC / 4;
    __shared__ u32x4 lds_t[kPlanes][kPieces], lds_h[kPlanes][kPieces], lds_g[GATED ? kPieces : 1];
    for (int i = threadIdx.x; i < kPieces; i += kRowThreads) {
        float v[VEC], h[VEC];
        E::unpack(load16(reinterpret_cast<const u32x4 *>(scale + b * C) + i), v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = 1.0f + v[j];
        E::round(v);  // t = 1 + scale in the element type
        E::unpack(load16(reinterpret_cast<const u32x4 *>(shift + b * C) + i), h);
#pragma unroll
        for (int p = 0; p < kPlanes; ++p) {
            lds_t[p][i] = u32x4{as_u32(v[4 * p]), as_u32(v[4 * p + 1]), as_u32(v[4 * p + 2]), as_u32(v[4 * p + 3])};
            lds_h[p][i] = u32x4{as_u32(h[4 * p]), as_u32(h[4 * p + 1]), as_u32(h[4 * p + 2]), as_u32(h[4 * p + 3])};
        }
        if constexpr (GATED) lds_g[i] = load16(reinterpret_cast<const u32x4 *>(gate + b * C) + i);
    }
    __syncthreads();

    const int64_t groups = (rows_per_sample + RPW - 1) / RPW;
    const int64_t stride = (int64_t)blocks_per_sample * kRowWaves;
    for (int64_t grp = (int64_t)slot * kRowWaves + wave; grp < groups; grp += stride) {
        const int64_t rs = grp * RPW + sub;  // row inside the sample
        const bool ok = rs < rows_per_sample;
        const int64_t row = lay.row(b, rs);
        // where the wavefront writes starts at its first row; the lane adds the distance to its own row
        const int64_t first = lay.row(b, grp * RPW) * C;
        const uint32_t lane_bytes = (uint32_t)(sub * lay.row_stride * C * sizeof(T)) + l * 16;
        const u32x4 *px = reinterpret_cast<const u32x4 *>(x + row * C) + l;
        u32x4 xr[CHUNKS];
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) xr[k] = ok ? load16_stream(px + k * LANES) : u32x4{0, 0, 0, 0};
        if constexpr (GATED) {
            const u32x4 *pa = reinterpret_cast<const u32x4 *>(attn + row * C) + l;
            const RowWriter<TTN_ADALN_FWD_STORE> wh(h2_out + first, lane_bytes);
            u32x4 ar[CHUNKS];
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k) ar[k] = ok ? load16_stream(pa + k * LANES) : u32x4{0, 0, 0, 0};
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k) {
                float hv[VEC], av[VEC], gv[VEC];
                E::unpack(xr[k], hv);
                E::unpack(ar[k], av);
                E::unpack(lds_g[k * LANES + l], gv);
#pragma unroll
                for (int j = 0; j < VEC; ++j) av[j] *= gv[j];
                E::round(av);  // attn * gate materialised in the element type
#pragma unroll
                for (int j = 0; j < VEC; ++j) hv[j] += av[j];
                xr[k] = E::pack(hv);  // h2: the new residual stream, and the row that is normalised
                if (ok) wh.put(k * LANES, xr[k]);
            }
        }

        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            if constexpr (kHasDot2<T>) {  // row sum straight from the packed pairs
#pragma unroll
                for (int i = 0; i < 4; ++i) s = dot2<T>(xr[k][i], kOnesPair<T>, s);
            } else {
                float v[VEC];
                E::unpack(xr[k], v);
#pragma unroll
                for (int j = 0; j < VEC; ++j) s += v[j];
            }
        }
        const float mu = group_sum<LANES>(s) / (float)C;
        float q = 0.0f;
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            float v[VEC];
            E::unpack(xr[k], v);
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const float d = v[j] - mu;
                q = fmaf(d, d, q);
            }
        }
        const float r = 1.0f / sqrtf(group_sum<LANES>(q) / (float)C + eps);
        if (ok && l == 0) {
            if (mean) mean[row] = mu;
            rstd[row] = r;
        }

        const float nmr = -(mu * r);
        const RowWriter<TTN_ADALN_FWD_STORE> wo(out + first, lane_bytes);
        const RowWriter<TTN_ADALN_FWD_STORE> wn(WRITE_XNORM ? xnorm + first : nullptr, lane_bytes);
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            float v[VEC], tv[VEC], hv[VEC];
            // keeps the LDS reads of later accesses from being hoisted up here, where they would all be live at once
            if constexpr (CHUNKS > 1) __builtin_amdgcn_sched_barrier(0);
            E::unpack(xr[k], v);
#pragma unroll
            for (int p = 0; p < kPlanes; ++p) {
                const u32x4 tq = lds_t[p][k * LANES + l], hq = lds_h[p][k * LANES + l];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    tv[4 * p + j] = as_f32(tq[j]);
                    hv[4 * p + j] = as_f32(hq[j]);
                }
            }
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] = centred<T>(v[j], mu, r, nmr);
            if constexpr (WRITE_XNORM) {
                const u32x4 xn = E::pack(v);
                if (ok) wn.put(k * LANES, xn);
                E::unpack(xn, v);
            } else {
                E::round(v);  // xn
            }
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] *= tv[j];
            E::round(v);  // xn * (1 + scale)
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] += hv[j];
            if (ok) wo.put(k * LANES, E::pack(v));
        }
    }
    wave_clock_mark(kClockAdalnFwd, 1);
}

// Backward.  FROM_XNORM = false: xin is the saved input x, statistics mean/rstd.
//            FROM_XNORM = true : xin is the saved normalised row rnd(LN(x)); only rstd is used.
//
// Same structure as the RMSNorm backward: one wavefront per SIMD at 3072
// columns, modulation row unpacked once, column sums in registers, next row in
// flight while the current one is processed.  With xhat = x*r - mu*r the row
// reductions reduce to sum_c gx and sum_c gx*x, both taken straight from packed
// bf16 pairs, and dx becomes r*gx + x*K1 + K0 with per-row scalars K1, K0.
//
// GATED = true (gated residual + AdaLN): xin is the saved h2; the gradient of h2 is
// dh = rnd(rnd(dx of the norm) + e) with e the gradient arriving at h2 from its other use (may be
// absent), written to dx; additionally da = rnd(dh * gate[b]) is written and
// dgate[b] += rnd(dh * attn) is accumulated as a third set of column sums.
//
// RES = true (plain AdaLN whose input has another consumer): e is the gradient the input receives from
// that consumer, and dx = rnd(rnd(dx of the norm) + e) -- the sum autograd would form in a pass of its own.
template <typename T, int C, bool FROM_XNORM, bool GATED, bool RES = false>
__global__ __launch_bounds__(kRowThreads) TTN_MIN_WAVES_PER_SIMD(C >= 1024 ? TTN_BWD_WAVES_PER_SIMD : 4) void adaln_bwd_kernel(
    T *__restrict__ dx, float *__restrict__ partial, const T *__restrict__ g,
    const T *__restrict__ xin, const T *__restrict__ scale, const float *__restrict__ mean,
    const float *__restrict__ rstd, T *__restrict__ da, const T *__restrict__ e,
    const T *__restrict__ attn, const T *__restrict__ gate, int64_t rows_per_sample,
    const SampleLayout lay, int blocks_per_sample) {
    static_assert(!(GATED && FROM_XNORM), "the gated form works from the saved h2");
    static_assert(!(GATED && RES), "the gated form handles e itself");
    constexpr int NSETS = GATED ? 3 : 2;
    using G = RowGeom<T, C>;
    using E = Elem<T>;
    constexpr int VEC = G::VEC, LANES = G::LANES, CHUNKS = G::CHUNKS, RPW = G::RPW;
    // row buffers in flight per wavefront; fp32 rows of 3072 take 96 registers each: one only
    constexpr int kRowBuffers = (sizeof(T) == 4 && C >= 1024) ? 1 : TTN_ADALN_BWD_ROW_BUFFERS;
    // A row's first pass starts only when the stores of the row before it have left the wavefront
    // (see the RMSNorm backward): 359 us with this wait, 366 us without, at 118 800 rows.
    constexpr bool kDrainStores = TTN_BWD_DRAIN_STORES && TTN_ADALN_BWD_STORE && !GATED && kRowBuffers == 2 && C >= 1024;
    __shared__ __align__(16) float lds[kFlushLdsFloats<NSETS, C>];
    const int lane = threadIdx.x & 63;
    const int sub = lane / LANES;
    const int l = lane % LANES;
    const int wave = wave_id_in_block();
    const int64_t smp = blockIdx.x / blocks_per_sample;
    const int slot = blockIdx.x % blocks_per_sample;
    wave_clock_mark(kClockAdalnBwd, 0);

    constexpr bool kPackedProducts = kHasDot2<T> && (TTN_BWD_PACKED_MATH & 1) != 0;
    constexpr bool kPackedColumnSums = kHasDot2<T> && (TTN_BWD_PACKED_MATH & 2) != 0;
    // t = rnd(1 + scale[sample]), resident for the whole kernel: unpacked to fp32, or (packed products) as
    // the masked pairs (t_lo, 0) and (0, t_hi)
    using Factor = PairFactor<std::conditional_t<kHasDot2<T>, T, bf16_t>>;  // (unused for 4-byte rows)
    [[maybe_unused]] const uint32_t one_lo = opaque_const(kOneLo<T>), one_hi = opaque_const(kOneHi<T>);
    [[maybe_unused]] float tv[kPackedProducts ? 1 : CHUNKS][VEC];
    [[maybe_unused]] Factor tf[kPackedProducts ? CHUNKS : 1];
    {
        u32x4 tr[CHUNKS];
        load_one_plus_scale<T, C>(tr, scale + smp * C, l);
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            if constexpr (kPackedProducts)
                tf[k].set(tr[k]);
            else
                E::unpack(tr[k], tv[k]);
        }
    }

    // gate[sample]: unpacked once for 2-byte elements; 4-byte rows have no registers to spare and
    // re-read it (cache hits) where it is used
    constexpr bool kGateResident = GATED && sizeof(T) == 2;
    constexpr bool kEarlyOperands = kGateResident && TTN_GATED_OPERANDS == 0;    // attn, e fetched with g, x
    constexpr bool kStartOperands = kGateResident && TTN_GATED_OPERANDS == 1;    // ... when processing starts
    [[maybe_unused]] float gatev[kGateResident ? CHUNKS : 1][VEC];
    if constexpr (kGateResident) {
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k)
            E::unpack(load16(reinterpret_cast<const u32x4 *>(gate + smp * C) + k * LANES + l), gatev[k]);
    }

    float acc[NSETS][CHUNKS][VEC];  // [0] = dscale, [1] = dshift, [2] = dgate
#pragma unroll
    for (int s = 0; s < NSETS; ++s)
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[s][k][j] = 0.0f;

    struct RowRegs {
        u32x4 g[CHUNKS], x[CHUNKS];
        u32x4 a[kEarlyOperands ? CHUNKS : 1], e[(kEarlyOperands || RES) ? CHUNKS : 1];
        float r, mu;
        int64_t row;
        int64_t first;  // element offset of the wavefront's first row (wave-uniform)
        bool ok;
    };
    auto fetch = [&](RowRegs &b, int64_t grp) {
        const int64_t rs = grp * RPW + sub;  // row inside the sample
        b.ok = rs < rows_per_sample;
#if TTN_BWD_ROW_WRAP > 0
        b.row = lay.row(smp, rs % TTN_BWD_ROW_WRAP);
        b.first = lay.row(smp, (grp * RPW) % TTN_BWD_ROW_WRAP) * C;
#else
        b.row = lay.row(smp, rs);
        b.first = lay.row(smp, grp * RPW) * C;
#endif
        const u32x4 *pg = reinterpret_cast<const u32x4 *>(g + b.row * C) + l;
        const u32x4 *px = reinterpret_cast<const u32x4 *>(xin + b.row * C) + l;
#if TTN_BWD_LOAD_POLICY >= 0
        if constexpr (LANES == kWaveSize) {
            const RowReader<TTN_BWD_LOAD_POLICY> rg(g + b.row * C, l * 16), rx(xin + b.row * C, l * 16);
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k) b.g[k] = b.ok ? rg.get(k * LANES) : u32x4{0, 0, 0, 0};
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k) b.x[k] = b.ok ? rx.get(k * LANES) : u32x4{0, 0, 0, 0};
        } else
#endif
#if TTN_BWD_LOAD_RUNS
        {
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) b.g[k] = b.ok ? load16_stream(pg + k * LANES) : u32x4{0, 0, 0, 0};
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) b.x[k] = b.ok ? load16_stream(px + k * LANES) : u32x4{0, 0, 0, 0};
        }
#else
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            b.g[k] = b.ok ? load16_stream(pg + k * LANES) : u32x4{0, 0, 0, 0};
            b.x[k] = b.ok ? load16_stream(px + k * LANES) : u32x4{0, 0, 0, 0};
        }
#endif
        if constexpr (RES) {
            const u32x4 *pe = reinterpret_cast<const u32x4 *>(e + b.row * C) + l;
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k) b.e[k] = b.ok ? load16_stream(pe + k * LANES) : u32x4{0, 0, 0, 0};
        }
        if constexpr (kEarlyOperands) {  // otherwise these two are fetched where they are used
            const u32x4 *pa = reinterpret_cast<const u32x4 *>(attn + b.row * C) + l;
            const u32x4 *pe = reinterpret_cast<const u32x4 *>(e + b.row * C) + l;
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k) b.a[k] = b.ok ? load16_stream(pa + k * LANES) : u32x4{0, 0, 0, 0};
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k)
                b.e[k] = (b.ok && e != nullptr) ? load16_stream(pe + k * LANES) : u32x4{0, 0, 0, 0};
        }
        // one row per wavefront: its statistics come through the scalar cache
        const int64_t srow = LANES == kWaveSize ? wave_uniform(b.row) : b.row;
        b.r = b.ok ? rstd[srow] : 0.0f;
        b.mu = (!FROM_XNORM && b.ok) ? mean[srow] : 0.0f;
    };
    auto process = [&](const RowRegs &b, auto &&between_passes) {
        const float r = b.r, mu = b.mu;
        const float nmr = -(mu * r);  // xhat = x*r + nmr
        [[maybe_unused]] u32x4 ar[kStartOperands ? CHUNKS : 1], er[kStartOperands ? CHUNKS : 1];
        if constexpr (kStartOperands) {
            const u32x4 *pa = reinterpret_cast<const u32x4 *>(attn + b.row * C) + l;
            const u32x4 *pe = reinterpret_cast<const u32x4 *>(e + b.row * C) + l;
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k) ar[k] = b.ok ? load16_stream(pa + k * LANES) : u32x4{0, 0, 0, 0};
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k)
                er[k] = (b.ok && e != nullptr) ? load16_stream(pe + k * LANES) : u32x4{0, 0, 0, 0};
        }
        // pass 1: gx = rnd(g*t) kept packed; s1 = sum_c gx; s2 = sum_c gx * xhat
        u32x4 gxp[CHUNKS];
        float s1 = 0.0f, s2 = 0.0f;
        if constexpr (kDrainStores) wait_memory_ops<0>();
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            if constexpr (kPackedProducts) {
                gxp[k] = rounded_products<T>(b.g[k], tf[k]);  // gx materialised in the element type
            } else {
                float gv[VEC];
                E::unpack(b.g[k], gv);
#pragma unroll
                for (int j = 0; j < VEC; ++j) gv[j] *= tv[k][j];
                gxp[k] = E::pack(gv);  // gx materialised in the element type
            }
            if constexpr (kHasDot2<T>) {
                // s2 accumulates sum_c gx * xin here; turned into sum_c gx * xhat below
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
                    s2 = fmaf(gx[j], FROM_XNORM ? xv[j] : centred<T>(xv[j], mu, r, nmr), s2);
                }
            }
        }
        s1 = group_sum<LANES>(s1);
        s2 = group_sum<LANES>(s2);
        between_passes();
        if constexpr (kHasDot2<T> && !FROM_XNORM) s2 = r * (s2 - mu * s1);
        const float m1 = s1 / (float)C, m2 = s2 / (float)C;
        // dx = r*gx + xhat*k1 + k0,  k1 = -r*m2, k0 = -r*m1;  in terms of xin: r*gx + xin*K1 + K0
        const float k1 = -(r * m2), k0 = -(r * m1);
        const float K1 = FROM_XNORM ? k1 : k1 * r;
        const float K0 = FROM_XNORM ? k0 : fmaf(k1, nmr, k0);

        const uint32_t lane_bytes = (uint32_t)(sub * lay.row_stride * C * sizeof(T)) + l * 16;
        constexpr int kDxStore = (GATED ? 0 : TTN_ADALN_BWD_STORE);
        const RowWriter<kDxStore> wd(dx + b.first, lane_bytes);
        const RowWriter<0> wa(GATED ? da + b.first : nullptr, lane_bytes);
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            [[maybe_unused]] float gv[VEC];
            float gx[VEC], xv[VEC], o[VEC], xn[VEC];
            if constexpr (!kPackedColumnSums) E::unpack(b.g[k], gv);
            E::unpack(gxp[k], gx);
            E::unpack(b.x[k], xv);
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                o[j] = fmaf(r, gx[j], fmaf(xv[j], K1, K0));
                xn[j] = FROM_XNORM ? xv[j] : centred<T>(xv[j], mu, r, nmr);
                if constexpr (!kPackedColumnSums) acc[1][k][j] += gv[j];
            }
            if constexpr (GATED) {
                float ev[VEC], av[VEC], dav[VEC];
                E::round(o);  // the norm's dx, materialised in the element type
                if constexpr (kEarlyOperands) {
                    E::unpack(b.e[k], ev);
                    E::unpack(b.a[k], av);
                } else if constexpr (kStartOperands) {
                    E::unpack(er[k], ev);
                    E::unpack(ar[k], av);
                } else {
                    const int64_t at = b.row * (C / VEC) + l + k * LANES;
                    const u32x4 zero{0, 0, 0, 0};
                    E::unpack((b.ok && e != nullptr) ? load16_stream(reinterpret_cast<const u32x4 *>(e) + at) : zero, ev);
                    E::unpack(b.ok ? load16_stream(reinterpret_cast<const u32x4 *>(attn) + at) : zero, av);
                }
#pragma unroll
                for (int j = 0; j < VEC; ++j) o[j] += ev[j];
                const u32x4 dhp = E::pack(o);  // dh: gradient of h2 = of the residual input
                if (b.ok) wd.put(k * LANES, dhp);
                E::unpack(dhp, o);
                if constexpr (kGateResident) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) dav[j] = o[j] * gatev[k][j];
                } else {
                    E::unpack(load16(reinterpret_cast<const u32x4 *>(gate + smp * C) + k * LANES + l), dav);
#pragma unroll
                    for (int j = 0; j < VEC; ++j) dav[j] *= o[j];
                }
#pragma unroll
                for (int j = 0; j < VEC; ++j) av[j] *= o[j];
                if (b.ok) wa.put(k * LANES, E::pack(dav));
                E::round(av);  // dh*attn materialised in the element type before the column sum
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc[2][k][j] += av[j];
            } else {
                if constexpr (RES) {
                    float ev[VEC];
                    E::round(o);  // the norm's dx, materialised in the element type
                    E::unpack(b.e[k], ev);
#pragma unroll
                    for (int j = 0; j < VEC; ++j) o[j] += ev[j];
                }
                if (b.ok) wd.put(k * LANES, E::pack(o));
            }
            if constexpr (kPackedColumnSums) {
                Factor nf;  // the normalised row in the element type
                if constexpr (FROM_XNORM)
                    nf.set(b.x[k]);
                else
                    nf.set_rounded(xn);
                const u32x4 pp = rounded_products<T>(b.g[k], nf);  // g*xn in the element type, then summed
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc[0][k][2 * i] = dot2<T>(pp[i], one_lo, acc[0][k][2 * i]);
                    acc[0][k][2 * i + 1] = dot2<T>(pp[i], one_hi, acc[0][k][2 * i + 1]);
                    acc[1][k][2 * i] = dot2<T>(b.g[k][i], one_lo, acc[1][k][2 * i]);
                    acc[1][k][2 * i + 1] = dot2<T>(b.g[k][i], one_hi, acc[1][k][2 * i + 1]);
                }
            } else {
                if constexpr (!FROM_XNORM) E::round(xn);  // the normalised row in the element type
#pragma unroll
                for (int j = 0; j < VEC; ++j) xn[j] *= gv[j];
                E::round(xn);  // g*xn materialised in the element type before the column sum
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc[0][k][j] += xn[j];
            }
        }
    };

    const int64_t groups = (rows_per_sample + RPW - 1) / RPW;
    const int64_t stride = (int64_t)blocks_per_sample * kRowWaves;
    int64_t grp = (int64_t)slot * kRowWaves + wave;
    if constexpr (kStartOperands)
        row_pipeline<2, true, RowRegs>(grp, groups, stride, fetch, process);
    else
        row_pipeline<kRowBuffers, TTN_ADALN_BWD_PREFETCH_MID != 0, RowRegs>(grp, groups, stride, fetch, process);
    wave_clock_mark(kClockAdalnBwd, 2);  // rows done; what follows is the workgroup's partial row
    flush_column_partials<G, NSETS>(acc, partial + (int64_t)blockIdx.x * (NSETS * C), lds);
    wave_clock_mark(kClockAdalnBwd, 1);
}

#if TTN_WAVE_CLOCK
int adaln_set_wave_clock(void *buf) {
    return hipMemcpyToSymbol(HIP_SYMBOL(ttn_wave_clock_buf), &buf, sizeof(buf)) == hipSuccess ? TT_NORM_OK : TT_NORM_EHIP;
}
#endif

// Same launch policy as RMSNorm: forward one-shot at 3072 columns, backward one
// workgroup per compute unit.
constexpr int kOneShotGrid = 1 << 20;
#ifndef TTN_ADALN_FWD_BLOCKS_PER_CU
#define TTN_ADALN_FWD_BLOCKS_PER_CU (C >= 1024 ? kOneShotGrid : 16)
#endif
#ifndef TTN_ADALN_BWD_BLOCKS_PER_CU
#define TTN_ADALN_BWD_BLOCKS_PER_CU (C >= 1024 ? 1 : 3)
#endif
template <typename T, int C>
struct AdalnTune {
    static constexpr int kFwdBlocksPerCu = TTN_ADALN_FWD_BLOCKS_PER_CU;
    static constexpr int kBwdBlocksPerCu = TTN_ADALN_BWD_BLOCKS_PER_CU;
};

struct AdalnArgs {
    int64_t batch, rows_per_sample;
    double eps;
    hipStream_t stream;
    bool seq_first = false;  // rows laid out [rows_per_sample, batch] instead of [batch, rows_per_sample]
    SampleLayout layout() const {
        return seq_first ? SampleLayout{1, batch} : SampleLayout{rows_per_sample, 1};
    }
};

struct GatedPtrs {  // the extra operands of the gated-residual form (all null otherwise)
    void *h2_or_da;    // forward: h2 out;   backward: da out
    const void *e;     // backward: gradient arriving at h2 from its other use, or null
    const void *attn;
    const void *gate;
};

template <typename T, int C, bool WRITE_XNORM, bool GATED = false>
static int adaln_forward_t(void *out, void *xnorm, float *mean, float *rstd, const void *x,
                           const void *scale, const void *shift, const AdalnArgs &a,
                           const GatedPtrs &gp = GatedPtrs{nullptr, nullptr, nullptr, nullptr}) {
    if (a.rows_per_sample == 0) return TT_NORM_OK;  // empty input: nothing to do
    int st = TT_NORM_OK;
    const int cus = current_device_cus(&st);
    if (st != TT_NORM_OK) return st;
    const RowPlan p = make_row_plan(a.batch, a.rows_per_sample, RowGeom<T, C>::RPW,
                                    AdalnTune<T, C>::kFwdBlocksPerCu, cus);
    if (p.blocks > 0x7fffffffLL) return fail(TT_NORM_EINVAL, "adaln forward: grid too large");
    {
        RowKernelProfile prof(a.stream);
        adaln_fwd_kernel<T, C, WRITE_XNORM, GATED><<<dim3((unsigned)p.blocks), dim3(kRowThreads), TTN_ADALN_FWD_DYN_LDS, a.stream>>>(
            (T *)out, (T *)xnorm, mean, rstd, (const T *)x, (const T *)scale, (const T *)shift,
            (T *)gp.h2_or_da, (const T *)gp.attn, (const T *)gp.gate, a.rows_per_sample, a.layout(),
            p.blocks_per_sample, (float)a.eps);
    }
    return check_launch("adaln forward launch");
}

template <typename T, int C>
static RowPlan adaln_backward_plan(int64_t batch, int64_t rows_per_sample, int cus) {
    const int share = C >= 1024 ? (cus * TTN_BWD_GRID_PERCENT + 99) / 100 : cus;
    return make_row_plan(batch, rows_per_sample, RowGeom<T, C>::RPW, AdalnTune<T, C>::kBwdBlocksPerCu, share);
}

template <typename T, int C, bool FROM_XNORM, bool GATED = false, bool RES = false>
static int adaln_backward_t(void *dx, void *dscale, void *dshift, const void *g, const void *xin,
                            const void *scale, const float *mean, const float *rstd, int dtype,
                            void *ws, size_t ws_bytes, const AdalnArgs &a, void *dgate = nullptr,
                            const GatedPtrs &gp = GatedPtrs{nullptr, nullptr, nullptr, nullptr}) {
    constexpr int NSETS = GATED ? 3 : 2;
    // empty input: the parameter gradients are empty sums, written by the reducer over zero partial rows
    if (a.rows_per_sample == 0)
        return launch_colreduce(dscale, dshift, dgate, nullptr, a.batch, 0, C, NSETS * C, dtype, a.stream);
    int st = TT_NORM_OK;
    const int cus = current_device_cus(&st);
    if (st != TT_NORM_OK) return st;
    const RowPlan p = adaln_backward_plan<T, C>(a.batch, a.rows_per_sample, cus);
    if (p.blocks > 0x7fffffffLL) return fail(TT_NORM_EINVAL, "adaln backward: grid too large");
    const size_t need = (size_t)p.blocks * NSETS * C * sizeof(float);
    if (!ws || ws_bytes < need)
        return fail(TT_NORM_EWORKSPACE, "adaln backward: workspace %zu B < required %zu B", ws_bytes, need);
    if (!aligned16(ws)) return fail(TT_NORM_EALIGN, "adaln backward: workspace %p not 16-byte aligned", ws);
    {
        RowKernelProfile prof(a.stream);
        adaln_bwd_kernel<T, C, FROM_XNORM, GATED, RES><<<dim3((unsigned)p.blocks), dim3(kRowThreads), 0, a.stream>>>(
            (T *)dx, (float *)ws, (const T *)g, (const T *)xin, (const T *)scale, mean, rstd,
            (T *)gp.h2_or_da, (const T *)gp.e, (const T *)gp.attn, (const T *)gp.gate, a.rows_per_sample,
            a.layout(), p.blocks_per_sample);
    }
    st = check_launch("adaln backward launch");
    if (st != TT_NORM_OK) return st;
    return launch_colreduce(dscale, dshift, dgate, (const float *)ws, a.batch, p.blocks_per_sample, C,
                            NSETS * C, dtype, a.stream);
}

// tuned_only: the entry point exists for the tuned shapes only (reference-contract and gated forms).
static int check_adaln_args(const char *who, int64_t batch, int64_t rows_per_sample, int64_t cols,
                            int dtype, std::initializer_list<const void *> ptrs, bool tuned_only = false) {
    if (batch <= 0 || rows_per_sample < 0 || cols <= 0)
        return fail(TT_NORM_EINVAL, "%s: batch=%lld rows_per_sample=%lld cols=%lld", who, (long long)batch,
                    (long long)rows_per_sample, (long long)cols);
    if (tuned_only && !tuned_shape(cols, dtype))
        return fail(TT_NORM_EUNSUPPORTED, "%s: cols=%lld dtype=%d (this entry point: cols 128/3072)", who,
                    (long long)cols, dtype);
    if (!tt_norm_supported(cols, dtype))
        return fail(TT_NORM_EUNSUPPORTED,
                    "%s: cols=%lld dtype=%d (cols must be a multiple of 16 bytes of elements, at most 8192 "
                    "two-byte or 4096 four-byte; dtype bf16, fp16 or fp32)", who, (long long)cols, dtype);
    if (rows_per_sample == 0) return TT_NORM_OK;  // empty input: nothing is dereferenced
    for (const void *p : ptrs) {
        if (!p) return fail(TT_NORM_EINVAL, "%s: null pointer", who);
        if (!aligned16(p)) return fail(TT_NORM_EALIGN, "%s: pointer %p not 16-byte aligned", who, p);
    }
    return TT_NORM_OK;
}

static int wide_form_unsupported(const char *who, int64_t cols) {
    return fail(TT_NORM_EUNSUPPORTED, "%s: cols=%lld (this form takes 3072 columns, or any row of up to 384 16-byte "
                "pieces: 3072 two-byte / 1536 four-byte columns)", who, (long long)cols);
}

// The rows a wavefront handles together (up to eight when rows are narrow) are addressed with 32-bit
// byte offsets from the first of them; in the sequence-first layout they lie batch rows apart.
static int check_seq_first(const char *who, int64_t batch, int64_t cols, int dtype) {
    if (batch * cols * (int64_t)elem_bytes(dtype) > kMaxRowStrideBytes)
        return fail(TT_NORM_EINVAL, "%s: batch * cols * element size exceeds 256 MiB", who);
    return TT_NORM_OK;
}

}  // namespace ttn

using namespace ttn;

#define TTN_DISPATCH(dtype, cols, CALL)                          \
    do {                                                         \
        if ((dtype) == TT_NORM_BF16) {                           \
            if ((cols) == 128) { CALL(bf16_t, 128); }            \
            else { CALL(bf16_t, 3072); }                         \
        } else if ((dtype) == TT_NORM_F16) {                     \
            if ((cols) == 128) { CALL(f16_t, 128); }             \
            else { CALL(f16_t, 3072); }                          \
        } else {                                                 \
            if ((cols) == 128) { CALL(float, 128); }             \
            else { CALL(float, 3072); }                          \
        }                                                        \
    } while (0)

extern "C" {

int tt_adaln_forward(void *out, float *mean, float *rstd, const void *x, const void *scale,
                     const void *shift, int64_t batch, int64_t rows_per_sample, int64_t cols,
                     double eps, int dtype, void *stream) {
    int st = check_adaln_args("tt_adaln_forward", batch, rows_per_sample, cols, dtype, {out, x, scale, shift});
    if (st != TT_NORM_OK) return st;
    if ((!mean || !rstd) && rows_per_sample > 0) return fail(TT_NORM_EINVAL, "tt_adaln_forward: null mean/rstd");
    if (!tuned_shape(cols, dtype))
        return anywidth_adaln_forward(out, mean, rstd, x, scale, shift, batch, rows_per_sample, cols, eps, dtype,
                                      (hipStream_t)stream);
    const AdalnArgs a{batch, rows_per_sample, eps, (hipStream_t)stream};
#define CALL(T, C) return adaln_forward_t<T, C, false>(out, nullptr, mean, rstd, x, scale, shift, a)
    TTN_DISPATCH(dtype, cols, CALL);
#undef CALL
}

int tt_adaln_forward_xnorm(void *out, void *x_norm, float *rstd, const void *x, const void *scale,
                           const void *shift, int64_t batch, int64_t rows_per_sample, int64_t cols,
                           double eps, int dtype, void *stream) {
    int st = check_adaln_args("tt_adaln_forward_xnorm", batch, rows_per_sample, cols, dtype,
                              {out, x_norm, x, scale, shift}, true);
    if (st != TT_NORM_OK) return st;
    if (!rstd && rows_per_sample > 0) return fail(TT_NORM_EINVAL, "tt_adaln_forward_xnorm: null rstd");
    const AdalnArgs a{batch, rows_per_sample, eps, (hipStream_t)stream};
#define CALL(T, C) return adaln_forward_t<T, C, true>(out, x_norm, nullptr, rstd, x, scale, shift, a)
    TTN_DISPATCH(dtype, cols, CALL);
#undef CALL
}

size_t tt_adaln_backward_workspace_bytes(int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype) {
    if (batch <= 0 || rows_per_sample <= 0 || !tt_norm_supported(cols, dtype)) return 0;
    if (!tuned_shape(cols, dtype) || dense_backward_on_wide_rows(cols, dtype))
        return anywidth_adaln_backward_workspace_bytes(batch, rows_per_sample, cols, dtype);
    int st = TT_NORM_OK;
    const int cus = current_device_cus(&st);
    if (st != TT_NORM_OK) return 0;
#define CALL(T, C) \
    return (size_t)adaln_backward_plan<T, C>(batch, rows_per_sample, cus).blocks * 2 * C * sizeof(float)
    TTN_DISPATCH(dtype, cols, CALL);
#undef CALL
}

int tt_adaln_backward(void *dx, void *dscale, void *dshift, const void *dout, const void *x,
                      const void *scale, const float *mean, const float *rstd, int64_t batch,
                      int64_t rows_per_sample, int64_t cols, int dtype, void *workspace,
                      size_t workspace_bytes, void *stream) {
    int st = check_adaln_args("tt_adaln_backward", batch, rows_per_sample, cols, dtype, {dx, dout, x, scale});
    if (st != TT_NORM_OK) return st;
    if (!dscale || !dshift || ((!mean || !rstd) && rows_per_sample > 0))
        return fail(TT_NORM_EINVAL, "tt_adaln_backward: null dscale/dshift/mean/rstd");
    if (!tuned_shape(cols, dtype) || dense_backward_on_wide_rows(cols, dtype))
        return anywidth_adaln_backward(dx, dscale, dshift, dout, x, scale, mean, rstd, batch, rows_per_sample, cols,
                                       dtype, workspace, workspace_bytes, (hipStream_t)stream);
    const AdalnArgs a{batch, rows_per_sample, 0.0, (hipStream_t)stream};
#define CALL(T, C)                                                                                \
    return adaln_backward_t<T, C, false>(dx, dscale, dshift, dout, x, scale, mean, rstd, dtype, workspace, \
                                         workspace_bytes, a)
    TTN_DISPATCH(dtype, cols, CALL);
#undef CALL
}

int tt_adaln_backward_from_xnorm(void *dx, void *dscale, void *dshift, const void *dout,
                                 const void *x_norm, const void *scale, const float *rstd,
                                 int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype,
                                 void *workspace, size_t workspace_bytes, void *stream) {
    int st = check_adaln_args("tt_adaln_backward_from_xnorm", batch, rows_per_sample, cols, dtype,
                              {dx, dout, x_norm, scale}, true);
    if (st != TT_NORM_OK) return st;
    if (!dscale || !dshift || (!rstd && rows_per_sample > 0))
        return fail(TT_NORM_EINVAL, "tt_adaln_backward_from_xnorm: null dscale/dshift/rstd");
    const AdalnArgs a{batch, rows_per_sample, 0.0, (hipStream_t)stream};
#define CALL(T, C)                                                                                 \
    return adaln_backward_t<T, C, true>(dx, dscale, dshift, dout, x_norm, scale, nullptr, rstd, dtype, \
                                        workspace, workspace_bytes, a)
    TTN_DISPATCH(dtype, cols, CALL);
#undef CALL
}

/* ---- sequence-first rows: x is [rows_per_sample, batch, cols] ---- */

int tt_adaln_forward_seq_first(void *out, float *mean, float *rstd, const void *x, const void *scale,
                               const void *shift, int64_t batch, int64_t rows_per_sample, int64_t cols,
                               double eps, int dtype, void *stream) {
    int st = check_adaln_args("tt_adaln_forward_seq_first", batch, rows_per_sample, cols, dtype, {out, x, scale, shift});
    if (st == TT_NORM_OK) st = check_seq_first("tt_adaln_forward_seq_first", batch, cols, dtype);
    if (st != TT_NORM_OK) return st;
    if ((!mean || !rstd) && rows_per_sample > 0) return fail(TT_NORM_EINVAL, "tt_adaln_forward_seq_first: null mean/rstd");
    if (!tuned_shape(cols, dtype))
        return anywidth_adaln_forward(out, mean, rstd, x, scale, shift, batch, rows_per_sample, cols, eps, dtype,
                                      (hipStream_t)stream, true);
    const AdalnArgs a{batch, rows_per_sample, eps, (hipStream_t)stream, true};
#define CALL(T, C) return adaln_forward_t<T, C, false>(out, nullptr, mean, rstd, x, scale, shift, a)
    TTN_DISPATCH(dtype, cols, CALL);
#undef CALL
}

int tt_adaln_backward_seq_first(void *dx, void *dscale, void *dshift, const void *dout, const void *x,
                                const void *scale, const float *mean, const float *rstd, int64_t batch,
                                int64_t rows_per_sample, int64_t cols, int dtype, void *workspace,
                                size_t workspace_bytes, void *stream) {
    int st = check_adaln_args("tt_adaln_backward_seq_first", batch, rows_per_sample, cols, dtype, {dx, dout, x, scale});
    if (st == TT_NORM_OK) st = check_seq_first("tt_adaln_backward_seq_first", batch, cols, dtype);
    if (st != TT_NORM_OK) return st;
    if (!dscale || !dshift || ((!mean || !rstd) && rows_per_sample > 0))
        return fail(TT_NORM_EINVAL, "tt_adaln_backward_seq_first: null dscale/dshift/mean/rstd");
    if (!tuned_shape(cols, dtype) || dense_backward_on_wide_rows(cols, dtype))
        return anywidth_adaln_backward(dx, dscale, dshift, dout, x, scale, mean, rstd, batch, rows_per_sample, cols,
                                       dtype, workspace, workspace_bytes, (hipStream_t)stream, true);
    const AdalnArgs a{batch, rows_per_sample, 0.0, (hipStream_t)stream, true};
#define CALL(T, C)                                                                                \
    return adaln_backward_t<T, C, false>(dx, dscale, dshift, dout, x, scale, mean, rstd, dtype, workspace, \
                                         workspace_bytes, a)
    TTN_DISPATCH(dtype, cols, CALL);
#undef CALL
}

/* ---- AdaLN backward that allocates nothing: scratch in a static device array ---- */

}  // extern "C"

namespace ttn {

// Partial column sums of tt_adaln_backward_static.  One copy per GPU the library runs on, held
// until the process ends; every call on a GPU uses that GPU's copy.
constexpr size_t kStaticScratchBytes = (size_t)TT_NORM_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device address of `scratch` on the current device.  The array's name is only a host-side handle;
// its address on each GPU is looked up once, with that GPU current, and kept.
static int static_scratch_address(void **out) {
    constexpr int kMaxDevices = 64;
    static std::atomic<void *> cache[kMaxDevices];  // zero-initialised: null = not looked up yet
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(TT_NORM_EHIP, "hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(TT_NORM_EINVAL, "device ordinal %d out of range", dev);
    void *p = cache[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return fail(TT_NORM_EHIP, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
        cache[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return TT_NORM_OK;
}

}  // namespace ttn

extern "C" {

int tt_adaln_backward_static(void *dx, void *dscale, void *dshift, const void *dout, const void *x,
                             const void *scale, const float *mean, const float *rstd, int64_t batch,
                             int64_t rows_per_sample, int64_t cols, int dtype, void *stream) {
    int st = check_adaln_args("tt_adaln_backward_static", batch, rows_per_sample, cols, dtype, {dx, dout, x, scale});
    if (st != TT_NORM_OK) return st;
    const size_t need = tt_adaln_backward_workspace_bytes(batch, rows_per_sample, cols, dtype);
    if (need > kStaticScratchBytes)
        return fail(TT_NORM_EWORKSPACE,
                    "tt_adaln_backward_static: batch=%lld rows_per_sample=%lld cols=%lld needs %zu B of scratch, the "
                    "static array holds %zu B; use tt_adaln_backward with caller-provided scratch",
                    (long long)batch, (long long)rows_per_sample, (long long)cols, need, kStaticScratchBytes);
    void *ws = nullptr;
    st = static_scratch_address(&ws);
    if (st != TT_NORM_OK) return st;
    if (rows_per_sample > 0) {
        // the array belongs to the current device; tensors on another one would be paired with the wrong copy
        int dev = -1;
        hipPointerAttribute_t attr;
        if (hipGetDevice(&dev) != hipSuccess || hipPointerGetAttributes(&attr, dx) != hipSuccess) {
            (void)hipGetLastError();
            return fail(TT_NORM_EINVAL, "tt_adaln_backward_static: dx is not a device pointer the runtime knows");
        }
        if (attr.device != dev)
            return fail(TT_NORM_EINVAL, "tt_adaln_backward_static: dx lives on device %d, the current device is %d",
                        attr.device, dev);
    }
    // every partial row the reducer reads is written in full by the row kernel of the same call:
    // nothing in the array has to start at zero
    return tt_adaln_backward(dx, dscale, dshift, dout, x, scale, mean, rstd, batch, rows_per_sample, cols, dtype, ws,
                             kStaticScratchBytes, stream);
}

/* ---- gated residual + AdaLN (3072 columns, or any row of up to 384 16-byte pieces) ---- */

int tt_gated_residual_adaln_forward(void *h2, void *out, float *mean, float *rstd, const void *h,
                                    const void *attn, const void *gate, const void *scale,
                                    const void *shift, int64_t batch, int64_t rows_per_sample,
                                    int64_t cols, double eps, int dtype, void *stream) {
    if (tt_norm_supported(cols, dtype) && !tt_norm_wide_forms_supported(cols, dtype))
        return wide_form_unsupported("tt_gated_residual_adaln_forward", cols);
    int st = check_adaln_args("tt_gated_residual_adaln_forward", batch, rows_per_sample, cols, dtype,
                              {h2, out, h, attn, gate, scale, shift});
    if (st != TT_NORM_OK) return st;
    if ((!mean || !rstd) && rows_per_sample > 0)
        return fail(TT_NORM_EINVAL, "tt_gated_residual_adaln_forward: null mean/rstd");
    if (cols != 3072 || gated_forward_on_wide_rows(cols, dtype)) {
        if (!anywidth_wide_forms_supported(cols, dtype)) return wide_form_unsupported("tt_gated_residual_adaln_forward", cols);
        return anywidth_gated_adaln_forward(h2, out, mean, rstd, h, attn, gate, scale, shift, batch, rows_per_sample, cols,
                                            eps, dtype, (hipStream_t)stream);
    }
    const AdalnArgs a{batch, rows_per_sample, eps, (hipStream_t)stream};
    const GatedPtrs gp{h2, nullptr, attn, gate};
    if (dtype == TT_NORM_BF16)
        return adaln_forward_t<bf16_t, 3072, false, true>(out, nullptr, mean, rstd, h, scale, shift, a, gp);
    if (dtype == TT_NORM_F16)
        return adaln_forward_t<f16_t, 3072, false, true>(out, nullptr, mean, rstd, h, scale, shift, a, gp);
    return adaln_forward_t<float, 3072, false, true>(out, nullptr, mean, rstd, h, scale, shift, a, gp);
}

size_t tt_gated_residual_adaln_backward_workspace_bytes(int64_t batch, int64_t rows_per_sample, int64_t cols,
                                                        int dtype) {
    if (!tt_norm_wide_forms_supported(cols, dtype)) return 0;
    // three sets of column sums (dscale, dshift, dgate) instead of two
    if (gated_forward_on_wide_rows(cols, dtype))
        return anywidth_gated_adaln_backward_workspace_bytes(batch, rows_per_sample, cols, dtype);
    return tt_adaln_backward_workspace_bytes(batch, rows_per_sample, cols, dtype) / 2 * 3;
}

int tt_gated_residual_adaln_backward(void *dh, void *dattn, void *dgate, void *dscale, void *dshift,
                                     const void *dout, const void *dh2, const void *h2, const void *attn,
                                     const void *gate, const void *scale, const float *mean,
                                     const float *rstd, int64_t batch, int64_t rows_per_sample,
                                     int64_t cols, int dtype, void *workspace, size_t workspace_bytes,
                                     void *stream) {
    if (tt_norm_supported(cols, dtype) && !tt_norm_wide_forms_supported(cols, dtype))
        return wide_form_unsupported("tt_gated_residual_adaln_backward", cols);
    int st = check_adaln_args("tt_gated_residual_adaln_backward", batch, rows_per_sample, cols, dtype,
                              {dh, dattn, dout, h2, attn, gate, scale});
    if (st != TT_NORM_OK) return st;
    if (dh2 && !aligned16(dh2)) return fail(TT_NORM_EALIGN, "tt_gated_residual_adaln_backward: dh2 not 16-byte aligned");
    if (!dgate || !dscale || !dshift || ((!mean || !rstd) && rows_per_sample > 0))
        return fail(TT_NORM_EINVAL, "tt_gated_residual_adaln_backward: null dgate/dscale/dshift/mean/rstd");
    if (cols != 3072 || dense_backward_on_wide_rows(cols, dtype) || gated_forward_on_wide_rows(cols, dtype)) {
        if (!anywidth_wide_forms_supported(cols, dtype)) return wide_form_unsupported("tt_gated_residual_adaln_backward", cols);
        return anywidth_gated_adaln_backward(dh, dattn, dgate, dscale, dshift, dout, dh2, h2, attn, gate, scale, mean, rstd,
                                             batch, rows_per_sample, cols, dtype, workspace, workspace_bytes,
                                             (hipStream_t)stream);
    }
    const AdalnArgs a{batch, rows_per_sample, 0.0, (hipStream_t)stream};
    const GatedPtrs gp{dattn, dh2, attn, gate};
    if (dtype == TT_NORM_BF16)
        return adaln_backward_t<bf16_t, 3072, false, true>(dh, dscale, dshift, dout, h2, scale, mean, rstd, dtype,
                                                           workspace, workspace_bytes, a, dgate, gp);
    if (dtype == TT_NORM_F16)
        return adaln_backward_t<f16_t, 3072, false, true>(dh, dscale, dshift, dout, h2, scale, mean, rstd, dtype,
                                                          workspace, workspace_bytes, a, dgate, gp);
    return adaln_backward_t<float, 3072, false, true>(dh, dscale, dshift, dout, h2, scale, mean, rstd, dtype,
                                                      workspace, workspace_bytes, a, dgate, gp);
}

/* ---- AdaLN backward with the input's other gradient added in (same shapes as the gated form) ---- */

int tt_adaln_backward_residual(void *dx, void *dscale, void *dshift, const void *dout, const void *dres,
                               const void *x, const void *scale, const float *mean, const float *rstd,
                               int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype,
                               void *workspace, size_t workspace_bytes, void *stream) {
    if (tt_norm_supported(cols, dtype) && !tt_norm_wide_forms_supported(cols, dtype))
        return wide_form_unsupported("tt_adaln_backward_residual", cols);
    int st = check_adaln_args("tt_adaln_backward_residual", batch, rows_per_sample, cols, dtype,
                              {dx, dout, dres, x, scale});
    if (st != TT_NORM_OK) return st;
    if (!dscale || !dshift || ((!mean || !rstd) && rows_per_sample > 0))
        return fail(TT_NORM_EINVAL, "tt_adaln_backward_residual: null dscale/dshift/mean/rstd");
    if (cols != 3072 || dense_backward_on_wide_rows(cols, dtype)) {
        if (!anywidth_wide_forms_supported(cols, dtype)) return wide_form_unsupported("tt_adaln_backward_residual", cols);
        return anywidth_adaln_backward_residual(dx, dscale, dshift, dout, dres, x, scale, mean, rstd, batch, rows_per_sample,
                                                cols, dtype, workspace, workspace_bytes, (hipStream_t)stream);
    }
    const AdalnArgs a{batch, rows_per_sample, 0.0, (hipStream_t)stream};
    const GatedPtrs gp{nullptr, dres, nullptr, nullptr};
    if (dtype == TT_NORM_BF16)
        return adaln_backward_t<bf16_t, 3072, false, false, true>(dx, dscale, dshift, dout, x, scale, mean, rstd, dtype,
                                                                  workspace, workspace_bytes, a, nullptr, gp);
    if (dtype == TT_NORM_F16)
        return adaln_backward_t<f16_t, 3072, false, false, true>(dx, dscale, dshift, dout, x, scale, mean, rstd, dtype,
                                                                 workspace, workspace_bytes, a, nullptr, gp);
    return adaln_backward_t<float, 3072, false, false, true>(dx, dscale, dshift, dout, x, scale, mean, rstd, dtype,
                                                             workspace, workspace_bytes, a, nullptr, gp);
}

}  // extern "C"
