// Fused RMSNorm for gfx950: forward, and a single-pass backward that produces
// dx together with per-workgroup partial column sums for dweight.
//
// Math (rounding points follow the eager graph of
// teletron/models/dit/dit_fusedlayers.py:360-370, "rnd" = round to the element
// type, identity for fp32):
//   forward   r = 1/sqrt(mean_c(x^2) + eps);  y = rnd(x*r);  out = rnd(y*w)
//   backward  gy = rnd(g*w);  dx = rnd(gy*r - x * r^3 * mean_c(gy*x))
//             dw[c] = sum_rows rnd(g * y)
// HBM traffic per row: forward reads x, writes out (+4 B of rstd); backward
// reads g and x, writes dx; dweight costs one fp32 row per workgroup.
#include "norm_device.h"
#include "norm_host.h"

// Backward pipeline shape at 3072 columns (measured back-to-back at 118 800 rows):
// two row buffers with the next row requested half-way through the current one.
#ifndef TTN_RMS_BWD_ROW_BUFFERS
#define TTN_RMS_BWD_ROW_BUFFERS 2
#endif
#ifndef TTN_RMS_BWD_PREFETCH_MID
#define TTN_RMS_BWD_PREFETCH_MID 1
#endif
// Dynamic LDS requested by the forward launch at 3072 columns: 50 KiB per workgroup lets a
// compute unit hold three one-shot workgroups (12 wavefronts, ~72 KiB of reads in flight),
// which streams 5 % faster than the five its registers would allow (232 vs 244 us at
// 118 800 rows).  The kernel does not touch this memory; it is only an occupancy throttle.
// 4-byte rows carry twice the bytes per wavefront: two workgroups per compute unit (75 KiB each;
// 234 vs 253 us at 59 400 rows).
#ifndef TTN_RMS_FWD_DYN_LDS
#define TTN_RMS_FWD_DYN_LDS (C >= 1024 ? (sizeof(T) == 2 ? 51200 : 76800) : 0)
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
// Backward arithmetic on 2-byte rows taken from the packed pairs (bit 0: gy = rnd(g*w) as one packed
// dot product per element against masked weight pairs instead of unpack + multiply; bit 1: the column
// sum dw += rnd(g*rnd(x*r)) as packed dot products, so g is never unpacked).  A product of two bf16 or
// fp16 values is exact in fp32, so every rounding point stays where it was.
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
// Stores of dx / out: 1 = write-through at device scope (RowWriter<1>), 0 = plain streaming store.
// Backward (2 reads + 1 write): 367 -> 353 us with write-through.  Forward (1 read + 1 write): the same
// either way at 3072 columns (one-shot grid), 62.6 -> 61.4 us at 128 columns (persistent grid).
#ifndef TTN_RMS_FWD_STORE
#define TTN_RMS_FWD_STORE (C < 1024)
#endif
#ifndef TTN_RMS_BWD_STORE
#define TTN_RMS_BWD_STORE 1
#endif

namespace ttn {

// ---- rotary embedding behind the norm -----------------------------------------
// The attention caller rotates the normalised query and key right after the per-head norm
// (teletron/models/dit/dit_attention.py:266-273, :435-443) with the real-pair form of
// diffusers' apply_rotary_emb: for tokens below `tokens`
//     out = cast(float(y) * cos + float(rotate_pairs(y)) * sin),   rotate_pairs(y)[2i, 2i+1] = (-y[2i+1], y[2i])
// with cos, sin fp32 tables [tokens, C]; each product and the sum are rounded to fp32, the result
// once to the element type.  Pairs are adjacent, so both halves sit in one lane's 16-byte piece.
struct NoRope {
    static constexpr bool kOn = false;
};
struct RopeTable {
    static constexpr bool kOn = true;
    const float *cos, *sin;  // [tokens, C] fp32, row = token index
    int64_t tokens;          // rows of the view at sequence index >= tokens are left unrotated
};

template <int VEC>
__device__ __forceinline__ void load_fp32_run(float (&dst)[VEC], const float *p) {
#pragma unroll
    for (int i = 0; i < VEC / 4; ++i) {
        const u32x4 t = load16(reinterpret_cast<const u32x4 *>(p) + i);  // cached: every head reuses the row
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[4 * i + j] = as_f32(t[j]);
    }
}

// Groups a wavefront takes per step: runs only pay where the index arithmetic and the shared side tables
// weigh against the row itself, i.e. for narrow rows.
// Forward without tables: single groups stream better (74 vs 77 us at 712 800 x 128), the divisions hide
// behind the loads of a kernel that has four times the wavefronts of the backward one.
template <int C, typename Map, bool SHARES_TABLES = true>
constexpr int run_length() { return (C < 1024 && SHARES_TABLES) ? Map::kRun : 1; }

// One row's share of the tables in registers: lane l holds the VEC columns of each of its CHUNKS pieces.
template <bool ON, int CHUNKS, int VEC>
struct RopeRows {};
template <int CHUNKS, int VEC>
struct RopeRows<true, CHUNKS, VEC> {
    float c[CHUNKS][VEC], s[CHUNKS][VEC];
    bool on;  // this lane's row is rotated (a row that exists, at a token index below rope.tokens)
    __device__ __forceinline__ void fetch(const RopeTable &rope, bool ok, int64_t seq, int C, int l, int LANES) {
        on = ok && seq < rope.tokens;
        if (on) {
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k) {
                const int64_t col0 = seq * C + (k * LANES + l) * VEC;
                load_fp32_run<VEC>(c[k], rope.cos + col0);
                load_fp32_run<VEC>(s[k], rope.sin + col0);
            }
        }
    }
};

// y -> y*cos + rotate_pairs(y)*sin in fp32 (y already rounded to the element type)
template <int VEC>
__device__ __forceinline__ void rotate_pairs_forward(float (&v)[VEC], const float (&c)[VEC], const float (&s)[VEC]) {
#pragma unroll
    for (int j = 0; j < VEC; j += 2) {
        const float a = v[j], b = v[j + 1];
        v[j] = a * c[j] - b * s[j];
        v[j + 1] = b * c[j + 1] + a * s[j + 1];
    }
}

// The gradient of the rotation as autograd forms it: g*cos and g*sin are each cast to the element
// type (the two branches of x.float() and rotate_pairs(x).float()), the latter routed back through
// the pair swap, and the two contributions are added in the element type.
template <typename E, int VEC>
__device__ __forceinline__ void rotate_pairs_backward(float (&g)[VEC], const float (&c)[VEC], const float (&s)[VEC]) {
    float direct[VEC], swapped[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        direct[j] = g[j] * c[j];
        swapped[j] = g[j] * s[j];
    }
    E::round(direct);
    E::round(swapped);
#pragma unroll
    for (int j = 0; j < VEC; j += 2) {
        g[j] = direct[j] + swapped[j + 1];
        g[j + 1] = direct[j + 1] - swapped[j];
    }
    E::round(g);
}

template <typename T, int C, typename Map, typename Rope = NoRope>
__global__ __launch_bounds__(kRowThreads) TTN_MIN_WAVES_PER_SIMD(sizeof(T) == 2 ? 4 : 3) void rmsnorm_fwd_kernel(
    T *__restrict__ out, float *__restrict__ rstd, const T *__restrict__ x,
    const T *__restrict__ w, const Map map, float eps, const Rope rope = Rope{}) {
    using G = RowGeom<T, C>;
    using E = Elem<T>;
    constexpr int VEC = G::VEC, LANES = G::LANES, CHUNKS = G::CHUNKS, RPW = G::RPW;
    const int lane = threadIdx.x & 63;
    const int sub = lane / LANES;  // which of the wavefront's rows
    const int l = lane % LANES;    // position inside the row
    const int wave = wave_id_in_block();

    u32x4 wr[CHUNKS];
#pragma unroll
    for (int k = 0; k < CHUNKS; ++k) wr[k] = load16(reinterpret_cast<const u32x4 *>(w) + k * LANES + l);

    // Narrow rows of a strided view: a wavefront takes kRun consecutive groups (see Strided3Rows).  In the
    // rotary form these are the heads of one token tile, which all read the same rows of the tables: fetched
    // per row, 1 KiB of table per 256-byte row would make the vector memory pipeline (64 bytes per clock per
    // compute unit), not HBM, the limit.
    constexpr int kRun = run_length<C, Map, Rope::kOn>();
    const int64_t groups = map.template groups<RPW>();
    const int64_t stride = (int64_t)gridDim.x * kRowWaves * kRun;
    [[maybe_unused]] bool aligned = false;
    if constexpr (kRun > 1) aligned = map.runs_aligned();
    for (int64_t first = ((int64_t)blockIdx.x * kRowWaves + wave) * kRun; first < groups; first += stride) {
        keep_packed(wr);
        RowAddr at[kRun];
        if constexpr (kRun > 1) {
            if (aligned) {
                const RowAddr head = map.template locate<RPW>(first, sub, C);
#pragma unroll
                for (int h = 0; h < kRun; ++h) at[h] = map.next_in_run(head, h);
            } else {
#pragma unroll
                for (int h = 0; h < kRun; ++h) {
                    at[h] = map.template locate<RPW>(first + h, sub, C);
                    at[h].ok = at[h].ok && first + h < groups;
                }
            }
        } else {
            at[0] = map.template locate<RPW>(first, sub, C);
        }
        u32x4 xr[kRun][CHUNKS];
#pragma unroll
        for (int h = 0; h < kRun; ++h) {
            const u32x4 *px = reinterpret_cast<const u32x4 *>(x + at[h].xoff) + l;
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k) xr[h][k] = at[h].ok ? load16_stream(px + k * LANES) : u32x4{0, 0, 0, 0};
        }
        RopeRows<Rope::kOn, CHUNKS, VEC> rot;
#pragma unroll
        for (int h = 0; h < kRun; ++h) {
            const bool ok = at[h].ok;
            if constexpr (Rope::kOn) {
                // the tables depend on the token index alone: fetched when it changes
                if (h == 0 || at[h].seq != at[h - 1].seq || !rot.on) rot.fetch(rope, ok, at[h].seq, C, l, LANES);
            }
            float ss = 0.0f;
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k) {
                float v[VEC];
                E::unpack(xr[h][k], v);
#pragma unroll
                for (int j = 0; j < VEC; ++j) ss = fmaf(v[j], v[j], ss);
            }
            ss = group_sum<LANES>(ss);
            const float r = 1.0f / sqrtf(ss / (float)C + eps);
            if (ok && l == 0) rstd[at[h].row] = r;

            // the wavefront's rows are consecutive in out: base = its first row
            const int64_t row0 = wave_uniform(at[h].row - sub);
            const RowWriter<TTN_RMS_FWD_STORE> wo(out + row0 * C, (uint32_t)((sub * C) * sizeof(T)) + l * 16);
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k) {
                float v[VEC], wv[VEC];
                E::unpack(xr[h][k], v);
                E::unpack(wr[k], wv);
#pragma unroll
                for (int j = 0; j < VEC; ++j) v[j] *= r;
                E::round(v);
#pragma unroll
                for (int j = 0; j < VEC; ++j) v[j] *= wv[j];
                if constexpr (Rope::kOn) {
                    if (rot.on) {
                        E::round(v);  // the norm's output in the element type, which the rotation reads
                        rotate_pairs_forward<VEC>(v, rot.c[k], rot.s[k]);
                    }
                }
                if (ok) wo.put(k * LANES, E::pack(v));
            }
        }
    }
}

// Backward.  FROM_OUT = false: xin is the saved input x.
//            FROM_OUT = true : xin is the saved forward output; xhat is recovered as out/w.
//
// One wavefront per SIMD at 3072 columns: the kernel is given the whole register
// file so that the weight stays unpacked, the column sums stay in registers and
// the NEXT row's g and x are already in flight while the current row is
// processed (two row buffers, ping-pong).  Few, fat, always-loading wavefronts
// keep about 48 KiB of reads in flight per compute unit, which is where this
// memory system streams best; more resident wavefronts only add queueing.
// Rope::kOn: dout is the gradient of the ROTATED output; it is turned back through the rotation
// (rotate_pairs_backward) as the row arrives, and everything below sees the gradient of the norm's output.
template <typename T, int C, bool FROM_OUT, typename Map, typename Rope = NoRope>
__global__ __launch_bounds__(kRowThreads) TTN_MIN_WAVES_PER_SIMD(C >= 1024 ? TTN_BWD_WAVES_PER_SIMD : 4) void rmsnorm_bwd_kernel(
    T *__restrict__ dx, float *__restrict__ partial, const T *__restrict__ g,
    const T *__restrict__ xin, const T *__restrict__ w, const float *__restrict__ rstd,
    const Map map, const Rope rope = Rope{}) {
    using G = RowGeom<T, C>;
    using E = Elem<T>;
    constexpr int VEC = G::VEC, LANES = G::LANES, CHUNKS = G::CHUNKS, RPW = G::RPW;
    constexpr bool kPackedDot = kHasDot2<T> && !FROM_OUT;  // sum_c gy*x straight from the packed pairs
    // row buffers in flight per wavefront; fp32 rows of 3072 take 96 registers each: one only
    constexpr int kRowBuffers = (sizeof(T) == 4 && C >= 1024) ? 1 : TTN_RMS_BWD_ROW_BUFFERS;
    // With the next row requested between the passes, a row's first pass starts only when the stores
    // of the row before it have left the wavefront (and with them this row's loads, which are older):
    // one wavefront never has more than one row of loads plus one row of stores outstanding.  Measured
    // at 118 800 rows: 354 us with this wait, 365 us when the first pass waits for its loads alone.
    constexpr bool kDrainStores = TTN_BWD_DRAIN_STORES && TTN_RMS_BWD_STORE && kRowBuffers == 2 && C >= 1024;
    __shared__ __align__(16) float lds[kFlushLdsFloats<1, C>];
    const int lane = threadIdx.x & 63;
    const int sub = lane / LANES;
    const int l = lane % LANES;
    const int wave = wave_id_in_block();

    constexpr bool kPackedProducts = kHasDot2<T> && (TTN_BWD_PACKED_MATH & 1) != 0;
    constexpr bool kPackedColumnSums = kPackedDot && (TTN_BWD_PACKED_MATH & 2) != 0;
    // the weight, resident for the whole kernel: unpacked to fp32, or (packed products) as the masked
    // pairs (w_lo, 0) and (0, w_hi)
    using Factor = PairFactor<std::conditional_t<kHasDot2<T>, T, bf16_t>>;  // (unused for 4-byte rows)
    [[maybe_unused]] const uint32_t one_lo = opaque_const(kOneLo<T>), one_hi = opaque_const(kOneHi<T>);
    [[maybe_unused]] float wv[(kPackedProducts && !FROM_OUT) ? 1 : CHUNKS][VEC];
    [[maybe_unused]] Factor wf[kPackedProducts ? CHUNKS : 1];
    [[maybe_unused]] float winv[FROM_OUT ? CHUNKS : 1][VEC];  // 1/weight for the saved-output variant
#pragma unroll
    for (int k = 0; k < CHUNKS; ++k) {
        const u32x4 wr = load16(reinterpret_cast<const u32x4 *>(w) + k * LANES + l);
        if constexpr (kPackedProducts) wf[k].set(wr);
        if constexpr (!kPackedProducts || FROM_OUT) E::unpack(wr, wv[k]);
        if constexpr (FROM_OUT) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) winv[k][j] = __builtin_amdgcn_rcpf(wv[k][j]);
        }
    }

    float acc[1][CHUNKS][VEC];
#pragma unroll
    for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[0][k][j] = 0.0f;

    struct RowRegs {
        u32x4 g[CHUNKS], x[CHUNKS];
        float r;
        int64_t doff0;   // element offset in dx of the wavefront's first row (wave-uniform)
        uint32_t dlane;  // this lane's byte offset from there
        int64_t seq;     // token index (rotary form only)
        bool ok;
    };
    // Narrow rows of a strided view: a wavefront walks runs of kRun consecutive groups (see Strided3Rows and
    // the forward kernel); the rotary form keeps the table rows it fetched until the token changes.
    constexpr int kRun = run_length<C, Map>();
    const int64_t groups = map.template groups<RPW>();
    const int64_t waves = (int64_t)gridDim.x * kRowWaves;
    const int64_t me = (int64_t)blockIdx.x * kRowWaves + wave;
    [[maybe_unused]] bool aligned = false;
    if constexpr (kRun > 1) aligned = map.runs_aligned();
    [[maybe_unused]] RowAddr run_head, run_head0;  // first group of the current aligned run: this lane's row, the wavefront's first row
    [[maybe_unused]] RopeRows<Rope::kOn, CHUNKS, VEC> rot;
    [[maybe_unused]] int64_t rot_seq = -1;
    // kRun == 1: at_step is the group.  Otherwise it is the wavefront's own step counter and fetch is called
    // with 0, 1, 2, ... in turn: step s is place s % kRun of the wavefront's run number s / kRun.
    auto fetch = [&](RowRegs &b, int64_t at_step) {
        RowAddr at, at0;
        if constexpr (kRun == 1) {
#if TTN_BWD_ROW_WRAP > 0
            at = map.template locate<RPW>(at_step % (TTN_BWD_ROW_WRAP / RPW), sub, C);
            at0 = map.template locate<RPW>(at_step % (TTN_BWD_ROW_WRAP / RPW), 0, C);
#else
            at = map.template locate<RPW>(at_step, sub, C);
            at0 = map.template locate<RPW>(at_step, 0, C);
#endif
        } else {
            const int h = (int)(at_step % kRun);
            const int64_t first = ((at_step / kRun) * waves + me) * kRun;
            if (aligned) {
                if (h == 0) {
                    run_head = map.template locate<RPW>(first, sub, C);
                    run_head0 = map.template locate<RPW>(first, 0, C);
                }
                at = map.next_in_run(run_head, h);
                at0 = map.next_in_run(run_head0, h);
            } else {
                at = map.template locate<RPW>(first + h, sub, C);
                at.ok = at.ok && first + h < groups;
                at0 = map.template locate<RPW>(first + h, 0, C);
            }
        }
        b.ok = at.ok;
        b.seq = at.seq;
        b.doff0 = at0.doff;
        b.dlane = (uint32_t)((at.doff - b.doff0) * (int64_t)sizeof(T)) + l * 16;
        const u32x4 *pg = reinterpret_cast<const u32x4 *>(g + at.row * C) + l;
        const u32x4 *px = reinterpret_cast<const u32x4 *>(xin + at.xoff) + l;
#if TTN_BWD_LOAD_POLICY >= 0
        if constexpr (LANES == kWaveSize) {
            const RowReader<TTN_BWD_LOAD_POLICY> rg(g + at.row * C, l * 16), rx(xin + at.xoff, l * 16);
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
        b.r = b.ok ? rstd[at.row] : 0.0f;
    };
    auto process = [&](RowRegs &b, auto &&between_passes) {
        const float r = b.r;
        if constexpr (Rope::kOn) {
            // dout arrives as the gradient of the rotated output: back through the rotation first
            if (b.seq != rot_seq) {
                rot.fetch(rope, b.ok, b.seq, C, l, LANES);
                rot_seq = rot.on ? b.seq : -1;
            }
            if (b.ok && rot.on) {
#pragma unroll
                for (int k = 0; k < CHUNKS; ++k) {
                    float gv[VEC];
                    E::unpack(b.g[k], gv);
                    rotate_pairs_backward<E, VEC>(gv, rot.c[k], rot.s[k]);
                    b.g[k] = E::pack(gv);
                }
            }
        }
        // pass 1: gy = rnd(g*w), kept packed in the element type; row dot  sum_c gy * xs
        //   xs = x (native) or xhat = out / w (from the saved output)
        u32x4 gyp[CHUNKS];
        float dot = 0.0f;
        if constexpr (kDrainStores) wait_memory_ops<0>();
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            if constexpr (kPackedProducts) {
                gyp[k] = rounded_products<T>(b.g[k], wf[k]);  // gy materialised in the element type
            } else {
                float gv[VEC];
                E::unpack(b.g[k], gv);
#pragma unroll
                for (int j = 0; j < VEC; ++j) gv[j] *= wv[k][j];
                gyp[k] = E::pack(gv);  // gy materialised in the element type
            }
            if constexpr (kPackedDot) {
#pragma unroll
                for (int i = 0; i < 4; ++i) dot = dot2<T>(gyp[k][i], b.x[k][i], dot);
            } else {
                float gy[VEC], xv[VEC];
                E::unpack(gyp[k], gy);
                E::unpack(b.x[k], xv);
#pragma unroll
                for (int j = 0; j < VEC; ++j) dot = fmaf(gy[j], FROM_OUT ? xv[j] * winv[k][j] : xv[j], dot);
            }
        }
        dot = group_sum<LANES>(dot);
        between_passes();
        // dx = gy*r + xs*coef
        const float coef = FROM_OUT ? -(r * (dot / (float)C)) : -((dot / (float)C) * r * r * r);

        const RowWriter<TTN_RMS_BWD_STORE> wd(dx + b.doff0, b.dlane);
#pragma unroll
        for (int k = 0; k < CHUNKS; ++k) {
            [[maybe_unused]] float gv[VEC];
            float gy[VEC], xv[VEC], o[VEC], y[VEC];
            if constexpr (!kPackedColumnSums) E::unpack(b.g[k], gv);
            E::unpack(gyp[k], gy);
            E::unpack(b.x[k], xv);
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const float xs = FROM_OUT ? xv[j] * winv[k][j] : xv[j];
                o[j] = fmaf(xs, coef, gy[j] * r);
                y[j] = FROM_OUT ? xs : xs * r;
            }
            if (b.ok) wd.put(k * LANES, E::pack(o));
            if constexpr (kPackedColumnSums) {
                Factor yf;  // y = the normalised row in the element type
                yf.set_rounded(y);
                const u32x4 pp = rounded_products<T>(b.g[k], yf);  // g*y in the element type, then summed
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc[0][k][2 * i] = dot2<T>(pp[i], one_lo, acc[0][k][2 * i]);
                    acc[0][k][2 * i + 1] = dot2<T>(pp[i], one_hi, acc[0][k][2 * i + 1]);
                }
            } else {
                E::round(y);  // y = normalised row in the element type
#pragma unroll
                for (int j = 0; j < VEC; ++j) y[j] *= gv[j];
                E::round(y);  // g*y materialised in the element type before the column sum
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc[0][k][j] += y[j];
            }
        }
    };

    if constexpr (kRun == 1) {
        row_pipeline<kRowBuffers, TTN_RMS_BWD_PREFETCH_MID != 0, RowRegs>(me, groups, waves, fetch, process);
    } else {
        // runs this wavefront starts: m = 0, 1, ... with (m * waves + me) * kRun < groups
        const int64_t all_runs = (groups + kRun - 1) / kRun;
        const int64_t my_runs = all_runs > me ? (all_runs - me + waves - 1) / waves : 0;
        row_pipeline<kRowBuffers, TTN_RMS_BWD_PREFETCH_MID != 0, RowRegs>(0, my_runs * kRun, 1, fetch, process);
    }
    flush_column_partials<G, 1>(acc, partial + (int64_t)blockIdx.x * C, lds);
}

// ---- rows of a contiguous tensor into a strided view --------------------------
// The value gradient of the QK-norm call site: v leaves the forward as a view of the fused projection, so its
// gradient arrives as a contiguous [B, H, S, D] tensor and belongs in the v slice of the projection's
// gradient, next to the dq and dk the backward kernels write there (torch.split's backward in the reference,
// teletron/models/dit/dit_attention.py:149-214).  Same traversal as the norm kernels: a wavefront takes
// 64 / LANES consecutive i2 of one (i0, i1), consecutive wavefronts consecutive i1.  Offsets of `map` count
// 16-byte pieces; a row is `pieces` of them.
template <int LANES>
__global__ __launch_bounds__(kRowThreads) void copy_rows_strided_kernel(u32x4 *__restrict__ dst,
                                                                        const u32x4 *__restrict__ src,
                                                                        const Strided3Rows map, int pieces) {
    constexpr int RPW = kWaveSize / LANES;
    const int lane = threadIdx.x & 63;
    const int sub = lane / LANES;
    const int l = lane % LANES;
    const int64_t groups = map.template groups<RPW>();
    const int64_t stride = (int64_t)gridDim.x * kRowWaves;
    for (int64_t grp = (int64_t)blockIdx.x * kRowWaves + wave_id_in_block(); grp < groups; grp += stride) {
        const RowAddr at = map.template locate<RPW>(grp, sub, 0);
        if (!at.ok) continue;
        const u32x4 *from = src + at.row * pieces;
        u32x4 *to = dst + at.doff;
        for (int p = l; p < pieces; p += LANES) store16_stream(to + p, load16_stream(from + p));
    }
}

// ---- tuning: workgroups per compute unit of the persistent grids ------------
// Forward at 3072 columns runs one-shot (one row per wavefront, then exit; the
// hardware dispatcher keeps a steady mix of loading and storing wavefronts, which
// streams ~6 % faster here than any persistent loop).  Forward at 128 columns and
// both backward kernels are persistent; backward at 3072 columns uses one
// workgroup per compute unit (one wavefront per SIMD).
constexpr int kOneShot = 1 << 20;
#ifndef TTN_RMS_FWD_BLOCKS_PER_CU
#define TTN_RMS_FWD_BLOCKS_PER_CU (C >= 1024 ? kOneShot : 16)
#endif
#ifndef TTN_RMS_BWD_BLOCKS_PER_CU
#define TTN_RMS_BWD_BLOCKS_PER_CU (C >= 1024 ? 1 : 3)
#endif
template <typename T, int C>
struct RmsTune {
    static constexpr int kFwdBlocksPerCu = TTN_RMS_FWD_BLOCKS_PER_CU;
    static constexpr int kBwdBlocksPerCu = TTN_RMS_BWD_BLOCKS_PER_CU;
};

template <typename T, int C, typename Map, typename Rope = NoRope>
static int rmsnorm_forward_t(void *out, float *rstd, const void *x, const void *w, const Map &map,
                             int64_t rows, double eps, hipStream_t stream, const Rope &rope = Rope{}) {
    if (rows == 0) return TT_NORM_OK;  // empty input: nothing to do
    int st = TT_NORM_OK;
    const int cus = current_device_cus(&st);
    if (st != TT_NORM_OK) return st;
    const RowPlan p = make_row_plan(1, rows, RowGeom<T, C>::RPW * run_length<C, Map, Rope::kOn>(), RmsTune<T, C>::kFwdBlocksPerCu, cus);
    if (p.blocks > 0x7fffffffLL) return fail(TT_NORM_EINVAL, "rmsnorm forward: grid too large");
    {
        RowKernelProfile prof(stream);
        rmsnorm_fwd_kernel<T, C, Map, Rope><<<dim3((unsigned)p.blocks), dim3(kRowThreads), TTN_RMS_FWD_DYN_LDS, stream>>>(
            (T *)out, rstd, (const T *)x, (const T *)w, map, (float)eps, rope);
    }
    return check_launch("rmsnorm forward launch");
}

// The backward grid (and with it the scratch size) depends on the row count only,
// also for strided views: a persistent grid covers any traversal.
template <typename T, int C>
static RowPlan rmsnorm_backward_plan(int64_t rows, int cus) {
    const int share = C >= 1024 ? (cus * TTN_BWD_GRID_PERCENT + 99) / 100 : cus;
    return make_row_plan(1, rows, RowGeom<T, C>::RPW, RmsTune<T, C>::kBwdBlocksPerCu, share);
}

template <typename T, int C, bool FROM_OUT, typename Map, typename Rope = NoRope>
static int rmsnorm_backward_t(void *dx, void *dw, const void *g, const void *xin, const void *w,
                              const float *rstd, const Map &map, int64_t rows, int dtype, void *ws,
                              size_t ws_bytes, hipStream_t stream, const Rope &rope = Rope{}) {
    // empty input: dweight is the empty sum, written by the reducer over zero partial rows
    if (rows == 0) return launch_colreduce(dw, nullptr, nullptr, nullptr, 1, 0, C, C, dtype, stream);
    int st = TT_NORM_OK;
    const int cus = current_device_cus(&st);
    if (st != TT_NORM_OK) return st;
    const RowPlan p = rmsnorm_backward_plan<T, C>(rows, cus);
    const size_t need = (size_t)p.blocks * C * sizeof(float);
    if (!ws || ws_bytes < need)
        return fail(TT_NORM_EWORKSPACE, "rmsnorm backward: workspace %zu B < required %zu B", ws_bytes, need);
    if (!aligned16(ws)) return fail(TT_NORM_EALIGN, "rmsnorm backward: workspace %p not 16-byte aligned", ws);
    {
        RowKernelProfile prof(stream);
        rmsnorm_bwd_kernel<T, C, FROM_OUT, Map, Rope><<<dim3((unsigned)p.blocks), dim3(kRowThreads), 0, stream>>>(
            (T *)dx, (float *)ws, (const T *)g, (const T *)xin, (const T *)w, rstd, map, rope);
    }
    st = check_launch("rmsnorm backward launch");
    if (st != TT_NORM_OK) return st;
    return launch_colreduce(dw, nullptr, nullptr, (const float *)ws, 1, p.blocks_per_sample, C, C, dtype, stream);
}

// tuned_only: the entry point exists for the tuned shapes only (reference-contract and strided forms).
static int check_rms_args(const char *who, int64_t rows, int64_t cols, int dtype,
                          std::initializer_list<const void *> ptrs, bool tuned_only = false) {
    if (rows < 0 || cols <= 0) return fail(TT_NORM_EINVAL, "%s: rows=%lld cols=%lld", who, (long long)rows, (long long)cols);
    if (tuned_only && !tuned_shape(cols, dtype))
        return fail(TT_NORM_EUNSUPPORTED, "%s: cols=%lld dtype=%d (this entry point: cols 128/3072)", who,
                    (long long)cols, dtype);
    if (!tt_norm_supported(cols, dtype))
        return fail(TT_NORM_EUNSUPPORTED,
                    "%s: cols=%lld dtype=%d (cols must be a multiple of 16 bytes of elements, at most 8192 "
                    "two-byte or 4096 four-byte; dtype bf16, fp16 or fp32)", who, (long long)cols, dtype);
    if (rows == 0) return TT_NORM_OK;  // empty input: nothing is dereferenced
    for (const void *p : ptrs) {
        if (!p) return fail(TT_NORM_EINVAL, "%s: null pointer", who);
        if (!aligned16(p)) return fail(TT_NORM_EALIGN, "%s: pointer %p not 16-byte aligned", who, p);
    }
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

int tt_rmsnorm_forward(void *out, float *rstd, const void *x, const void *weight, int64_t rows,
                       int64_t cols, double eps, int dtype, void *stream) {
    int st = check_rms_args("tt_rmsnorm_forward", rows, cols, dtype, {out, x, weight});
    if (st != TT_NORM_OK) return st;
    if (!rstd && rows > 0) return fail(TT_NORM_EINVAL, "tt_rmsnorm_forward: null rstd");
    if (!tuned_shape(cols, dtype))
        return anywidth_rmsnorm_forward(out, rstd, x, weight, rows, cols, eps, dtype, (hipStream_t)stream);
#define CALL(T, C) return rmsnorm_forward_t<T, C>(out, rstd, x, weight, DenseRows{rows}, rows, eps, (hipStream_t)stream)
    TTN_DISPATCH(dtype, cols, CALL);
#undef CALL
}

size_t tt_rmsnorm_backward_workspace_bytes(int64_t rows, int64_t cols, int dtype) {
    if (rows <= 0 || !tt_norm_supported(cols, dtype)) return 0;
    if (!tuned_shape(cols, dtype) || dense_backward_on_wide_rows(cols, dtype))
        return anywidth_rmsnorm_backward_workspace_bytes(rows, cols, dtype);
    int st = TT_NORM_OK;
    const int cus = current_device_cus(&st);
    if (st != TT_NORM_OK) return 0;
#define CALL(T, C) return (size_t)rmsnorm_backward_plan<T, C>(rows, cus).blocks * C * sizeof(float)
    TTN_DISPATCH(dtype, cols, CALL);
#undef CALL
}

int tt_rmsnorm_backward(void *dx, void *dweight, const void *dout, const void *x, const void *weight,
                        const float *rstd, int64_t rows, int64_t cols, int dtype, void *workspace,
                        size_t workspace_bytes, void *stream) {
    int st = check_rms_args("tt_rmsnorm_backward", rows, cols, dtype, {dx, dout, x, weight});
    if (st != TT_NORM_OK) return st;
    if (!dweight || (!rstd && rows > 0)) return fail(TT_NORM_EINVAL, "tt_rmsnorm_backward: null dweight/rstd");
    if (!tuned_shape(cols, dtype) || dense_backward_on_wide_rows(cols, dtype))
        return anywidth_rmsnorm_backward(dx, dweight, dout, x, weight, rstd, rows, cols, dtype, workspace,
                                         workspace_bytes, (hipStream_t)stream);
#define CALL(T, C)                                                                                  \
    return rmsnorm_backward_t<T, C, false>(dx, dweight, dout, x, weight, rstd, DenseRows{rows}, rows, dtype, \
                                           workspace, workspace_bytes, (hipStream_t)stream)
    TTN_DISPATCH(dtype, cols, CALL);
#undef CALL
}

int tt_rmsnorm_backward_from_out(void *dx, void *dweight, const void *dout, const void *out,
                                 const void *weight, const float *rstd, int64_t rows, int64_t cols,
                                 int dtype, void *workspace, size_t workspace_bytes, void *stream) {
    int st = check_rms_args("tt_rmsnorm_backward_from_out", rows, cols, dtype, {dx, dout, out, weight}, true);
    if (st != TT_NORM_OK) return st;
    if (!dweight || (!rstd && rows > 0)) return fail(TT_NORM_EINVAL, "tt_rmsnorm_backward_from_out: null dweight/rstd");
#define CALL(T, C)                                                                                   \
    return rmsnorm_backward_t<T, C, true>(dx, dweight, dout, out, weight, rstd, DenseRows{rows}, rows, dtype, \
                                          workspace, workspace_bytes, (hipStream_t)stream)
    TTN_DISPATCH(dtype, cols, CALL);
#undef CALL
}

static int check_strided(const char *who, int64_t n0, int64_t n1, int64_t n2, int64_t cols, int dtype,
                         const int64_t (&strides)[3], const char *what) {
    if (n0 < 0 || n1 < 0 || n2 < 0)
        return fail(TT_NORM_EINVAL, "%s: sizes [%lld, %lld, %lld]", who, (long long)n0, (long long)n1, (long long)n2);
    if (!tt_norm_supported(cols, dtype)) return TT_NORM_OK;  // reported by the common check
    const int64_t vec = 16 / (int64_t)elem_bytes(dtype);
    for (int64_t s : strides)
        if (s < 0 || s % vec != 0)
            return fail(TT_NORM_EALIGN, "%s: %s stride %lld is not a non-negative multiple of %lld elements (16 bytes)",
                        who, what, (long long)s, (long long)vec);
    // the rows one wavefront handles together (up to kMaxRowsPerWave consecutive indices of the last dimension:
    // eight for the narrowest any-width rows, four for 128 two-byte columns, two for 128 four-byte ones) are
    // addressed with 32-bit byte offsets from the first of them: (kMaxRowsPerWave - 1) * stride < 4 GiB
    if (strides[2] > kMaxRowStrideBytes / (int64_t)elem_bytes(dtype))
        return fail(TT_NORM_EINVAL, "%s: %s stride %lld of the row dimension exceeds 256 MiB", who, what,
                    (long long)strides[2]);
    return TT_NORM_OK;
}

int tt_rmsnorm_forward_strided(void *out, float *rstd, const void *x, const void *weight, int64_t n0,
                               int64_t n1, int64_t n2, int64_t xs0, int64_t xs1, int64_t xs2, int64_t cols,
                               double eps, int dtype, void *stream) {
    const int64_t xs[3] = {xs0, xs1, xs2};
    int st = check_strided("tt_rmsnorm_forward_strided", n0, n1, n2, cols, dtype, xs, "x");
    if (st != TT_NORM_OK) return st;
    const int64_t rows = n0 * n1 * n2;
    st = check_rms_args("tt_rmsnorm_forward_strided", rows, cols, dtype, {out, x, weight});
    if (st != TT_NORM_OK) return st;
    if (!rstd && rows > 0) return fail(TT_NORM_EINVAL, "tt_rmsnorm_forward_strided: null rstd");
    const Strided3Rows map{n0, n1, n2, xs0, xs1, xs2, 0, 0, 0};
    if (!tuned_shape(cols, dtype))
        return anywidth_rmsnorm_forward_strided(out, rstd, x, weight, map, cols, eps, dtype, (hipStream_t)stream);
#define CALL(T, C) return rmsnorm_forward_t<T, C>(out, rstd, x, weight, map, rows, eps, (hipStream_t)stream)
    TTN_DISPATCH(dtype, cols, CALL);
#undef CALL
}

int tt_rmsnorm_backward_strided(void *dx, void *dweight, const void *dout, const void *x, const void *weight,
                                const float *rstd, int64_t n0, int64_t n1, int64_t n2, int64_t xs0,
                                int64_t xs1, int64_t xs2, int64_t dxs0, int64_t dxs1, int64_t dxs2,
                                int64_t cols, int dtype, void *workspace, size_t workspace_bytes,
                                void *stream) {
    const int64_t xs[3] = {xs0, xs1, xs2}, ds[3] = {dxs0, dxs1, dxs2};
    int st = check_strided("tt_rmsnorm_backward_strided", n0, n1, n2, cols, dtype, xs, "x");
    if (st == TT_NORM_OK) st = check_strided("tt_rmsnorm_backward_strided", n0, n1, n2, cols, dtype, ds, "dx");
    if (st != TT_NORM_OK) return st;
    const int64_t rows = n0 * n1 * n2;
    st = check_rms_args("tt_rmsnorm_backward_strided", rows, cols, dtype, {dx, dout, x, weight});
    if (st != TT_NORM_OK) return st;
    if (!dweight || (!rstd && rows > 0)) return fail(TT_NORM_EINVAL, "tt_rmsnorm_backward_strided: null dweight/rstd");
    const Strided3Rows map{n0, n1, n2, xs0, xs1, xs2, dxs0, dxs1, dxs2};
    if (!tuned_shape(cols, dtype))
        return anywidth_rmsnorm_backward_strided(dx, dweight, dout, x, weight, rstd, map, cols, dtype, workspace,
                                                 workspace_bytes, (hipStream_t)stream);
#define CALL(T, C)                                                                                       \
    return rmsnorm_backward_t<T, C, false>(dx, dweight, dout, x, weight, rstd, map, rows, dtype, workspace, \
                                           workspace_bytes, (hipStream_t)stream)
    TTN_DISPATCH(dtype, cols, CALL);
#undef CALL
}

int tt_norm_copy_rows_strided(void *dst, const void *src, int64_t n0, int64_t n1, int64_t n2, int64_t ds0,
                              int64_t ds1, int64_t ds2, int64_t cols, int dtype, void *stream) {
    const char *who = "tt_norm_copy_rows_strided";
    if (dtype != TT_NORM_BF16 && dtype != TT_NORM_F16 && dtype != TT_NORM_F32)
        return fail(TT_NORM_EUNSUPPORTED, "%s: dtype %d", who, dtype);
    const int64_t vec = 16 / (int64_t)elem_bytes(dtype);
    if (cols <= 0 || cols % vec != 0 || cols / vec > (1 << 20))
        return fail(TT_NORM_EUNSUPPORTED, "%s: cols=%lld is not a whole number of 16-byte pieces", who, (long long)cols);
    if (n0 < 0 || n1 < 0 || n2 < 0)
        return fail(TT_NORM_EINVAL, "%s: sizes [%lld, %lld, %lld]", who, (long long)n0, (long long)n1, (long long)n2);
    for (int64_t s : {ds0, ds1, ds2})
        if (s < 0 || s % vec != 0)
            return fail(TT_NORM_EALIGN, "%s: dst stride %lld is not a non-negative multiple of %lld elements (16 bytes)",
                        who, (long long)s, (long long)vec);
    const int64_t rows = n0 * n1 * n2;
    if (rows == 0) return TT_NORM_OK;
    if (!dst || !src) return fail(TT_NORM_EINVAL, "%s: null pointer", who);
    if (!aligned16(dst) || !aligned16(src)) return fail(TT_NORM_EALIGN, "%s: pointer not 16-byte aligned", who);
    int st = TT_NORM_OK;
    const int cus = current_device_cus(&st);
    if (st != TT_NORM_OK) return st;
    const int pieces = (int)(cols / vec);
    const Strided3Rows map{n0, n1, n2, 0, 0, 0, ds0 / vec, ds1 / vec, ds2 / vec};
    const int lanes = pieces <= 4 ? 4 : pieces <= 8 ? 8 : pieces <= 16 ? 16 : pieces <= 32 ? 32 : 64;
    const RowPlan p = make_row_plan(1, rows, kWaveSize / lanes, 16, cus);
    if (p.blocks > 0x7fffffffLL) return fail(TT_NORM_EINVAL, "%s: grid too large", who);
    const dim3 grid((unsigned)p.blocks), block(kRowThreads);
    const hipStream_t s = (hipStream_t)stream;
    u32x4 *d = (u32x4 *)dst;
    const u32x4 *f = (const u32x4 *)src;
    switch (lanes) {
        case 4: copy_rows_strided_kernel<4><<<grid, block, 0, s>>>(d, f, map, pieces); break;
        case 8: copy_rows_strided_kernel<8><<<grid, block, 0, s>>>(d, f, map, pieces); break;
        case 16: copy_rows_strided_kernel<16><<<grid, block, 0, s>>>(d, f, map, pieces); break;
        case 32: copy_rows_strided_kernel<32><<<grid, block, 0, s>>>(d, f, map, pieces); break;
        default: copy_rows_strided_kernel<64><<<grid, block, 0, s>>>(d, f, map, pieces); break;
    }
    return check_launch("strided row copy launch");
}

/* ---- strided QK-norm with the rotary embedding applied behind it (head dimension 128) ---- */

static int check_rope(const char *who, int64_t cols, const float *cos, const float *sin, int64_t rope_tokens,
                      int64_t n2) {
    if (cols != 128) return fail(TT_NORM_EUNSUPPORTED, "%s: built for cols 128 (the head dimension) only", who);
    if (rope_tokens < 0 || rope_tokens > n2)
        return fail(TT_NORM_EINVAL, "%s: rope_tokens=%lld outside [0, n2=%lld]", who, (long long)rope_tokens, (long long)n2);
    if (rope_tokens > 0 && (!cos || !sin)) return fail(TT_NORM_EINVAL, "%s: null cos/sin table", who);
    if (!aligned16(cos) || !aligned16(sin)) return fail(TT_NORM_EALIGN, "%s: cos/sin table not 16-byte aligned", who);
    return TT_NORM_OK;
}

int tt_rmsnorm_rope_forward_strided(void *out, float *rstd, const void *x, const void *weight, const float *cos,
                                    const float *sin, int64_t rope_tokens, int64_t n0, int64_t n1, int64_t n2,
                                    int64_t xs0, int64_t xs1, int64_t xs2, int64_t cols, double eps, int dtype,
                                    void *stream) {
    const int64_t xs[3] = {xs0, xs1, xs2};
    int st = check_strided("tt_rmsnorm_rope_forward_strided", n0, n1, n2, cols, dtype, xs, "x");
    if (st != TT_NORM_OK) return st;
    const int64_t rows = n0 * n1 * n2;
    st = check_rms_args("tt_rmsnorm_rope_forward_strided", rows, cols, dtype, {out, x, weight}, true);
    if (st == TT_NORM_OK) st = check_rope("tt_rmsnorm_rope_forward_strided", cols, cos, sin, rope_tokens, n2);
    if (st != TT_NORM_OK) return st;
    if (!rstd && rows > 0) return fail(TT_NORM_EINVAL, "tt_rmsnorm_rope_forward_strided: null rstd");
    const Strided3Rows map{n0, n1, n2, xs0, xs1, xs2, 0, 0, 0};
    const RopeTable rope{cos, sin, rope_tokens};
    const hipStream_t s = (hipStream_t)stream;
    if (dtype == TT_NORM_BF16)
        return rmsnorm_forward_t<bf16_t, 128, Strided3Rows, RopeTable>(out, rstd, x, weight, map, rows, eps, s, rope);
    if (dtype == TT_NORM_F16)
        return rmsnorm_forward_t<f16_t, 128, Strided3Rows, RopeTable>(out, rstd, x, weight, map, rows, eps, s, rope);
    return rmsnorm_forward_t<float, 128, Strided3Rows, RopeTable>(out, rstd, x, weight, map, rows, eps, s, rope);
}

int tt_rmsnorm_rope_backward_strided(void *dx, void *dweight, const void *dout, const void *x, const void *weight,
                                     const float *rstd, const float *cos, const float *sin, int64_t rope_tokens,
                                     int64_t n0, int64_t n1, int64_t n2, int64_t xs0, int64_t xs1, int64_t xs2,
                                     int64_t dxs0, int64_t dxs1, int64_t dxs2, int64_t cols, int dtype,
                                     void *workspace, size_t workspace_bytes, void *stream) {
    const int64_t xs[3] = {xs0, xs1, xs2}, ds[3] = {dxs0, dxs1, dxs2};
    int st = check_strided("tt_rmsnorm_rope_backward_strided", n0, n1, n2, cols, dtype, xs, "x");
    if (st == TT_NORM_OK) st = check_strided("tt_rmsnorm_rope_backward_strided", n0, n1, n2, cols, dtype, ds, "dx");
    if (st != TT_NORM_OK) return st;
    const int64_t rows = n0 * n1 * n2;
    st = check_rms_args("tt_rmsnorm_rope_backward_strided", rows, cols, dtype, {dx, dout, x, weight}, true);
    if (st == TT_NORM_OK) st = check_rope("tt_rmsnorm_rope_backward_strided", cols, cos, sin, rope_tokens, n2);
    if (st != TT_NORM_OK) return st;
    if (!dweight || (!rstd && rows > 0))
        return fail(TT_NORM_EINVAL, "tt_rmsnorm_rope_backward_strided: null dweight/rstd");
    const Strided3Rows map{n0, n1, n2, xs0, xs1, xs2, dxs0, dxs1, dxs2};
    const RopeTable rope{cos, sin, rope_tokens};
    const hipStream_t s = (hipStream_t)stream;
    if (dtype == TT_NORM_BF16)
        return rmsnorm_backward_t<bf16_t, 128, false, Strided3Rows, RopeTable>(dx, dweight, dout, x, weight, rstd, map, rows,
                                                                               dtype, workspace, workspace_bytes, s, rope);
    if (dtype == TT_NORM_F16)
        return rmsnorm_backward_t<f16_t, 128, false, Strided3Rows, RopeTable>(dx, dweight, dout, x, weight, rstd, map, rows,
                                                                              dtype, workspace, workspace_bytes, s, rope);
    return rmsnorm_backward_t<float, 128, false, Strided3Rows, RopeTable>(dx, dweight, dout, x, weight, rstd, map, rows, dtype,
                                                                          workspace, workspace_bytes, s, rope);
}

}  // extern "C"
