// Device-side building blocks shared by the gfx950 normalization kernels:
// 128-bit row access, bf16 <-> fp32 packing with the hardware RNE convert,
// wave64 DPP reductions, and the row -> lane geometry.
//
// Geometry.  A row of C elements is owned by LANES lanes of one wavefront;
// every lane moves 16 bytes (VEC elements) per access and a row takes CHUNKS
// accesses per lane, so each access of a wavefront is one contiguous,
// fully-coalesced 1 KiB (LANES = 64) segment:
//     column(chunk k, lane l, element j) = (k * LANES + l) * VEC + j
//   C = 3072 bf16 : LANES 64, CHUNKS 6  -> one wavefront per row, no LDS
//   C = 3072 fp32 : LANES 64, CHUNKS 12
//   C =  128 bf16 : LANES 16, CHUNKS 1  -> four rows per wavefront (one DPP row each)
//   C =  128 fp32 : LANES 32, CHUNKS 1  -> two rows per wavefront
// A lane owns the same columns for every row it ever sees, which is what lets
// the backward kernels keep parameter-gradient partial sums in registers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace ttn {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

// Storage-only tags for 2-byte elements (arithmetic is always fp32).
struct bf16_t {
    uint16_t bits;
};
struct f16_t {
    uint16_t bits;
};

constexpr int kWaveSize = 64;
constexpr int kRowWaves = 4;  // wavefronts per workgroup of every row kernel
// The narrowest row geometry any kernel is instantiated with (tuned: 16 lanes; any-width: 8), hence the most rows
// one wavefront handles together.  Rows of a wavefront are addressed with 32-bit byte offsets from the first of
// them, so (kMaxRowsPerWave - 1) row strides must stay below 4 GiB: the host caps a row stride at kMaxRowStrideBytes.
constexpr int kMinRowLanes = 8;
constexpr int kMaxRowsPerWave = kWaveSize / kMinRowLanes;
constexpr int64_t kMaxRowStrideBytes = (int64_t)1 << 28;
static_assert((kMaxRowsPerWave - 1) * kMaxRowStrideBytes + (1 << 20) < ((int64_t)1 << 32),
              "rows of one wavefront must stay within a 32-bit byte offset of the first");
constexpr int kRowThreads = kRowWaves * kWaveSize;

// Caps a kernel's register use so that at least N wavefronts fit on each SIMD
// (512 registers per lane per SIMD: N = 4 -> 128 registers, N = 2 -> 256).
#define TTN_MIN_WAVES_PER_SIMD(N) __attribute__((amdgpu_waves_per_eu(N)))

__device__ __forceinline__ float as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }

// Two fp32 -> one dword of two bf16, round-to-nearest-even (v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    bf16x2_t v;
    v[0] = (__bf16)lo;
    v[1] = (__bf16)hi;
    return __builtin_bit_cast(uint32_t, v);
}

template <typename T>
inline constexpr bool kIsBf16 = std::is_same<T, bf16_t>::value;
// 2-byte element types have a packed dot-product instruction.
template <typename T>
inline constexpr bool kHasDot2 = sizeof(T) == 2;

// (1.0, 1.0) as two elements of T in one dword.
template <typename T>
inline constexpr uint32_t kOnesPair = kIsBf16<T> ? 0x3F803F80u : 0x3C003C00u;

// (1, 0) and (0, 1) as pairs of T: a packed dot product against one of them adds one half of a pair
// to an fp32 accumulator, and a pair with one half cleared turns the packed dot product into the
// exact fp32 product of the other halves -- "unpack and multiply" / "unpack and add" in one
// instruction per element instead of two.
template <typename T>
inline constexpr uint32_t kOneLo = kIsBf16<T> ? 0x00003F80u : 0x00003C00u;
template <typename T>
inline constexpr uint32_t kOneHi = kIsBf16<T> ? 0x3F800000u : 0x3C000000u;

// A 32-bit constant handed to the compiler in a scalar register whose value it cannot see.  Needed for
// pair constants that are operands of the packed bf16 dot product: the compiler encodes the pair
// (1.0, 0) as the inline operand 1.0, which the hardware reads as the fp32 number 1.0 -- the pair
// (0, 1.0) -- so both halves of a column-sum update would add the upper element.
__device__ __forceinline__ uint32_t opaque_const(uint32_t v) {
    asm("" : "+s"(v));
    return v;
}

// acc + a.lo*b.lo + a.hi*b.hi over one dword of two elements each (v_dot2c_f32_bf16 /
// v_dot2_f32_f16): products of bf16 or fp16 pairs are exact in fp32, so this is a row
// reduction step taken straight from the packed registers, with no unpacking.
template <typename T>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
    if constexpr (kIsBf16<T>)
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), acc,
                                               false);
    else
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, a), __builtin_bit_cast(f16x2_t, b), acc, false);
}

template <typename T>
struct Elem;

template <>
struct Elem<bf16_t> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ void unpack(const u32x4 &r, float (&v)[8]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = as_f32(r[i] << 16);
            v[2 * i + 1] = as_f32(r[i] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }
    static __device__ __forceinline__ u32x4 pack(const float (&v)[8]) {
        u32x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
        return r;
    }
    // Round every value to bf16 and back: the eager graph materialises this
    // tensor in bf16 at this point.
    static __device__ __forceinline__ void round(float (&v)[8]) {
        u32x4 r = pack(v);
        unpack(r, v);
    }
};

// IEEE half: conversions are the hardware's (v_cvt_f32_f16 exact, v_cvt_f16_f32 in the default
// round-to-nearest-even mode, subnormals kept).
template <>
struct Elem<f16_t> {
    static constexpr int VEC = 8;
    static __device__ __forceinline__ void unpack(const u32x4 &r, float (&v)[8]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const f16x2_t h = __builtin_bit_cast(f16x2_t, (uint32_t)r[i]);
            v[2 * i] = (float)h[0];
            v[2 * i + 1] = (float)h[1];
        }
    }
    // The value is an fp32 number before it is converted, as in the eager formulas (an fp32 op, then
    // .to(half)).  Left to itself the compiler folds the producing multiply into a mixed-precision
    // instruction in some kernels and not in others, and one element in ten thousand then differs
    // by an ulp from kernel to kernel.
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        asm("" : "+v"(lo), "+v"(hi));
        f16x2_t h;
        h[0] = (_Float16)lo;
        h[1] = (_Float16)hi;
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ u32x4 pack(const float (&v)[8]) {
        u32x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = pack2(v[2 * i], v[2 * i + 1]);
        return r;
    }
    static __device__ __forceinline__ void round(float (&v)[8]) {
        u32x4 r = pack(v);
        unpack(r, v);
    }
};

template <>
struct Elem<float> {
    static constexpr int VEC = 4;
    static __device__ __forceinline__ void unpack(const u32x4 &r, float (&v)[4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = as_f32(r[i]);
    }
    static __device__ __forceinline__ u32x4 pack(const float (&v)[4]) {
        u32x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = as_u32(v[i]);
        return r;
    }
    static __device__ __forceinline__ void round(float (&)[4]) {}
};

// ---- rounded products straight from packed pairs ------------------------------------
// rnd(a*b) for the eight elements of a 16-byte piece, both factors 2-byte values: the product of two
// bf16 or fp16 values is exact in fp32, so rounding it once to the element type is what the eager
// formulas do when they multiply two tensors of that type.
//   fp16: the packed half multiply (v_pk_mul_f16) is that operation, one instruction per pair.
//   bf16: there is no packed bf16 multiply; the packed dot product  a.lo*b.lo + a.hi*b.hi + 0  against a
//     pair with one half cleared is the exact product of the other halves: one instruction per
//     element where unpacking and multiplying takes two.  The second factor is therefore held as the
//     two masked pairs (b.lo, 0) and (0, b.hi).
// PairFactor<T> is the second factor in the form its type wants; it can be set from packed pairs or
// from eight fp32 values that are rounded to the element type on the way.
template <typename T>
struct PairFactor;

template <>
struct PairFactor<bf16_t> {
    uint32_t lo[4], hi[4];
    __device__ __forceinline__ void set(const u32x4 &p) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            lo[i] = p[i] & 0x0000ffffu;
            hi[i] = p[i] & 0xffff0000u;
        }
    }
    __device__ __forceinline__ void set_rounded(const float (&v)[8]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // (rnd(v), 0) and (0, rnd(v)) in one conversion each; written out because the compiler builds
            // the pair with a constant half from a conversion plus a byte permute
            asm("v_cvt_pk_bf16_f32 %0, %1, 0" : "=v"(lo[i]) : "v"(v[2 * i]));
            asm("v_cvt_pk_bf16_f32 %0, 0, %1" : "=v"(hi[i]) : "v"(v[2 * i + 1]));
        }
    }
};

template <>
struct PairFactor<f16_t> {
    u32x4 p;
    __device__ __forceinline__ void set(const u32x4 &v) { p = v; }
    __device__ __forceinline__ void set_rounded(const float (&v)[8]) { p = Elem<f16_t>::pack(v); }
};

template <typename T>
__device__ __forceinline__ u32x4 rounded_products(const u32x4 &a, const PairFactor<T> &b);

template <>
__device__ __forceinline__ u32x4 rounded_products<f16_t>(const u32x4 &a, const PairFactor<f16_t> &b) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        r[i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2_t, (uint32_t)a[i]) *
                                                __builtin_bit_cast(f16x2_t, (uint32_t)b.p[i]));
    return r;
}

// Written as one block of instructions because the compiler only knows the accumulating form of the
// bf16 dot product (it clears a register first: two instructions per product again), and because a
// register written by a dot-product instruction may be read by another kind of instruction only three
// or more instructions later: the block keeps that distance itself (each conversion reads products
// issued at least three instructions before it), and what leaves the block was written by conversions.
template <>
__device__ __forceinline__ u32x4 rounded_products<bf16_t>(const u32x4 &a, const PairFactor<bf16_t> &b) {
    uint32_t r0, r1, r2, r3, q0, q1, q2, q3;
    asm("v_dot2_f32_bf16 %0, %8, %12, 0\n\t"
        "v_dot2_f32_bf16 %4, %8, %16, 0\n\t"
        "v_dot2_f32_bf16 %1, %9, %13, 0\n\t"
        "v_dot2_f32_bf16 %5, %9, %17, 0\n\t"
        "v_dot2_f32_bf16 %2, %10, %14, 0\n\t"
        "v_dot2_f32_bf16 %6, %10, %18, 0\n\t"
        "v_dot2_f32_bf16 %3, %11, %15, 0\n\t"
        "v_dot2_f32_bf16 %7, %11, %19, 0\n\t"
        "v_cvt_pk_bf16_f32 %0, %0, %4\n\t"
        "v_cvt_pk_bf16_f32 %1, %1, %5\n\t"
        "v_cvt_pk_bf16_f32 %2, %2, %6\n\t"
        "v_cvt_pk_bf16_f32 %3, %3, %7"
        : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3), "=&v"(q0), "=&v"(q1), "=&v"(q2), "=&v"(q3)
        : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(b.lo[0]), "v"(b.lo[1]), "v"(b.lo[2]), "v"(b.lo[3]),
          "v"(b.hi[0]), "v"(b.hi[1]), "v"(b.hi[2]), "v"(b.hi[3]));
    return u32x4{r0, r1, r2, r3};
}

template <typename T, int C>
struct RowGeom {
    static constexpr int VEC = Elem<T>::VEC;
    static constexpr int LANES = (C / VEC) < kWaveSize ? (C / VEC) : kWaveSize;
    static constexpr int CHUNKS = C / (VEC * LANES);
    static constexpr int RPW = kWaveSize / LANES;  // rows per wavefront
    static_assert(C % (VEC * LANES) == 0, "row must split into whole 16-byte accesses");
    static_assert(LANES == 16 || LANES == 32 || LANES == 64, "row must fill whole DPP rows");
};

// Streaming 16-byte accesses.  Activations are touched once per kernel, so
// they carry the non-temporal hint; parameters use the plain cached forms.
__device__ __forceinline__ u32x4 load16_stream(const u32x4 *p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void store16_stream(u32x4 *p, const u32x4 &v) { __builtin_nontemporal_store(v, p); }
__device__ __forceinline__ u32x4 load16(const u32x4 *p) { return *p; }

// Where a wavefront writes the rows of one loop iteration: a wave-uniform base address (the first of
// the wavefront's rows) plus a per-lane byte offset below 2 GiB; put(piece, v) stores 16 bytes at
// 16-byte piece `piece` (a compile-time multiple of LANES) past the lane's position.
//   THROUGH = 0: plain streaming store (non-temporal hint).
//   THROUGH = 1: the same store marked write-through at device scope (sc1) as well as non-temporal:
//     the line goes to memory as it is written instead of waiting dirty in L2 for an eviction.
//     Measured on the backward kernels (2 reads + 1 write): 367 -> 354 us; no gain on 1 read +
//     1 write.  Issued as a buffer store, the one store form whose cache-policy bits the compiler
//     exposes, so the compiler sees a store: it keeps the wait states after it and counts it in the
//     memory-operation counter, and a wait for the NEXT row's loads (requested before these stores)
//     does not wait for these stores as well.
template <int THROUGH>
struct RowWriter;

template <>
struct RowWriter<0> {
    u32x4 *p;
    __device__ __forceinline__ RowWriter(void *wave_base, uint32_t lane_bytes)
        : p(reinterpret_cast<u32x4 *>(static_cast<char *>(wave_base) + lane_bytes)) {}
    __device__ __forceinline__ void put(int piece, const u32x4 &v) const { store16_stream(p + piece, v); }
};

template <>
struct RowWriter<1> {
    static constexpr uint32_t kRawDwords = 0x00020000u;  // word 3 of a raw (untyped, unswizzled) resource
    static constexpr int kSc1Nt = 16 | 2;                // cache policy: sc1 (bit 4) | nt (bit 1)
    __amdgpu_buffer_rsrc_t rsrc;
    uint32_t off;
    __device__ __forceinline__ RowWriter(void *wave_base, uint32_t lane_bytes) : off(lane_bytes) {
        // the base lives in scalar registers; every caller passes a wave-uniform address
        const uint64_t a = reinterpret_cast<uint64_t>(wave_base);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
        rsrc = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void *>(((uint64_t)hi << 32) | lo), 0, 0xffffffffu,
                                                 kRawDwords);
    }
    __device__ __forceinline__ void put(int piece, const u32x4 &v) const {
        __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, off, piece * 16, kSc1Nt);
    }
};

// Where a wavefront reads one row from when the row's address is wave-uniform (one row per wavefront):
// the base in scalar registers, as RowWriter<1>, so that the load can carry any cache-policy bits
// (sc0 = 1, nt = 2, sc1 = 16); get(piece) loads the lane's 16 bytes at 16-byte piece `piece`.
template <int POLICY>
struct RowReader {
    __amdgpu_buffer_rsrc_t rsrc;
    uint32_t off;
    __device__ __forceinline__ RowReader(const void *wave_base, uint32_t lane_bytes) : off(lane_bytes) {
        const uint64_t a = reinterpret_cast<uint64_t>(wave_base);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
        rsrc = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void *>(((uint64_t)hi << 32) | lo), 0, 0xffffffffu,
                                                 RowWriter<1>::kRawDwords);
    }
    __device__ __forceinline__ u32x4 get(int piece) const {
        return __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, piece * 16, POLICY);
    }
};

// Waits until at most N of this wavefront's vector-memory operations (loads and stores, which
// complete in issue order) are outstanding.
template <int N>
__device__ __forceinline__ void wait_memory_ops() {
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}


// xhat = (x - mu) * r.  Two-byte element types take it as one fused multiply-add, x*r + (-mu*r): the
// rounding of mu*r (half an fp32 ulp of |mu|*r) is far below what the result is rounded to next.
// Four-byte rows subtract first, as the eager LayerNorm does: for a row whose mean is many standard
// deviations away, the fused form would cost a few fp32 ulps of |mu|*r in every element.
template <typename T>
__device__ __forceinline__ float centred(float x, float mu, float r, float nmr) {
    if constexpr (sizeof(T) == 4)
        return (x - mu) * r;
    else
        return fmaf(x, r, nmr);
}

// Makes the compiler forget what it knows about a packed register array (no
// instruction is emitted).  Used on loop-invariant packed parameters at the
// top of each row iteration: without it the unpacked fp32 copies are hoisted
// out of the loop and held live across it, which costs two registers per
// packed dword and pushes the kernels into spilling.
template <int N>
__device__ __forceinline__ void keep_packed(u32x4 (&a)[N]) {
#pragma unroll
    for (int k = 0; k < N; ++k) asm volatile("" : "+v"(a[k]));
}

// ---- wave64 reductions ---------------------------------------------------
// DPP control words (GCN3/CDNA "data parallel primitives").
constexpr int kDppQuadXor1 = 0xB1;      // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;      // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;
constexpr int kDppRowBcast15 = 0x142;   // lane 15 of each row -> next row
constexpr int kDppRowBcast31 = 0x143;   // lane 31 -> rows 2 and 3

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_take(float v) {
    // Lanes outside ROW_MASK receive 0.
    return as_f32((uint32_t)__builtin_amdgcn_update_dpp(0, (int)as_u32(v), CTRL, ROW_MASK, 0xf, false));
}

// Sum over each aligned group of 16 lanes; every lane gets its group's sum.
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_take<kDppQuadXor1, 0xf>(v);
    v += dpp_take<kDppQuadXor2, 0xf>(v);
    v += dpp_take<kDppRowHalfMirror, 0xf>(v);
    v += dpp_take<kDppRowMirror, 0xf>(v);
    return v;
}

// Sum over each aligned group of 8 lanes; every lane gets its group's sum.
__device__ __forceinline__ float row8_sum(float v) {
    v += dpp_take<kDppQuadXor1, 0xf>(v);
    v += dpp_take<kDppQuadXor2, 0xf>(v);
    v += dpp_take<kDppRowHalfMirror, 0xf>(v);
    return v;
}

// Sum over each aligned group of LANES lanes (8, 16, 32 or 64); every lane of the
// group gets the sum.  The 64-lane form funnels the four DPP-row sums into
// lane 63 with two row broadcasts and returns it through a scalar register,
// so it costs no LDS traffic at all.
template <int LANES>
__device__ __forceinline__ float group_sum(float v) {
    if constexpr (LANES == 8) return row8_sum(v);
    v = row16_sum(v);
    if constexpr (LANES == 32) {
        v += __shfl_xor(v, 16, kWaveSize);
    } else if constexpr (LANES == 64) {
        v += dpp_take<kDppRowBcast15, 0xa>(v);
        v += dpp_take<kDppRowBcast31, 0xc>(v);
        v = as_f32((uint32_t)__builtin_amdgcn_readlane((int)as_u32(v), 63));
    }
    return v;
}

// Adds, for every lane, the values held by the lanes that own the SAME columns
// in the other rows of this wavefront (RPW rows per wavefront).
template <int LANES>
__device__ __forceinline__ float fold_rows_of_wave(float v) {
    if constexpr (LANES <= 32) v += __shfl_xor(v, 32, kWaveSize);
    if constexpr (LANES <= 16) v += __shfl_xor(v, 16, kWaveSize);
    if constexpr (LANES <= 8) v += __shfl_xor(v, 8, kWaveSize);
    return v;
}

// A 64-bit value every lane of the wavefront holds alike, moved to scalar registers: indexing a per-row
// array with it is then a scalar load instead of a vector load that queues behind the row's own loads.
__device__ __forceinline__ int64_t wave_uniform(int64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

__device__ __forceinline__ int wave_id_in_block() {
    return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
}

// Measurement builds only (-DTTN_WAVE_CLOCK=1): every wavefront of an instrumented kernel records the constant
// 100 MHz clock when it starts and when its last memory operation has completed, into a buffer the host hands
// over with tt_norm_debug_wave_clock(): entry ((kernel_id * kWaveClockSlots + wavefront) * 4 + which), which = 0
// start, 1 end, 2 an intermediate point of the kernel's choosing.  The
// pointer is one variable per translation unit; a null pointer records nothing.  0 in a shipped build: the
// calls compile to nothing.
#ifndef TTN_WAVE_CLOCK
#define TTN_WAVE_CLOCK 0
#endif
constexpr int kWaveClockSlots = 1 << 20;
enum WaveClockKernel { kClockAdalnFwd = 0, kClockAdalnBwd = 1, kClockColReduce = 2, kClockKernels = 3 };
#if TTN_WAVE_CLOCK
static __device__ unsigned long long *ttn_wave_clock_buf = nullptr;
__device__ __forceinline__ void wave_clock_mark(int kernel_id, int which) {
    unsigned long long *buf = ttn_wave_clock_buf;
    if (!buf) return;
    if (which) __builtin_amdgcn_s_waitcnt(0);  // loads and stores of this wavefront have completed
    const unsigned long long t = __builtin_amdgcn_s_memrealtime();
    const size_t w = (size_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if ((threadIdx.x & 63) == 0 && w < (size_t)kWaveClockSlots)
        buf[((size_t)kernel_id * kWaveClockSlots + w) * 4 + which] = t;
}
#else
__device__ __forceinline__ void wave_clock_mark(int, int) {}
#endif

// Software pipeline over the rows of one wavefront.  `fetch(buf, grp)` issues the
// loads of a row, `process(buf, mid)` consumes them and calls `mid()` once
// between its two register passes.  grp advances by `stride` and is
// wave-uniform, so every branch here is too.
//   NBUF = 1 : plain loop (load, process, store; nothing else in flight).
//   NBUF = 2, MID = false : the next row is requested before the current one is processed.
//   NBUF = 2, MID = true  : the next row is requested half-way through the current one.
template <int NBUF, bool MID, typename RowRegs, typename Fetch, typename Process>
__device__ __forceinline__ void row_pipeline(int64_t grp, int64_t groups, int64_t stride, Fetch &&fetch,
                                             Process &&process) {
    static_assert(NBUF == 1 || NBUF == 2, "one or two row buffers");
    auto nothing = [] {};
    if constexpr (NBUF == 1) {
        for (; grp < groups; grp += stride) {
            RowRegs a;
            fetch(a, grp);
            process(a, nothing);
        }
    } else {
        if (grp >= groups) return;
        RowRegs buf0, buf1;
        fetch(buf0, grp);
        // one row: process `cur`, requesting the row after it into `nxt`; false when it was the last
        auto step = [&](RowRegs &cur, RowRegs &nxt) -> bool {
            const int64_t ahead = grp + stride;
            const bool more = ahead < groups;
            auto request = [&] {
                if (more) fetch(nxt, ahead);
            };
            if constexpr (MID) {
                process(cur, request);
            } else {
                request();
                process(cur, nothing);
            }
            grp = ahead;
            return more;
        };
        for (;;) {
            if (!step(buf0, buf1)) return;
            if (!step(buf1, buf0)) return;
        }
    }
}

// Consecutive groups a wavefront takes per step over a strided view of narrow rows (see Strided3Rows)
#ifndef TTN_STRIDED_RUN
#define TTN_STRIDED_RUN 6
#endif

// ---- where a wavefront's rows live ---------------------------------------------
// A row map turns (wavefront group index, row within the wavefront) into the
// row's logical number -- its index in the contiguous tensors (out, dout) and in
// the per-row statistics -- and its element offsets in the tensors that may be
// strided (x and, for backward, dx).
struct RowAddr {
    int64_t row;   // logical row number
    int64_t xoff;  // element offset of the row in x
    int64_t doff;  // element offset of the row in dx (backward only)
    int64_t seq;   // index along the view's last leading dimension (the token of a [B, H, S, D] view)
    bool ok;
};

// Row-major contiguous [rows, C].
struct DenseRows {
    static constexpr int kRun = 1;
    int64_t rows;
    template <int RPW>
    __device__ __forceinline__ int64_t groups() const { return (rows + RPW - 1) / RPW; }
    template <int RPW>
    __device__ __forceinline__ RowAddr locate(int64_t grp, int sub, int C) const {
        RowAddr a;
        a.row = grp * RPW + sub;
        a.ok = a.row < rows;
        a.xoff = a.doff = a.row * C;
        a.seq = a.row;
        return a;
    }
};

// A 4-D view [n0, n1, n2, C] with contiguous last dimension and arbitrary other
// strides (in elements); logical row number (i0*n1 + i1)*n2 + i2.  This is the
// per-head QK-norm input: query.transpose(1, 2) is [B, H, S, D] with strides
// (S*H*3D, 3D, H*3D, 1) inside the fused QKV projection output.
// Traversal: a wavefront takes RPW consecutive i2 of one (i0, i1) -- so what it
// writes to the contiguous side is one unbroken run -- and consecutive wavefronts
// take consecutive i1 for the same i2 tile, so the workgroups running at the
// same time read neighbouring pieces of the strided side.
struct Strided3Rows {
    // Narrow rows: a wavefront takes kRun consecutive groups at a time.  Consecutive groups are consecutive
    // i1 of one (i0, i2 tile), so when n1 is a multiple of kRun the run needs the divisions of locate() once
    // (they cost more than a 128-column row itself) and its groups share whatever is indexed by i2 alone.
    static constexpr int kRun = TTN_STRIDED_RUN;
    int64_t n0, n1, n2;
    int64_t xs0, xs1, xs2;
    int64_t ds0, ds1, ds2;
    __device__ __forceinline__ bool runs_aligned() const { return n1 % kRun == 0; }
    // the group h places after `a` inside an aligned run: same i0 and i2, i1 + h
    __device__ __forceinline__ RowAddr next_in_run(RowAddr a, int h) const {
        a.row += h * n2;
        a.xoff += h * xs1;
        a.doff += h * ds1;
        return a;
    }
    template <int RPW>
    __device__ __forceinline__ int64_t groups() const { return n0 * n1 * ((n2 + RPW - 1) / RPW); }
    template <int RPW>
    __device__ __forceinline__ RowAddr locate(int64_t grp, int sub, int /*C*/) const {
        const int64_t tiles2 = (n2 + RPW - 1) / RPW;
        const int64_t i1 = grp % n1;
        const int64_t q = grp / n1;
        const int64_t i2 = (q % tiles2) * RPW + sub;
        const int64_t i0 = q / tiles2;
        RowAddr a;
        a.ok = i2 < n2;
        a.seq = i2;
        a.row = (i0 * n1 + i1) * n2 + i2;
        a.xoff = i0 * xs0 + i1 * xs1 + i2 * xs2;
        a.doff = i0 * ds0 + i1 * ds1 + i2 * ds2;
        return a;
    }
};

// Where the rows of a sample live in the AdaLN tensors (x, out, dout, dx and the per-row statistics all
// share it), in units of rows: row(b, r) = b * sample_stride + r * row_stride.
//   sample-major [batch, rows_per_sample, C]: {rows_per_sample, 1}
//   sequence-first [rows_per_sample, batch, C] (the layout of the blocks' callers, where the modulation row
//   of sample b applies to rows b, b + batch, ...; teletron/models/dit/dit_layerspec.py:72-78): {1, batch}
struct SampleLayout {
    int64_t sample_stride, row_stride;
    __device__ __forceinline__ int64_t row(int64_t b, int64_t r) const { return b * sample_stride + r * row_stride; }
};

// How a workgroup folds the column sums of its four wavefronts into its partial row:
//   1: every wavefront deposits its sums in an LDS region of its own, one barrier, then all threads add the four
//      regions in wavefront order and write the row in 16-byte pieces (kRowWaves * NSETS * C floats of LDS);
//   0: wavefront 0 deposits, wavefronts 1.. add in turn into one region (four barriers), 4-byte writes.
// Both form ((w0 + w1) + w2) + w3 per column: bit-identical.  At 3072 columns and two sets the first takes
// about 1.5 us less per workgroup, which is time at the end of the kernel that nothing overlaps.
#ifndef TTN_FLUSH_PARALLEL
#define TTN_FLUSH_PARALLEL 1
#endif
template <int NSETS, int C>
inline constexpr int kFlushLdsFloats = (TTN_FLUSH_PARALLEL ? kRowWaves : 1) * NSETS * C;

// Adds this workgroup's per-lane column accumulators (acc[k][j] belongs to
// column (k*LANES + l)*VEC + j) across the rows of each wavefront and across
// wavefronts in fixed order, and writes one fp32 row of NSETS*C partial sums
// (16-byte aligned).  `lds` holds kFlushLdsFloats<NSETS, C> floats.
template <typename G, int NSETS>
__device__ __forceinline__ void flush_column_partials(float (&acc)[NSETS][G::CHUNKS][G::VEC],
                                                      float *__restrict__ partial_row, float *lds) {
    constexpr int VEC = G::VEC, LANES = G::LANES, CHUNKS = G::CHUNKS;
    constexpr int C = VEC * LANES * CHUNKS;
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

#if TTN_FLUSH_PARALLEL
    static_assert(VEC % 4 == 0 && (NSETS * C) % 4 == 0, "columns come in 16-byte pieces of fp32");
    if (sub == 0) {
        u32x4 *mine = reinterpret_cast<u32x4 *>(lds + wave * (NSETS * C));
#pragma unroll
        for (int s = 0; s < NSETS; ++s)
#pragma unroll
            for (int k = 0; k < CHUNKS; ++k)
#pragma unroll
                for (int q = 0; q < VEC / 4; ++q) {
                    // copies the compiler cannot see through: the 16-byte write wants four consecutive registers, and
                    // without the copies it keeps the accumulators themselves in such groups for the whole kernel,
                    // which costs the row loop a register move per accumulator and row
                    float a0 = acc[s][k][4 * q], a1 = acc[s][k][4 * q + 1], a2 = acc[s][k][4 * q + 2], a3 = acc[s][k][4 * q + 3];
                    asm volatile("" : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3));
                    mine[(s * C + (k * LANES + l) * VEC) / 4 + q] = u32x4{as_u32(a0), as_u32(a1), as_u32(a2), as_u32(a3)};
                }
    }
    __syncthreads();
    const u32x4 *all = reinterpret_cast<const u32x4 *>(lds);
    u32x4 *dst = reinterpret_cast<u32x4 *>(partial_row);
    constexpr int kPieces = NSETS * C / 4;
    for (int i = threadIdx.x; i < kPieces; i += kRowThreads) {
        u32x4 sum = all[i];
#pragma unroll
        for (int wv = 1; wv < kRowWaves; ++wv) {  // wavefront order: one fixed association
            const u32x4 v = all[wv * kPieces + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) sum[j] = as_u32(as_f32(sum[j]) + as_f32(v[j]));
        }
        dst[i] = sum;
    }
#else
    // wavefront 0 deposits, wavefronts 1.. add in turn: one fixed order
    for (int wv = 0; wv < kRowWaves; ++wv) {
        if (wave == wv && sub == 0) {
#pragma unroll
            for (int s = 0; s < NSETS; ++s)
#pragma unroll
                for (int k = 0; k < CHUNKS; ++k) {
                    float *p = lds + s * C + (k * LANES + l) * VEC;
#pragma unroll
                    for (int j = 0; j < VEC; ++j) p[j] = (wv == 0) ? acc[s][k][j] : p[j] + acc[s][k][j];
                }
        }
        __syncthreads();
    }
    for (int i = threadIdx.x; i < NSETS * C; i += kRowThreads) partial_row[i] = lds[i];
#endif
}

}  // namespace ttn
