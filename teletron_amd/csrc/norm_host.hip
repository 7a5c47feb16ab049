// Status handling, device facts, launch geometry, the fixed-order column
// reducer (stage 2 of every parameter-gradient reduction) and the streaming
// copy used as the bandwidth yardstick.
#include "norm_host.h"

#include <atomic>
#include <string.h>

#include "norm_device.h"

namespace ttn {

static thread_local char g_last_error[512] = "";

int fail(int status, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return status;
}

int current_device_cus(int *status) {
    constexpr int kMaxDevices = 64;
    static std::atomic<int> cache[kMaxDevices];  // zero-initialised: 0 = unknown
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        *status = fail(TT_NORM_EHIP, "hipGetDevice: %s", hipGetErrorString(e));
        return 0;
    }
    if (dev >= 0 && dev < kMaxDevices) {
        int c = cache[dev].load(std::memory_order_relaxed);
        if (c > 0) return c;
    }
    int cus = 0;
    e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess || cus <= 0) {
        *status = fail(TT_NORM_EHIP, "hipDeviceGetAttribute(multiprocessor count): %s",
                       hipGetErrorString(e));
        return 0;
    }
    if (dev >= 0 && dev < kMaxDevices) cache[dev].store(cus, std::memory_order_relaxed);
    return cus;
}

static thread_local hipEvent_t g_profile_start = nullptr;
static thread_local hipEvent_t g_profile_stop = nullptr;

RowKernelProfile::RowKernelProfile(hipStream_t stream) : stream_(stream), stop_(g_profile_stop) {
    if (g_profile_start) (void)hipEventRecord(g_profile_start, stream_);
    g_profile_start = nullptr;
    g_profile_stop = nullptr;
}

RowKernelProfile::~RowKernelProfile() {
    if (stop_) (void)hipEventRecord(stop_, stream_);
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(TT_NORM_EHIP, "%s: %s", what, hipGetErrorString(e));
    return TT_NORM_OK;
}

RowPlan make_row_plan(int64_t batch, int64_t rows_per_sample, int rows_per_wave,
                      int blocks_per_cu, int cus) {
    RowPlan p;
    p.rows_per_wave = rows_per_wave;
    const int64_t rows_per_block = (int64_t)kRowWaves * rows_per_wave;
    const int64_t needed = (rows_per_sample + rows_per_block - 1) / rows_per_block;  // per sample
    int64_t budget = ((int64_t)cus * blocks_per_cu) / batch;  // share of the persistent grid
    if (budget < 1) budget = 1;
    int64_t bps = needed < budget ? needed : budget;
    if (bps < 1) bps = 1;
    p.blocks_per_sample = (int)bps;
    p.blocks = batch * bps;
    return p;
}

// ---- stage 2: fixed-order column reduction ---------------------------------
// partial[b][g][ncols] -> out0/out1/out2[b][c] (ncols = 1, 2 or 3 sets of C columns).  A workgroup of 32 x 32 threads owns 32
// adjacent columns of one sample; thread (tx, ty) adds partial rows ty, ty+32,
// ... of column tx in ascending order, then one thread per column adds the 32
// strands in ascending ty.  Every sum has one fixed association order, so the
// result is bit-identical from run to run.
constexpr int kRedCols = 32;
constexpr int kRedStrands = 32;

template <typename T>
__device__ __forceinline__ void store_scalar(T *p, float v);
template <>
__device__ __forceinline__ void store_scalar<float>(float *p, float v) { *p = v; }
template <>
__device__ __forceinline__ void store_scalar<bf16_t>(bf16_t *p, float v) {
    p->bits = (uint16_t)(pack_bf16x2(v, 0.0f) & 0xffffu);
}
template <>
__device__ __forceinline__ void store_scalar<f16_t>(f16_t *p, float v) {
    p->bits = __builtin_bit_cast(uint16_t, (_Float16)v);
}

template <typename T>
__global__ __launch_bounds__(kRedCols *kRedStrands) void colreduce_kernel(
    T *__restrict__ out0, T *__restrict__ out1, T *__restrict__ out2, const float *__restrict__ partial,
    int blocks_per_sample, int C, int ncols, int col_blocks) {
    __shared__ float strands[kRedStrands][kRedCols + 1];
    const int tx = threadIdx.x % kRedCols;
    const int ty = threadIdx.x / kRedCols;
    const int64_t b = blockIdx.x / col_blocks;
    const int col = (int)(blockIdx.x % col_blocks) * kRedCols + tx;
    float acc = 0.0f;
    if (col < ncols) {
        const float *p = partial + (b * blocks_per_sample) * (int64_t)ncols + col;
        int g = ty;
        // four loads in flight per thread; the additions stay in ascending-g order
        for (; g + 3 * kRedStrands < blocks_per_sample; g += 4 * kRedStrands) {
            const float v0 = p[(int64_t)g * ncols];
            const float v1 = p[(int64_t)(g + kRedStrands) * ncols];
            const float v2 = p[(int64_t)(g + 2 * kRedStrands) * ncols];
            const float v3 = p[(int64_t)(g + 3 * kRedStrands) * ncols];
            acc = (((acc + v0) + v1) + v2) + v3;
        }
        for (; g < blocks_per_sample; g += kRedStrands) acc += p[(int64_t)g * ncols];
    }
    strands[ty][tx] = acc;
    __syncthreads();
    if (ty == 0 && col < ncols) {
        float s = strands[0][tx];
#pragma unroll
        for (int i = 1; i < kRedStrands; ++i) s += strands[i][tx];
        T *dst = col < C ? out0 : (col < 2 * C ? out1 : out2);  // column sets of C columns each
        store_scalar<T>(dst + b * C + col % C, s);
    }
}

int launch_colreduce(void *out0, void *out1, void *out2, const float *partial, int64_t batch,
                     int blocks_per_sample, int64_t C, int64_t ncols, int dtype,
                     hipStream_t stream) {
    const int col_blocks = (int)((ncols + kRedCols - 1) / kRedCols);
    const int64_t grid = batch * col_blocks;
    if (grid > 0x7fffffffLL) return fail(TT_NORM_EINVAL, "column reducer grid too large");
    dim3 g((unsigned)grid), blk(kRedCols * kRedStrands);
    if (dtype == TT_NORM_BF16)
        colreduce_kernel<bf16_t><<<g, blk, 0, stream>>>((bf16_t *)out0, (bf16_t *)out1, (bf16_t *)out2, partial,
                                                        blocks_per_sample, (int)C, (int)ncols, col_blocks);
    else if (dtype == TT_NORM_F16)
        colreduce_kernel<f16_t><<<g, blk, 0, stream>>>((f16_t *)out0, (f16_t *)out1, (f16_t *)out2, partial,
                                                       blocks_per_sample, (int)C, (int)ncols, col_blocks);
    else
        colreduce_kernel<float><<<g, blk, 0, stream>>>((float *)out0, (float *)out1, (float *)out2, partial,
                                                       blocks_per_sample, (int)C, (int)ncols, col_blocks);
    return check_launch("column reducer launch");
}

// ---- streaming copy ----------------------------------------------------------
// The fastest plain copy found on this part, used as the yardstick next to the
// kernels: one-shot grid, every wavefront copies one contiguous 6 KiB run (six
// 16-byte accesses per lane, the shape of a 3072-wide bf16 row) and exits.
__global__ __launch_bounds__(kRowThreads) void stream_copy_kernel(u32x4 *__restrict__ dst,
                                                                  const u32x4 *__restrict__ src, size_t n16) {
    constexpr int kDepth = 6;
    const int lane = threadIdx.x & 63;
    const size_t wave = (size_t)blockIdx.x * kRowWaves + wave_id_in_block();
    const size_t base = wave * (kDepth * kWaveSize) + lane;
    u32x4 v[kDepth];
#pragma unroll
    for (int k = 0; k < kDepth; ++k) {
        const size_t i = base + (size_t)k * kWaveSize;
        if (i < n16) v[k] = load16_stream(src + i);
    }
#pragma unroll
    for (int k = 0; k < kDepth; ++k) {
        const size_t i = base + (size_t)k * kWaveSize;
        if (i < n16) store16_stream(dst + i, v[k]);
    }
}

// ---- streaming probe -----------------------------------------------------------
// Plain streams with the access shapes the row kernels can choose from, for measuring what this
// memory system gives each read/write mix: NR tensors read (0..4), NW written (0..2);
// every wavefront moves one contiguous run of D KiB per tensor (D 16-byte accesses per lane; 6 is
// a 3072-column two-byte row) and either exits (one-shot grid) or strides on (persistent grid).
// Loads carry the non-temporal hint; THROUGH picks the store (see RowWriter).
struct ProbeTensors {
    const u32x4 *read[4];
    u32x4 *write[2];
};

template <int NR, int NW, int D, int THROUGH>
__global__ __launch_bounds__(kRowThreads) void stream_probe_kernel(const ProbeTensors t, int64_t runs,
                                                                   u32x4 *__restrict__ sink) {
    const int lane = threadIdx.x & 63;
    u32x4 keep{0, 0, 0, 0};
    const int64_t stride = (int64_t)gridDim.x * kRowWaves;
    for (int64_t run = (int64_t)blockIdx.x * kRowWaves + wave_id_in_block(); run < runs; run += stride) {
        const int64_t at = run * (D * kWaveSize);
        u32x4 v[NR > 0 ? NR : 1][D];
        if constexpr (NR == 0) {
#pragma unroll
            for (int k = 0; k < D; ++k) v[0][k] = u32x4{(uint32_t)run, 1, 2, 3};
        }
#pragma unroll
        for (int i = 0; i < NR; ++i)
#pragma unroll
            for (int k = 0; k < D; ++k) v[i][k] = load16_stream(t.read[i] + at + lane + k * kWaveSize);
#pragma unroll
        for (int i = 1; i < NR; ++i)
#pragma unroll
            for (int k = 0; k < D; ++k) v[0][k] += v[i][k];
        if constexpr (NW >= 1) {
#pragma unroll
            for (int j = 0; j < NW; ++j) {
                const RowWriter<THROUGH> wr(t.write[j] + at, lane * 16);
#pragma unroll
                for (int k = 0; k < D; ++k) wr.put(k * kWaveSize, v[0][k] + (uint32_t)j);
            }
        } else {
#pragma unroll
            for (int k = 0; k < D; ++k) keep += v[0][k];
        }
    }
    // read-only probes: keep the loads alive without ever storing
    if (NW == 0 && keep[0] == 0x12345678u && keep[1] == 0x9abcdef0u && keep[2] == 0x0fedcba9u) *sink = keep;
}

template <int NR, int NW, int D, int THROUGH>
static int launch_stream_probe(const ProbeTensors &t, int64_t runs, int64_t blocks, hipStream_t stream) {
    RowKernelProfile prof(stream);
    stream_probe_kernel<NR, NW, D, THROUGH><<<dim3((unsigned)blocks), dim3(kRowThreads), 0, stream>>>(t, runs, t.write[0]);
    return TT_NORM_OK;
}

}  // namespace ttn

using namespace ttn;

extern "C" {

int tt_norm_abi_version(void) { return TT_NORM_ABI_VERSION; }

const char *tt_norm_status_string(int status) {
    switch (status) {
        case TT_NORM_OK: return "ok";
        case TT_NORM_EINVAL: return "invalid argument";
        case TT_NORM_EUNSUPPORTED: return "unsupported cols/dtype for this entry point";
        case TT_NORM_EALIGN: return "pointer not 16-byte aligned";
        case TT_NORM_EWORKSPACE: return "workspace missing or too small";
        case TT_NORM_EHIP: return "HIP runtime error";
        default: return "unknown status";
    }
}

const char *tt_norm_last_error(void) { return g_last_error; }

int tt_norm_supported(int64_t cols, int dtype) {
    return (tuned_shape(cols, dtype) || anywidth_supported(cols, dtype)) ? 1 : 0;
}

int tt_norm_tuned(int64_t cols, int dtype) { return tuned_shape(cols, dtype) ? 1 : 0; }

int tt_norm_profile_next_row_kernel(void *start_event, void *stop_event) {
    if ((start_event == nullptr) != (stop_event == nullptr))
        return fail(TT_NORM_EINVAL, "profile_next_row_kernel: pass both events or neither");
    g_profile_start = (hipEvent_t)start_event;
    g_profile_stop = (hipEvent_t)stop_event;
    return TT_NORM_OK;
}

int tt_norm_stream_copy(void *dst, const void *src, size_t bytes, void *stream) {
    if (!dst || !src) return fail(TT_NORM_EINVAL, "stream_copy: null pointer");
    if (bytes % 16) return fail(TT_NORM_EINVAL, "stream_copy: bytes (%zu) not a multiple of 16", bytes);
    if (!aligned16(dst) || !aligned16(src)) return fail(TT_NORM_EALIGN, "stream_copy: unaligned pointer");
    if (bytes == 0) return TT_NORM_OK;
    const size_t n16 = bytes / 16;
    const size_t per_block = (size_t)kRowWaves * 6 * kWaveSize;
    const size_t blocks = (n16 + per_block - 1) / per_block;
    if (blocks > 0x7fffffffULL) return fail(TT_NORM_EINVAL, "stream_copy: %zu bytes is too large for one launch", bytes);
    stream_copy_kernel<<<dim3((unsigned)blocks), dim3(kRowThreads), 0, (hipStream_t)stream>>>(
        (u32x4 *)dst, (const u32x4 *)src, n16);
    return check_launch("stream copy launch");
}

int tt_norm_stream_probe(void *dst, const void *a, const void *b, size_t bytes, int reads, int writes,
                         int accesses_per_lane, int persistent_blocks, int write_through, void *stream) {
    if (reads < 0 || reads > 4 || writes < 0 || writes > 2 || reads + writes == 0)
        return fail(TT_NORM_EINVAL, "stream_probe: reads=%d (0..4) writes=%d (0..2), at least one stream", reads, writes);
    if (accesses_per_lane != 1 && accesses_per_lane != 2 && accesses_per_lane != 6)
        return fail(TT_NORM_EUNSUPPORTED, "stream_probe: accesses_per_lane=%d (built for 1, 2 and 6)", accesses_per_lane);
    if (persistent_blocks < 0) return fail(TT_NORM_EINVAL, "stream_probe: persistent_blocks=%d", persistent_blocks);
    const size_t run_bytes = (size_t)accesses_per_lane * kWaveSize * 16;
    if (bytes == 0 || bytes % run_bytes)
        return fail(TT_NORM_EINVAL, "stream_probe: bytes (%zu) must be a positive multiple of %zu", bytes, run_bytes);
    if (!dst || (reads >= 1 && !a) || (reads >= 2 && !b)) return fail(TT_NORM_EINVAL, "stream_probe: null pointer");
    if (!aligned16(dst) || !aligned16(a) || !aligned16(b)) return fail(TT_NORM_EALIGN, "stream_probe: unaligned pointer");
    const int64_t runs = (int64_t)(bytes / run_bytes);
    const int64_t blocks = persistent_blocks ? persistent_blocks : (runs + kRowWaves - 1) / kRowWaves;
    if (blocks > 0x7fffffffLL) return fail(TT_NORM_EINVAL, "stream_probe: grid too large");
    const hipStream_t s = (hipStream_t)stream;
    const int through = (write_through && writes) ? 1 : 0;
    // tensors 3 and 4 read, and the second one written, follow the first ones in the same allocations
    const char *ca = (const char *)a, *cb = (const char *)b;
    char *cd = (char *)dst;
    const ProbeTensors t{{(const u32x4 *)ca, (const u32x4 *)cb, (const u32x4 *)(ca + bytes), (const u32x4 *)(cb + bytes)},
                         {(u32x4 *)cd, (u32x4 *)(cd + bytes)}};
#define TTN_PROBE(NR, NW, D, TH)                                                          \
    if (reads == NR && writes == NW && accesses_per_lane == D && through == TH) {         \
        launch_stream_probe<NR, NW, D, TH>(t, runs, blocks, s);                           \
        return check_launch("stream probe launch");                                       \
    }
#define TTN_PROBE_D(NR, NW, TH) TTN_PROBE(NR, NW, 1, TH) TTN_PROBE(NR, NW, 2, TH) TTN_PROBE(NR, NW, 6, TH)
    TTN_PROBE_D(1, 0, 0) TTN_PROBE_D(2, 0, 0)
    TTN_PROBE_D(0, 1, 0) TTN_PROBE_D(1, 1, 0) TTN_PROBE_D(2, 1, 0)
    TTN_PROBE_D(0, 1, 1) TTN_PROBE_D(1, 1, 1) TTN_PROBE_D(2, 1, 1)
#undef TTN_PROBE_D
    // the mixes of the gated residual kernels (forward 2 reads + 2 writes, backward 4 + 2) and of the
    // backward with a residual gradient (3 + 1), in the one-row and the 1 KiB shapes
#define TTN_PROBE_W(NR, NW) TTN_PROBE(NR, NW, 1, 0) TTN_PROBE(NR, NW, 6, 0) TTN_PROBE(NR, NW, 1, 1) TTN_PROBE(NR, NW, 6, 1)
    TTN_PROBE_W(3, 1) TTN_PROBE_W(2, 2) TTN_PROBE_W(4, 2)
#undef TTN_PROBE_W
#undef TTN_PROBE
    return fail(TT_NORM_EUNSUPPORTED, "stream_probe: no kernel for this combination");
}

}  // extern "C"
