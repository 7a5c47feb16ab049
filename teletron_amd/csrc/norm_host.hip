// Status handling, device facts, launch geometry and the fixed-order column
// reducer (stage 2 of every parameter-gradient reduction).
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
    wave_clock_mark(kClockColReduce, 0);
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
    wave_clock_mark(kClockColReduce, 1);
}

// The same sums, 128 columns per workgroup: thread (tx, ty) of 32 x 32 owns the four adjacent columns of one
// 16-byte piece and adds partial rows ty, ty+32, ... in ascending order with up to eight loads in flight; then
// one thread per column adds the 32 strands in ascending ty.  Same association order as colreduce_kernel (so
// the same bits), a quarter of the workgroups, 16-byte loads.  ncols must be a multiple of four and the partial
// rows 16-byte aligned.
constexpr int kRedWideCols = 4 * kRedCols;

template <typename T>
__global__ __launch_bounds__(kRedCols *kRedStrands) void colreduce_wide_kernel(
    T *__restrict__ out0, T *__restrict__ out1, T *__restrict__ out2, const float *__restrict__ partial,
    int blocks_per_sample, int C, int ncols, int col_blocks) {
    __shared__ float strands[kRedStrands][kRedWideCols + 4];
    wave_clock_mark(kClockColReduce, 0);
    const int tx = threadIdx.x % kRedCols;
    const int ty = threadIdx.x / kRedCols;
    const int64_t b = blockIdx.x / col_blocks;
    const int col0 = (int)(blockIdx.x % col_blocks) * kRedWideCols;
    const int col = col0 + 4 * tx;
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (col < ncols) {
        const float *p = partial + (b * blocks_per_sample) * (int64_t)ncols + col;
        int g = ty;
        for (; g + 7 * kRedStrands < blocks_per_sample; g += 8 * kRedStrands) {
            u32x4 v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = *reinterpret_cast<const u32x4 *>(p + (int64_t)(g + i * kRedStrands) * ncols);
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[j] += as_f32(v[i][j]);
        }
        for (; g < blocks_per_sample; g += kRedStrands) {
            const u32x4 v = *reinterpret_cast<const u32x4 *>(p + (int64_t)g * ncols);
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] += as_f32(v[j]);
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) strands[ty][4 * tx + j] = acc[j];
    __syncthreads();
    const int c = col0 + (int)threadIdx.x;
    if (threadIdx.x < kRedWideCols && c < ncols) {
        float s = strands[0][threadIdx.x];
#pragma unroll
        for (int i = 1; i < kRedStrands; ++i) s += strands[i][threadIdx.x];
        T *dst = c < C ? out0 : (c < 2 * C ? out1 : out2);  // column sets of C columns each
        store_scalar<T>(dst + b * C + c % C, s);
    }
    wave_clock_mark(kClockColReduce, 1);
}

// 1: colreduce_wide_kernel where its conditions hold; 0: colreduce_kernel always.  Measured inside cfg3's step with
// the per-wavefront clocks (256 partial rows of 6144 columns): 3.1 us from first wavefront start to last end for
// the wide form against 2.3 us for the narrow one, whose 192 workgroups spread the same loads over four times
// as many wavefronts; the narrow one stays.
#ifndef TTN_COLREDUCE_WIDE
#define TTN_COLREDUCE_WIDE 0
#endif

int launch_colreduce(void *out0, void *out1, void *out2, const float *partial, int64_t batch,
                     int blocks_per_sample, int64_t C, int64_t ncols, int dtype,
                     hipStream_t stream) {
    if (TTN_COLREDUCE_WIDE && ncols % 4 == 0 && aligned16(partial)) {
        const int col_blocks = (int)((ncols + kRedWideCols - 1) / kRedWideCols);
        const int64_t grid = batch * col_blocks;
        if (grid > 0x7fffffffLL) return fail(TT_NORM_EINVAL, "column reducer grid too large");
        dim3 g((unsigned)grid), blk(kRedCols * kRedStrands);
        if (dtype == TT_NORM_BF16)
            colreduce_wide_kernel<bf16_t><<<g, blk, 0, stream>>>((bf16_t *)out0, (bf16_t *)out1, (bf16_t *)out2, partial,
                                                                 blocks_per_sample, (int)C, (int)ncols, col_blocks);
        else if (dtype == TT_NORM_F16)
            colreduce_wide_kernel<f16_t><<<g, blk, 0, stream>>>((f16_t *)out0, (f16_t *)out1, (f16_t *)out2, partial,
                                                                blocks_per_sample, (int)C, (int)ncols, col_blocks);
        else
            colreduce_wide_kernel<float><<<g, blk, 0, stream>>>((float *)out0, (float *)out1, (float *)out2, partial,
                                                                blocks_per_sample, (int)C, (int)ncols, col_blocks);
        return check_launch("column reducer launch");
    }
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

#if TTN_WAVE_CLOCK
// Measurement builds only: hands the instrumented kernels a device buffer of kClockKernels * kWaveClockSlots * 4
// 64-bit entries (null switches the recording off).  Synchronous; call it while nothing is running.
int tt_norm_debug_wave_clock(void *buf) {
    if (hipMemcpyToSymbol(HIP_SYMBOL(ttn_wave_clock_buf), &buf, sizeof(buf)) != hipSuccess) return TT_NORM_EHIP;
    return adaln_set_wave_clock(buf);
}
size_t tt_norm_debug_wave_clock_bytes(void) { return (size_t)kClockKernels * kWaveClockSlots * 4 * sizeof(unsigned long long); }
#endif

int tt_norm_supported(int64_t cols, int dtype) {
    return (tuned_shape(cols, dtype) || anywidth_supported(cols, dtype)) ? 1 : 0;
}

int tt_norm_tuned(int64_t cols, int dtype) { return tuned_shape(cols, dtype) ? 1 : 0; }

int tt_norm_wide_forms_supported(int64_t cols, int dtype) {
    if (dtype != TT_NORM_BF16 && dtype != TT_NORM_F16 && dtype != TT_NORM_F32) return 0;
    return (cols == 3072 || anywidth_wide_forms_supported(cols, dtype)) ? 1 : 0;
}

int tt_norm_profile_next_row_kernel(void *start_event, void *stop_event) {
    if ((start_event == nullptr) != (stop_event == nullptr))
        return fail(TT_NORM_EINVAL, "profile_next_row_kernel: pass both events or neither");
    g_profile_start = (hipEvent_t)start_event;
    g_profile_stop = (hipEvent_t)stop_event;
    return TT_NORM_OK;
}

}  // extern "C"
