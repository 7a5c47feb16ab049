// Host-side plumbing shared by the C-ABI entry points: status + thread-local
// error text, argument checks, cached device facts and the launch geometry
// ("plan") that both the workspace queries and the launches derive from.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/teletron_norm.h"
#include "norm_device.h"

namespace ttn {

int fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

// Number of compute units of the current device (cached per device ordinal).
int current_device_cus(int *status);

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline size_t elem_bytes(int dtype) { return dtype == TT_NORM_F32 ? 4 : 2; }

// (cols, dtype) the tuned kernels of rmsnorm.hip / adaln.hip are built for.
inline bool tuned_shape(int64_t cols, int dtype) {
    return (cols == 128 || cols == 3072) && (dtype == TT_NORM_BF16 || dtype == TT_NORM_F32 || dtype == TT_NORM_F16);
}

// Checks the last launch on this thread; returns TT_NORM_OK or TT_NORM_EHIP.
int check_launch(const char *what);

// Brackets the row-kernel launch made inside its scope with the event pair armed by
// tt_norm_profile_next_row_kernel (if any), on `stream`; disarms the pair.
class RowKernelProfile {
public:
    explicit RowKernelProfile(hipStream_t stream);
    ~RowKernelProfile();
    RowKernelProfile(const RowKernelProfile &) = delete;
    RowKernelProfile &operator=(const RowKernelProfile &) = delete;

private:
    hipStream_t stream_;
    hipEvent_t stop_;
};

// ---- launch geometry -------------------------------------------------------
// Every row kernel runs as a persistent 1-D grid of `batch * blocks_per_sample`
// workgroups of kRowWaves wavefronts.  Workgroup i serves sample
// i / blocks_per_sample only, and walks that sample's rows with stride
// blocks_per_sample * kRowWaves * RPW, so per-sample parameters are loaded once
// per workgroup and backward partial sums are naturally segmented by sample.

struct RowPlan {
    int rows_per_wave;       // RPW of the geometry
    int blocks_per_sample;   // >= 1
    int64_t blocks;          // batch * blocks_per_sample
};

// `blocks_per_cu`: how many workgroups per compute unit the kernel is tuned for.
RowPlan make_row_plan(int64_t batch, int64_t rows_per_sample, int rows_per_wave,
                      int blocks_per_cu, int cus);

// Stage-2 reducer: partial[batch][blocks_per_sample][ncols] fp32 ->
// out0[batch][C] (columns [0, C)), out1[batch][C] (columns [C, 2C)) when ncols >= 2C,
// out2[batch][C] (columns [2C, 3C)) when ncols == 3C.
int launch_colreduce(void *out0, void *out1, void *out2, const float *partial, int64_t batch,
                     int blocks_per_sample, int64_t C, int64_t ncols, int dtype,
                     hipStream_t stream);

// ---- any-width kernels (anywidth.hip): every other supported (cols, dtype) -----
// Native contract only (saved input + row statistics); same argument meaning as the
// C-ABI entry points that forward to them.
bool anywidth_supported(int64_t cols, int dtype);
int anywidth_rmsnorm_forward(void *out, float *rstd, const void *x, const void *w, int64_t rows, int64_t cols,
                             double eps, int dtype, hipStream_t stream);
size_t anywidth_rmsnorm_backward_workspace_bytes(int64_t rows, int64_t cols, int dtype);
int anywidth_rmsnorm_backward(void *dx, void *dw, const void *g, const void *x, const void *w,
                              const float *rstd, int64_t rows, int64_t cols, int dtype, void *ws,
                              size_t ws_bytes, hipStream_t stream);
// The same over a strided 4-D view (see Strided3Rows): out / dout / rstd contiguous in logical row order.
int anywidth_rmsnorm_forward_strided(void *out, float *rstd, const void *x, const void *w, const Strided3Rows &map,
                                     int64_t cols, double eps, int dtype, hipStream_t stream);
int anywidth_rmsnorm_backward_strided(void *dx, void *dw, const void *g, const void *x, const void *w,
                                      const float *rstd, const Strided3Rows &map, int64_t cols, int dtype,
                                      void *ws, size_t ws_bytes, hipStream_t stream);
// seq_first: rows laid out [rows_per_sample, batch] (sample b owns rows b, b + batch, ...) instead of
// [batch, rows_per_sample]; x, out, dout, dx and the statistics all share the layout.
int anywidth_adaln_forward(void *out, float *mean, float *rstd, const void *x, const void *scale,
                           const void *shift, int64_t batch, int64_t rows_per_sample, int64_t cols, double eps,
                           int dtype, hipStream_t stream, bool seq_first = false);
size_t anywidth_adaln_backward_workspace_bytes(int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype);
int anywidth_adaln_backward(void *dx, void *dscale, void *dshift, const void *g, const void *x,
                            const void *scale, const float *mean, const float *rstd, int64_t batch,
                            int64_t rows_per_sample, int64_t cols, int dtype, void *ws, size_t ws_bytes,
                            hipStream_t stream, bool seq_first = false);
// The gated residual and residual forms, for rows of up to six 16-byte accesses per lane
// (anywidth_wide_forms_supported): same argument meaning as the C-ABI entry points that forward to them.
bool anywidth_wide_forms_supported(int64_t cols, int dtype);
int anywidth_gated_adaln_forward(void *h2, void *out, float *mean, float *rstd, const void *h, const void *attn,
                                 const void *gate, const void *scale, const void *shift, int64_t batch,
                                 int64_t rows_per_sample, int64_t cols, double eps, int dtype, hipStream_t stream);
size_t anywidth_gated_adaln_backward_workspace_bytes(int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype);
int anywidth_gated_adaln_backward(void *dh, void *dattn, void *dgate, void *dscale, void *dshift, const void *g,
                                  const void *dh2, const void *h2, const void *attn, const void *gate,
                                  const void *scale, const float *mean, const float *rstd, int64_t batch,
                                  int64_t rows_per_sample, int64_t cols, int dtype, void *ws, size_t ws_bytes,
                                  hipStream_t stream);
int anywidth_adaln_backward_residual(void *dx, void *dscale, void *dshift, const void *g, const void *dres,
                                     const void *x, const void *scale, const float *mean, const float *rstd,
                                     int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype, void *ws,
                                     size_t ws_bytes, hipStream_t stream);

// 1: dense rows of more than 384 pieces go to the kernels of widerow.hip (four wavefronts per row); 0: they stay
// with the one-wavefront-per-row kernels of anywidth.hip (8, 12 or 16 accesses per lane), which strided views always use.
#ifndef TTN_WIDE_ROWS
#define TTN_WIDE_ROWS 1
#endif

// Measurement builds only (-DTTN_WAVE_CLOCK=1): sets the timestamp buffer of the kernels in adaln.hip.
int adaln_set_wave_clock(void *buf);

// ---- wide rows (widerow.hip): more than 384 16-byte pieces per row, four wavefronts per row -----
// Dense rows only (contiguous, or sample-major / sequence-first AdaLN); same argument meaning as above.
bool widerow_takes(int64_t cols, int dtype);
// Dense backward calls at a tuned width that run on the wide-row kernels all the same (fp32 rows of 3072 columns: a
// wavefront that owns such a row has registers for one row buffer only).
bool dense_backward_on_wide_rows(int64_t cols, int dtype);
// Measurement builds (-DTTN_GATED_3072_WIDE=1): the gated residual form at 3072 two-byte columns on the wide-row
// kernels instead of the tuned ones.  False in a shipped build.
bool gated_forward_on_wide_rows(int64_t cols, int dtype);
size_t widerow_backward_workspace_bytes(int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype, int nsets);
int widerow_rmsnorm_forward(void *out, float *rstd, const void *x, const void *w, int64_t rows, int64_t cols,
                            double eps, int dtype, hipStream_t stream);
int widerow_rmsnorm_backward(void *dx, void *dw, const void *g, const void *x, const void *w, const float *rstd,
                             int64_t rows, int64_t cols, int dtype, void *ws, size_t ws_bytes, hipStream_t stream);
int widerow_adaln_forward(void *out, float *mean, float *rstd, const void *x, const void *scale, const void *shift,
                          int64_t batch, int64_t rows_per_sample, int64_t cols, double eps, int dtype, bool seq_first,
                          hipStream_t stream);
int widerow_adaln_backward(void *dx, void *dscale, void *dshift, const void *g, const void *x, const void *scale,
                           const float *mean, const float *rstd, int64_t batch, int64_t rows_per_sample, int64_t cols,
                           int dtype, void *ws, size_t ws_bytes, bool seq_first, hipStream_t stream);
int widerow_gated_adaln_forward(void *h2, void *out, float *mean, float *rstd, const void *h, const void *attn,
                                const void *gate, const void *scale, const void *shift, int64_t batch,
                                int64_t rows_per_sample, int64_t cols, double eps, int dtype, hipStream_t stream);
int widerow_gated_adaln_backward(void *dh, void *dattn, void *dgate, void *dscale, void *dshift, const void *g,
                                 const void *dh2, const void *h2, const void *attn, const void *gate,
                                 const void *scale, const float *mean, const float *rstd, int64_t batch,
                                 int64_t rows_per_sample, int64_t cols, int dtype, void *ws, size_t ws_bytes,
                                 hipStream_t stream);
int widerow_adaln_backward_residual(void *dx, void *dscale, void *dshift, const void *g, const void *dres,
                                    const void *x, const void *scale, const float *mean, const float *rstd,
                                    int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype, void *ws,
                                    size_t ws_bytes, hipStream_t stream);

}  // namespace ttn
