/* teletron_norm.h -- C ABI of the gfx950 fused normalization library
 * (libteletron_norm.so): fused RMSNorm and fused AdaLayerNorm, forward and
 * backward.  Tuned kernels for bf16, fp16 and fp32 rows of 128 or 3072 columns (the
 * shapes the reference's kernels are built for, teletron/models/dit/
 * dit_fusedlayers.py:91,301); any-width kernels for every other row of whole
 * 16-byte pieces, bf16 / fp16 / fp32, up to 8192 two-byte or 4096 four-byte
 * columns, behind the same native entry points.
 *
 * This is the seam the reference has between its pybind glue and its kernel
 * launchers (teletron_op/fused_rmsnorm/include/rmsnorm_kernel.h:5-25 and
 * teletron_op/fused_adaln/include/adaln_kernel.h:20-45): plain device
 * pointers and sizes in, nothing returned but a status.  Differences from
 * those launchers, all additive:
 *   - every call takes the HIP stream to enqueue on (the reference launches
 *     on the legacy default stream) and returns a status instead of void;
 *   - the element type is an argument (the reference is bf16 only);
 *   - AdaLN takes one scale/shift row PER SAMPLE ([batch, cols]), as the
 *     eager path does (teletron/models/dit/dit_fusedlayers.py:223); the
 *     reference kernels read a single row;
 *   - the backward entry points come in two flavours: the native one works
 *     from the saved INPUT x and row statistics (forward writes 1 tensor),
 *     the *_from_out / *_from_xnorm ones work from what the reference's
 *     Python functions save (forward output / normalised x) so the
 *     reference's autograd classes run unmodified;
 *   - scratch memory for the parameter-gradient partial sums is passed in by
 *     the caller (query the size first); the library never allocates.
 *
 * All pointers are device pointers, 16-byte aligned, row-major contiguous.
 * Zero rows is a valid input: forward does nothing, backward writes zeros to the
 * parameter gradients (no scratch needed); negative sizes are TT_NORM_EINVAL.
 * All calls are asynchronous on `stream` (a hipStream_t passed as void*;
 * NULL = the null stream).  Nothing here synchronises.
 */
#ifndef TELETRON_NORM_H_
#define TELETRON_NORM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 2: adds tt_norm_wide_forms_supported; the gated residual and residual entry points take every row of
 *    up to 384 16-byte pieces (they took 3072 columns only); the measurement kernels tt_norm_stream_copy
 *    and tt_norm_stream_probe left this library for libteletron_probe.so (include/teletron_probe.h).
 * 3: the gated residual and residual entry points take every supported row (up to 1024 pieces); scratch passed
 *    to a backward entry point must be 16-byte aligned; TT_NORM_STATIC_SCRATCH_BYTES is 32 MiB. */
#define TT_NORM_ABI_VERSION 3

enum tt_norm_status {
    TT_NORM_OK = 0,
    TT_NORM_EINVAL = 1,       /* null pointer, negative size, non-positive cols or batch */
    TT_NORM_EUNSUPPORTED = 2, /* cols or dtype this entry point is not built for */
    TT_NORM_EALIGN = 3,       /* a tensor pointer is not 16-byte aligned */
    TT_NORM_EWORKSPACE = 4,   /* workspace missing or smaller than *_workspace_bytes() */
    TT_NORM_EHIP = 5          /* the HIP runtime refused the launch; see tt_norm_last_error() */
};

enum tt_norm_dtype {
    TT_NORM_BF16 = 0,
    TT_NORM_F32 = 1,
    TT_NORM_F16 = 2
};

/* ABI version of the loaded library (TT_NORM_ABI_VERSION at build time). */
int tt_norm_abi_version(void);

/* Static description of a status code. */
const char *tt_norm_status_string(int status);

/* Thread-local detail of the last non-OK status returned on this thread. */
const char *tt_norm_last_error(void);

/* 1 if the native entry points (tt_rmsnorm_forward/backward, tt_adaln_forward/backward and
 * their workspace queries) accept (cols, dtype), else 0. */
int tt_norm_supported(int64_t cols, int dtype);

/* 1 if (cols, dtype) is one of the tuned shapes (cols 128 or 3072; bf16, fp16 or fp32): the only
 * ones the reference-contract entry points (*_from_out, *_xnorm, *_from_xnorm) take; the rotary
 * entry points take cols 128 only.  The strided and sequence-first entry points take whatever
 * tt_norm_supported accepts. */
int tt_norm_tuned(int64_t cols, int dtype);

/* 1 if the gated residual and residual entry points (tt_gated_residual_adaln_forward / _backward,
 * tt_adaln_backward_residual) accept (cols, dtype): every row tt_norm_supported accepts (whole 16-byte pieces,
 * at most 1024 of them: 8192 two-byte / 4096 four-byte columns).  For other rows those entry points return
 * TT_NORM_EUNSUPPORTED. */
int tt_norm_wide_forms_supported(int64_t cols, int dtype);

/* ------------------------------------------------------------------ RMSNorm
 * out = round(round(x * rstd) * weight),  rstd = 1/sqrt(mean_c(x^2) + eps)
 * (intermediate rounding to the element type as the eager path does,
 * teletron/models/dit/dit_fusedlayers.py:360-370).
 */

/* Replaces launch_rms_forward (rmsnorm_kernel.h:5-12, rms_forward.cu:102).
 * out [rows, cols], rstd [rows] fp32 (the reference's inv_variance). */
int tt_rmsnorm_forward(void *out, float *rstd, const void *x, const void *weight,
                       int64_t rows, int64_t cols, double eps, int dtype, void *stream);

/* Bytes of scratch tt_rmsnorm_backward* need for this shape.  Scratch passed to any backward entry point must be
 * 16-byte aligned (TT_NORM_EALIGN otherwise), like every tensor. */
size_t tt_rmsnorm_backward_workspace_bytes(int64_t rows, int64_t cols, int dtype);

/* Native backward from the saved input: dx [rows, cols], dweight [cols].
 * One pass over dout and x produces dx and per-workgroup partial column sums;
 * a second small kernel reduces the partials in a fixed order (deterministic).
 * Covers launch_rms_backward + launch_rms_weight_backward
 * (rms_backward.cu:91, weight_backward.cu:212). */
int tt_rmsnorm_backward(void *dx, void *dweight, const void *dout, const void *x,
                        const void *weight, const float *rstd,
                        int64_t rows, int64_t cols, int dtype,
                        void *workspace, size_t workspace_bytes, void *stream);

/* Same contract as the reference's launch_rms_backward (rmsnorm_kernel.h:19-24):
 * `out` is the saved FORWARD OUTPUT; the normalised row is recovered as
 * out / weight (weight must be non-zero, as in the reference). */
int tt_rmsnorm_backward_from_out(void *dx, void *dweight, const void *dout, const void *out,
                                 const void *weight, const float *rstd,
                                 int64_t rows, int64_t cols, int dtype,
                                 void *workspace, size_t workspace_bytes, void *stream);

/* Strided input: x is a 4-D view [n0, n1, n2, cols] whose last dimension is
 * contiguous and whose other strides xs0..xs2 (in ELEMENTS, multiples of 16 bytes,
 * >= 0) are arbitrary; out, dout and rstd are contiguous in logical order, i.e.
 * row (i0*n1 + i1)*n2 + i2.  This is the per-head QK-norm call site: the reference
 * normalises query.transpose(1, 2) (teletron/models/dit/dit_attention.py:201-212),
 * a [B, H, S, D] view into the fused QKV projection, and first materialises a
 * contiguous copy of it (teletron/models/dit/dit_fusedlayers.py:296); here the view
 * is read in place.  dx is written through its own strides dxs0..dxs2, so the caller
 * picks its layout.  Scratch: tt_rmsnorm_backward_workspace_bytes(n0*n1*n2, cols, dtype). */
int tt_rmsnorm_forward_strided(void *out, float *rstd, const void *x, const void *weight,
                               int64_t n0, int64_t n1, int64_t n2,
                               int64_t xs0, int64_t xs1, int64_t xs2,
                               int64_t cols, double eps, int dtype, void *stream);

int tt_rmsnorm_backward_strided(void *dx, void *dweight, const void *dout, const void *x,
                                const void *weight, const float *rstd,
                                int64_t n0, int64_t n1, int64_t n2,
                                int64_t xs0, int64_t xs1, int64_t xs2,
                                int64_t dxs0, int64_t dxs1, int64_t dxs2,
                                int64_t cols, int dtype,
                                void *workspace, size_t workspace_bytes, void *stream);

/* Rows of a contiguous [n0, n1, n2, cols] tensor `src` copied into a strided view `dst` of that shape
 * (strides in elements, multiples of 16 bytes; contiguous last dimension).  The QK-norm call site's
 * value gradient: v is a view of the fused projection, so dv [B, H, S, D] belongs in the v slice of the
 * projection's gradient beside the dq and dk that tt_rmsnorm_backward_strided writes there -- what
 * torch.split's backward does in the reference by concatenating three separate gradients
 * (teletron/models/dit/dit_attention.py:149-214).  Any cols that make whole 16-byte pieces. */
int tt_norm_copy_rows_strided(void *dst, const void *src, int64_t n0, int64_t n1, int64_t n2, int64_t ds0,
                              int64_t ds1, int64_t ds2, int64_t cols, int dtype, void *stream);

/* The strided QK-norm with the rotary embedding the attention caller applies right behind it
 * (teletron/models/dit/dit_attention.py:266-273 and :435-443: apply_rotary_emb(query, (freqs_cos,
 * freqs_sin)) on the [B, H, S, D] result of q_layernorm / k_layernorm, a separate read + write pass
 * per tensor in the reference; in the single-stream block only the first S_img tokens are rotated).
 * x is the [n0, n1, n2, cols] view as above with n2 the token dimension; cos, sin are fp32 tables
 * [rope_tokens, cols], row = token; tokens i2 >= rope_tokens are normalised only.  The rotation is
 * the real-pair form of diffusers' apply_rotary_emb (use_real=True, unbind dim -1):
 *   out[2i]   = y[2i] * cos[2i]     - y[2i+1] * sin[2i]
 *   out[2i+1] = y[2i+1] * cos[2i+1] + y[2i]   * sin[2i+1]      (fp32, rounded once to the element type)
 * with y the norm's output rounded to the element type.  Backward takes the gradient of the ROTATED
 * output and returns dx and dweight of the norm.  cols must be 128 (the head dimension). */
int tt_rmsnorm_rope_forward_strided(void *out, float *rstd, const void *x, const void *weight,
                                    const float *cos, const float *sin, int64_t rope_tokens,
                                    int64_t n0, int64_t n1, int64_t n2,
                                    int64_t xs0, int64_t xs1, int64_t xs2,
                                    int64_t cols, double eps, int dtype, void *stream);
int tt_rmsnorm_rope_backward_strided(void *dx, void *dweight, const void *dout, const void *x,
                                     const void *weight, const float *rstd,
                                     const float *cos, const float *sin, int64_t rope_tokens,
                                     int64_t n0, int64_t n1, int64_t n2,
                                     int64_t xs0, int64_t xs1, int64_t xs2,
                                     int64_t dxs0, int64_t dxs1, int64_t dxs2,
                                     int64_t cols, int dtype,
                                     void *workspace, size_t workspace_bytes, void *stream);

/* -------------------------------------------------------------------- AdaLN
 * out = round(round(LN(x) * round(1 + scale[b])) + shift[b]),  LN without affine,
 * b = row / rows_per_sample  (teletron/models/dit/dit_fusedlayers.py:198,223).
 * x, out [batch * rows_per_sample, cols]; scale, shift [batch, cols].
 */

/* Native forward: writes out and the per-row statistics mean, rstd [rows] fp32. */
int tt_adaln_forward(void *out, float *mean, float *rstd, const void *x,
                     const void *scale, const void *shift,
                     int64_t batch, int64_t rows_per_sample, int64_t cols,
                     double eps, int dtype, void *stream);

/* Replaces launch_adaln_forward (adaln_kernel.h:20-29, adaln_forward.cu:198):
 * additionally writes x_norm [rows, cols] = round(LN(x)); rstd is the
 * reference's inv_variance. */
int tt_adaln_forward_xnorm(void *out, void *x_norm, float *rstd, const void *x,
                           const void *scale, const void *shift,
                           int64_t batch, int64_t rows_per_sample, int64_t cols,
                           double eps, int dtype, void *stream);

size_t tt_adaln_backward_workspace_bytes(int64_t batch, int64_t rows_per_sample,
                                         int64_t cols, int dtype);

/* Native backward from the saved input and statistics: dx [rows, cols],
 * dscale, dshift [batch, cols].  Covers launch_adaln_backward +
 * launch_adaln_scale_shift_backward (adaln_backward.cu:129,
 * scale_shift_backward.cu:129) in one pass plus the fixed-order reducer. */
int tt_adaln_backward(void *dx, void *dscale, void *dshift, const void *dout, const void *x,
                      const void *scale, const float *mean, const float *rstd,
                      int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype,
                      void *workspace, size_t workspace_bytes, void *stream);

/* tt_adaln_forward / tt_adaln_backward on sequence-first rows: x, out, dout and dx are
 * [rows_per_sample, batch, cols] (the layout of the blocks' callers; the output norm broadcasts its
 * per-sample modulation over it, teletron/models/dit/dit_layerspec.py:72-78): sample b owns rows
 * b, b + batch, ...  mean and rstd are indexed by the same row numbers.  Same scratch as
 * tt_adaln_backward.  batch * cols * element size must not exceed 256 MiB. */
int tt_adaln_forward_seq_first(void *out, float *mean, float *rstd, const void *x,
                               const void *scale, const void *shift,
                               int64_t batch, int64_t rows_per_sample, int64_t cols,
                               double eps, int dtype, void *stream);
int tt_adaln_backward_seq_first(void *dx, void *dscale, void *dshift, const void *dout, const void *x,
                                const void *scale, const float *mean, const float *rstd,
                                int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype,
                                void *workspace, size_t workspace_bytes, void *stream);

/* tt_adaln_backward without a scratch argument, for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has
 * no counterpart in the reference.  The partial column sums go to a static device array of
 * TT_NORM_STATIC_SCRATCH_BYTES inside the library (one copy per GPU, held until the process
 * ends); the call allocates and frees nothing.  Shapes whose scratch need
 * (tt_adaln_backward_workspace_bytes) exceeds the array return TT_NORM_EWORKSPACE: at 3072
 * columns that is batch > 1365; every supported width fits for batch <= 256.  Results are
 * bit-identical to tt_adaln_backward.  All calls on one GPU share that GPU's array: calls that
 * overlap in time on one GPU (different streams or threads) race; on one stream they are safe.
 * The array used is the CURRENT device's (hipGetDevice), which must be the device that holds the
 * tensors: a dx that lives on another device is refused with TT_NORM_EINVAL. */
#define TT_NORM_STATIC_SCRATCH_BYTES (32u << 20)
int tt_adaln_backward_static(void *dx, void *dscale, void *dshift, const void *dout, const void *x,
                             const void *scale, const float *mean, const float *rstd,
                             int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype,
                             void *stream);

/* Same contract as the reference's launch_adaln_backward (adaln_kernel.h:36-45):
 * works from the saved normalised rows x_norm and rstd. */
int tt_adaln_backward_from_xnorm(void *dx, void *dscale, void *dshift, const void *dout,
                                 const void *x_norm, const void *scale, const float *rstd,
                                 int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype,
                                 void *workspace, size_t workspace_bytes, void *stream);

/* tt_adaln_backward for an input that has another consumer (the residual stream continues past the
 * norm, teletron/models/dit/dit_layerspec.py:126-131,152): dres [rows, cols] is the gradient the input
 * receives from that consumer, and dx = round(round(dx of the norm) + dres), the sum autograd would
 * otherwise form in a separate pass.  Same scratch as tt_adaln_backward.  Shapes:
 * tt_norm_wide_forms_supported(cols, dtype), else TT_NORM_EUNSUPPORTED. */
int tt_adaln_backward_residual(void *dx, void *dscale, void *dshift, const void *dout, const void *dres,
                               const void *x, const void *scale, const float *mean, const float *rstd,
                               int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype,
                               void *workspace, size_t workspace_bytes, void *stream);

/* ----------------------------------------------- gated residual + AdaLN
 * The transformer blocks update the residual stream and then normalise it:
 *     h2  = round(h + round(attn * gate[b]))
 *     out = AdaLN(h2; scale[b], shift[b])
 * (teletron/models/dit/dit_layerspec.py:152-167 in the double-stream block; the
 * single-stream block ends with the same update, :351-352, feeding the next block's
 * norm).  The reference runs these as separate elementwise kernels plus the norm; here
 * one pass reads h and attn and writes h2 and out, and one backward pass produces every
 * gradient.  h, attn, h2, out [batch * rows_per_sample, cols]; gate, scale, shift
 * [batch, cols].  Shapes: tt_norm_wide_forms_supported(cols, dtype) -- every supported row -- else
 * TT_NORM_EUNSUPPORTED.
 */

int tt_gated_residual_adaln_forward(void *h2, void *out, float *mean, float *rstd,
                                    const void *h, const void *attn, const void *gate,
                                    const void *scale, const void *shift,
                                    int64_t batch, int64_t rows_per_sample, int64_t cols,
                                    double eps, int dtype, void *stream);

size_t tt_gated_residual_adaln_backward_workspace_bytes(int64_t batch, int64_t rows_per_sample,
                                                        int64_t cols, int dtype);

/* dout is the gradient of `out`; dh2 the gradient reaching h2 through its other uses
 * (the residual stream continues past the norm), or NULL when there is none.
 * Writes dh (gradient of h, = total gradient of h2), dattn = round(dh * gate[b])
 * [rows, cols] and dgate = sum_rows round(dh * attn), dscale, dshift [batch, cols].
 * mean, rstd are what the forward wrote; h2 is the forward's first output. */
int tt_gated_residual_adaln_backward(void *dh, void *dattn, void *dgate, void *dscale, void *dshift,
                                     const void *dout, const void *dh2, const void *h2,
                                     const void *attn, const void *gate, const void *scale,
                                     const float *mean, const float *rstd,
                                     int64_t batch, int64_t rows_per_sample, int64_t cols, int dtype,
                                     void *workspace, size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------- measurement only
 * Not part of the operator interface, and no counterpart in the reference (which has no
 * instrumentation).  Arms a pair of HIP events (hipEvent_t passed as void*, created by the caller
 * with timing enabled) for the NEXT row kernel launched from this thread: `start` is recorded on that
 * launch's stream immediately before the row kernel and `stop` immediately after it, i.e. before the
 * column reducer of a backward call.  One shot: the pair is disarmed once used.  It exists so that a
 * benchmark can time exactly the kernel a profiler reports; it has to live in this library because
 * the launch it brackets does.  Pass NULLs to disarm.  The plain streaming kernels the benchmark
 * compares against are in libteletron_probe.so (teletron_probe.h), not here. */
int tt_norm_profile_next_row_kernel(void *start_event, void *stop_event);

#ifdef __cplusplus
}
#endif
#endif /* TELETRON_NORM_H_ */
