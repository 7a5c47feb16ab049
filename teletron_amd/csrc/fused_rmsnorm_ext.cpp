// Python module `fused_rmsnorm`: the two functions of the reference's module of
// the same name, with the same argument order
// (teletron_op/fused_rmsnorm/rms_ops.cpp:6-13,25-33,47-55), plus the native
// backward that works from the saved input.  Unlike the reference glue, every
// argument is checked, the launch goes to PyTorch's current stream, and a
// failed launch raises.
#include "torch_glue.h"

using namespace ttn_glue;

// output[rows, cols] = rmsnorm(input) * weight;  inv_variance[rows] = 1/rms  (fp32)
void torch_launch_rms_forward(torch::Tensor &output, const torch::Tensor &input,
                              const torch::Tensor &weight, int64_t rows, int64_t cols, double epsilon,
                              torch::Tensor &inv_variance) {
    const auto dev = input.device();
    check_dense_on(input, dev, "input");
    check_dense_on(output, dev, "output");
    check_dense_on(weight, dev, "weight");
    check_dense_on(inv_variance, dev, "inv_variance");
    const int dt = dtype_code(input, "input");
    TORCH_CHECK(rows >= 0 && cols > 0, "rows must be non-negative and cols positive");
    check_elems(input, rows * cols, input.scalar_type(), "input");
    check_elems(output, rows * cols, input.scalar_type(), "output");
    check_elems(weight, cols, input.scalar_type(), "weight");
    check_elems(inv_variance, rows, at::kFloat, "inv_variance");
    c10::DeviceGuard guard(dev);
    raise_on(tt_rmsnorm_forward(output.data_ptr(), inv_variance.data_ptr<float>(), input.data_ptr(),
                                weight.data_ptr(), rows, cols, epsilon, dt, current_stream(input)),
             "tt_rmsnorm_forward");
}

static void rms_backward_impl(torch::Tensor &dinp, torch::Tensor &dweight, const torch::Tensor &dout,
                              const torch::Tensor &saved, const torch::Tensor &weight,
                              const torch::Tensor &inv_variance, int64_t rows, int64_t cols,
                              bool saved_is_output) {
    const auto dev = dout.device();
    check_dense_on(dout, dev, "dout");
    check_dense_on(dinp, dev, "dinp");
    check_dense_on(dweight, dev, "dweight");
    check_dense_on(saved, dev, saved_is_output ? "x_norm" : "input");
    check_dense_on(weight, dev, "weight");
    check_dense_on(inv_variance, dev, "inv_variance");
    const int dt = dtype_code(dout, "dout");
    TORCH_CHECK(rows >= 0 && cols > 0, "rows must be non-negative and cols positive");
    check_elems(dout, rows * cols, dout.scalar_type(), "dout");
    check_elems(dinp, rows * cols, dout.scalar_type(), "dinp");
    check_elems(saved, rows * cols, dout.scalar_type(), saved_is_output ? "x_norm" : "input");
    check_elems(weight, cols, dout.scalar_type(), "weight");
    check_elems(dweight, cols, dout.scalar_type(), "dweight");
    check_elems(inv_variance, rows, at::kFloat, "inv_variance");
    c10::DeviceGuard guard(dev);
    const size_t need = tt_rmsnorm_backward_workspace_bytes(rows, cols, dt);
    TORCH_CHECK(need > 0 || rows == 0, "unsupported RMSNorm shape: cols=", cols);
    at::Tensor ws = scratch(need, dout);
    auto fn = saved_is_output ? tt_rmsnorm_backward_from_out : tt_rmsnorm_backward;
    raise_on(fn(dinp.data_ptr(), dweight.data_ptr(), dout.data_ptr(), saved.data_ptr(), weight.data_ptr(),
                inv_variance.data_ptr<float>(), rows, cols, dt, ws.data_ptr(), need, current_stream(dout)),
             saved_is_output ? "tt_rmsnorm_backward_from_out" : "tt_rmsnorm_backward");
}

// Reference contract: x_norm is the tensor torch_launch_rms_forward wrote to `output`.
void torch_launch_rms_backward(torch::Tensor &dinp, torch::Tensor &dweight, const torch::Tensor &dout,
                               const torch::Tensor &x_norm, const torch::Tensor &weight,
                               const torch::Tensor &inv_variance, int64_t rows, int64_t cols) {
    rms_backward_impl(dinp, dweight, dout, x_norm, weight, inv_variance, rows, cols, true);
}

// Native contract: `input` is the tensor that was normalised (forward then keeps no copy of its output).
void torch_launch_rms_backward_x(torch::Tensor &dinp, torch::Tensor &dweight, const torch::Tensor &dout,
                                 const torch::Tensor &input, const torch::Tensor &weight,
                                 const torch::Tensor &inv_variance, int64_t rows, int64_t cols) {
    rms_backward_impl(dinp, dweight, dout, input, weight, inv_variance, rows, cols, false);
}

// ---- strided views (no reference counterpart: the reference copies to contiguous first) ----
struct View3 {
    int64_t n[3], s[3];
};

// Leading dimensions of a <= 4-D view with contiguous last dimension, padded to three.
static View3 view3(const torch::Tensor &t, int64_t cols, const char *name) {
    TORCH_CHECK(t.dim() >= 1 && t.dim() <= 4, name, " must have 1 to 4 dimensions, got ", t.dim());
    TORCH_CHECK(t.size(-1) == cols && t.stride(-1) == 1, name, " needs a contiguous last dimension of ", cols);
    View3 v{{1, 1, 1}, {0, 0, 0}};
    const int64_t lead = t.dim() - 1;
    for (int64_t d = 0; d < lead; ++d) {
        v.n[3 - lead + d] = t.size(d);
        v.s[3 - lead + d] = t.stride(d);
    }
    return v;
}

// output (contiguous, input's shape) = rmsnorm(input view) * weight; inv_variance in output row order.
void torch_launch_rms_forward_strided(torch::Tensor &output, const torch::Tensor &input,
                                      const torch::Tensor &weight, double epsilon,
                                      torch::Tensor &inv_variance) {
    const auto dev = input.device();
    TORCH_CHECK(input.is_cuda(), "input must be a GPU tensor");
    check_dense_on(output, dev, "output");
    check_dense_on(weight, dev, "weight");
    check_dense_on(inv_variance, dev, "inv_variance");
    const int dt = dtype_code(input, "input");
    const int64_t cols = weight.numel();
    const View3 v = view3(input, cols, "input");
    const int64_t rows = v.n[0] * v.n[1] * v.n[2];
    check_elems(output, rows * cols, input.scalar_type(), "output");
    check_elems(weight, cols, input.scalar_type(), "weight");
    check_elems(inv_variance, rows, at::kFloat, "inv_variance");
    c10::DeviceGuard guard(dev);
    raise_on(tt_rmsnorm_forward_strided(output.data_ptr(), inv_variance.data_ptr<float>(), input.data_ptr(),
                                        weight.data_ptr(), v.n[0], v.n[1], v.n[2], v.s[0], v.s[1], v.s[2], cols,
                                        epsilon, dt, current_stream(input)),
             "tt_rmsnorm_forward_strided");
}

// dinp: any view of input's shape (its strides choose the layout dx is written in); dout contiguous.
void torch_launch_rms_backward_strided(torch::Tensor &dinp, torch::Tensor &dweight, const torch::Tensor &dout,
                                       const torch::Tensor &input, const torch::Tensor &weight,
                                       const torch::Tensor &inv_variance) {
    const auto dev = dout.device();
    TORCH_CHECK(input.is_cuda() && dinp.is_cuda(), "input and dinp must be GPU tensors");
    TORCH_CHECK(input.device() == dev && dinp.device() == dev, "tensors are on different devices");
    check_dense_on(dout, dev, "dout");
    check_dense_on(dweight, dev, "dweight");
    check_dense_on(weight, dev, "weight");
    check_dense_on(inv_variance, dev, "inv_variance");
    const int dt = dtype_code(dout, "dout");
    const int64_t cols = weight.numel();
    const View3 vx = view3(input, cols, "input");
    const View3 vd = view3(dinp, cols, "dinp");
    TORCH_CHECK(input.sizes() == dinp.sizes(), "dinp must have input's shape");
    const int64_t rows = vx.n[0] * vx.n[1] * vx.n[2];
    TORCH_CHECK(input.scalar_type() == dout.scalar_type() && dinp.scalar_type() == dout.scalar_type(),
                "input, dinp and dout must share a dtype");
    check_elems(dout, rows * cols, dout.scalar_type(), "dout");
    check_elems(weight, cols, dout.scalar_type(), "weight");
    check_elems(dweight, cols, dout.scalar_type(), "dweight");
    check_elems(inv_variance, rows, at::kFloat, "inv_variance");
    c10::DeviceGuard guard(dev);
    const size_t need = tt_rmsnorm_backward_workspace_bytes(rows, cols, dt);
    TORCH_CHECK(need > 0 || rows == 0, "unsupported RMSNorm shape: cols=", cols);
    at::Tensor ws = scratch(need, dout);
    raise_on(tt_rmsnorm_backward_strided(dinp.data_ptr(), dweight.data_ptr(), dout.data_ptr(), input.data_ptr(),
                                         weight.data_ptr(), inv_variance.data_ptr<float>(), vx.n[0], vx.n[1],
                                         vx.n[2], vx.s[0], vx.s[1], vx.s[2], vd.s[0], vd.s[1], vd.s[2], cols, dt,
                                         ws.data_ptr(), need, current_stream(dout)),
             "tt_rmsnorm_backward_strided");
}

// dst: any view (<= 4-D, contiguous last dimension) of src's shape; src contiguous.  The value gradient of the
// QK-norm call site goes into its slice of the fused projection's gradient with this.
void torch_launch_copy_rows_strided(torch::Tensor &dst, const torch::Tensor &src) {
    const auto dev = src.device();
    TORCH_CHECK(dst.is_cuda() && dst.device() == dev, "dst and src must be on the same GPU");
    check_dense_on(src, dev, "src");
    TORCH_CHECK(dst.sizes() == src.sizes() && dst.scalar_type() == src.scalar_type(), "dst must have src's shape and dtype");
    const int dt = dtype_code(src, "src");
    const int64_t cols = src.size(-1);
    const View3 vd = view3(dst, cols, "dst");
    c10::DeviceGuard guard(dev);
    raise_on(tt_norm_copy_rows_strided(dst.data_ptr(), src.data_ptr(), vd.n[0], vd.n[1], vd.n[2], vd.s[0], vd.s[1],
                                       vd.s[2], cols, dt, current_stream(src)),
             "tt_norm_copy_rows_strided");
}

// ---- strided QK-norm with the rotary embedding behind it (no reference counterpart: the reference
// runs apply_rotary_emb as separate PyTorch ops on the norm's output) ----
static int64_t check_rope_tables(const torch::Tensor &cos, const torch::Tensor &sin, const at::Device &dev,
                                 int64_t cols, int64_t seq) {
    check_dense_on(cos, dev, "freqs_cos");
    check_dense_on(sin, dev, "freqs_sin");
    TORCH_CHECK(cos.scalar_type() == at::kFloat && sin.scalar_type() == at::kFloat, "freqs_cos/freqs_sin must be float32");
    TORCH_CHECK(cos.dim() == 2 && cos.size(1) == cols && cos.sizes() == sin.sizes(),
                "freqs_cos/freqs_sin must both be [tokens, ", cols, "]");
    TORCH_CHECK(cos.size(0) <= seq, "rotary tables hold ", cos.size(0), " tokens, the view only ", seq);
    return cos.size(0);
}

// input: a [B, H, S, D] view (or fewer leading dimensions); rows at token index >= freqs_cos.size(0) are
// normalised but not rotated.
void torch_launch_rms_rope_forward_strided(torch::Tensor &output, const torch::Tensor &input,
                                           const torch::Tensor &weight, double epsilon,
                                           torch::Tensor &inv_variance, const torch::Tensor &freqs_cos,
                                           const torch::Tensor &freqs_sin) {
    const auto dev = input.device();
    TORCH_CHECK(input.is_cuda(), "input must be a GPU tensor");
    check_dense_on(output, dev, "output");
    check_dense_on(weight, dev, "weight");
    check_dense_on(inv_variance, dev, "inv_variance");
    const int dt = dtype_code(input, "input");
    const int64_t cols = weight.numel();
    const View3 v = view3(input, cols, "input");
    const int64_t rows = v.n[0] * v.n[1] * v.n[2];
    const int64_t tokens = check_rope_tables(freqs_cos, freqs_sin, dev, cols, v.n[2]);
    check_elems(output, rows * cols, input.scalar_type(), "output");
    check_elems(weight, cols, input.scalar_type(), "weight");
    check_elems(inv_variance, rows, at::kFloat, "inv_variance");
    c10::DeviceGuard guard(dev);
    raise_on(tt_rmsnorm_rope_forward_strided(output.data_ptr(), inv_variance.data_ptr<float>(), input.data_ptr(),
                                             weight.data_ptr(), freqs_cos.data_ptr<float>(),
                                             freqs_sin.data_ptr<float>(), tokens, v.n[0], v.n[1], v.n[2], v.s[0],
                                             v.s[1], v.s[2], cols, epsilon, dt, current_stream(input)),
             "tt_rmsnorm_rope_forward_strided");
}

// dout: gradient of the rotated output (contiguous); dinp as in torch_launch_rms_backward_strided.
void torch_launch_rms_rope_backward_strided(torch::Tensor &dinp, torch::Tensor &dweight, const torch::Tensor &dout,
                                            const torch::Tensor &input, const torch::Tensor &weight,
                                            const torch::Tensor &inv_variance, const torch::Tensor &freqs_cos,
                                            const torch::Tensor &freqs_sin) {
    const auto dev = dout.device();
    TORCH_CHECK(input.is_cuda() && dinp.is_cuda(), "input and dinp must be GPU tensors");
    TORCH_CHECK(input.device() == dev && dinp.device() == dev, "tensors are on different devices");
    check_dense_on(dout, dev, "dout");
    check_dense_on(dweight, dev, "dweight");
    check_dense_on(weight, dev, "weight");
    check_dense_on(inv_variance, dev, "inv_variance");
    const int dt = dtype_code(dout, "dout");
    const int64_t cols = weight.numel();
    const View3 vx = view3(input, cols, "input");
    const View3 vd = view3(dinp, cols, "dinp");
    TORCH_CHECK(input.sizes() == dinp.sizes(), "dinp must have input's shape");
    const int64_t rows = vx.n[0] * vx.n[1] * vx.n[2];
    const int64_t tokens = check_rope_tables(freqs_cos, freqs_sin, dev, cols, vx.n[2]);
    TORCH_CHECK(input.scalar_type() == dout.scalar_type() && dinp.scalar_type() == dout.scalar_type(),
                "input, dinp and dout must share a dtype");
    check_elems(dout, rows * cols, dout.scalar_type(), "dout");
    check_elems(weight, cols, dout.scalar_type(), "weight");
    check_elems(dweight, cols, dout.scalar_type(), "dweight");
    check_elems(inv_variance, rows, at::kFloat, "inv_variance");
    c10::DeviceGuard guard(dev);
    const size_t need = tt_rmsnorm_backward_workspace_bytes(rows, cols, dt);
    TORCH_CHECK(need > 0 || rows == 0, "unsupported RMSNorm shape: cols=", cols);
    at::Tensor ws = scratch(need, dout);
    raise_on(tt_rmsnorm_rope_backward_strided(dinp.data_ptr(), dweight.data_ptr(), dout.data_ptr(), input.data_ptr(),
                                              weight.data_ptr(), inv_variance.data_ptr<float>(),
                                              freqs_cos.data_ptr<float>(), freqs_sin.data_ptr<float>(), tokens,
                                              vx.n[0], vx.n[1], vx.n[2], vx.s[0], vx.s[1], vx.s[2], vd.s[0], vd.s[1],
                                              vd.s[2], cols, dt, ws.data_ptr(), need, current_stream(dout)),
             "tt_rmsnorm_rope_backward_strided");
}

PYBIND11_MODULE(fused_rmsnorm, m) {
    m.def("torch_launch_copy_rows_strided", &torch_launch_copy_rows_strided,
          "rows of a contiguous tensor into a strided view of the same shape");
    m.def("torch_launch_rms_rope_forward_strided", &torch_launch_rms_rope_forward_strided,
          "strided RMSNorm forward with the rotary embedding applied to the result");
    m.def("torch_launch_rms_rope_backward_strided", &torch_launch_rms_rope_backward_strided,
          "backward of the strided RMSNorm + rotary embedding");
    m.def("torch_launch_rms_forward", &torch_launch_rms_forward, "RMSNorm forward kernel");
    m.def("torch_launch_rms_backward", &torch_launch_rms_backward,
          "RMSNorm backward kernel (from the saved forward output)");
    m.def("torch_launch_rms_backward_x", &torch_launch_rms_backward_x,
          "RMSNorm backward kernel (from the saved input)");
    m.def("torch_launch_rms_forward_strided", &torch_launch_rms_forward_strided,
          "RMSNorm forward kernel reading a strided view (contiguous last dimension) in place");
    m.def("torch_launch_rms_backward_strided", &torch_launch_rms_backward_strided,
          "RMSNorm backward kernel for a strided input view; dx is written through dinp's strides");
    m.def("supported", [](int64_t cols, const torch::Tensor &like) {
        return tt_norm_supported(cols, like.scalar_type() == at::kBFloat16 ? TT_NORM_BF16
                                       : like.scalar_type() == at::kFloat  ? TT_NORM_F32
                                       : like.scalar_type() == at::kHalf   ? TT_NORM_F16 : -1) != 0;
    }, "whether the kernels are built for this column count and dtype");
}

// Same operator namespace as the reference registers (rms_ops.cpp:58-61).
TORCH_LIBRARY(Fused_RMSNorm, m) {
    m.def("torch_launch_rms_forward(Tensor(a!) output, Tensor input, Tensor weight, int rows, int cols, "
          "float epsilon, Tensor(b!) inv_variance) -> ()",
          &torch_launch_rms_forward);
    m.def("torch_launch_rms_backward(Tensor(a!) dinp, Tensor(b!) dweight, Tensor dout, Tensor x_norm, "
          "Tensor weight, Tensor inv_variance, int rows, int cols) -> ()",
          &torch_launch_rms_backward);
}
