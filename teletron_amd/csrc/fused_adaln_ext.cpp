// Python module `fused_adaln`: the two functions of the reference's module of
// the same name, with the same argument order
// (teletron_op/fused_adaln/adaln_ops.cpp:6-15,29-38,52-60), plus the native
// pair that saves row statistics instead of a second full-size tensor.
// scale/shift may hold one row per sample ([batch, cols]); rows are then
// grouped by sample, rows/batch consecutive rows each.
#include "torch_glue.h"

using namespace ttn_glue;

struct AdalnShape {
    int64_t batch, rows_per_sample;
    int dt;
};

static AdalnShape adaln_shape(const torch::Tensor &x, const torch::Tensor &scale, int64_t rows, int64_t cols) {
    TORCH_CHECK(rows >= 0 && cols > 0, "rows must be non-negative and cols positive");
    TORCH_CHECK(scale.numel() > 0 && scale.numel() % cols == 0, "scale has ", scale.numel(),
                " elements, not a multiple of cols=", cols);
    const int64_t batch = scale.numel() / cols;
    TORCH_CHECK(rows % batch == 0, "rows=", rows, " is not a multiple of the ", batch, " modulation rows");
    return {batch, rows / batch, dtype_code(x, "input")};
}

void torch_launch_adaln_forward(torch::Tensor &output, torch::Tensor &x_norm, const torch::Tensor &input,
                                const torch::Tensor &scale, const torch::Tensor &shift, int64_t rows,
                                int64_t cols, double epsilon, torch::Tensor &inv_variance) {
    const auto dev = input.device();
    for (auto *t : {&output, &x_norm, &inv_variance}) check_dense_on(*t, dev, "output tensor");
    for (auto *t : {&input, &scale, &shift}) check_dense_on(*t, dev, "input tensor");
    const AdalnShape s = adaln_shape(input, scale, rows, cols);
    const auto st = input.scalar_type();
    check_elems(input, rows * cols, st, "input");
    check_elems(output, rows * cols, st, "output");
    check_elems(x_norm, rows * cols, st, "x_norm");
    check_elems(shift, scale.numel(), st, "shift");
    check_elems(scale, scale.numel(), st, "scale");
    check_elems(inv_variance, rows, at::kFloat, "inv_variance");
    c10::DeviceGuard guard(dev);
    raise_on(tt_adaln_forward_xnorm(output.data_ptr(), x_norm.data_ptr(), inv_variance.data_ptr<float>(),
                                    input.data_ptr(), scale.data_ptr(), shift.data_ptr(), s.batch,
                                    s.rows_per_sample, cols, epsilon, s.dt, current_stream(input)),
             "tt_adaln_forward_xnorm");
}

static void adaln_forward_stats_impl(torch::Tensor &output, const torch::Tensor &input,
                                     const torch::Tensor &scale, const torch::Tensor &shift, int64_t rows,
                                     int64_t cols, double epsilon, torch::Tensor &mean,
                                     torch::Tensor &inv_variance, bool seq_first) {
    const auto dev = input.device();
    for (auto *t : {&output, &mean, &inv_variance}) check_dense_on(*t, dev, "output tensor");
    for (auto *t : {&input, &scale, &shift}) check_dense_on(*t, dev, "input tensor");
    const AdalnShape s = adaln_shape(input, scale, rows, cols);
    const auto st = input.scalar_type();
    check_elems(input, rows * cols, st, "input");
    check_elems(output, rows * cols, st, "output");
    check_elems(shift, scale.numel(), st, "shift");
    check_elems(scale, scale.numel(), st, "scale");
    check_elems(mean, rows, at::kFloat, "mean");
    check_elems(inv_variance, rows, at::kFloat, "inv_variance");
    c10::DeviceGuard guard(dev);
    if (seq_first)
        raise_on(tt_adaln_forward_seq_first(output.data_ptr(), mean.data_ptr<float>(), inv_variance.data_ptr<float>(),
                                            input.data_ptr(), scale.data_ptr(), shift.data_ptr(), s.batch,
                                            s.rows_per_sample, cols, epsilon, s.dt, current_stream(input)),
                 "tt_adaln_forward_seq_first");
    else
        raise_on(tt_adaln_forward(output.data_ptr(), mean.data_ptr<float>(), inv_variance.data_ptr<float>(),
                                  input.data_ptr(), scale.data_ptr(), shift.data_ptr(), s.batch, s.rows_per_sample,
                                  cols, epsilon, s.dt, current_stream(input)),
                 "tt_adaln_forward");
}

void torch_launch_adaln_forward_stats(torch::Tensor &output, const torch::Tensor &input,
                                      const torch::Tensor &scale, const torch::Tensor &shift, int64_t rows,
                                      int64_t cols, double epsilon, torch::Tensor &mean,
                                      torch::Tensor &inv_variance) {
    adaln_forward_stats_impl(output, input, scale, shift, rows, cols, epsilon, mean, inv_variance, false);
}

// input is [rows / batch, batch, cols] (sequence first): sample b owns rows b, b + batch, ...
void torch_launch_adaln_forward_stats_seq_first(torch::Tensor &output, const torch::Tensor &input,
                                                const torch::Tensor &scale, const torch::Tensor &shift, int64_t rows,
                                                int64_t cols, double epsilon, torch::Tensor &mean,
                                                torch::Tensor &inv_variance) {
    adaln_forward_stats_impl(output, input, scale, shift, rows, cols, epsilon, mean, inv_variance, true);
}

static void adaln_backward_impl(torch::Tensor &dinp, torch::Tensor &dscale, torch::Tensor &dshift,
                                const torch::Tensor &dout, const torch::Tensor &saved,
                                const torch::Tensor &scale, const torch::Tensor *mean,
                                const torch::Tensor &inv_variance, int64_t rows, int64_t cols,
                                bool seq_first = false) {
    const auto dev = dout.device();
    for (auto *t : {&dinp, &dscale, &dshift}) check_dense_on(*t, dev, "output tensor");
    for (auto *t : {&dout, &saved, &scale, &inv_variance}) check_dense_on(*t, dev, "input tensor");
    const AdalnShape s = adaln_shape(dout, scale, rows, cols);
    const auto st = dout.scalar_type();
    check_elems(dout, rows * cols, st, "dout");
    check_elems(dinp, rows * cols, st, "dinp");
    check_elems(saved, rows * cols, st, mean ? "input" : "x_norm");
    check_elems(scale, scale.numel(), st, "scale");
    check_elems(dscale, scale.numel(), st, "dscale");
    check_elems(dshift, scale.numel(), st, "dshift");
    check_elems(inv_variance, rows, at::kFloat, "inv_variance");
    if (mean) {
        check_dense_on(*mean, dev, "mean");
        check_elems(*mean, rows, at::kFloat, "mean");
    }
    c10::DeviceGuard guard(dev);
    const size_t need = tt_adaln_backward_workspace_bytes(s.batch, s.rows_per_sample, cols, s.dt);
    TORCH_CHECK(need > 0 || rows == 0, "unsupported AdaLN shape: cols=", cols);
    at::Tensor ws = scratch(need, dout);
    if (mean && seq_first)
        raise_on(tt_adaln_backward_seq_first(dinp.data_ptr(), dscale.data_ptr(), dshift.data_ptr(), dout.data_ptr(),
                                             saved.data_ptr(), scale.data_ptr(), mean->data_ptr<float>(),
                                             inv_variance.data_ptr<float>(), s.batch, s.rows_per_sample, cols, s.dt,
                                             ws.data_ptr(), need, current_stream(dout)),
                 "tt_adaln_backward_seq_first");
    else if (mean)
        raise_on(tt_adaln_backward(dinp.data_ptr(), dscale.data_ptr(), dshift.data_ptr(), dout.data_ptr(),
                                   saved.data_ptr(), scale.data_ptr(), mean->data_ptr<float>(),
                                   inv_variance.data_ptr<float>(), s.batch, s.rows_per_sample, cols, s.dt,
                                   ws.data_ptr(), need, current_stream(dout)),
                 "tt_adaln_backward");
    else
        raise_on(tt_adaln_backward_from_xnorm(dinp.data_ptr(), dscale.data_ptr(), dshift.data_ptr(),
                                              dout.data_ptr(), saved.data_ptr(), scale.data_ptr(),
                                              inv_variance.data_ptr<float>(), s.batch, s.rows_per_sample, cols,
                                              s.dt, ws.data_ptr(), need, current_stream(dout)),
                 "tt_adaln_backward_from_xnorm");
}

// Reference contract: x_norm is what torch_launch_adaln_forward wrote to `x_norm`.
void torch_launch_adaln_backward(torch::Tensor &dinp, torch::Tensor &dscale, torch::Tensor &dshift,
                                 const torch::Tensor &dout, const torch::Tensor &x_norm,
                                 const torch::Tensor &scale, const torch::Tensor &inv_variance, int64_t rows,
                                 int64_t cols) {
    adaln_backward_impl(dinp, dscale, dshift, dout, x_norm, scale, nullptr, inv_variance, rows, cols);
}

// Native contract: `input`, `mean`, `inv_variance` as seen / written by torch_launch_adaln_forward_stats.
void torch_launch_adaln_backward_x(torch::Tensor &dinp, torch::Tensor &dscale, torch::Tensor &dshift,
                                   const torch::Tensor &dout, const torch::Tensor &input,
                                   const torch::Tensor &scale, const torch::Tensor &mean,
                                   const torch::Tensor &inv_variance, int64_t rows, int64_t cols) {
    adaln_backward_impl(dinp, dscale, dshift, dout, input, scale, &mean, inv_variance, rows, cols);
}

void torch_launch_adaln_backward_x_seq_first(torch::Tensor &dinp, torch::Tensor &dscale, torch::Tensor &dshift,
                                             const torch::Tensor &dout, const torch::Tensor &input,
                                             const torch::Tensor &scale, const torch::Tensor &mean,
                                             const torch::Tensor &inv_variance, int64_t rows, int64_t cols) {
    adaln_backward_impl(dinp, dscale, dshift, dout, input, scale, &mean, inv_variance, rows, cols, true);
}

// Native backward for an input with another consumer: `dres` is the gradient the input receives from it,
// dinp = dx of the norm + dres.  No counterpart in the reference's module.
void torch_launch_adaln_backward_residual(torch::Tensor &dinp, torch::Tensor &dscale, torch::Tensor &dshift,
                                          const torch::Tensor &dout, const torch::Tensor &dres,
                                          const torch::Tensor &input, const torch::Tensor &scale,
                                          const torch::Tensor &mean, const torch::Tensor &inv_variance,
                                          int64_t rows, int64_t cols) {
    const auto dev = dout.device();
    for (auto *t : {&dinp, &dscale, &dshift}) check_dense_on(*t, dev, "output tensor");
    for (auto *t : {&dout, &dres, &input, &scale, &mean, &inv_variance}) check_dense_on(*t, dev, "input tensor");
    const AdalnShape s = adaln_shape(dout, scale, rows, cols);
    const auto st = dout.scalar_type();
    for (auto *t : {&dout, &dres, &input}) check_elems(*t, rows * cols, st, "dout/dres/input");
    check_elems(dinp, rows * cols, st, "dinp");
    check_elems(scale, scale.numel(), st, "scale");
    for (auto *t : {&dscale, &dshift}) check_elems(*t, scale.numel(), st, "dscale/dshift");
    check_elems(mean, rows, at::kFloat, "mean");
    check_elems(inv_variance, rows, at::kFloat, "inv_variance");
    c10::DeviceGuard guard(dev);
    const size_t need = tt_adaln_backward_workspace_bytes(s.batch, s.rows_per_sample, cols, s.dt);
    TORCH_CHECK(need > 0 || rows == 0, "unsupported AdaLN shape: cols=", cols);
    at::Tensor ws = scratch(need, dout);
    raise_on(tt_adaln_backward_residual(dinp.data_ptr(), dscale.data_ptr(), dshift.data_ptr(), dout.data_ptr(),
                                        dres.data_ptr(), input.data_ptr(), scale.data_ptr(),
                                        mean.data_ptr<float>(), inv_variance.data_ptr<float>(), s.batch,
                                        s.rows_per_sample, cols, s.dt, ws.data_ptr(), need, current_stream(dout)),
             "tt_adaln_backward_residual");
}

// Gated residual update fused with the norm that follows it:
// h2 = input + attn * gate[b];  output = AdaLN(h2).  No counterpart in the reference's module.
void torch_launch_gated_adaln_forward(torch::Tensor &h2, torch::Tensor &output, const torch::Tensor &input,
                                      const torch::Tensor &attn, const torch::Tensor &gate,
                                      const torch::Tensor &scale, const torch::Tensor &shift, int64_t rows,
                                      int64_t cols, double epsilon, torch::Tensor &mean,
                                      torch::Tensor &inv_variance) {
    const auto dev = input.device();
    for (auto *t : {&h2, &output, &mean, &inv_variance}) check_dense_on(*t, dev, "output tensor");
    for (auto *t : {&input, &attn, &gate, &scale, &shift}) check_dense_on(*t, dev, "input tensor");
    const AdalnShape s = adaln_shape(input, scale, rows, cols);
    const auto st = input.scalar_type();
    for (auto *t : {&input, &attn}) check_elems(*t, rows * cols, st, "input/attn");
    check_elems(h2, rows * cols, st, "h2");
    check_elems(output, rows * cols, st, "output");
    for (auto *t : {&gate, &scale, &shift}) check_elems(*t, scale.numel(), st, "gate/scale/shift");
    check_elems(mean, rows, at::kFloat, "mean");
    check_elems(inv_variance, rows, at::kFloat, "inv_variance");
    c10::DeviceGuard guard(dev);
    raise_on(tt_gated_residual_adaln_forward(h2.data_ptr(), output.data_ptr(), mean.data_ptr<float>(),
                                             inv_variance.data_ptr<float>(), input.data_ptr(), attn.data_ptr(),
                                             gate.data_ptr(), scale.data_ptr(), shift.data_ptr(), s.batch,
                                             s.rows_per_sample, cols, epsilon, s.dt, current_stream(input)),
             "tt_gated_residual_adaln_forward");
}

// dh2: gradient reaching h2 from its other uses, or None.
void torch_launch_gated_adaln_backward(torch::Tensor &dinp, torch::Tensor &dattn, torch::Tensor &dgate,
                                       torch::Tensor &dscale, torch::Tensor &dshift, const torch::Tensor &dout,
                                       const c10::optional<torch::Tensor> &dh2, const torch::Tensor &h2,
                                       const torch::Tensor &attn, const torch::Tensor &gate,
                                       const torch::Tensor &scale, const torch::Tensor &mean,
                                       const torch::Tensor &inv_variance, int64_t rows, int64_t cols) {
    const auto dev = dout.device();
    for (auto *t : {&dinp, &dattn, &dgate, &dscale, &dshift}) check_dense_on(*t, dev, "output tensor");
    for (auto *t : {&dout, &h2, &attn, &gate, &scale, &mean, &inv_variance}) check_dense_on(*t, dev, "input tensor");
    const AdalnShape s = adaln_shape(dout, scale, rows, cols);
    const auto st = dout.scalar_type();
    for (auto *t : {&dout, &h2, &attn}) check_elems(*t, rows * cols, st, "dout/h2/attn");
    for (auto *t : {&dinp, &dattn}) check_elems(*t, rows * cols, st, "dinp/dattn");
    for (auto *t : {&gate, &scale}) check_elems(*t, scale.numel(), st, "gate/scale");
    for (auto *t : {&dgate, &dscale, &dshift}) check_elems(*t, scale.numel(), st, "dgate/dscale/dshift");
    check_elems(mean, rows, at::kFloat, "mean");
    check_elems(inv_variance, rows, at::kFloat, "inv_variance");
    const void *dh2_ptr = nullptr;
    if (dh2.has_value() && dh2->defined()) {
        check_dense_on(*dh2, dev, "dh2");
        check_elems(*dh2, rows * cols, st, "dh2");
        dh2_ptr = dh2->data_ptr();
    }
    c10::DeviceGuard guard(dev);
    const size_t need = tt_gated_residual_adaln_backward_workspace_bytes(s.batch, s.rows_per_sample, cols, s.dt);
    TORCH_CHECK(need > 0 || rows == 0, "unsupported gated AdaLN shape: cols=", cols);
    at::Tensor ws = scratch(need, dout);
    raise_on(tt_gated_residual_adaln_backward(dinp.data_ptr(), dattn.data_ptr(), dgate.data_ptr(),
                                              dscale.data_ptr(), dshift.data_ptr(), dout.data_ptr(), dh2_ptr,
                                              h2.data_ptr(), attn.data_ptr(), gate.data_ptr(), scale.data_ptr(),
                                              mean.data_ptr<float>(), inv_variance.data_ptr<float>(), s.batch,
                                              s.rows_per_sample, cols, s.dt, ws.data_ptr(), need,
                                              current_stream(dout)),
             "tt_gated_residual_adaln_backward");
}

PYBIND11_MODULE(fused_adaln, m) {
    m.def("torch_launch_adaln_backward_residual", &torch_launch_adaln_backward_residual,
          "AdaLN backward kernel with the input's other gradient added in");
    m.def("torch_launch_gated_adaln_forward", &torch_launch_gated_adaln_forward,
          "gated residual update + AdaLN forward kernel");
    m.def("torch_launch_gated_adaln_backward", &torch_launch_gated_adaln_backward,
          "gated residual update + AdaLN backward kernel");
    m.def("torch_launch_adaln_forward", &torch_launch_adaln_forward, "AdaLN forward kernel");
    m.def("torch_launch_adaln_backward", &torch_launch_adaln_backward,
          "AdaLN backward kernel (from the saved normalised rows)");
    m.def("torch_launch_adaln_forward_stats", &torch_launch_adaln_forward_stats,
          "AdaLN forward kernel that saves mean and inv_variance instead of x_norm");
    m.def("torch_launch_adaln_backward_x", &torch_launch_adaln_backward_x,
          "AdaLN backward kernel (from the saved input and statistics)");
    m.def("torch_launch_adaln_forward_stats_seq_first", &torch_launch_adaln_forward_stats_seq_first,
          "AdaLN forward kernel on sequence-first rows [S, B, C]");
    m.def("torch_launch_adaln_backward_x_seq_first", &torch_launch_adaln_backward_x_seq_first,
          "AdaLN backward kernel on sequence-first rows [S, B, C]");
    m.def("supported", [](int64_t cols, const torch::Tensor &like) {
        return tt_norm_supported(cols, like.scalar_type() == at::kBFloat16 ? TT_NORM_BF16
                                       : like.scalar_type() == at::kFloat  ? TT_NORM_F32
                                       : like.scalar_type() == at::kHalf   ? TT_NORM_F16 : -1) != 0;
    }, "whether the kernels are built for this column count and dtype");
}

// Same operator namespace as the reference registers (adaln_ops.cpp:62-65).
TORCH_LIBRARY(layernorm_block_smem, m) {
    m.def("torch_launch_adaln_forward(Tensor(a!) output, Tensor(b!) x_norm, Tensor input, Tensor scale, "
          "Tensor shift, int rows, int cols, float epsilon, Tensor(c!) inv_variance) -> ()",
          &torch_launch_adaln_forward);
    m.def("torch_launch_adaln_backward(Tensor(a!) dinp, Tensor(b!) dscale, Tensor(c!) dshift, Tensor dout, "
          "Tensor x_norm, Tensor scale, Tensor inv_variance, int rows, int cols) -> ()",
          &torch_launch_adaln_backward);
}
