// Shared host-side glue of the two PyTorch extension modules: argument checks,
// element-type mapping, the current HIP stream, scratch from the caching
// allocator, and status -> exception.  No kernels here; everything goes
// through the C ABI of libteletron_norm.so.
#pragma once

#include <torch/extension.h>
#include <c10/hip/HIPStream.h>

#include "teletron_norm.h"

namespace ttn_glue {

inline int dtype_code(const at::Tensor &t, const char *name) {
    if (t.scalar_type() == at::kBFloat16) return TT_NORM_BF16;
    if (t.scalar_type() == at::kFloat) return TT_NORM_F32;
    if (t.scalar_type() == at::kHalf) return TT_NORM_F16;
    TORCH_CHECK(false, name, ": expected a bfloat16, float16 or float32 tensor, got ", t.scalar_type());
}

inline void check_dense_on(const at::Tensor &t, const at::Device &dev, const char *name) {
    TORCH_CHECK(t.defined(), name, " is undefined");
    TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
    TORCH_CHECK(t.device() == dev, name, " is on ", t.device(), ", expected ", dev);
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

inline void check_elems(const at::Tensor &t, int64_t n, at::ScalarType st, const char *name) {
    TORCH_CHECK(t.numel() == n, name, " has ", t.numel(), " elements, expected ", n);
    TORCH_CHECK(t.scalar_type() == st, name, " has dtype ", t.scalar_type(), ", expected ", st);
}

inline void *current_stream(const at::Tensor &t) {
    return (void *)c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

inline at::Tensor scratch(size_t bytes, const at::Tensor &like) {
    return at::empty({(int64_t)(bytes ? bytes : 16)}, like.options().dtype(at::kByte));
}

inline void raise_on(int status, const char *what) {
    TORCH_CHECK(status == TT_NORM_OK, what, " failed: ", tt_norm_status_string(status), " -- ",
                tt_norm_last_error());
}

}  // namespace ttn_glue
