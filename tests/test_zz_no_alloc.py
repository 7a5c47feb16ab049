"""tt_adaln_backward_static: the AdaLN backward that allocates nothing (scratch in a static device
array inside the library), called through the C ABI and compared, bit for bit, with
tt_adaln_backward on the same inputs.  Two calls in a row, the second on a smaller input, so that
what the first call left in the shared array cannot leak into the second."""
import ctypes

import pytest
import torch

from oracle import norm_oracle as O

pytestmark = pytest.mark.gpu
EPS = 1e-6


_CALLED_BEFORE = {}


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _both_ways(capi, device, batch, rows_per_sample, cols, dtype, seed):
    L = capi.lib()
    code = capi._DTYPES[dtype]
    d = O.make_adaln_inputs(batch, rows_per_sample, cols, dtype, seed=seed)
    x, scale, shift, grad = (d[k].to(device) for k in ("x", "scale", "shift", "grad"))
    out, mean, rstd = capi.adaln_forward(x, scale, shift, EPS)
    want_dx, want_ds, want_dh = capi.adaln_backward(grad, x, scale, mean, rstd)
    # outputs pre-filled with a pattern the kernels must overwrite
    dx = torch.full_like(x, 7.0)
    ds, dh = torch.full_like(scale, 7.0), torch.full_like(scale, 7.0)
    stream = ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(device)[0]      # hipMemGetInfo: device memory not held by any allocation
    st = L.tt_adaln_backward_static(_p(dx), _p(ds), _p(dh), _p(grad), _p(x), _p(scale), _p(mean), _p(rstd),
                                    batch, rows_per_sample, cols, code, stream)
    assert st == 0, (st, L.tt_norm_last_error())
    torch.cuda.synchronize()
    # the first call on a device may load the library's code object (and with it the static array); later calls
    # must leave the device's free memory exactly where it was
    if _CALLED_BEFORE.get(str(device)):
        assert torch.cuda.mem_get_info(device)[0] == free_before, "tt_adaln_backward_static changed the free device memory"
    _CALLED_BEFORE[str(device)] = True
    what = f"batch={batch} rows_per_sample={rows_per_sample} cols={cols} {dtype}"
    assert torch.equal(dx, want_dx), "dx " + what
    assert torch.equal(ds, want_ds), "dscale " + what
    assert torch.equal(dh, want_dh), "dshift " + what
    # and the pair agrees with the eager oracle (the bar of the parity tests)
    if dtype == torch.bfloat16 and cols == 3072:
        _, e_dx, e_ds, e_dh = O.eager_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], d["grad"])
        assert O.frac_outside(dx.cpu(), e_dx, 1e-2, 1e-3) <= 1e-5, what
        assert O.frac_outside(ds.cpu(), e_ds, 1e-2, 1e-3) == 0.0, what
        assert O.frac_outside(dh.cpu(), e_dh, 1e-2, 1e-3) == 0.0, what


def test_static_scratch_backward_matches_tt_adaln_backward(gpu_device):
    from teletron_amd import capi
    capi.lib()
    # large first (every workgroup of the persistent grid writes its partial row), then smaller
    # inputs that use fewer partial rows and a narrower row: stale contents must not be read
    _both_ways(capi, gpu_device, 2, 4099, 3072, torch.bfloat16, seed=11)
    _both_ways(capi, gpu_device, 1, 37, 3072, torch.bfloat16, seed=12)
    _both_ways(capi, gpu_device, 3, 5, 1536, torch.float16, seed=13)
    _both_ways(capi, gpu_device, 1, 700, 128, torch.float32, seed=14)
    # rows of more than 384 pieces (four wavefronts per row, two workgroups per compute unit), then fewer of them
    _both_ways(capi, gpu_device, 2, 1301, 8192, torch.bfloat16, seed=15)
    _both_ways(capi, gpu_device, 1, 9, 3072, torch.float32, seed=16)


def test_static_scratch_backward_rejects_what_does_not_fit(gpu_device):
    from teletron_amd import capi
    L = capi.lib()
    cols, batch = 3072, 1400                     # 1400 workgroups x 24 KiB of partial sums > 32 MiB
    assert L.tt_adaln_backward_workspace_bytes(batch, 4, cols, capi.BF16) > 32 << 20
    t = torch.zeros(batch * 4 * cols, dtype=torch.bfloat16, device=gpu_device)
    s = torch.zeros(batch * cols, dtype=torch.bfloat16, device=gpu_device)
    f = torch.zeros(batch * 4, dtype=torch.float32, device=gpu_device)
    st = L.tt_adaln_backward_static(_p(t), _p(s), _p(s), _p(t), _p(t), _p(s), _p(f), _p(f), batch, 4, cols,
                                    capi.BF16, None)
    assert st == 4, (st, L.tt_norm_last_error())        # TT_NORM_EWORKSPACE, decided on the host: nothing ran
    assert b"static array holds" in L.tt_norm_last_error()
    torch.cuda.synchronize()
