"""Out-of-bounds evidence: every tensor a C-ABI call writes (out, dx, h2, dattn, rstd, mean, the
parameter gradients and the scratch) is carved out of a larger device buffer pre-filled with a byte
pattern, 4 KiB of it before and after, and the margins -- for strided outputs also the gaps between
the slices -- must still hold the pattern after the call.  All of the memory is valid, so a stray
store cannot fault; it shows up here instead.  The cases are the ones where a kernel's last piece of
work is partial: ragged last groups of rows, rows whose last 16-byte access per lane lies partly or
wholly outside the row in every any-width geometry, strided views whose head count is not a multiple
of the run length, sequence-first rows with three samples, zero rows, and the entry point that keeps
its scratch in the library.  Each case also checks the results against a second run into ordinary
tensors, so a kernel that wrote nothing would not pass either."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
EPS = 1e-6
MARGIN = 4096
PATTERN = 0xA5


@pytest.fixture(scope="module")
def capi(gpu_device):
    from teletron_amd import capi as c
    c.lib()
    return c


def _p(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


class Guarded:
    """Output tensors with pattern-filled margins around each of them."""

    def __init__(self, device):
        self.device = device
        self.bufs = []

    def new(self, shape, dtype):
        n = 1
        for s in shape:
            n *= s
        nbytes = n * torch.empty((), dtype=dtype).element_size()
        buf = torch.full((MARGIN + nbytes + MARGIN,), PATTERN, dtype=torch.uint8, device=self.device)
        self.bufs.append((buf, nbytes))
        return buf[MARGIN:MARGIN + nbytes].view(dtype).view(shape)

    def bytes(self, nbytes):
        return self.new((max(nbytes, 16),), torch.uint8)

    def check(self, what=""):
        for i, (buf, nbytes) in enumerate(self.bufs):
            lo, hi = buf[:MARGIN], buf[MARGIN + nbytes:]
            assert bool((lo == PATTERN).all()), f"{what}: output {i} ({nbytes} B): bytes BEFORE it were overwritten"
            assert bool((hi == PATTERN).all()), f"{what}: output {i} ({nbytes} B): bytes AFTER it were overwritten"


def _stream(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _ok(L, st):
    assert st == 0, (st, L.tt_norm_last_error())


def _inputs(rows, cols, dtype, device, batch=1, seed=0):
    gen = torch.Generator(device=device).manual_seed(seed * 7919 + rows * 31 + cols)
    mk = lambda *shape, k=1.0, b=0.0: (b + k * torch.randn(*shape, device=device, generator=gen)).to(dtype)
    return dict(x=mk(rows, cols), g=mk(rows, cols), w=mk(cols, k=0.02, b=1.0), scale=mk(batch, cols, k=0.1),
                shift=mk(batch, cols, k=0.1), gate=mk(batch, cols, k=0.3), attn=mk(rows, cols), e=mk(rows, cols, k=0.1))


# (cols, dtype): the tuned shapes, and for every any-width geometry (8, 16, 32 lanes x 1 access; 64 lanes x 1, 2, 3,
# 4, 6, 8, 12, 16 accesses) a width whose last access per lane is partly outside the row, in two- and four-byte types
WIDTHS = [(3072, torch.bfloat16), (3072, torch.float32), (128, torch.bfloat16), (128, torch.float32),
          (40, torch.bfloat16), (72, torch.float16), (200, torch.bfloat16), (320, torch.bfloat16),
          (1000, torch.bfloat16), (1496, torch.float16), (2000, torch.bfloat16), (3000, torch.bfloat16),
          (4000, torch.bfloat16), (6000, torch.float16), (8000, torch.bfloat16), (8192, torch.bfloat16),
          (20, torch.float32), (100, torch.float32), (500, torch.float32), (1500, torch.float32),
          (2996, torch.float32), (4092, torch.float32)]
# row counts that leave the last group of every rows-per-wavefront (1, 2, 4, 8) and the last workgroup ragged
ROWS = [1, 2, 3, 5, 7, 1029, 1031]


@pytest.mark.parametrize("cols,dtype", WIDTHS, ids=lambda v: str(v).replace("torch.", ""))
def test_rmsnorm_writes_stay_inside(capi, gpu_device, cols, dtype):
    L, dt, s = capi.lib(), capi._DTYPES[dtype], _stream(gpu_device)
    for rows in ROWS:
        d = _inputs(rows, cols, dtype, gpu_device)
        G = Guarded(gpu_device)
        out, rstd = G.new((rows, cols), dtype), G.new((rows,), torch.float32)
        dx, dw = G.new((rows, cols), dtype), G.new((cols,), dtype)
        n = L.tt_rmsnorm_backward_workspace_bytes(rows, cols, dt)
        ws = G.bytes(n)
        _ok(L, L.tt_rmsnorm_forward(_p(out), _p(rstd), _p(d["x"]), _p(d["w"]), rows, cols, EPS, dt, s))
        _ok(L, L.tt_rmsnorm_backward(_p(dx), _p(dw), _p(d["g"]), _p(d["x"]), _p(d["w"]), _p(rstd), rows, cols, dt,
                                     _p(ws), n, s))
        torch.cuda.synchronize()
        G.check(f"rmsnorm rows={rows} cols={cols} {dtype}")
        out2, rstd2 = capi.rmsnorm_forward(d["x"], d["w"], EPS)
        dx2, dw2 = capi.rmsnorm_backward(d["g"], d["x"], d["w"], rstd2)
        assert torch.equal(out, out2) and torch.equal(rstd, rstd2) and torch.equal(dx, dx2) and torch.equal(dw, dw2)


@pytest.mark.parametrize("cols,dtype", WIDTHS, ids=lambda v: str(v).replace("torch.", ""))
def test_adaln_writes_stay_inside(capi, gpu_device, cols, dtype):
    L, dt, s = capi.lib(), capi._DTYPES[dtype], _stream(gpu_device)
    for batch, rps in ((1, 1), (1, 3), (3, 5), (2, 1031), (3, 7)):
        rows = batch * rps
        d = _inputs(rows, cols, dtype, gpu_device, batch)
        for seq_first in (False, True):
            G = Guarded(gpu_device)
            out, mean, rstd = G.new((rows, cols), dtype), G.new((rows,), torch.float32), G.new((rows,), torch.float32)
            dx, dsc, dsh = G.new((rows, cols), dtype), G.new((batch, cols), dtype), G.new((batch, cols), dtype)
            n = L.tt_adaln_backward_workspace_bytes(batch, rps, cols, dt)
            ws = G.bytes(n)
            fwd = L.tt_adaln_forward_seq_first if seq_first else L.tt_adaln_forward
            bwd = L.tt_adaln_backward_seq_first if seq_first else L.tt_adaln_backward
            _ok(L, fwd(_p(out), _p(mean), _p(rstd), _p(d["x"]), _p(d["scale"]), _p(d["shift"]), batch, rps, cols, EPS, dt, s))
            _ok(L, bwd(_p(dx), _p(dsc), _p(dsh), _p(d["g"]), _p(d["x"]), _p(d["scale"]), _p(mean), _p(rstd), batch, rps,
                       cols, dt, _p(ws), n, s))
            torch.cuda.synchronize()
            G.check(f"adaln batch={batch} rows_per_sample={rps} cols={cols} {dtype} seq_first={seq_first}")
            x3 = d["x"].view(rps, batch, cols) if seq_first else d["x"].view(batch, rps, cols)
            out2, mean2, rstd2 = capi.adaln_forward(x3, d["scale"], d["shift"], EPS, seq_first=seq_first)
            dx2, dsc2, dsh2 = capi.adaln_backward(d["g"].view_as(x3), x3, d["scale"], mean2, rstd2, seq_first=seq_first)
            assert torch.equal(out.view_as(out2), out2) and torch.equal(mean, mean2) and torch.equal(rstd, rstd2)
            assert torch.equal(dx.view_as(dx2), dx2) and torch.equal(dsc, dsc2) and torch.equal(dsh, dsh2)


@pytest.mark.parametrize("cols,dtype", [(3072, torch.bfloat16), (3072, torch.float32), (3072, torch.float16),
                                        (40, torch.bfloat16), (1000, torch.float16), (2000, torch.bfloat16),
                                        (3000, torch.bfloat16), (1500, torch.float32), (100, torch.float32)],
                         ids=lambda v: str(v).replace("torch.", ""))
def test_gated_and_residual_writes_stay_inside(capi, gpu_device, cols, dtype):
    L, dt, s = capi.lib(), capi._DTYPES[dtype], _stream(gpu_device)
    assert L.tt_norm_wide_forms_supported(cols, dt) == 1
    for batch, rps in ((1, 1), (3, 5), (2, 1031)):
        rows = batch * rps
        d = _inputs(rows, cols, dtype, gpu_device, batch, seed=1)
        for with_e in (True, False):
            G = Guarded(gpu_device)
            h2, out = G.new((rows, cols), dtype), G.new((rows, cols), dtype)
            mean, rstd = G.new((rows,), torch.float32), G.new((rows,), torch.float32)
            dh, da = G.new((rows, cols), dtype), G.new((rows, cols), dtype)
            dgate, dsc, dsh = (G.new((batch, cols), dtype) for _ in range(3))
            n = L.tt_gated_residual_adaln_backward_workspace_bytes(batch, rps, cols, dt)
            ws = G.bytes(n)
            _ok(L, L.tt_gated_residual_adaln_forward(_p(h2), _p(out), _p(mean), _p(rstd), _p(d["x"]), _p(d["attn"]),
                                                     _p(d["gate"]), _p(d["scale"]), _p(d["shift"]), batch, rps, cols, EPS,
                                                     dt, s))
            _ok(L, L.tt_gated_residual_adaln_backward(_p(dh), _p(da), _p(dgate), _p(dsc), _p(dsh), _p(d["g"]),
                                                      _p(d["e"]) if with_e else None, _p(h2), _p(d["attn"]), _p(d["gate"]),
                                                      _p(d["scale"]), _p(mean), _p(rstd), batch, rps, cols, dt, _p(ws), n, s))
            torch.cuda.synchronize()
            G.check(f"gated batch={batch} rows_per_sample={rps} cols={cols} {dtype} dh2={with_e}")
            x3, a3 = d["x"].view(batch, rps, cols), d["attn"].view(batch, rps, cols)
            h2b, outb, meanb, rstdb = capi.gated_residual_adaln_forward(x3, a3, d["gate"], d["scale"], d["shift"], EPS)
            ref = capi.gated_residual_adaln_backward(d["g"].view_as(x3), d["e"].view_as(x3) if with_e else None, h2b, a3,
                                                     d["gate"], d["scale"], meanb, rstdb)
            assert torch.equal(h2.view_as(h2b), h2b) and torch.equal(out.view_as(outb), outb)
            for got, want in zip((dh, da, dgate, dsc, dsh), ref):
                assert torch.equal(got.view_as(want), want)
        # the plain backward with the input's other gradient added in
        G = Guarded(gpu_device)
        dx, dsc, dsh = G.new((rows, cols), dtype), G.new((batch, cols), dtype), G.new((batch, cols), dtype)
        n = L.tt_adaln_backward_workspace_bytes(batch, rps, cols, dt)
        ws = G.bytes(n)
        x3 = d["x"].view(batch, rps, cols)
        _, mean, rstd = capi.adaln_forward(x3, d["scale"], d["shift"], EPS)
        _ok(L, L.tt_adaln_backward_residual(_p(dx), _p(dsc), _p(dsh), _p(d["g"]), _p(d["e"]), _p(d["x"]), _p(d["scale"]),
                                            _p(mean), _p(rstd), batch, rps, cols, dt, _p(ws), n, s))
        torch.cuda.synchronize()
        G.check(f"residual batch={batch} rows_per_sample={rps} cols={cols} {dtype}")
        ref = capi.adaln_backward_residual(d["g"].view_as(x3), d["e"].view_as(x3), x3, d["scale"], mean, rstd)
        for got, want in zip((dx, dsc, dsh), ref):
            assert torch.equal(got.view_as(want), want)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,S,H,D", [(1, 1001, 5, 128), (2, 37, 7, 128), (1, 3, 1, 128), (2, 130, 13, 128),
                                     (1, 1030, 12, 128), (2, 131, 5, 40), (1, 61, 7, 64), (1, 9, 2, 3072)])
def test_strided_writes_stay_inside_their_slices(capi, gpu_device, dtype, B, S, H, D):
    """The QK-norm call site: q and k are [B, H, S, D] views into the fused projection [B, S, H, 3D]; the backward
    writes dq and dk into their slices of the projection's gradient and the row copy writes dv into its slice.
    Head counts that are not multiples of the run length; the gradient buffer carries margins, and each call may
    touch its own slice only."""
    L, dt, s = capi.lib(), capi._DTYPES[dtype], _stream(gpu_device)
    gen = torch.Generator(device=gpu_device).manual_seed(B * 1000 + S * 10 + H)
    mixed = torch.randn(B, S, H, 3 * D, device=gpu_device, generator=gen).to(dtype)
    w = (1 + 0.02 * torch.randn(D, device=gpu_device, generator=gen)).to(dtype)
    grads = [torch.randn(B, H, S, D, device=gpu_device, generator=gen).to(dtype) for _ in range(3)]
    G = Guarded(gpu_device)
    dmixed = G.new((B, S, H, 3 * D), dtype)
    fill = dmixed.clone()
    outs = [G.new((B, H, S, D), dtype) for _ in range(2)]
    rstds = [G.new((B * H * S,), torch.float32) for _ in range(2)]
    dws = [G.new((D,), dtype) for _ in range(2)]
    n = L.tt_rmsnorm_backward_workspace_bytes(B * H * S, D, dt)
    ws = G.bytes(n)
    written = torch.zeros_like(dmixed, dtype=torch.bool)
    for i in range(2):
        view = mixed[..., i * D:(i + 1) * D].transpose(1, 2)
        dview = dmixed[..., i * D:(i + 1) * D].transpose(1, 2)
        xs, ds = view.stride(), dview.stride()
        _ok(L, L.tt_rmsnorm_forward_strided(_p(outs[i]), _p(rstds[i]), _p(view), _p(w), B, H, S, xs[0], xs[1], xs[2], D,
                                            EPS, dt, s))
        _ok(L, L.tt_rmsnorm_backward_strided(_p(dmixed[..., i * D:]), _p(dws[i]), _p(grads[i]), _p(view), _p(w),
                                             _p(rstds[i]), B, H, S, xs[0], xs[1], xs[2], ds[0], ds[1], ds[2], D, dt,
                                             _p(ws), n, s))
        torch.cuda.synchronize()
        written[..., i * D:(i + 1) * D] = True
        G.check(f"strided slice {i} B={B} S={S} H={H} D={D} {dtype}")
        assert torch.equal(dmixed[~written], fill[~written]), f"slice {i}: wrote outside its slice of the gradient"
        out2, rstd2 = capi.rmsnorm_forward(view.contiguous(), w, EPS)
        dx2, dw2 = capi.rmsnorm_backward(grads[i], view.contiguous(), w, rstd2)
        assert torch.equal(outs[i], out2) and torch.equal(rstds[i], rstd2)
        if D * mixed.element_size() // 16 > 384:
            # dense rows of more than 384 pieces run their backward on other kernels (four wavefronts per row) than
            # a strided view does: the row sums are formed in another order
            torch.testing.assert_close(dview.contiguous(), dx2, rtol=1e-5, atol=1e-6)
        else:
            assert torch.equal(dview.contiguous(), dx2)
    dv = dmixed[..., 2 * D:].transpose(1, 2)
    ds = dv.stride()
    before = dmixed.clone()
    _ok(L, L.tt_norm_copy_rows_strided(_p(dv), _p(grads[2]), B, H, S, ds[0], ds[1], ds[2], D, dt, s))
    torch.cuda.synchronize()
    G.check("value-gradient row copy")
    assert torch.equal(dmixed[..., :2 * D], before[..., :2 * D]) and torch.equal(dv, grads[2])


@pytest.mark.parametrize("B,S,H,n_rot", [(1, 1001, 5, 1001), (2, 37, 7, 20), (1, 130, 13, 129)])
def test_rotary_strided_writes_stay_inside(capi, gpu_device, B, S, H, n_rot):
    from oracle import norm_oracle as O
    D, dtype = 128, torch.bfloat16
    L, dt, s = capi.lib(), capi.BF16, _stream(gpu_device)
    gen = torch.Generator(device=gpu_device).manual_seed(S)
    mixed = torch.randn(B, S, H, 3 * D, device=gpu_device, generator=gen).to(dtype)
    w = (1 + 0.02 * torch.randn(D, device=gpu_device, generator=gen)).to(dtype)
    grad = torch.randn(B, H, S, D, device=gpu_device, generator=gen).to(dtype)
    cos, sin = (t.to(gpu_device) for t in O.make_rope_tables(n_rot, D, seed=S))
    G = Guarded(gpu_device)
    dmixed = G.new((B, S, H, 3 * D), dtype)
    fill = dmixed.clone()
    out, rstd, dw = G.new((B, H, S, D), dtype), G.new((B * H * S,), torch.float32), G.new((D,), dtype)
    n = L.tt_rmsnorm_backward_workspace_bytes(B * H * S, D, dt)
    ws = G.bytes(n)
    view = mixed[..., D:2 * D].transpose(1, 2)
    dview = dmixed[..., D:2 * D].transpose(1, 2)
    xs, ds = view.stride(), dview.stride()
    _ok(L, L.tt_rmsnorm_rope_forward_strided(_p(out), _p(rstd), _p(view), _p(w), _p(cos), _p(sin), n_rot, B, H, S, xs[0],
                                             xs[1], xs[2], D, EPS, dt, s))
    _ok(L, L.tt_rmsnorm_rope_backward_strided(_p(dview), _p(dw), _p(grad), _p(view), _p(w), _p(rstd), _p(cos), _p(sin),
                                              n_rot, B, H, S, xs[0], xs[1], xs[2], ds[0], ds[1], ds[2], D, dt, _p(ws), n, s))
    torch.cuda.synchronize()
    G.check(f"rotary strided B={B} S={S} H={H}")
    assert torch.equal(dmixed[..., :D], fill[..., :D]) and torch.equal(dmixed[..., 2 * D:], fill[..., 2 * D:])
    out2, rstd2 = capi.rmsnorm_rope_forward_strided(view, w, cos, sin, EPS)
    dx2, dw2 = capi.rmsnorm_rope_backward_strided(grad, view, w, rstd2, cos, sin)
    assert torch.equal(out, out2) and torch.equal(dview, dx2) and torch.equal(dw, dw2)


def test_reference_contract_writes_stay_inside(capi, gpu_device):
    """The entry points with the reference's saved tensors (forward output / normalised rows)."""
    L, s = capi.lib(), _stream(gpu_device)
    for cols, rows in ((128, 1031), (128, 3), (3072, 7), (3072, 1029)):
        dt, dtype = capi.BF16, torch.bfloat16
        d = _inputs(rows, cols, dtype, gpu_device, seed=2)
        G = Guarded(gpu_device)
        out, xn, rstd = G.new((rows, cols), dtype), G.new((rows, cols), dtype), G.new((rows,), torch.float32)
        dx, dsc, dsh, dw = G.new((rows, cols), dtype), G.new((1, cols), dtype), G.new((1, cols), dtype), G.new((cols,), dtype)
        n = max(L.tt_adaln_backward_workspace_bytes(1, rows, cols, dt), L.tt_rmsnorm_backward_workspace_bytes(rows, cols, dt))
        ws = G.bytes(n)
        _ok(L, L.tt_adaln_forward_xnorm(_p(out), _p(xn), _p(rstd), _p(d["x"]), _p(d["scale"]), _p(d["shift"]), 1, rows,
                                        cols, EPS, dt, s))
        _ok(L, L.tt_adaln_backward_from_xnorm(_p(dx), _p(dsc), _p(dsh), _p(d["g"]), _p(xn), _p(d["scale"]), _p(rstd), 1,
                                              rows, cols, dt, _p(ws), n, s))
        torch.cuda.synchronize()
        G.check(f"adaln reference contract rows={rows} cols={cols}")
        _ok(L, L.tt_rmsnorm_forward(_p(out), _p(rstd), _p(d["x"]), _p(d["w"]), rows, cols, EPS, dt, s))
        _ok(L, L.tt_rmsnorm_backward_from_out(_p(dx), _p(dw), _p(d["g"]), _p(out), _p(d["w"]), _p(rstd), rows, cols, dt,
                                              _p(ws), n, s))
        torch.cuda.synchronize()
        G.check(f"rmsnorm reference contract rows={rows} cols={cols}")
        assert bool(torch.isfinite(dx.float()).all()) and bool(torch.isfinite(dw.float()).all())


def test_zero_rows_and_the_static_scratch_path(capi, gpu_device):
    L, s = capi.lib(), _stream(gpu_device)
    dt, dtype, cols = capi.BF16, torch.bfloat16, 3072
    # zero rows: forward is a no-op, backward writes zeros to the parameter gradients and nothing else
    G = Guarded(gpu_device)
    out, dx = G.new((0, cols), dtype), G.new((0, cols), dtype)
    dw, dsc, dsh = G.new((cols,), dtype), G.new((2, cols), dtype), G.new((2, cols), dtype)
    rstd = G.new((0,), torch.float32)
    z = torch.zeros(2, cols, dtype=dtype, device=gpu_device)
    _ok(L, L.tt_rmsnorm_forward(_p(out), _p(rstd), _p(out), _p(z), 0, cols, EPS, dt, s))
    _ok(L, L.tt_rmsnorm_backward(_p(dx), _p(dw), _p(out), _p(out), _p(z), _p(rstd), 0, cols, dt, None, 0, s))
    _ok(L, L.tt_adaln_forward(_p(out), _p(rstd), _p(rstd), _p(out), _p(z), _p(z), 2, 0, cols, EPS, dt, s))
    _ok(L, L.tt_adaln_backward(_p(dx), _p(dsc), _p(dsh), _p(out), _p(out), _p(z), _p(rstd), _p(rstd), 2, 0, cols, dt,
                               None, 0, s))
    torch.cuda.synchronize()
    G.check("zero rows")
    assert not dw.any() and not dsc.any() and not dsh.any()
    # the backward whose scratch lives in the library: outputs guarded, results equal to the ordinary entry point
    for batch, rps, c, ty in ((2, 1031, 3072, torch.bfloat16), (3, 5, 1000, torch.float16), (1, 7, 100, torch.float32)):
        code = capi._DTYPES[ty]
        d = _inputs(batch * rps, c, ty, gpu_device, batch, seed=3)
        x3 = d["x"].view(batch, rps, c)
        _, mean, rstd = capi.adaln_forward(x3, d["scale"], d["shift"], EPS)
        G = Guarded(gpu_device)
        dx, dsc, dsh = G.new((batch * rps, c), ty), G.new((batch, c), ty), G.new((batch, c), ty)
        _ok(L, L.tt_adaln_backward_static(_p(dx), _p(dsc), _p(dsh), _p(d["g"]), _p(d["x"]), _p(d["scale"]), _p(mean),
                                          _p(rstd), batch, rps, c, code, s))
        torch.cuda.synchronize()
        G.check(f"static scratch batch={batch} rows_per_sample={rps} cols={c}")
        ref = capi.adaln_backward(d["g"].view_as(x3), x3, d["scale"], mean, rstd)
        for got, want in zip((dx, dsc, dsh), ref):
            assert torch.equal(got.view_as(want), want)


def test_scratch_is_used_only_up_to_the_size_asked_for(capi, gpu_device):
    """The workspace queries are exact upper bounds: a scratch buffer of exactly that size, with margins."""
    L, s = capi.lib(), _stream(gpu_device)
    for cols, dtype, batch, rps in ((3072, torch.bfloat16, 4, 11056), (128, torch.bfloat16, 1, 40000),
                                    (1000, torch.float16, 3, 3000), (8192, torch.bfloat16, 2, 600)):
        dt = capi._DTYPES[dtype]
        rows = batch * rps
        d = _inputs(rows, cols, dtype, gpu_device, batch, seed=4)
        x3 = d["x"].view(batch, rps, cols)
        _, mean, rstd = capi.adaln_forward(x3, d["scale"], d["shift"], EPS)
        _, rrstd = capi.rmsnorm_forward(d["x"], d["w"], EPS)
        dx = torch.empty_like(d["x"])
        for which in ("adaln", "rmsnorm"):
            G = Guarded(gpu_device)
            dsc, dsh, dw = G.new((batch, cols), dtype), G.new((batch, cols), dtype), G.new((cols,), dtype)
            if which == "adaln":
                n = L.tt_adaln_backward_workspace_bytes(batch, rps, cols, dt)
                ws = G.bytes(n)
                _ok(L, L.tt_adaln_backward(_p(dx), _p(dsc), _p(dsh), _p(d["g"]), _p(d["x"]), _p(d["scale"]), _p(mean),
                                           _p(rstd), batch, rps, cols, dt, _p(ws), n, s))
            else:
                n = L.tt_rmsnorm_backward_workspace_bytes(rows, cols, dt)
                ws = G.bytes(n)
                _ok(L, L.tt_rmsnorm_backward(_p(dx), _p(dw), _p(d["g"]), _p(d["x"]), _p(d["w"]), _p(rrstd), rows, cols, dt,
                                             _p(ws), n, s))
            torch.cuda.synchronize()
            G.check(f"{which} scratch of {n} B, cols={cols} batch={batch} rows_per_sample={rps}")
