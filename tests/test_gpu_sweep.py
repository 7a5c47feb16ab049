"""Seeded random sweep over widths, row counts, element types and layouts, through the C ABI, against the
eager oracle with the bars of tests/test_gpu_anywidth.py.  The fixed lists of the other files name the
geometries on purpose; this file asks the questions nobody thought of (the seed is fixed, so a failure names a
reproducible case)."""
import random

import pytest
import torch

from oracle import norm_oracle as O
from tests.test_gpu_anywidth import BF, EPS, F32, HF, colsum_ok, fwd_16bit_ok, grad_ok

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def capi(gpu_device):
    from teletron_amd import capi as c
    c.lib()
    return c


def _cases(seed, n):
    rng = random.Random(seed)
    out = []
    for _ in range(n):
        dtype = rng.choice([BF, BF, HF, F32])
        piece = 4 if dtype == F32 else 8
        pieces = rng.choice([rng.randint(1, 16), rng.randint(1, 64), rng.randint(1, 400), rng.randint(1, 1024)])
        out.append((pieces * piece, dtype, rng.randint(1, 1200), rng.randint(1, 4)))
    return out


@pytest.mark.parametrize("cols,dtype,rows,batch", _cases(2024, 40))
def test_random_rmsnorm_dense_and_strided(capi, gpu_device, cols, dtype, rows, batch):
    d = O.make_rmsnorm_inputs((rows,), cols, dtype, seed=cols + rows)
    want_out, want_dx, want_dw = O.eager_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
    x, w, g = (d[k].to(gpu_device) for k in ("x", "weight", "grad"))
    out, rstd = capi.rmsnorm_forward(x, w, EPS)
    if dtype == F32:
        torch.testing.assert_close(out.cpu(), want_out, rtol=1e-5, atol=1e-6)
    else:
        fwd_16bit_ok(out, want_out, O.rmsnorm_excuse(want_out), "out")
    dx, dw = capi.rmsnorm_backward(g, x, w, rstd)
    grad_ok(dx, want_dx, "dx")
    colsum_ok(dw, want_dw, d["grad"].float() * want_out.float(), 0, "dweight")
    # the same rows as a strided view: every `batch`-th slot of a wider buffer, transposed leading dimensions
    heads = batch + 1
    if rows % heads == 0 and rows >= heads:
        seq = rows // heads
        wide = torch.zeros(seq, heads, 3 * cols, dtype=dtype, device=gpu_device)
        view = wide[:, :, cols:2 * cols]
        view.copy_(x.reshape(heads, seq, cols).transpose(0, 1))
        xv = view.transpose(0, 1)                                  # [heads, seq, cols], strided
        assert not xv.is_contiguous()
        out_s, rstd_s = capi.rmsnorm_forward_strided(xv, w, EPS)
        dx_s, dw_s = capi.rmsnorm_backward_strided(g.reshape(heads, seq, cols), xv, w, rstd_s)
        out_s, dx_s = out_s.reshape(rows, cols), dx_s.contiguous().reshape(rows, cols)
        if cols * x.element_size() // 16 <= 384:
            assert torch.equal(out_s, out) and torch.equal(rstd_s, rstd) and torch.equal(dx_s, dx)
        else:
            # dense rows of more than 384 pieces run on other kernels (four wavefronts per row) than a strided view of
            # them: the row sums are formed in another order, so the two agree to fp32 rounding, not bit for bit
            torch.testing.assert_close(rstd_s, rstd, rtol=1e-6, atol=0)
            tol = dict(rtol=1e-5, atol=1e-6) if dtype == F32 else dict(rtol=2.0 ** -7, atol=1e-6)
            torch.testing.assert_close(out_s.float(), out.float(), **tol)
            torch.testing.assert_close(dx_s.float(), dx.float(), **tol)
            assert (out_s != out).float().mean() <= 1e-3 and (dx_s != dx).float().mean() <= 1e-2
        colsum_ok(dw_s, want_dw, d["grad"].float() * want_out.float(), 0, "dweight (strided)")


@pytest.mark.parametrize("cols,dtype,seq,batch", _cases(4202, 40))
def test_random_adaln_both_layouts(capi, gpu_device, cols, dtype, seq, batch):
    seq = min(seq, 600)
    d = O.make_adaln_inputs(batch, seq, cols, dtype, seed=cols + seq, sigma=1.5)
    want_out, want_dx, want_ds, want_dh = O.eager_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], d["grad"])
    x, sc, sh, g = (d[k].to(gpu_device) for k in ("x", "scale", "shift", "grad"))
    out, mean, rstd = capi.adaln_forward(x, sc, sh, EPS)
    if dtype == F32:
        torch.testing.assert_close(out.cpu(), want_out, rtol=1e-5, atol=1e-5)
    else:
        fwd_16bit_ok(out, want_out, O.adaln_excuse(d["x"], d["scale"], d["shift"], want_out), "out")
    dx, ds, dh = capi.adaln_backward(g, x, sc, mean, rstd)
    if dtype == F32:
        grad_ok(dx, want_dx, "dx")
    else:
        terms = O.adaln_dx_terms(d["x"], d["scale"], d["grad"])
        assert O.frac_outside(dx.cpu(), want_dx, 1e-2, 1e-3, magnitude=terms) <= max(1e-4, 2.0 / dx.numel()), "dx"
    xn = torch.nn.functional.layer_norm(d["x"].float(), (cols,), None, None, EPS)
    colsum_ok(ds, want_ds, d["grad"].float() * xn, 1, "dscale")
    colsum_ok(dh, want_dh, d["grad"].float(), 1, "dshift")
    # sequence-first rows [seq, batch, cols]: the same numbers, row for row
    xs, gs = x.transpose(0, 1).contiguous(), g.transpose(0, 1).contiguous()
    out_s, mean_s, rstd_s = capi.adaln_forward(xs, sc, sh, EPS, seq_first=True)
    assert torch.equal(out_s.transpose(0, 1), out)
    dx_s, ds_s, dh_s = capi.adaln_backward(gs, xs, sc, mean_s, rstd_s, seq_first=True)
    assert torch.equal(dx_s.transpose(0, 1), dx)
    colsum_ok(ds_s, want_ds, d["grad"].float() * xn, 1, "dscale (sequence-first)")
    colsum_ok(dh_s, want_dh, d["grad"].float(), 1, "dshift (sequence-first)")


def _wide_cases(seed, n):
    rng = random.Random(seed)
    out = []
    for _ in range(n):
        dtype = rng.choice([BF, BF, HF, F32])
        piece = 4 if dtype == F32 else 8
        pieces = rng.choice([rng.randint(1, 16), rng.randint(1, 64), rng.randint(1, 384), 384, rng.randint(385, 1024)])
        out.append((pieces * piece, dtype, rng.randint(1, 4), rng.randint(1, 400), rng.random() < 0.7))
    return out


@pytest.mark.parametrize("C,dtype,B,S,with_h2", _wide_cases(777, 30))
def test_random_gated_and_residual_forms_equal_their_parts(capi, gpu_device, C, dtype, B, S, with_h2):
    """The fused call-site forms at random widths: bit for bit what the elementwise update, the plain AdaLN
    and the plain backward plus autograd's accumulation give when run one after the other."""
    h, a, q, sc, sh, go, g2 = O.make_gated_inputs(B, S, C, dtype, seed=C + S, with_grad_h2=with_h2)
    to = lambda t: None if t is None else t.to(gpu_device)
    H, A, Q, SC, SH, GO, G2 = (to(t) for t in (h, a, q, sc, sh, go, g2))
    h2, out, mean, rstd = capi.gated_residual_adaln_forward(H, A, Q, SC, SH, EPS)
    dh, da, dq, dsc, dsh = capi.gated_residual_adaln_backward(GO, G2, h2, A, Q, SC, mean, rstd)
    h2_parts = H + A * Q[:, None]
    assert torch.equal(h2, h2_parts)
    out_p, mean_p, rstd_p = capi.adaln_forward(h2_parts, SC, SH, EPS)
    assert torch.equal(out, out_p) and torch.equal(mean, mean_p) and torch.equal(rstd, rstd_p)
    dxn, dsc_p, dsh_p = capi.adaln_backward(GO, h2_parts, SC, mean_p, rstd_p)
    dh_parts = dxn + G2 if with_h2 else dxn
    assert torch.equal(dh, dh_parts) and torch.equal(da, dh_parts * Q[:, None])
    assert torch.equal(dsc, dsc_p) and torch.equal(dsh, dsh_p)
    # dgate = sum over the sample's rows of rnd(dh * attn): against an fp32 reduction of the same products
    want_dq = (dh_parts * A).float().sum(1)
    l1 = (dh_parts * A).float().abs().sum(1)
    tol = 1e-5 if dtype == F32 else 2.0 ** -8
    assert ((dq.float() - want_dq).abs() <= tol * want_dq.abs() + 1e-5 * l1 + 1e-6).all()
    if with_h2:
        dxr, dsr, dhr = capi.adaln_backward_residual(GO, G2, h2_parts, SC, mean_p, rstd_p)
        assert torch.equal(dxr, dh_parts) and torch.equal(dsr, dsc_p) and torch.equal(dhr, dsh_p)
