"""GPU parity: the HIP kernels, called through the C ABI (teletron_amd.capi ->
libteletron_norm.so), against the CPU oracle on identical seeded inputs.

Bars (stated once, used everywhere below):
  forward, bf16 : >= 99.9 % of elements bit-identical to eager and every element
                  within 1 bf16 ulp, with one excusable exception.  The kernels
                  and eager sum a row in different orders, so the normalised
                  value (y or xn) can land on the other side of a rounding
                  boundary (one ulp, <= 2^-7 relative); eager then multiplies it
                  (by w or 1+scale) and rounds, and for AdaLN adds shift and
                  rounds again, so the result can move by 2-3 of its own ulp, or
                  by many where the add cancels.  Such elements must lie within
                  what that chain allows -- 2^-6 |out| for RMSNorm,
                  2^-6 |xn*(1+scale)| + 2^-7 |out| for AdaLN -- and number
                  < 1e-4 of all elements (measured: ~2e-6);
  forward, fp32 : rel 1e-5 (abs 1e-6);
  gradients bf16: |got - want| <= 1e-3 + 1e-2 * |want| on every element
                  (AdaLN dx: on all but 1e-5 of elements);
  gradients fp32: rel 1e-4 / abs 1e-5 (column sums: rel 1e-4 of the column's L1 mass).
"""
import ctypes

import pytest
import torch

from oracle import norm_oracle as O
from tests.golden_util import load_golden

pytestmark = pytest.mark.gpu
EPS = 1e-6


@pytest.fixture(scope="module")
def capi(gpu_device):
    from teletron_amd import capi as c
    c.lib()
    return c


def dev(d, device):
    return {k: (v.to(device) if torch.is_tensor(v) else v) for k, v in d.items()}


def assert_fwd_bf16(got, want, guard=None, what=""):
    if guard is None:
        guard = O.rmsnorm_excuse(want)
    rep = O.compare_bf16_ulp(got.cpu(), want, excuse_abs=guard)
    assert rep.n_gt1 == 0, (what, rep)
    assert rep.n_excused <= 1e-4 * rep.n, (what, rep)
    assert rep.frac_exact >= 0.999, (what, rep)


def assert_grad_bf16(got, want, what="", allow=0.0):
    frac = O.frac_outside(got.cpu(), want, 1e-2, 1e-3)
    assert frac <= allow, (what, frac)


def adaln_guard(d, want_out, eps=EPS):
    return O.adaln_excuse(d["x"], d["scale"], d["shift"], want_out, eps)


# ------------------------------------------------------------------ goldens

def test_golden_vectors(capi, gpu_device):
    for name, d in load_golden().items():
        g = dev(d, gpu_device)
        loose = {}          # fields whose bound scales with the terms that are summed
        if name.startswith("rms"):
            out, rstd = capi.rmsnorm_forward(g["x"], g["weight"], EPS)
            dx, dw = capi.rmsnorm_backward(g["grad"], g["x"], g["weight"], rstd)
            got = {"out": out, "dx": dx, "dweight": dw}
            guard = None
        elif name.startswith("adaln"):
            out, mean, rstd = capi.adaln_forward(g["x"], g["scale"], g["shift"], EPS)
            dx, ds, dh = capi.adaln_backward(g["grad"], g["x"], g["scale"], mean, rstd)
            got = {"out": out, "dx": dx, "dscale": ds, "dshift": dh}
            guard = adaln_guard(d, d["out"]) if d["is_16bit"] else None
            loose["dx"] = O.adaln_dx_terms(d["x"], d["scale"], d["grad"])
        else:
            h2, out, mean, rstd = capi.gated_residual_adaln_forward(g["h"], g["attn"], g["gate"], g["scale"],
                                                                    g["shift"], EPS)
            assert torch.equal(h2.cpu(), d["h2"]), name
            grads = capi.gated_residual_adaln_backward(g["grad"], g["grad_h2"], h2, g["attn"], g["gate"], g["scale"],
                                                       mean, rstd)
            got = dict(zip(("dh", "dattn", "dgate", "dscale", "dshift"), grads), out=out)
            guard = O.adaln_excuse(d["h2"], d["scale"], d["shift"], d["out"])
            terms = d["dh"].float().abs() + d["grad_h2"].float().abs()
            loose = {"dh": terms, "dattn": terms * d["gate"].float().abs()[:, None]}
            assert O.colsum_outside(got.pop("dgate").cpu(), d["dgate"], terms * d["attn"].float(), dim=1) == 0, name
        for k, v in got.items():
            if d["is_16bit"]:
                if k == "out":
                    assert_fwd_bf16(v, d[k], guard, f"{name}/{k}")
                elif k in loose:
                    assert O.frac_outside(v.cpu(), d[k], 1e-2, 1e-3, magnitude=loose[k]) <= 1e-4, f"{name}/{k}"
                else:
                    assert_grad_bf16(v, d[k], f"{name}/{k}")
            else:
                torch.testing.assert_close(v.cpu(), d[k], rtol=1e-4, atol=1e-5, msg=f"{name}/{k}")


# ------------------------------------------------------------------ RMSNorm

@pytest.mark.parametrize("cols,rows", [(128, 1), (128, 3), (128, 4), (128, 4099), (128, 100003),
                                       (3072, 1), (3072, 5), (3072, 1031), (3072, 9001)])
def test_rmsnorm_bf16_vs_eager(capi, gpu_device, cols, rows):
    d = O.make_rmsnorm_inputs((rows,), cols, torch.bfloat16, seed=100 + rows % 97)
    want_out, want_dx, want_dw = O.eager_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
    g = dev(d, gpu_device)
    out, rstd = capi.rmsnorm_forward(g["x"], g["weight"], EPS)
    assert_fwd_bf16(out, want_out, None, "out")
    _, want_r = O.staged_rmsnorm_fwd(d["x"], d["weight"])
    torch.testing.assert_close(rstd.cpu(), want_r.reshape(-1), rtol=1e-6, atol=0)
    dx, dw = capi.rmsnorm_backward(g["grad"], g["x"], g["weight"], rstd)
    assert_grad_bf16(dx, want_dx, "dx")
    assert_grad_bf16(dw, want_dw, "dweight")
    # dx is also nearly bit-identical to eager (same rounding points)
    assert O.compare_bf16_ulp(dx.cpu(), want_dx).frac_exact > 0.99


@pytest.mark.parametrize("cols,rows", [(128, 777), (3072, 8192 // 16)])
def test_rmsnorm_fp32_vs_eager(capi, gpu_device, cols, rows):
    d = O.make_rmsnorm_inputs((rows,), cols, torch.float32, seed=7)
    want_out, want_dx, want_dw = O.eager_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
    g = dev(d, gpu_device)
    out, rstd = capi.rmsnorm_forward(g["x"], g["weight"], EPS)
    torch.testing.assert_close(out.cpu(), want_out, rtol=1e-5, atol=1e-6)
    dx, dw = capi.rmsnorm_backward(g["grad"], g["x"], g["weight"], rstd)
    torch.testing.assert_close(dx.cpu(), want_dx, rtol=1e-4, atol=1e-5)
    l1 = (d["grad"].abs() * want_out.abs()).sum(0)
    assert ((dw.cpu() - want_dw).abs() <= 1e-4 * l1 + 1e-5).all()


@pytest.mark.parametrize("cols,rows", [(128, 5001), (3072, 515)])
def test_rmsnorm_backward_from_saved_output(capi, gpu_device, cols, rows):
    """The reference-compatible entry point works from the forward OUTPUT."""
    d = O.make_rmsnorm_inputs((rows,), cols, torch.bfloat16, seed=5)
    want_out, want_dx, want_dw = O.eager_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
    g = dev(d, gpu_device)
    out, rstd = capi.rmsnorm_forward(g["x"], g["weight"], EPS)
    dx, dw = capi.rmsnorm_backward(g["grad"], out, g["weight"], rstd, from_out=True)
    # xhat = out / w is known to bf16 only (relative error up to 2^-8 per element), as in
    # the reference kernel: dx meets the gradient bar on >= 99.9 % of elements and 10x the
    # bar everywhere; a dweight column carries the random sum of `rows` such errors.
    assert O.frac_outside(dx.cpu(), want_dx, 1e-2, 1e-3) < 1e-3
    assert O.frac_outside(dx.cpu(), want_dx, 1e-1, 1e-2) == 0.0
    l2 = (d["grad"].float() * want_out.float()).pow(2).reshape(-1, cols).sum(0).sqrt()
    assert ((dw.cpu().float() - want_dw.float()).abs() <= 1e-2 * want_dw.float().abs() + 2.0 ** -7 * l2).all()


# -------------------------------------------------------------------- AdaLN

@pytest.mark.parametrize("batch,seq", [(1, 1), (1, 7), (1, 2053), (4, 333), (3, 1), (5, 1001), (300, 2)])
def test_adaln_bf16_vs_eager(capi, gpu_device, batch, seq):
    d = O.make_adaln_inputs(batch, seq, 3072, torch.bfloat16, seed=200 + seq % 89, sigma=1.5)
    want_out, want_dx, want_ds, want_dh = O.eager_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], d["grad"])
    g = dev(d, gpu_device)
    out, mean, rstd = capi.adaln_forward(g["x"], g["scale"], g["shift"], EPS)
    assert_fwd_bf16(out, want_out, adaln_guard(d, want_out), "out")
    _, want_mu, want_r = O.staged_adaln_fwd(d["x"], d["scale"], d["shift"])
    torch.testing.assert_close(rstd.cpu(), want_r.reshape(-1), rtol=2e-6, atol=0)
    torch.testing.assert_close(mean.cpu(), want_mu.reshape(-1), rtol=0, atol=2e-6)
    dx, ds, dh = capi.adaln_backward(g["grad"], g["x"], g["scale"], mean, rstd)
    assert_grad_bf16(dx, want_dx, "dx", allow=1e-5)
    assert_grad_bf16(ds, want_ds, "dscale")
    assert_grad_bf16(dh, want_dh, "dshift")


def test_adaln_fp32_vs_eager(capi, gpu_device):
    d = O.make_adaln_inputs(3, 171, 3072, torch.float32, seed=9)
    want_out, want_dx, want_ds, want_dh = O.eager_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], d["grad"])
    g = dev(d, gpu_device)
    out, mean, rstd = capi.adaln_forward(g["x"], g["scale"], g["shift"], EPS)
    torch.testing.assert_close(out.cpu(), want_out, rtol=1e-5, atol=1e-5)
    dx, ds, dh = capi.adaln_backward(g["grad"], g["x"], g["scale"], mean, rstd)
    torch.testing.assert_close(dx.cpu(), want_dx, rtol=1e-4, atol=1e-5)
    l1 = d["grad"].abs().sum(1)
    assert ((dh.cpu() - want_dh).abs() <= 1e-4 * l1 + 1e-5).all()
    assert ((ds.cpu() - want_ds).abs() <= 1e-4 * 3 * l1 + 1e-5).all()


def test_adaln_reference_compatible_entry_points(capi, gpu_device):
    """forward that also writes x_norm + backward from x_norm (what the
    reference's autograd class saves)."""
    d = O.make_adaln_inputs(2, 409, 3072, torch.bfloat16, seed=31)
    want_out, want_dx, want_ds, want_dh = O.eager_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], d["grad"])
    g = dev(d, gpu_device)
    out, xn, rstd = capi.adaln_forward(g["x"], g["scale"], g["shift"], EPS, want_xnorm=True)
    out2, mean, rstd2 = capi.adaln_forward(g["x"], g["scale"], g["shift"], EPS)
    assert torch.equal(out, out2) and torch.equal(rstd, rstd2)
    want_xn = torch.nn.functional.layer_norm(d["x"], (3072,), None, None, EPS)
    rep = O.compare_bf16_ulp(xn.cpu(), want_xn)
    assert rep.n_gt1 == 0 and rep.frac_exact > 0.999
    dx, ds, dh = capi.adaln_backward(g["grad"], xn, g["scale"], None, rstd, from_xnorm=True)
    assert O.frac_outside(dx.cpu(), want_dx, 1e-2, 1e-3) < 1e-3     # xhat known to bf16 only
    assert O.frac_outside(dx.cpu(), want_dx, 1e-1, 1e-2) == 0.0
    assert_grad_bf16(ds, want_ds, "dscale")
    assert_grad_bf16(dh, want_dh, "dshift")


# -------------------------------------------- properties at the full shapes

def _full_rows():
    return 118800


def test_full_size_rmsnorm_properties(capi, gpu_device):
    """118 800 x 3072 bf16: determinism, exact linearity in the upstream grad,
    and agreement with eager on a strided sample of rows."""
    rows, C = _full_rows(), 3072
    gen = torch.Generator(device=gpu_device).manual_seed(0)
    x = torch.randn(rows, C, device=gpu_device, generator=gen).bfloat16()
    grad = torch.randn(rows, C, device=gpu_device, generator=gen).bfloat16()
    w = (1 + 0.02 * torch.randn(C, device=gpu_device, generator=gen)).bfloat16()
    out, rstd = capi.rmsnorm_forward(x, w, EPS)
    out2, rstd2 = capi.rmsnorm_forward(x, w, EPS)
    assert torch.equal(out, out2) and torch.equal(rstd, rstd2)
    dx, dw = capi.rmsnorm_backward(grad, x, w, rstd)
    dx2, dw2 = capi.rmsnorm_backward(grad, x, w, rstd)
    assert torch.equal(dx, dx2) and torch.equal(dw, dw2)           # deterministic reduction
    dx4, dw4 = capi.rmsnorm_backward(grad * 4, x, w, rstd)          # exact power-of-two scaling
    assert torch.equal(dx4, dx * 4)
    torch.testing.assert_close(dw4.float(), dw.float() * 4, rtol=2 ** -7, atol=0)
    # sampled rows against eager on the CPU
    idx = torch.arange(0, rows, 997, device=gpu_device)
    xs, gs = x[idx].cpu(), grad[idx].cpu()
    want_out, want_dx, _ = O.eager_rmsnorm_fwd_bwd(xs, w.cpu(), gs)
    assert_fwd_bf16(out[idx], want_out, None, "out rows")
    assert_grad_bf16(dx[idx], want_dx, "dx rows")
    # dweight against an independent fp32 column reduction on the GPU (torch ops)
    y = (x.float() * rstd[:, None]).bfloat16()
    want_dw = (grad * y).float().sum(0)
    assert O.frac_outside(dw.cpu(), want_dw.cpu(), 1e-2, 1e-3) == 0.0


def test_full_size_adaln_properties(capi, gpu_device):
    rows, C = _full_rows(), 3072
    gen = torch.Generator(device=gpu_device).manual_seed(1)
    x = torch.randn(1, rows, C, device=gpu_device, generator=gen).bfloat16()
    grad = torch.randn(1, rows, C, device=gpu_device, generator=gen).bfloat16()
    scale = (0.1 * torch.randn(1, C, device=gpu_device, generator=gen)).bfloat16()
    shift = (0.1 * torch.randn(1, C, device=gpu_device, generator=gen)).bfloat16()
    out, mean, rstd = capi.adaln_forward(x, scale, shift, EPS)
    out2, _, _ = capi.adaln_forward(x, scale, shift, EPS)
    assert torch.equal(out, out2)
    dx, ds, dh = capi.adaln_backward(grad, x, scale, mean, rstd)
    dx2, ds2, dh2 = capi.adaln_backward(grad, x, scale, mean, rstd)
    assert torch.equal(dx, dx2) and torch.equal(ds, ds2) and torch.equal(dh, dh2)
    dx4, ds4, dh4 = capi.adaln_backward(grad * 4, x, scale, mean, rstd)
    assert torch.equal(dx4, dx * 4)
    # LayerNorm backward is orthogonal to the ones vector: before the final rounding each
    # row of dx sums to zero, and rounding moves an element by at most 2^-8 of itself
    assert (dx.float().sum(-1).abs() <= 2.0 ** -8 * dx.float().abs().sum(-1) + 1e-3).all()
    # dshift = column sums of the upstream gradient
    want_dh = grad.float().sum(1)
    assert O.frac_outside(dh.cpu(), want_dh.cpu(), 1e-2, 1e-3) == 0.0
    # dscale against an independent fp32 column reduction (torch ops) of rnd(g * rnd(xhat)), xhat from the
    # statistics the forward wrote
    # (summed in float64: over 118 800 terms an fp32 reduction of its own carries ~1e-3 of rounding); the plain
    # gradient bar on all but 1e-3 of the columns, and every column within 1e-2 |want| + 2^-8 of its L2 mass
    xn = ((x.float() - mean.view(1, rows, 1)) * rstd.view(1, rows, 1)).bfloat16()
    terms = grad * xn
    del xn
    want_ds = terms.double().sum(1)
    l2 = terms.float().pow(2).sum(1).sqrt().double()
    del terms
    assert O.frac_outside(ds.cpu(), want_ds.cpu(), 1e-2, 1e-3) <= 1e-3
    assert bool(((ds.double() - want_ds).abs() <= 1e-2 * want_ds.abs() + 2.0 ** -8 * l2).all())
    # the input's other gradient added inside the kernel == plain backward, then the addition
    other = (0.5 * torch.randn(1, rows, C, device=gpu_device, generator=gen)).bfloat16()
    dxr, dsr, dhr = capi.adaln_backward_residual(grad, other, x, scale, mean, rstd)
    assert torch.equal(dxr, dx + other) and torch.equal(dsr, ds) and torch.equal(dhr, dh)
    del dxr, other
    idx = torch.arange(0, rows, 991, device=gpu_device)
    d = {"x": x[:, idx].cpu(), "scale": scale.cpu(), "shift": shift.cpu(), "grad": grad[:, idx].cpu()}
    want_out, want_dx, _, _ = O.eager_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], d["grad"])
    assert_fwd_bf16(out[:, idx], want_out, adaln_guard(d, want_out), "out rows")
    assert_grad_bf16(dx[:, idx], want_dx, "dx rows", allow=1e-5)


# ---------------------------------------------------- gated residual + AdaLN

def _gated_terms(want_dh, grad_h2):
    t = want_dh.float().abs()
    return t if grad_h2 is None else t + grad_h2.float().abs()


@pytest.mark.parametrize("batch,seq,with_h2_grad", [(1, 1, True), (1, 7, False), (2, 1031, True),
                                                     (3, 333, False), (5, 1001, True), (260, 3, True)])
def test_gated_residual_adaln_bf16_vs_eager(capi, gpu_device, batch, seq, with_h2_grad):
    h, a, q, sc, sh, go, g2 = O.make_gated_inputs(batch, seq, 3072, torch.bfloat16, seed=300 + seq % 83,
                                                  with_grad_h2=with_h2_grad)
    want = O.eager_gated_residual_adaln_fwd_bwd(h, a, q, sc, sh, go, g2)
    w_h2, w_out, w_dh, w_da, w_dq, w_dsc, w_dsh = want
    to = lambda t: None if t is None else t.to(gpu_device)
    H, A, Q, SC, SH, GO, G2 = (to(t) for t in (h, a, q, sc, sh, go, g2))
    h2, out, mean, rstd = capi.gated_residual_adaln_forward(H, A, Q, SC, SH, EPS)
    assert torch.equal(h2.cpu(), w_h2)                      # two roundings, both fixed by the expression
    assert_fwd_bf16(out, w_out, O.adaln_excuse(w_h2, sc, sh, w_out), "out")
    _, want_mu, want_r = O.staged_adaln_fwd(w_h2, sc, sh)
    torch.testing.assert_close(rstd.cpu(), want_r.reshape(-1), rtol=2e-6, atol=0)
    torch.testing.assert_close(mean.cpu(), want_mu.reshape(-1), rtol=0, atol=2e-6)
    dh, da, dq, dsc, dsh = capi.gated_residual_adaln_backward(GO, G2, h2, A, Q, SC, mean, rstd)
    # gradients: |got - want| <= 1e-3 + 1e-2 * m on all but 1e-5 of elements; m = |want| except for
    # dh = round(dx of the norm) + grad_h2, a sum of separately rounded terms that may cancel, where
    # m is the size of the terms; dgate sums dh * attn with dh known to an ulp: random-walk bound
    terms = _gated_terms(w_dh, g2)
    assert O.frac_outside(dh.cpu(), w_dh, 1e-2, 1e-3, magnitude=terms) <= 1e-5
    assert O.frac_outside(da.cpu(), w_da, 1e-2, 1e-3, magnitude=terms * q.float().abs()[:, None]) <= 1e-5
    assert O.colsum_outside(dq.cpu(), w_dq, terms * a.float(), dim=1) == 0
    assert_grad_bf16(dsc, w_dsc, "dscale")
    assert_grad_bf16(dsh, w_dsh, "dshift")


def test_gated_residual_adaln_fp32_vs_eager(capi, gpu_device):
    h, a, q, sc, sh, go, g2 = O.make_gated_inputs(3, 171, 3072, torch.float32, seed=12)
    want = O.eager_gated_residual_adaln_fwd_bwd(h, a, q, sc, sh, go, g2)
    H, A, Q, SC, SH, GO, G2 = (t.to(gpu_device) for t in (h, a, q, sc, sh, go, g2))
    h2, out, mean, rstd = capi.gated_residual_adaln_forward(H, A, Q, SC, SH, EPS)
    dh, da, dq, dsc, dsh = capi.gated_residual_adaln_backward(GO, G2, h2, A, Q, SC, mean, rstd)
    torch.testing.assert_close(h2.cpu(), want[0], rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(out.cpu(), want[1], rtol=1e-5, atol=1e-6)   # forward fp32: rel 1e-5
    for got, w in zip((dh, da), want[2:4]):                                # gradients fp32: rel 1e-4
        torch.testing.assert_close(got.cpu(), w, rtol=1e-4, atol=1e-5)
    l1 = (want[2].abs() * a.abs()).sum(1)
    assert ((dq.cpu() - want[4]).abs() <= 1e-4 * l1 + 1e-5).all()          # column sums: 1e-4 of the L1 mass
    for got, w in zip((dsc, dsh), want[5:7]):
        torch.testing.assert_close(got.cpu(), w, rtol=1e-4, atol=1e-4)


def test_full_size_gated_residual_adaln_properties(capi, gpu_device):
    """118 800 x 3072 bf16.  The fused op must be bit-identical to its parts run one after the
    other: h2 to the elementwise update, out / mean / rstd to the plain AdaLN forward of h2, and the
    backward to the plain AdaLN backward followed by the elementwise gradient formulas."""
    rows, C = _full_rows(), 3072
    gen = torch.Generator(device=gpu_device).manual_seed(2)
    rnd = lambda *shape, s=1.0: (s * torch.randn(*shape, device=gpu_device, generator=gen)).bfloat16()
    h, a, go = rnd(1, rows, C), rnd(1, rows, C), rnd(1, rows, C, s=0.1)
    q, sc, sh = rnd(1, C, s=0.3), rnd(1, C, s=0.3), rnd(1, C, s=0.3)
    h2, out, mean, rstd = capi.gated_residual_adaln_forward(h, a, q, sc, sh, EPS)
    assert torch.equal(h2, h + a * q[:, None])
    out_p, mean_p, rstd_p = capi.adaln_forward(h2, sc, sh, EPS)
    assert torch.equal(out, out_p) and torch.equal(mean, mean_p) and torch.equal(rstd, rstd_p)
    del out_p, h
    dh, da, dq, dsc, dsh = capi.gated_residual_adaln_backward(go, None, h2, a, q, sc, mean, rstd)
    dx_p, dsc_p, dsh_p = capi.adaln_backward(go, h2, sc, mean, rstd)
    assert torch.equal(dh, dx_p) and torch.equal(dsc, dsc_p) and torch.equal(dsh, dsh_p)
    del dx_p
    assert torch.equal(da, dh * q[:, None])
    want_dq = (dh * a).float().sum(1)
    assert O.colsum_outside(dq.cpu(), want_dq.cpu(), (dh * a).float().cpu(), dim=1, ulp=2.0 ** -9) == 0
    del da
    # with an upstream gradient on h2: dh = round(dx of the norm + that gradient), run twice -> identical
    g2 = rnd(1, rows, C, s=0.1)
    dh2a = capi.gated_residual_adaln_backward(go, g2, h2, a, q, sc, mean, rstd)
    assert torch.equal(dh2a[0], dh + g2)
    dh2b = capi.gated_residual_adaln_backward(go, g2, h2, a, q, sc, mean, rstd)
    assert all(torch.equal(x, y) for x, y in zip(dh2a, dh2b))
    # gate = 0: the residual stream passes through, attn receives no gradient
    z = torch.zeros_like(q)
    h2z, _, mz, rz = capi.gated_residual_adaln_forward(h2, a, z, sc, sh, EPS)
    assert torch.equal(h2z, h2)
    daz = capi.gated_residual_adaln_backward(go, None, h2z, a, z, sc, mz, rz)[1]
    assert not daz.any()


def test_gated_residual_adaln_rejects_other_widths(capi, gpu_device):
    mk = lambda *shape: torch.zeros(*shape, device=gpu_device, dtype=torch.bfloat16)
    with pytest.raises(capi.NormError) as e:     # rows that are not whole 16-byte pieces, or too wide
        capi.gated_residual_adaln_forward(mk(1, 8, 4100), mk(1, 8, 4100), mk(1, 4100), mk(1, 4100), mk(1, 4100), EPS)
    assert e.value.status == 2
    with pytest.raises(capi.NormError) as e:
        capi.gated_residual_adaln_forward(mk(1, 8, 8200), mk(1, 8, 8200), mk(1, 8200), mk(1, 8200), mk(1, 8200), EPS)
    assert e.value.status == 2
    # zero rows: a no-op forward and all-zero parameter gradients
    h2, out, mean, rstd = capi.gated_residual_adaln_forward(mk(2, 0, 3072), mk(2, 0, 3072), mk(2, 3072),
                                                            mk(2, 3072), mk(2, 3072), EPS)
    grads = capi.gated_residual_adaln_backward(mk(2, 0, 3072), None, h2, mk(2, 0, 3072), mk(2, 3072),
                                               mk(2, 3072), mean, rstd)
    assert all(g.shape == (2, 3072) and not g.any() for g in grads[2:])


def test_qk_norm_shape_one_cp_rank(capi, gpu_device):
    """q of one CP=4 rank: [1, 29700, 24, 128] bf16 = 712 800 rows of 128."""
    d = O.make_rmsnorm_inputs((1, 29700, 24), 128, torch.bfloat16, seed=0)
    want_out, want_dx, want_dw = O.eager_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
    g = dev(d, gpu_device)
    out, rstd = capi.rmsnorm_forward(g["x"], g["weight"], EPS)
    assert_fwd_bf16(out, want_out, None, "out")
    dx, dw = capi.rmsnorm_backward(g["grad"], g["x"], g["weight"], rstd)
    assert_grad_bf16(dx, want_dx, "dx")
    assert_grad_bf16(dw, want_dw, "dweight")


def test_batched_per_sample_modulation_chain(capi, gpu_device):
    """batch 4 x (10800 + 256) tokens, sigma 2, distinct modulation per sample:
    AdaLN then RMSNorm(3072), forward and backward of the chain."""
    B, S, C = 4, 11056, 3072
    d = O.make_adaln_inputs(B, S, C, torch.bfloat16, seed=0, sigma=2.0)
    w = (1 + 0.02 * torch.randn(C, generator=torch.Generator().manual_seed(3))).bfloat16()
    xr = d["x"].clone().requires_grad_(True)
    sc = d["scale"].clone().requires_grad_(True)
    sh = d["shift"].clone().requires_grad_(True)
    wr = w.clone().requires_grad_(True)
    y = O.eager_adaln(xr, sc, sh, EPS)
    z = O.eager_rmsnorm(y, wr, EPS)
    z.backward(d["grad"])
    g = dev(d, gpu_device)
    wg = w.to(gpu_device)
    y_g, mean, rstd = capi.adaln_forward(g["x"], g["scale"], g["shift"], EPS)
    z_g, rstd2 = capi.rmsnorm_forward(y_g, wg, EPS)
    assert_fwd_bf16(y_g, y.detach(), adaln_guard(d, y.detach()), "adaln out")
    # z sees y's occasional 1-ulp differences re-normalised: same bar, exact fraction relaxed
    rep = O.compare_bf16_ulp(z_g.cpu(), z.detach())
    assert rep.frac_exact > 0.995 and O.frac_outside(z_g.cpu(), z.detach(), 1e-2, 1e-3) < 1e-5
    dy, dw = capi.rmsnorm_backward(g["grad"], y_g, wg, rstd2)
    dx, ds, dh = capi.adaln_backward(dy, g["x"], g["scale"], mean, rstd)
    # The reduced gradients sum 11 056 (dscale, dshift) or 44 224 (dweight) rows whose inputs are
    # the previous op's outputs, which already differ from eager's by the occasional one-ulp flip;
    # a column whose sum nearly cancels can then miss the absolute part of the bar.  Such columns
    # must be few and stay within 5x of it.
    for name, got, want in (("dweight", dw, wr.grad), ("dscale", ds, sc.grad), ("dshift", dh, sh.grad)):
        assert_grad_bf16(got, want, name, allow=3e-3)
        assert O.frac_outside(got.cpu(), want, 5e-2, 5e-3) == 0.0, name
    assert_grad_bf16(dx, xr.grad, "dx", allow=1e-4)


# ---------------------------------------------------------------- boundary

def test_non_default_stream_and_output_reuse(capi, gpu_device):
    d = dev(O.make_rmsnorm_inputs((4096,), 3072, torch.bfloat16, seed=1), gpu_device)
    ref, _ = capi.rmsnorm_forward(d["x"], d["weight"], EPS)
    side = torch.cuda.Stream(device=gpu_device)
    side.wait_stream(torch.cuda.current_stream(gpu_device))
    with torch.cuda.stream(side):
        out, _ = capi.rmsnorm_forward(d["x"], d["weight"], EPS)
    side.synchronize()
    assert torch.equal(out, ref)


def test_calls_capture_into_a_hip_graph_and_replay(capi, gpu_device):
    """The entry points only launch kernels on the stream they are given (no allocation, no memset, no
    synchronisation), so a caller can capture a forward+backward into a HIP graph.  Every replay, with
    new input values and eager work in between, must equal the directly launched result bit for bit."""
    C, S = 3072, 700
    mk = lambda seed: O.make_adaln_inputs(2, S, C, torch.bfloat16, seed=seed)
    static = {k: v.to(gpu_device) for k, v in mk(900).items()}
    q = {k: v.to(gpu_device) for k, v in O.make_rmsnorm_inputs((S * 24,), 128, torch.bfloat16, seed=901).items()}

    def run():
        out, mean, rstd = capi.adaln_forward(static["x"], static["scale"], static["shift"], EPS)
        grads = capi.adaln_backward(static["grad"], static["x"], static["scale"], mean, rstd)
        qo, qr = capi.rmsnorm_forward(q["x"], q["weight"], EPS)
        qg = capi.rmsnorm_backward(q["grad"], q["x"], q["weight"], qr)
        return (out, *grads, qo, *qg)

    run()                                   # warm: first-use device queries happen outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run()
    for replay in range(3):
        fresh = mk(910 + replay)
        for k in static:
            static[k].copy_(fresh[k].to(gpu_device))
        q["x"].copy_(torch.roll(q["x"], 1 + replay, 0))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = run()                        # eager launches of the same calls on the same inputs
        torch.cuda.synchronize()
        for i, (g, w) in enumerate(zip(got, want)):
            assert torch.equal(g, w), (replay, i)


def test_error_statuses(capi, gpu_device):
    L = capi.lib()
    x = torch.zeros(8, 3072, dtype=torch.bfloat16, device=gpu_device)
    w = torch.ones(3072, dtype=torch.bfloat16, device=gpu_device)
    r = torch.zeros(8, dtype=torch.float32, device=gpu_device)
    vp = lambda t, off=0: ctypes.c_void_p(t.data_ptr() + off)
    # unsupported column count
    assert L.tt_rmsnorm_forward(vp(x), vp(r), vp(x), vp(w), 8, 100, 1e-6, 0, None) == 2
    assert b"cols=100" in L.tt_norm_last_error()
    # unsupported dtype
    assert L.tt_rmsnorm_forward(vp(x), vp(r), vp(x), vp(w), 8, 3072, 1e-6, 7, None) == 2
    # misaligned pointer
    assert L.tt_rmsnorm_forward(vp(x, 2), vp(r), vp(x), vp(w), 4, 3072, 1e-6, 0, None) == 3
    # null pointer / bad sizes
    assert L.tt_rmsnorm_forward(None, vp(r), vp(x), vp(w), 8, 3072, 1e-6, 0, None) == 1
    assert L.tt_rmsnorm_forward(vp(x), vp(r), vp(x), vp(w), -1, 3072, 1e-6, 0, None) == 1
    assert L.tt_rmsnorm_forward(vp(x), vp(r), vp(x), vp(w), 0, 3072, 1e-6, 0, None) == 0   # zero rows: valid no-op
    # workspace too small
    need = L.tt_rmsnorm_backward_workspace_bytes(8, 3072, 0)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device=gpu_device)
    assert L.tt_rmsnorm_backward(vp(x), vp(w), vp(x), vp(x), vp(w), vp(r), 8, 3072, 0, vp(ws), need - 1, None) == 4
    assert L.tt_rmsnorm_backward(vp(x), vp(w), vp(x), vp(x), vp(w), vp(r), 8, 3072, 0, None, 0, None) == 4
    with pytest.raises(capi.NormError):   # rows that are not whole 16-byte pieces
        capi.rmsnorm_forward(torch.zeros(4, 260, dtype=torch.bfloat16, device=gpu_device),
                             torch.ones(260, dtype=torch.bfloat16, device=gpu_device), EPS)
    torch.cuda.synchronize()


# ------------------------------------------- strided views (QK-norm call site)

def _qkv_views(B, S, H, D, dtype, seed, device):
    """query/key as the attention caller sees them: slices of a fused [B, S, H, 3D] projection,
    transposed to [B, H, S, D] (dit_attention.py:149-203)."""
    gen = torch.Generator().manual_seed(seed)
    mixed = torch.randn(B, S, H, 3 * D, generator=gen).to(dtype)
    q_cpu, k_cpu, _ = torch.split(mixed, [D, D, D], dim=3)
    mixed_g = mixed.to(device)
    q_g, k_g, _ = torch.split(mixed_g, [D, D, D], dim=3)
    return q_cpu.transpose(1, 2), k_cpu.transpose(1, 2), q_g.transpose(1, 2), k_g.transpose(1, 2)


@pytest.mark.parametrize("B,S,H", [(1, 1001, 24), (2, 37, 6), (1, 3, 1), (1, 129, 13), (2, 4001, 10)])
def test_rmsnorm_strided_qk_view_matches_eager(capi, gpu_device, B, S, H):
    D = 128
    q_cpu, k_cpu, q_g, k_g = _qkv_views(B, S, H, D, torch.bfloat16, 5, gpu_device)
    gen = torch.Generator().manual_seed(6)
    w = (1 + 0.02 * torch.randn(D, generator=gen)).bfloat16()
    grad = torch.randn(B, H, S, D, generator=gen).bfloat16()
    for x_cpu, x_g in ((q_cpu, q_g), (k_cpu, k_g)):
        assert not x_g.is_contiguous()
        want_out, want_dx, want_dw = O.eager_rmsnorm_fwd_bwd(x_cpu, w, grad)
        out, rstd = capi.rmsnorm_forward_strided(x_g, w.to(gpu_device), EPS)
        assert out.is_contiguous() and out.shape == (B, H, S, D)
        assert_fwd_bf16(out, want_out, None, "out")
        # identical to the dense kernel on a materialised copy (same per-row arithmetic)
        out_dense, rstd_dense = capi.rmsnorm_forward(x_g.contiguous(), w.to(gpu_device), EPS)
        assert torch.equal(out, out_dense) and torch.equal(rstd, rstd_dense)
        dx, dw = capi.rmsnorm_backward_strided(grad.to(gpu_device), x_g, w.to(gpu_device), rstd)
        assert dx.shape == x_g.shape and dx.transpose(1, 2).is_contiguous()   # laid out in x's dimension order
        assert_grad_bf16(dx, want_dx, "dx")
        assert_grad_bf16(dw, want_dw, "dweight")
        dx_dense, _ = capi.rmsnorm_backward(grad.to(gpu_device), x_g.contiguous(), w.to(gpu_device), rstd_dense)
        assert torch.equal(dx.contiguous(), dx_dense)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("B,S,H,D", [(1, 1001, 24, 128), (2, 37, 6, 64), (1, 3, 1, 8), (2, 130, 5, 40), (1, 9, 2, 3072)])
def test_copy_rows_strided_into_the_value_slice(capi, gpu_device, dtype, B, S, H, D):
    """dv [B, H, S, D] into the v slice of the fused projection's gradient [B, S, H, 3D], bit for bit what
    Tensor.copy_ writes there, and nothing outside the slice."""
    gen = torch.Generator().manual_seed(B * 1000 + S)
    src = torch.randn(B, H, S, D, generator=gen).to(dtype).to(gpu_device)
    whole = torch.full((B, S, H, 3 * D), 7.0, dtype=dtype, device=gpu_device)
    want = whole.clone()
    want[..., 2 * D:].transpose(1, 2).copy_(src)
    got = capi.copy_rows_strided(whole[..., 2 * D:].transpose(1, 2), src)
    assert got.data_ptr() == whole[..., 2 * D:].data_ptr()
    assert torch.equal(whole, want)
    # a 3-D and a 2-D view, and no rows at all
    flat = torch.zeros(S * H, 2 * D, dtype=dtype, device=gpu_device)
    capi.copy_rows_strided(flat[:, D:], src[0].reshape(H * S, D).contiguous())
    assert torch.equal(flat[:, D:], src[0].reshape(H * S, D)) and not flat[:, :D].any()
    capi.copy_rows_strided(whole[:0, :, :, :D].transpose(1, 2), src[:0])


def test_copy_rows_strided_rejects_what_it_cannot_address(capi, gpu_device):
    L = capi.lib()
    buf = torch.zeros(64, 3 * 128 + 4, dtype=torch.bfloat16, device=gpu_device)
    src = torch.zeros(64, 128, dtype=torch.bfloat16, device=gpu_device)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    # row stride of 388 elements = 776 bytes: not a multiple of 16
    assert L.tt_norm_copy_rows_strided(p(buf), p(src), 1, 1, 64, 0, 0, 388, 128, capi.BF16, None) == 3
    # misaligned base, a row that is not whole 16-byte pieces, an unknown dtype
    ok = torch.zeros(64, 384, dtype=torch.bfloat16, device=gpu_device)
    assert L.tt_norm_copy_rows_strided(ctypes.c_void_p(ok.data_ptr() + 2), p(src), 1, 1, 64, 0, 0, 384, 128,
                                       capi.BF16, None) == 3
    assert L.tt_norm_copy_rows_strided(p(ok), p(src), 1, 1, 64, 0, 0, 384, 100, capi.BF16, None) == 2
    assert L.tt_norm_copy_rows_strided(p(ok), p(src), 1, 1, 64, 0, 0, 384, 128, 9, None) == 2
    assert not ok.any()
    with pytest.raises(ValueError):
        capi.copy_rows_strided(ok[:, :128], src.float())


# ------------------------------- rotary embedding fused behind the strided QK-norm

@pytest.mark.parametrize("B,S,H,n_rot", [(1, 1001, 24, 1001), (2, 37, 6, 20), (1, 5, 1, 0), (1, 300, 3, 299), (1, 4, 2, 3),
                                          (1, 50, 7, 50), (2, 4001, 10, 3999), (3, 2049, 12, 2049)])
def test_rmsnorm_rope_strided_vs_eager(capi, gpu_device, B, S, H, n_rot):
    """q_layernorm / k_layernorm on the transposed views, then apply_rotary_emb on the first n_rot tokens
    (dit_attention.py:266-273, :435-443), as one kernel each way, against the eager sequence."""
    D = 128
    q_cpu, k_cpu, q_g, k_g = _qkv_views(B, S, H, D, torch.bfloat16, 15, gpu_device)
    gen = torch.Generator().manual_seed(16)
    w = (1 + 0.02 * torch.randn(D, generator=gen)).bfloat16()
    grad = torch.randn(B, H, S, D, generator=gen).bfloat16()
    cos, sin = O.make_rope_tables(n_rot, D, seed=S)
    cos_g, sin_g = cos.to(gpu_device), sin.to(gpu_device)
    for x_cpu, x_g in ((q_cpu, q_g), (k_cpu, k_g)):
        want_out, want_dx, want_dw = O.eager_qk_norm_rope_fwd_bwd(x_cpu, w, cos, sin, grad)
        y = O.eager_rmsnorm(x_cpu, w)
        out, rstd = capi.rmsnorm_rope_forward_strided(x_g, w.to(gpu_device), cos_g, sin_g, EPS)
        assert out.is_contiguous() and out.shape == (B, H, S, D)
        assert_fwd_bf16(out, want_out, O.rope_excuse(y, want_out), "out")
        # tokens past the table: exactly the plain strided norm; same statistics everywhere
        plain, rstd_plain = capi.rmsnorm_forward_strided(x_g, w.to(gpu_device), EPS)
        assert torch.equal(out[:, :, n_rot:], plain[:, :, n_rot:]) and torch.equal(rstd, rstd_plain)
        dx, dw = capi.rmsnorm_rope_backward_strided(grad.to(gpu_device), x_g, w.to(gpu_device), rstd, cos_g, sin_g)
        assert dx.shape == x_g.shape
        assert_grad_bf16(dx, want_dx, "dx", allow=1e-5)
        assert_grad_bf16(dw, want_dw, "dweight")
        # the fused backward equals "rotate the gradient back, then the plain backward", bit for bit
        gy = grad.clone().requires_grad_(False)
        yl = y.detach().clone().requires_grad_(True)
        O.eager_qk_norm_rope(x_cpu, w, cos, sin)  # (shape check of the oracle path)
        rot = (O.apply_rotary_emb_real(yl[:, :, :n_rot], cos, sin) if n_rot else yl[:, :, :0])
        torch.cat([rot, yl[:, :, n_rot:]], dim=2).backward(gy)
        dx2, dw2 = capi.rmsnorm_backward_strided(yl.grad.contiguous().to(gpu_device), x_g, w.to(gpu_device), rstd_plain)
        assert torch.equal(dx, dx2) and torch.equal(dw, dw2)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("B,S,H,n_rot", [(1, 1001, 24, 1001), (2, 131, 5, 100)])
def test_rmsnorm_strided_and_rope_in_fp16_and_fp32(capi, gpu_device, dtype, B, S, H, n_rot):
    """The other element types through the strided and the rotary kernels at head dimension 128 (two rows
    per wavefront in fp32): identities that hold bit for bit whatever the type, and the truth in float64."""
    D = 128
    q_cpu, _, q_g, _ = _qkv_views(B, S, H, D, dtype, 25, gpu_device)
    gen = torch.Generator().manual_seed(26)
    w = (1 + 0.02 * torch.randn(D, generator=gen)).to(dtype)
    grad = torch.randn(B, H, S, D, generator=gen).to(dtype)
    cos, sin = O.make_rope_tables(n_rot, D, seed=S)
    w_g, grad_g, cos_g, sin_g = w.to(gpu_device), grad.to(gpu_device), cos.to(gpu_device), sin.to(gpu_device)
    # plain strided norm == dense norm on a materialised copy, forward and backward
    out, rstd = capi.rmsnorm_forward_strided(q_g, w_g, EPS)
    out_dense, rstd_dense = capi.rmsnorm_forward(q_g.contiguous(), w_g, EPS)
    assert torch.equal(out, out_dense) and torch.equal(rstd, rstd_dense)
    dx, dw = capi.rmsnorm_backward_strided(grad_g, q_g, w_g, rstd)
    dx_dense, dw_dense = capi.rmsnorm_backward(grad_g, q_g.contiguous(), w_g, rstd_dense)
    assert torch.equal(dx.contiguous(), dx_dense)
    torch.testing.assert_close(dw.float(), dw_dense.float(), rtol=2e-3 if dtype == torch.float16 else 1e-5, atol=1e-3)
    # rotary form: rows past the table are the plain norm; the backward equals "gradient rotated back by
    # autograd on the host, then the plain strided backward"
    out_r, rstd_r = capi.rmsnorm_rope_forward_strided(q_g, w_g, cos_g, sin_g, EPS)
    assert torch.equal(out_r[:, :, n_rot:], out[:, :, n_rot:]) and torch.equal(rstd_r, rstd)
    dx_r, dw_r = capi.rmsnorm_rope_backward_strided(grad_g, q_g, w_g, rstd, cos_g, sin_g)
    yl = out.cpu().requires_grad_(True)
    torch.cat([O.apply_rotary_emb_real(yl[:, :, :n_rot], cos, sin), yl[:, :, n_rot:]], dim=2).backward(grad)
    dx2, dw2 = capi.rmsnorm_backward_strided(yl.grad.contiguous().to(gpu_device), q_g, w_g, rstd)
    assert torch.equal(dx_r, dx2) and torch.equal(dw_r, dw2)
    # against the float64 truth: one rounding of the result in fp32, the element type's grid in fp16
    t_out, t_dx, t_dw = O.truth_qk_norm_rope_fwd_bwd(q_cpu, w, cos, sin, grad)
    tol = dict(rtol=4e-3, atol=4e-3) if dtype == torch.float16 else dict(rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(out_r.cpu().double(), t_out, **tol)
    torch.testing.assert_close(dx_r.cpu().double(), t_dx, **tol)
    rows = B * H * S
    torch.testing.assert_close(dw_r.cpu().double(), t_dw, rtol=0, atol=(4e-3 if dtype == torch.float16 else 1e-5) * rows ** 0.5)


def test_rmsnorm_rope_rejects_other_head_dims_and_bad_tables(capi, gpu_device):
    x = torch.zeros(1, 2, 8, 3072, dtype=torch.bfloat16, device=gpu_device)
    w = torch.ones(3072, dtype=torch.bfloat16, device=gpu_device)
    t = torch.zeros(8, 3072, device=gpu_device)
    with pytest.raises(capi.NormError) as e:
        capi.rmsnorm_rope_forward_strided(x, w, t, t, EPS)
    assert e.value.status == 2                       # head dimension 128 only
    x = torch.zeros(1, 2, 8, 128, dtype=torch.bfloat16, device=gpu_device)
    w = torch.ones(128, dtype=torch.bfloat16, device=gpu_device)
    t = torch.zeros(9, 128, device=gpu_device)       # more table rows than tokens
    with pytest.raises(capi.NormError) as e:
        capi.rmsnorm_rope_forward_strided(x, w, t, t, EPS)
    assert e.value.status == 1


def test_rmsnorm_strided_3072_transposed_and_fp32(capi, gpu_device):
    """[S, B, C] activations viewed as [B, S, C] (the blocks transpose between the two layouts)."""
    S, B, C = 301, 2, 3072
    for dtype in (torch.bfloat16, torch.float32):
        d = O.make_rmsnorm_inputs((S, B), C, dtype, seed=9)
        xv_cpu = d["x"].transpose(0, 1)
        gv = d["grad"].transpose(0, 1).contiguous()
        want_out, want_dx, want_dw = O.eager_rmsnorm_fwd_bwd(xv_cpu, d["weight"], gv)
        x_g = d["x"].to(gpu_device).transpose(0, 1)
        w_g = d["weight"].to(gpu_device)
        out, rstd = capi.rmsnorm_forward_strided(x_g, w_g, EPS)
        dx, dw = capi.rmsnorm_backward_strided(gv.to(gpu_device), x_g, w_g, rstd)
        if dtype == torch.bfloat16:
            assert_fwd_bf16(out, want_out, None, "out")
            assert_grad_bf16(dx, want_dx, "dx")
            assert_grad_bf16(dw, want_dw, "dweight")
        else:
            torch.testing.assert_close(out.cpu(), want_out, rtol=1e-5, atol=1e-6)
            torch.testing.assert_close(dx.cpu(), want_dx, rtol=1e-4, atol=1e-5)


def test_rmsnorm_strided_rejects_unaligned_strides(capi, gpu_device):
    base = torch.zeros(4, 10, 132, dtype=torch.bfloat16, device=gpu_device)
    view = base[:, :, :128]                      # row stride 132 elements = 264 bytes: not 16-byte aligned
    w = torch.ones(128, dtype=torch.bfloat16, device=gpu_device)
    with pytest.raises(capi.NormError) as e:
        capi.rmsnorm_forward_strided(view, w, EPS)
    assert e.value.status == 3


@pytest.mark.parametrize("dtype,code", [(torch.float16, 2), (torch.bfloat16, 0), (torch.float32, 1)])
def test_strided_entry_points_reject_strides_that_are_not_16_bytes(capi, gpu_device, dtype, code):
    """The header promises TT_NORM_EALIGN for strides that are not multiples of 16 bytes, for every
    element type; checked on the C ABI itself (the Python wrapper has a check of its own in front).
    The rejection happens on the host: no kernel runs."""
    L = capi.lib()
    D, esz = 128, torch.empty(0, dtype=dtype).element_size()
    half = 8 // esz                                  # elements in 8 bytes: aligned to 8 bytes, not to 16
    n0, n1, n2 = 2, 3, 5
    x = torch.zeros(n0 * n1 * n2 * (D + half) + 64, dtype=dtype, device=gpu_device)
    out = torch.zeros(n0 * n1 * n2 * D, dtype=dtype, device=gpu_device)
    w = torch.ones(D, dtype=dtype, device=gpu_device)
    rstd = torch.zeros(n0 * n1 * n2, dtype=torch.float32, device=gpu_device)
    dw = torch.zeros(D, dtype=dtype, device=gpu_device)
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device=gpu_device)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    bad = D + half                                   # row stride of D elements + 8 bytes
    st = L.tt_rmsnorm_forward_strided(p(out), p(rstd), p(x), p(w), n0, n1, n2, n1 * n2 * bad, n2 * bad, bad, D,
                                      EPS, code, None)
    assert st == 3, (st, L.tt_norm_last_error())
    for xs2, ds2 in ((bad, D), (D, bad)):            # the check covers x's strides and dx's strides
        st = L.tt_rmsnorm_backward_strided(p(out), p(dw), p(out), p(x), p(w), p(rstd), n0, n1, n2,
                                           n1 * n2 * xs2, n2 * xs2, xs2, n1 * n2 * ds2, n2 * ds2, ds2, D, code,
                                           p(ws), ws.numel(), None)
        assert st == 3, (st, L.tt_norm_last_error())
    torch.cuda.synchronize()


def test_profile_hook_brackets_the_row_kernel(capi, gpu_device):
    """tt_norm_profile_next_row_kernel: one shot, records on the launch stream around the row kernel."""
    hip = ctypes.CDLL("libamdhip64.so")
    ev = [ctypes.c_void_p() for _ in range(2)]
    for e in ev:
        assert hip.hipEventCreate(ctypes.byref(e)) == 0
    L = capi.lib()
    assert L.tt_norm_profile_next_row_kernel(ev[0], None) == 1          # both or neither
    d = dev(O.make_rmsnorm_inputs((20000,), 3072, torch.bfloat16, seed=2), gpu_device)
    out, rstd = capi.rmsnorm_forward(d["x"], d["weight"], EPS)
    assert L.tt_norm_profile_next_row_kernel(ev[0], ev[1]) == 0
    dx, dw = capi.rmsnorm_backward(d["grad"], d["x"], d["weight"], rstd)
    torch.cuda.synchronize()
    ms = ctypes.c_float()
    assert hip.hipEventElapsedTime(ctypes.byref(ms), ev[0], ev[1]) == 0
    assert 0.01 < ms.value < 5.0                                         # 20 000 rows: tens of microseconds
    # disarmed after one use: a second call must not re-record (elapsed time unchanged)
    capi.rmsnorm_backward(d["grad"], d["x"], d["weight"], rstd)
    torch.cuda.synchronize()
    ms2 = ctypes.c_float()
    assert hip.hipEventElapsedTime(ctypes.byref(ms2), ev[0], ev[1]) == 0 and ms2.value == ms.value
    for e in ev:
        hip.hipEventDestroy(e)


def test_rows_past_two_to_the_31_elements(capi, gpu_device):
    """700 000 x 3072 = 2.15e9 elements per tensor: row offsets need 64 bits (the reference kernels index
    with a 32-bit row*cols, adaln_backward.cu:78).  The first and the last rows are checked against eager."""
    rows, C = 700_000, 3072
    assert rows * C > 2 ** 31
    gen = torch.Generator(device=gpu_device).manual_seed(5)
    x = torch.empty(1, rows, C, device=gpu_device, dtype=torch.bfloat16)
    grad = torch.empty_like(x)
    for lo in range(0, rows, 100_000):     # filled in slices: no 8.6 GB fp32 temporary
        n = min(100_000, rows - lo)
        x[0, lo:lo + n] = torch.randn(n, C, device=gpu_device, generator=gen).bfloat16()
        grad[0, lo:lo + n] = torch.randn(n, C, device=gpu_device, generator=gen).bfloat16()
    scale = (0.1 * torch.randn(1, C, device=gpu_device, generator=gen)).bfloat16()
    shift = (0.1 * torch.randn(1, C, device=gpu_device, generator=gen)).bfloat16()
    w = (1 + 0.02 * torch.randn(C, device=gpu_device, generator=gen)).bfloat16()
    idx = torch.cat([torch.arange(0, 8), torch.arange(rows - 8, rows)]).to(gpu_device)
    xs, gs = x[:, idx].cpu(), grad[:, idx].cpu()
    out, mean, rstd = capi.adaln_forward(x, scale, shift, EPS)
    want_out, want_dx, _, _ = O.eager_adaln_fwd_bwd(xs, scale.cpu(), shift.cpu(), gs)
    assert_fwd_bf16(out[:, idx], want_out, O.adaln_excuse(xs, scale.cpu(), shift.cpu(), want_out), "adaln out")
    dx, ds, dh = capi.adaln_backward(grad, x, scale, mean, rstd)
    del out
    assert_grad_bf16(dx[:, idx], want_dx, "adaln dx", allow=1e-4)
    want_dh = torch.zeros(C, device=gpu_device)
    for lo in range(0, rows, 100_000):
        want_dh += grad[0, lo:lo + 100_000].float().sum(0)
    assert O.frac_outside(dh.cpu(), want_dh.cpu().reshape(1, C), 1e-2, 1e-2) == 0.0
    del dx
    out, rstd = capi.rmsnorm_forward(x[0], w, EPS)
    want_out, want_dx, _ = O.eager_rmsnorm_fwd_bwd(xs[0], w.cpu(), gs[0])
    assert_fwd_bf16(out[idx], want_out, None, "rms out")
    dx, dw = capi.rmsnorm_backward(grad[0], x[0], w, rstd)
    assert_grad_bf16(dx[idx], want_dx, "rms dx")
    # dweight against an independent fp32 reduction of rnd(g * rnd(x * rstd)) in torch, slice by slice
    want_dw = torch.zeros(C, device=gpu_device)
    for lo in range(0, rows, 50_000):
        xs_, gs_, rs_ = x[0, lo:lo + 50_000].float(), grad[0, lo:lo + 50_000], rstd[lo:lo + 50_000]
        y = (xs_ * rs_[:, None]).bfloat16()
        want_dw += (gs_ * y).float().sum(0)
    assert O.frac_outside(dw.cpu(), want_dw.cpu(), 1e-2, 1e-2) == 0.0
