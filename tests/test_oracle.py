"""Pins the CPU oracle: every check here would fail for a plausible mistake
(dropped eps, sum instead of mean, unbiased variance, scale instead of 1+scale,
shift sign, scale/shift applied to the wrong sample, a missing rounding point).
None of them re-types the oracle's own formula."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import c_oracle as Cc
from oracle import norm_oracle as O
from tests.golden_util import load_golden

EPS = 1e-6


# ------------------------------------------------------------------ RMSNorm

@pytest.mark.parametrize("cols", [128, 3072])
def test_rmsnorm_matches_library_rms_norm(cols):
    d = O.make_rmsnorm_inputs((64,), cols, torch.float32, seed=3)
    got = O.eager_rmsnorm(d["x"], d["weight"], EPS)
    want = F.rms_norm(d["x"], (cols,), d["weight"], EPS)
    torch.testing.assert_close(got, want, rtol=2e-6, atol=1e-7)
    db = O.make_rmsnorm_inputs((64,), cols, torch.bfloat16, seed=3)
    gotb = O.eager_rmsnorm(db["x"], db["weight"], EPS)
    wantb = F.rms_norm(db["x"].float(), (cols,), db["weight"].float(), EPS)
    # eager rounds twice (y, then y*w): at most one bf16 ulp from the single-rounded value
    assert O.compare_bf16_ulp(gotb, wantb.bfloat16()).n_gt1 == 0


def test_rmsnorm_constant_row_closed_form():
    cols = 128
    for c in (0.5, -3.0, 1e-3, 0.0):
        x = torch.full((1, cols), c)
        w = torch.linspace(0.5, 1.5, cols)
        want = w * (c / math.sqrt(c * c + EPS))
        torch.testing.assert_close(O.eager_rmsnorm(x, w, EPS)[0], want, rtol=1e-6, atol=1e-12)


def test_rmsnorm_unit_weight_mean_square():
    x = 3.0 * torch.randn(16, 3072, generator=torch.Generator().manual_seed(1))
    out = O.eager_rmsnorm(x, torch.ones(3072), EPS).double()
    ms = (x.double() ** 2).mean(-1)
    torch.testing.assert_close((out ** 2).mean(-1), ms / (ms + EPS), rtol=1e-5, atol=0)


def test_rmsnorm_eps_matters_and_scale_invariance():
    x = torch.randn(8, 128, generator=torch.Generator().manual_seed(2))
    w = torch.ones(128)
    # eps -> 0: f(a x) = f(x)
    torch.testing.assert_close(O.eager_rmsnorm(7.0 * x, w, 0.0), O.eager_rmsnorm(x, w, 0.0),
                               rtol=1e-6, atol=1e-7)
    # tiny rows: eps dominates, out ~= x / sqrt(eps)
    tiny = 1e-6 * x
    torch.testing.assert_close(O.eager_rmsnorm(tiny, w, EPS),
                               tiny / torch.sqrt((tiny ** 2).mean(-1, keepdim=True) + EPS),
                               rtol=1e-5, atol=0)
    assert (O.eager_rmsnorm(tiny, w, EPS).abs() < 0.01).all()


def _brute_rmsnorm(x, w, g, eps):
    """float64 python loops straight from the definitions; d/dx by the quotient rule."""
    N, C = x.shape
    out = [[0.0] * C for _ in range(N)]
    dx = [[0.0] * C for _ in range(N)]
    dw = [0.0] * C
    for n in range(N):
        ms = sum(float(v) ** 2 for v in x[n]) / C
        r = 1.0 / math.sqrt(ms + eps)
        for c in range(C):
            out[n][c] = float(x[n, c]) * r * float(w[c])
            dw[c] += float(g[n, c]) * float(x[n, c]) * r
        # d out[n,k] / d x[n,c] = w_k * (delta_kc * r - x_k * x_c * r^3 / C)
        for c in range(C):
            s = 0.0
            for k in range(C):
                j = float(w[k]) * ((r if k == c else 0.0) - float(x[n, k]) * float(x[n, c]) * r ** 3 / C)
                s += float(g[n, k]) * j
            dx[n][c] = s
    return (torch.tensor(out, dtype=torch.float64), torch.tensor(dx, dtype=torch.float64),
            torch.tensor(dw, dtype=torch.float64))


def test_rmsnorm_truth_vs_bruteforce_and_autograd():
    gen = torch.Generator().manual_seed(5)
    x = torch.randn(3, 16, generator=gen, dtype=torch.float64)
    w = 1 + 0.1 * torch.randn(16, generator=gen, dtype=torch.float64)
    g = torch.randn(3, 16, generator=gen, dtype=torch.float64)
    bo, bdx, bdw = _brute_rmsnorm(x, w, g, EPS)
    to, tdx, tdw = O.truth_rmsnorm_fwd_bwd(x, w, g, EPS)
    for a, b in ((bo, to), (bdx, tdx), (bdw, tdw)):
        torch.testing.assert_close(a.double(), b, rtol=1e-12, atol=1e-13)
    eo, edx, edw = O.eager_rmsnorm_fwd_bwd(x, w, g, EPS)  # float64 in, so .float() is the only loss
    for a, b in ((eo, to), (edx, tdx), (edw, tdw)):
        torch.testing.assert_close(a.double(), b, rtol=1e-5, atol=1e-6)


def test_rmsnorm_gradcheck_on_eager_formula():
    gen = torch.Generator().manual_seed(6)
    x = torch.randn(2, 8, generator=gen, dtype=torch.float64, requires_grad=True)
    w = (1 + 0.1 * torch.randn(8, generator=gen, dtype=torch.float64)).requires_grad_(True)

    def f(x, w):  # the eager formula without the .float() down-cast
        return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + EPS)) * w
    assert torch.autograd.gradcheck(f, (x, w), eps=1e-6, atol=1e-6)
    # and the analytic float64 form agrees with autograd of that same formula
    g = torch.randn(2, 8, generator=gen, dtype=torch.float64)
    f(x, w).backward(g)
    _, tdx, tdw = O.truth_rmsnorm_fwd_bwd(x.detach(), w.detach(), g, EPS)
    torch.testing.assert_close(x.grad, tdx, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(w.grad, tdw, rtol=1e-10, atol=1e-12)


def test_rmsnorm_backward_invariants():
    d = O.make_rmsnorm_inputs((32,), 3072, torch.float32, seed=7)
    _, dx, dw = O.eager_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"], eps=0.0)
    # with eps = 0 the output is invariant to scaling a row, so x . dx = 0 per row
    dots = (d["x"].double() * dx.double()).sum(-1)
    scale = (d["x"].double().abs() * dx.double().abs()).sum(-1)
    assert (dots.abs() / scale).max() < 1e-5
    # g = 1  =>  dw = column sums of the normalised rows
    ones = torch.ones_like(d["x"])
    out1, _, dw1 = O.eager_rmsnorm_fwd_bwd(d["x"], torch.ones(3072), ones)
    torch.testing.assert_close(dw1, out1.sum(0), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("cols,rows", [(128, 2048), (3072, 96)])
def test_rmsnorm_staged_and_c_agree_with_eager_bf16(cols, rows):
    d = O.make_rmsnorm_inputs((rows,), cols, torch.bfloat16, seed=8)
    out, dx, dw = O.eager_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
    so, sr = O.staged_rmsnorm_fwd(d["x"], d["weight"])
    assert torch.equal(so.view(torch.int16), out.view(torch.int16))       # rounding points are right
    co, cr = Cc.rmsnorm_fwd(d["x"], d["weight"], EPS)
    rep = O.compare_bf16_ulp(co, out)
    assert rep.n_gt1 == 0 and rep.frac_exact > 0.999                       # only summation order differs
    torch.testing.assert_close(cr, sr, rtol=3e-7, atol=0)
    # dropping the intermediate rounding of y would show up here as ~20 % one-ulp differences
    single = (d["x"].float() * sr[:, None] * d["weight"].float()).bfloat16()
    assert O.compare_bf16_ulp(single, out).frac_exact < 0.9
    cdx, cdw = Cc.rmsnorm_bwd(d["x"], d["weight"], cr, d["grad"])
    sdx, sdw = O.staged_rmsnorm_bwd(d["x"], d["weight"], sr, d["grad"])
    for got in (cdx, sdx):
        rep = O.compare_bf16_ulp(got, dx)
        assert rep.frac_exact > 0.999 and O.frac_outside(got, dx, 1e-2, 1e-3) == 0.0
    for got in (cdw, sdw):
        assert O.frac_outside(got, dw, 1e-2, 1e-3) == 0.0
        assert O.compare_bf16_ulp(got, dw).max_ulp <= 2


def test_rmsnorm_c_f32_matches_eager():
    d = O.make_rmsnorm_inputs((64,), 3072, torch.float32, seed=9)
    out, dx, dw = O.eager_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
    co, cr = Cc.rmsnorm_fwd(d["x"], d["weight"], EPS)
    cdx, cdw = Cc.rmsnorm_bwd(d["x"], d["weight"], cr, d["grad"])
    torch.testing.assert_close(co, out, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(cdx, dx, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(cdw, dw, rtol=1e-5, atol=1e-5)


# -------------------------------------------------------------------- AdaLN

def test_adaln_matches_library_layer_norm_affine():
    d = O.make_adaln_inputs(1, 40, 3072, torch.float32, seed=21)
    got = O.eager_adaln(d["x"], d["scale"], d["shift"], EPS)
    want = F.layer_norm(d["x"], (3072,), 1 + d["scale"][0], d["shift"][0], EPS)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)


def test_adaln_zero_modulation_moments_and_affine_invariance():
    gen = torch.Generator().manual_seed(22)
    x = 2.5 * torch.randn(2, 6, 3072, generator=gen) + 1.0
    z = torch.zeros(2, 3072)
    out = O.eager_adaln(x, z, z, EPS).double()
    var = x.double().var(-1, unbiased=False)
    assert out.mean(-1).abs().max() < 1e-6
    torch.testing.assert_close(out.var(-1, unbiased=False), var / (var + EPS), rtol=1e-5, atol=0)
    # the unbiased estimator would differ by C/(C-1) ~ 3e-4: make sure the check can see that
    assert ((out.var(-1, unbiased=True) - var / (var + EPS)).abs() > 1e-4).all()
    # LN(a x + b) = LN(x) for a > 0 (eps negligible against var)
    torch.testing.assert_close(O.eager_adaln(3.0 * x + 5.0, z, z, 0.0), O.eager_adaln(x, z, z, 0.0),
                               rtol=1e-4, atol=1e-5)


def test_adaln_per_sample_modulation_bruteforce():
    d = O.make_adaln_inputs(3, 5, 3072, torch.float32, seed=23)
    got = O.eager_adaln(d["x"], d["scale"], d["shift"], EPS)
    for b in range(3):
        xb = d["x"][b].double()
        mu = xb.mean(-1, keepdim=True)
        sd = torch.sqrt(((xb - mu) ** 2).mean(-1, keepdim=True) + EPS)
        want = (xb - mu) / sd * (1 + d["scale"][b].double()) + d["shift"][b].double()
        torch.testing.assert_close(got[b].double(), want, rtol=1e-5, atol=1e-5)
    # a sample swapped with its neighbour must be detectable
    swapped = O.eager_adaln(d["x"], d["scale"].flip(0), d["shift"].flip(0), EPS)
    assert (swapped[0] - got[0]).abs().max() > 0.05


def test_adaln_truth_vs_autograd_fp64_and_invariants():
    gen = torch.Generator().manual_seed(24)
    B, S, C = 2, 3, 24
    x = torch.randn(B, S, C, generator=gen, dtype=torch.float64, requires_grad=True)
    sc = (0.1 * torch.randn(B, C, generator=gen, dtype=torch.float64)).requires_grad_(True)
    sh = (0.1 * torch.randn(B, C, generator=gen, dtype=torch.float64)).requires_grad_(True)
    g = torch.randn(B, S, C, generator=gen, dtype=torch.float64)
    assert torch.autograd.gradcheck(lambda a, b, c: O.eager_adaln(a, b, c, EPS), (x, sc, sh),
                                    eps=1e-6, atol=1e-6)
    out = O.eager_adaln(x, sc, sh, EPS)
    out.backward(g)
    to, tdx, tds, tdh = O.truth_adaln_fwd_bwd(x.detach(), sc.detach(), sh.detach(), g, EPS)
    torch.testing.assert_close(out.detach(), to, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(x.grad, tdx, rtol=1e-9, atol=1e-11)
    torch.testing.assert_close(sc.grad, tds, rtol=1e-9, atol=1e-11)
    torch.testing.assert_close(sh.grad, tdh, rtol=1e-9, atol=1e-11)
    # LayerNorm's backward is orthogonal to the all-ones vector and to xhat
    xd = x.detach()
    mu = xd.mean(-1, keepdim=True)
    xhat = (xd - mu) / torch.sqrt(((xd - mu) ** 2).mean(-1, keepdim=True) + EPS)
    assert tdx.sum(-1).abs().max() < 1e-10
    # exact only for eps = 0; with eps = 1e-6 and unit variance the residue is O(eps)
    assert (tdx * xhat).sum(-1).abs().max() < 1e-4


def test_adaln_staged_and_c_agree_with_eager_bf16():
    d = O.make_adaln_inputs(3, 70, 3072, torch.bfloat16, seed=25)
    out, dx, ds, dh = O.eager_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], d["grad"])
    so, smu, sr = O.staged_adaln_fwd(d["x"], d["scale"], d["shift"])
    co, cmu, cr = Cc.adaln_fwd(d["x"], d["scale"], d["shift"], EPS)
    excuse = O.adaln_excuse(d["x"], d["scale"], d["shift"], out)
    for got, mu, r in ((so, smu, sr), (co, cmu, cr)):
        rep = O.compare_bf16_ulp(got, out, excuse_abs=excuse)
        assert rep.n_gt1 == 0 and rep.n_excused < 1e-4 * rep.n and rep.frac_exact > 0.999, rep
    torch.testing.assert_close(cr, sr.reshape(-1), rtol=1e-6, atol=0)
    torch.testing.assert_close(cmu, smu.reshape(-1), rtol=0, atol=1e-6)
    # a single final rounding (no intermediate bf16 steps) is visibly different from eager
    single = ((d["x"].float() - smu.view(3, 70, 1)) * sr.view(3, 70, 1) * (1 + d["scale"].float()[:, None])
              + d["shift"].float()[:, None]).bfloat16()
    assert O.compare_bf16_ulp(single, out).frac_exact < 0.95
    cdx, cds, cdh = Cc.adaln_bwd(d["x"], d["scale"], cmu, cr, d["grad"])
    sdx, sds, sdh = O.staged_adaln_bwd(d["x"], d["scale"], smu, sr, d["grad"])
    for gdx, gds, gdh in ((cdx, cds, cdh), (sdx, sds, sdh)):
        assert O.frac_outside(gdx, dx, 1e-2, 1e-3) < 1e-5
        assert O.frac_outside(gds, ds, 1e-2, 1e-3) == 0.0
        assert O.frac_outside(gdh, dh, 1e-2, 1e-3) == 0.0
    # and against the float64 truth (bf16 rounding noise only)
    _, tdx, tds, tdh = O.truth_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], d["grad"], EPS)
    assert O.frac_outside(cdx, tdx, 2e-2, 2e-2) < 1e-4


def test_adaln_c_f32_matches_eager():
    d = O.make_adaln_inputs(2, 9, 3072, torch.float32, seed=26)
    out, dx, ds, dh = O.eager_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], d["grad"])
    co, cmu, cr = Cc.adaln_fwd(d["x"], d["scale"], d["shift"], EPS)
    cdx, cds, cdh = Cc.adaln_bwd(d["x"], d["scale"], cmu, cr, d["grad"])
    torch.testing.assert_close(co, out, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(cdx, dx, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(cds, ds, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(cdh, dh, rtol=1e-5, atol=1e-5)


# ------------------------------------------------------------ golden vectors

# ----------------------------------------------------- gated residual + AdaLN

def test_gated_bruteforce_loops_fp64():
    """Scalar loops over a tiny case: catches gate applied to h instead of attn, gate of the wrong
    sample, the norm taken of h instead of h2, a gradient of h2 that misses either of its two uses."""
    gen = torch.Generator().manual_seed(31)
    B, S, C = 2, 3, 8
    h, a, go, g2 = (torch.randn(B, S, C, generator=gen, dtype=torch.float64) for _ in range(4))
    q, sc, sh = (0.5 * torch.randn(B, C, generator=gen, dtype=torch.float64) for _ in range(3))
    h2, out, dh, da, dq, dsc, dsh = O.eager_gated_residual_adaln_fwd_bwd(h, a, q, sc, sh, go, g2, EPS)
    for b in range(B):
        dq_want = [0.0] * C
        for s in range(S):
            row = [float(h[b, s, c]) + float(a[b, s, c]) * float(q[b, c]) for c in range(C)]
            mu = sum(row) / C
            var = sum((v - mu) ** 2 for v in row) / C
            r = 1.0 / math.sqrt(var + EPS)
            xhat = [(v - mu) * r for v in row]
            gx = [float(go[b, s, c]) * (1.0 + float(sc[b, c])) for c in range(C)]
            m1 = sum(gx) / C
            m2 = sum(gx[c] * xhat[c] for c in range(C)) / C
            for c in range(C):
                assert abs(float(h2[b, s, c]) - row[c]) < 1e-12
                want = xhat[c] * (1.0 + float(sc[b, c])) + float(sh[b, c])
                assert abs(float(out[b, s, c]) - want) < 1e-9
                dh_want = r * (gx[c] - m1 - xhat[c] * m2) + float(g2[b, s, c])
                assert abs(float(dh[b, s, c]) - dh_want) < 1e-9
                assert abs(float(da[b, s, c]) - dh_want * float(q[b, c])) < 1e-9
                dq_want[c] += dh_want * float(a[b, s, c])
        for c in range(C):
            assert abs(float(dq[b, c]) - dq_want[c]) < 1e-9
    # the float64 closed form agrees with autograd on every output
    truth = O.truth_gated_residual_adaln_fwd_bwd(h, a, q, sc, sh, go, g2, EPS)
    for got, want in zip((h2, out, dh, da, dq, dsc, dsh), truth):
        torch.testing.assert_close(got, want, rtol=1e-9, atol=1e-11)
    # without a gradient at h2, dh is the norm's dx alone
    no2 = O.eager_gated_residual_adaln_fwd_bwd(h, a, q, sc, sh, go, None, EPS)
    torch.testing.assert_close(no2[2] + g2, dh, rtol=1e-9, atol=1e-11)


def test_gated_gradcheck_and_special_cases():
    gen = torch.Generator().manual_seed(32)
    B, S, C = 2, 2, 12
    mk = lambda *shape: torch.randn(*shape, generator=gen, dtype=torch.float64)
    leaves = [mk(B, S, C), mk(B, S, C), 0.3 * mk(B, C), 0.3 * mk(B, C), 0.3 * mk(B, C)]
    for t in leaves:
        t.requires_grad_(True)
    assert torch.autograd.gradcheck(lambda *a: O.eager_gated_residual_adaln(*a, EPS), leaves, eps=1e-6, atol=1e-6)
    h, a, q, sc, sh = (t.detach() for t in leaves)
    # gate = 0: the residual stream passes through untouched and the op is the plain modulated norm
    h2, out = O.eager_gated_residual_adaln(h, a, torch.zeros_like(q), sc, sh, EPS)
    assert torch.equal(h2, h)
    torch.testing.assert_close(out, O.eager_adaln(h, sc, sh, EPS), rtol=0, atol=0)
    # gate = 1, attn = -h: h2 = 0, every row is constant, the norm returns shift
    h2, out = O.eager_gated_residual_adaln(h, -h, torch.ones_like(q), sc, sh, EPS)
    assert h2.abs().max() == 0
    torch.testing.assert_close(out, sh[:, None].expand_as(out), rtol=0, atol=1e-12)


def test_gated_staged_agrees_with_eager_bf16():
    h, a, q, sc, sh, go, g2 = O.make_gated_inputs(2, 48, 3072, torch.bfloat16, seed=33)
    eh2, eout, edh, eda, edq, edsc, edsh = O.eager_gated_residual_adaln_fwd_bwd(h, a, q, sc, sh, go, g2)
    sh2, sout, smu, sr = O.staged_gated_residual_adaln_fwd(h, a, q, sc, sh)
    assert torch.equal(sh2, eh2)  # two roundings, both fixed by the eager expression
    rep = O.compare_bf16_ulp(sout, eout, excuse_abs=O.adaln_excuse(eh2, sc, sh, eout))
    assert rep.n_gt1 == 0 and rep.n_excused < 1e-4 * rep.n and rep.frac_exact > 0.999, rep
    # dropping the rounding of attn*gate is visible in h2
    single = (h.float() + a.float() * q.float()[:, None]).bfloat16()
    assert (single != eh2).float().mean() > 0.02
    sdh, sda, sdq, sdsc, sdsh = O.staged_gated_residual_adaln_bwd(eh2, a, q, sc, smu, sr, go, g2)
    # dh sums two rounded terms: a one-ulp disagreement in the norm's dx survives a cancelling sum,
    # so its bound scales with the terms (|dh| + |grad_h2| >= |dx of the norm|)
    terms = edh.float().abs() + g2.float().abs()
    assert O.frac_outside(sdh, edh, 1e-2, 1e-3, magnitude=terms) < 1e-5
    assert O.frac_outside(sda, eda, 1e-2, 1e-3, magnitude=terms * q.float().abs()[:, None]) < 1e-5
    for got, want in ((sdsc, edsc), (sdsh, edsh)):
        assert O.frac_outside(got, want, 1e-2, 1e-3) == 0.0
    # dgate sums dh*attn, and dh is known to an ulp only: random-walk bound on the column
    assert O.colsum_outside(sdq, edq, terms * a.float(), dim=1) == 0
    # the scalar C restatement (explicit RNE, double accumulation) tells the same story
    ch2, cout, cmu, cr = Cc.gated_residual_adaln_fwd(h, a, q, sc, sh, EPS)
    assert torch.equal(ch2, eh2)
    rep = O.compare_bf16_ulp(cout, eout, excuse_abs=O.adaln_excuse(eh2, sc, sh, eout))
    assert rep.n_gt1 == 0 and rep.n_excused < 1e-4 * rep.n and rep.frac_exact > 0.999, rep
    for with_h2 in (True, False):
        want = (edh, eda, edq) if with_h2 else O.eager_gated_residual_adaln_fwd_bwd(h, a, q, sc, sh, go, None)[2:5]
        cdh, cda, cdq, cdsc, cdsh = Cc.gated_residual_adaln_bwd(eh2, a, q, sc, cmu, cr, go, g2 if with_h2 else None)
        t = want[0].float().abs() + (g2.float().abs() if with_h2 else 0)
        assert O.frac_outside(cdh, want[0], 1e-2, 1e-3, magnitude=t) < 1e-5
        assert O.frac_outside(cda, want[1], 1e-2, 1e-3, magnitude=t * q.float().abs()[:, None]) < 1e-5
        assert O.colsum_outside(cdq, want[2], t * a.float(), dim=1) == 0
        assert O.frac_outside(cdsc, edsc, 1e-2, 1e-3) == 0.0 and O.frac_outside(cdsh, edsh, 1e-2, 1e-3) == 0.0
    # and the float64 truth is within bf16 rounding noise of both
    truth = O.truth_gated_residual_adaln_fwd_bwd(h, a, q, sc, sh, go, g2)
    assert O.frac_outside(sdh, truth[2], 2e-2, 2e-2) < 1e-4
    assert O.colsum_outside(sdq, truth[4], terms * a.float(), dim=1) == 0


@pytest.mark.parametrize("cols", [64, 1000, 5120])
def test_staged_rounding_points_hold_for_fp16_and_other_widths(cols):
    """The rounding chain is a property of the element type, not of the width: fp16 rows of any
    width follow the same staged forms (the arithmetic itself is pinned above on bf16 / fp32 / fp64)."""
    d = O.make_rmsnorm_inputs((37,), cols, torch.float16, seed=60 + cols)
    out, dx, dw = O.eager_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
    so, sr = O.staged_rmsnorm_fwd(d["x"], d["weight"])
    rep = O.compare_bf16_ulp(so, out, excuse_abs=O.rmsnorm_excuse(out))
    assert rep.n_gt1 == 0 and rep.frac_exact > 0.999, rep
    sdx, sdw = O.staged_rmsnorm_bwd(d["x"], d["weight"], sr, d["grad"])
    assert O.frac_outside(sdx, dx, 1e-2, 1e-3) == 0.0 and O.frac_outside(sdw, dw, 1e-2, 1e-3) == 0.0
    a = O.make_adaln_inputs(3, 19, cols, torch.float16, seed=61 + cols)
    aout, adx, ads, adh = O.eager_adaln_fwd_bwd(a["x"], a["scale"], a["shift"], a["grad"])
    s_out, smu, s_r = O.staged_adaln_fwd(a["x"], a["scale"], a["shift"])
    rep = O.compare_bf16_ulp(s_out, aout, excuse_abs=O.adaln_excuse(a["x"], a["scale"], a["shift"], aout))
    assert rep.n_gt1 == 0 and rep.n_excused < 1e-3 * rep.n and rep.frac_exact > 0.99, rep
    tdx, tds, tdh = O.staged_adaln_bwd(a["x"], a["scale"], smu, s_r, a["grad"])
    assert O.frac_outside(tdx, adx, 1e-2, 1e-3) < 1e-4
    assert O.frac_outside(tds, ads, 1e-2, 1e-3) == 0.0 and O.frac_outside(tdh, adh, 1e-2, 1e-3) == 0.0
    # fp16 and bf16 round differently: the fp16 result is not what a bf16 chain would give
    assert not torch.equal(aout.bfloat16(), O.eager_adaln(a["x"].bfloat16(), a["scale"].bfloat16(), a["shift"].bfloat16()))


def test_golden_vectors_reproduce():
    gold = load_golden()
    assert len(gold) == 11
    for name, d in gold.items():
        if name.startswith("rms"):
            out, dx, dw = O.eager_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
            got = {"out": out, "dx": dx, "dweight": dw}
        elif name.startswith("adaln"):
            out, dx, ds, dh = O.eager_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], d["grad"])
            got = {"out": out, "dx": dx, "dscale": ds, "dshift": dh}
        else:
            res = O.eager_gated_residual_adaln_fwd_bwd(d["h"], d["attn"], d["gate"], d["scale"], d["shift"],
                                                       d["grad"], d["grad_h2"])
            got = dict(zip(("h2", "out", "dh", "dattn", "dgate", "dscale", "dshift"), res))
        for k, v in got.items():
            if d["is_16bit"]:
                # thread count may change a summation order: allow 1 ulp on a handful of elements
                rep = O.compare_bf16_ulp(v, d[k])
                assert rep.frac_exact > 0.995 and O.frac_outside(v, d[k], 1e-2, 1e-3) == 0.0, (name, k, rep)
            else:
                torch.testing.assert_close(v, d[k], rtol=1e-5, atol=1e-5)


def test_bf16_ulp_comparator():
    a = torch.tensor([1.0, 1.0, -1.0, 0.0, 2.0 ** -126]).bfloat16()
    b = torch.tensor([1.0078125, 1.015625, -1.0078125, -0.0, 0.0]).bfloat16()
    assert O.bf16_ulp_distance(a, b).tolist() == [1, 2, 1, 0, 128]


# ------------------------------------------------- rotary embedding (restated)
# apply_rotary_emb_real restates a third-party routine (diffusers 0.32.1, absent here).  What follows pins the
# restatement by what a rotation of adjacent pairs must satisfy; none of it re-types its formula.

def _angles(S, D, seed):
    g = torch.Generator().manual_seed(seed)
    th = (torch.rand(S, D // 2, generator=g, dtype=torch.float64) - 0.5) * 12.0
    rep = lambda t: t.repeat_interleave(2, dim=1)
    return th, rep(th.cos()).float(), rep(th.sin()).float()


def test_rotary_identity_at_angle_zero_is_bit_exact():
    x = torch.randn(2, 3, 5, 16, generator=torch.Generator().manual_seed(1))
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        xt = x.to(dtype)
        out = O.apply_rotary_emb_real(xt, torch.ones(5, 16), torch.zeros(5, 16))
        assert out.dtype == dtype and torch.equal(out, xt)


def test_rotary_is_a_complex_multiplication_per_pair_brute_force():
    B, H, S, D = 2, 2, 3, 8
    x = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(2), dtype=torch.float64)
    th, cos, sin = _angles(S, D, 3)
    got = O.apply_rotary_emb_real(x.float(), cos, sin).double()
    for b in range(B):
        for h in range(H):
            for s in range(S):
                for i in range(D // 2):
                    z = complex(x[b, h, s, 2 * i], x[b, h, s, 2 * i + 1]) * complex(math.cos(th[s, i]), math.sin(th[s, i]))
                    assert abs(got[b, h, s, 2 * i] - z.real) < 1e-5 and abs(got[b, h, s, 2 * i + 1] - z.imag) < 1e-5


def test_rotary_preserves_pair_norms_and_composes_angles():
    B, H, S, D = 1, 2, 7, 32
    x = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(4))
    th1, c1, s1 = _angles(S, D, 5)
    th2, c2, s2 = _angles(S, D, 6)
    y = O.apply_rotary_emb_real(x, c1, s1)
    pair = lambda t: t.reshape(B, H, S, D // 2, 2).pow(2).sum(-1)
    torch.testing.assert_close(pair(y), pair(x), rtol=1e-5, atol=1e-6)
    rep = lambda t: t.repeat_interleave(2, dim=1).float()
    both = O.apply_rotary_emb_real(x, rep((th1 + th2).cos()), rep((th1 + th2).sin()))
    torch.testing.assert_close(O.apply_rotary_emb_real(y, c2, s2), both, rtol=1e-4, atol=1e-5)
    # a quarter turn maps (a, b) to (-b, a): fixes the direction of rotation and which element is "real"
    q = O.apply_rotary_emb_real(x, torch.zeros(S, D), torch.ones(S, D))
    assert torch.equal(q[..., 0::2], -x[..., 1::2]) and torch.equal(q[..., 1::2], x[..., 0::2])


def test_rotary_other_conventions_are_visibly_different():
    B, H, S, D = 1, 1, 4, 16
    x = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(7))
    _, cos, sin = _angles(S, D, 8)
    want = O.apply_rotary_emb_real(x, cos, sin)
    a, b = x[..., 0::2], x[..., 1::2]
    clockwise = torch.stack([b, -a], dim=-1).flatten(3)                 # rotate_pairs with the sign on the other element
    assert (x * cos + clockwise * sin - want).abs().max() > 0.1
    h1, h2 = x[..., : D // 2], x[..., D // 2:]                          # halves instead of adjacent pairs (unbind dim -2)
    halves = torch.cat([-h2, h1], dim=-1)
    assert (x * cos + halves * sin - want).abs().max() > 0.1


def test_rotary_gradient_is_the_inverse_rotation():
    B, H, S, D = 1, 2, 3, 8
    th, cos, sin = _angles(S, D, 9)
    x = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(10)).requires_grad_(True)
    g = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(11))
    O.apply_rotary_emb_real(x, cos, sin).backward(g)
    rep = lambda t: t.repeat_interleave(2, dim=1).float()
    torch.testing.assert_close(x.grad, O.apply_rotary_emb_real(g, rep(th.cos()), rep((-th).sin())), rtol=1e-5, atol=1e-6)
    # (the map is linear in x, so its gradient is its transpose; for a rotation that is the inverse rotation.
    # gradcheck does not apply: the routine computes in float32 whatever the input type.)
    u = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(12))
    lhs = (O.apply_rotary_emb_real(u, cos, sin) * g).sum()
    rhs = (u * x.grad).sum()
    torch.testing.assert_close(lhs, rhs, rtol=1e-4, atol=1e-4)                  # <R u, g> = <u, R^T g>


def test_qk_norm_rope_composition_and_partial_rotation():
    B, H, S, D, n = 1, 3, 9, 128, 6
    d = O.make_rmsnorm_inputs((B, H, S), D, torch.bfloat16, seed=12)
    cos, sin = O.make_rope_tables(n, D, seed=1)
    assert cos.shape == (n, D) and torch.equal(cos[:, 0::2], cos[:, 1::2])          # one angle per pair
    torch.testing.assert_close(cos * cos + sin * sin, torch.ones(n, D), rtol=1e-6, atol=1e-6)
    out, dx, dw = O.eager_qk_norm_rope_fwd_bwd(d["x"], d["weight"], cos, sin, d["grad"])
    y = O.eager_rmsnorm(d["x"], d["weight"])
    assert torch.equal(out[:, :, n:], y[:, :, n:])                                   # text tokens: norm only
    assert torch.equal(out[:, :, :n], O.apply_rotary_emb_real(y[:, :, :n], cos, sin))
    t_out, t_dx, t_dw = O.truth_qk_norm_rope_fwd_bwd(d["x"], d["weight"], cos, sin, d["grad"])
    assert (out.double() - t_out).abs().max() < 0.05
    assert O.frac_outside(dx, t_dx.float(), 3e-2, 3e-2) == 0.0
    assert O.frac_outside(dw, t_dw.float(), 3e-2, 0.1) == 0.0
    # no rotation at all (n = 0 tokens) is the plain norm, gradient included
    o0, dx0, dw0 = O.eager_qk_norm_rope_fwd_bwd(d["x"], d["weight"], cos[:0], sin[:0], d["grad"])
    p0 = O.eager_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
    assert torch.equal(o0, p0[0]) and torch.equal(dx0, p0[1]) and torch.equal(dw0, p0[2])
