"""GPU parity at the benchmark configurations' full shapes, judged two ways at once:

  * against the eager oracle, to the bars of tests/test_gpu_parity.py (the excused / outside fractions
    that those bars allow are measured here and reported in the assertion messages);
  * against the float64 truth: for every output, the kernel's error to the truth must not exceed eager's
    own error to the truth by more than 5 % (max and RMS).  Where a bar against eager had to be widened
    (elements excused in the forward, a fraction of AdaLN dx, reduced gradients of the two-op chain,
    the gated op's gradients) this is what shows that the kernels are not the cause: they sit as close
    to the exact result as eager does.

Also here: rows with a large mean and with outlier channels through the AdaLN backward's one-pass row
sums (tuned and any-width kernels).

Set TT_PARITY_REPORT=<file> to have the measured fractions and error ratios written out as JSON.
"""
import json
import os

import pytest
import torch

from oracle import norm_oracle as O

pytestmark = pytest.mark.gpu
EPS = 1e-6
REPORT = {}


@pytest.fixture(scope="module")
def capi(gpu_device):
    from teletron_amd import capi as c
    c.lib()
    yield c
    path = os.environ.get("TT_PARITY_REPORT")
    if path:
        with open(path, "w") as f:
            json.dump(REPORT, f, indent=1, sort_keys=True)


def _err(t, truth):
    d = (t.detach().double().cpu().reshape(truth.shape) - truth).abs()
    return float(d.max()), float(d.pow(2).mean().sqrt())


def no_worse_than_eager(case, name, got, eager, truth, slack=1.05, slack_max=1.25):
    """RMS err(kernel, truth) <= slack * RMS err(eager, truth), and the same for the maximum with slack_max:
    the population statistic gets the tight factor; the maximum is decided by which way ONE element's last
    rounding fell (measured over every 16-bit case below: <= 1.02 except a single 1.17)."""
    kmax, krms = _err(got, truth)
    emax, erms = _err(eager, truth)
    REPORT.setdefault(case, {})[name] = {"kernel_max": kmax, "eager_max": emax, "kernel_rms": krms, "eager_rms": erms,
                                         "max_ratio": kmax / emax if emax else None,
                                         "rms_ratio": krms / erms if erms else None}
    msg = f"{case}/{name}: kernel max {kmax:.4g} rms {krms:.4g} vs eager max {emax:.4g} rms {erms:.4g}"
    assert krms <= slack * erms + 1e-30, msg
    assert kmax <= max(slack, slack_max) * emax + 1e-30, msg


def forward_bar(case, name, got, want, excuse):
    rep = O.compare_bf16_ulp(got.detach().cpu(), want, excuse_abs=excuse)
    REPORT.setdefault(case, {})[name + "_vs_eager"] = {"frac_exact": rep.frac_exact, "frac_excused": rep.n_excused / rep.n,
                                                       "n_gt1": rep.n_gt1}
    assert rep.n_gt1 == 0 and rep.n_excused <= 1e-4 * rep.n and rep.frac_exact >= 0.999, (case, name, rep)


def grad_bar(case, name, got, want, allow=0.0, magnitude=None):
    frac = O.frac_outside(got.detach().cpu(), want, 1e-2, 1e-3, magnitude=magnitude)
    REPORT.setdefault(case, {})[name + "_vs_eager"] = {"frac_outside": frac, "allowed": allow}
    assert frac <= allow, (case, name, frac)


def dev(d, device):
    return {k: v.to(device) for k, v in d.items()}


# ------------------------------------------------------------------ config 1

def test_cfg1_rmsnorm_fp32_full_shape(capi, gpu_device):
    """x [2, 4096, 3072] fp32: forward rel 1e-5; gradients rel 1e-4; and no further from the truth than eager."""
    _, d = O.make_config_inputs("cfg1_rms_fp32", seed=0)
    want_out, want_dx, want_dw = O.eager_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
    t_out, t_dx, t_dw = O.truth_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
    g = dev(d, gpu_device)
    out, rstd = capi.rmsnorm_forward(g["x"], g["weight"], EPS)
    dx, dw = capi.rmsnorm_backward(g["grad"], g["x"], g["weight"], rstd)
    torch.testing.assert_close(out.cpu(), want_out, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(dx.cpu(), want_dx, rtol=1e-4, atol=1e-5)
    l1 = (d["grad"].abs() * want_out.abs()).reshape(-1, 3072).sum(0)
    assert ((dw.cpu() - want_dw).abs() <= 1e-4 * l1 + 1e-5).all()
    # fp32: no bar against eager was widened; both sit a few fp32 ulps from the truth and differ in summation
    # order only (torch's CPU sum is pairwise, the kernels add rows in sequence per wavefront)
    no_worse_than_eager("cfg1", "out", out, want_out, t_out, slack=1.25)
    no_worse_than_eager("cfg1", "dx", dx, want_dx, t_dx, slack=1.25)
    no_worse_than_eager("cfg1", "dweight", dw, want_dw, t_dw, slack=1.25, slack_max=3.0)


# ------------------------------------------------------------------ config 2

@pytest.mark.parametrize("which,seed", [("q", 0), ("k", 1)])
def test_cfg2_qk_rmsnorm_full_shape(capi, gpu_device, which, seed):
    """q and k of one CP=4 rank: [1, 29700, 24, 128] bf16 each."""
    d = O.make_rmsnorm_inputs((1, 29700, 24), 128, torch.bfloat16, seed=seed)
    want_out, want_dx, want_dw = O.eager_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
    t_out, t_dx, t_dw = O.truth_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
    g = dev(d, gpu_device)
    out, rstd = capi.rmsnorm_forward(g["x"], g["weight"], EPS)
    dx, dw = capi.rmsnorm_backward(g["grad"], g["x"], g["weight"], rstd)
    case = "cfg2_" + which
    forward_bar(case, "out", out, want_out, O.rmsnorm_excuse(want_out))
    grad_bar(case, "dx", dx, want_dx)
    grad_bar(case, "dweight", dw, want_dw)
    no_worse_than_eager(case, "out", out, want_out, t_out)
    no_worse_than_eager(case, "dx", dx, want_dx, t_dx)
    no_worse_than_eager(case, "dweight", dw, want_dw, t_dw)


@pytest.mark.parametrize("n_rot", [29700, 29700 - 256])
def test_cfg2_qk_norm_with_rotary_embedding_full_shape(capi, gpu_device, n_rot):
    """The QK-norm call site end to end at one CP=4 rank's shape: q is the transposed [1, 24, 29700, 128] view
    into the fused [1, 29700, 24, 384] projection; norm + rotary embedding in one kernel each way (all tokens
    rotated as in the double-stream block, or all but 256 text tokens as in the single-stream block)."""
    B, S, H, D = 1, 29700, 24, 128
    gen = torch.Generator().manual_seed(21)
    mixed = torch.randn(B, S, H, 3 * D, generator=gen).bfloat16()
    w = (1 + 0.02 * torch.randn(D, generator=gen)).bfloat16()
    grad = torch.randn(B, H, S, D, generator=gen).bfloat16()
    cos, sin = O.make_rope_tables(n_rot, D, seed=2)
    q_cpu = mixed[..., :D].transpose(1, 2)
    want = O.eager_qk_norm_rope_fwd_bwd(q_cpu, w, cos, sin, grad)
    truth = O.truth_qk_norm_rope_fwd_bwd(q_cpu, w, cos, sin, grad)
    mixed_g = mixed.to(gpu_device)
    q_g = mixed_g[..., :D].transpose(1, 2)
    out, rstd = capi.rmsnorm_rope_forward_strided(q_g, w.to(gpu_device), cos.to(gpu_device), sin.to(gpu_device), EPS)
    dx, dw = capi.rmsnorm_rope_backward_strided(grad.to(gpu_device), q_g, w.to(gpu_device), rstd,
                                                cos.to(gpu_device), sin.to(gpu_device))
    case = f"cfg2_rope_{n_rot}"
    forward_bar(case, "out", out, want[0], O.rope_excuse(O.eager_rmsnorm(q_cpu, w), want[0]))
    grad_bar(case, "dx", dx, want[1], allow=1e-5)
    grad_bar(case, "dweight", dw, want[2])
    for name, got, wnt, t in zip(("out", "dx", "dweight"), (out, dx, dw), want, truth):
        no_worse_than_eager(case, name, got, wnt, t)


# ------------------------------------------------------------------ config 3

def test_cfg3_adaln_full_shape(capi, gpu_device):
    """x [1, 29700, 3072] bf16, one modulation row."""
    _, d = O.make_config_inputs("cfg3_adaln_bf16", seed=0)
    want = O.eager_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], d["grad"])
    truth = O.truth_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], d["grad"])
    g = dev(d, gpu_device)
    out, mean, rstd = capi.adaln_forward(g["x"], g["scale"], g["shift"], EPS)
    dx, ds, dh = capi.adaln_backward(g["grad"], g["x"], g["scale"], mean, rstd)
    forward_bar("cfg3", "out", out, want[0], O.adaln_excuse(d["x"], d["scale"], d["shift"], want[0]))
    grad_bar("cfg3", "dx", dx, want[1], allow=1e-5)
    grad_bar("cfg3", "dscale", ds, want[2])
    grad_bar("cfg3", "dshift", dh, want[3])
    for name, got, w, t in zip(("out", "dx", "dscale", "dshift"), (out, dx, ds, dh), want, truth):
        no_worse_than_eager("cfg3", name, got, w, t)


# ------------------------------------------------------------------ config 5

def test_cfg5_chain_against_the_truth(capi, gpu_device):
    """batch 4 x 11056 tokens, sigma 2, per-sample modulation: AdaLN then RMSNorm(3072), forward and backward of
    the chain.  The reduced gradients sum rows whose inputs already carry the first operator's one-ulp flips,
    which is why their bar against eager is wider (tests/test_gpu_parity.py); against the truth the chain on the
    GPU is as accurate as the eager chain."""
    B, S, C = 4, 11056, 3072
    d = O.make_adaln_inputs(B, S, C, torch.bfloat16, seed=0, sigma=2.0)
    w = (1 + 0.02 * torch.randn(C, generator=torch.Generator().manual_seed(3))).bfloat16()
    leaves = [t.clone().requires_grad_(True) for t in (d["x"], d["scale"], d["shift"], w)]
    y = O.eager_adaln(leaves[0], leaves[1], leaves[2], EPS)
    z = O.eager_rmsnorm(y, leaves[3], EPS)
    z.backward(d["grad"])
    # truth of the chain in float64 from the same inputs
    t_y, _, _, _ = O.truth_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], d["grad"])
    t_z, t_dy, t_dw = O.truth_rmsnorm_fwd_bwd(t_y, w, d["grad"])
    _, t_dx, t_ds, t_dh = O.truth_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], t_dy)
    g = dev(d, gpu_device)
    wg = w.to(gpu_device)
    y_g, mean, rstd = capi.adaln_forward(g["x"], g["scale"], g["shift"], EPS)
    z_g, rstd2 = capi.rmsnorm_forward(y_g, wg, EPS)
    dy, dw = capi.rmsnorm_backward(g["grad"], y_g, wg, rstd2)
    dx, ds, dh = capi.adaln_backward(dy, g["x"], g["scale"], mean, rstd)
    no_worse_than_eager("cfg5", "z", z_g, z.detach(), t_z)
    no_worse_than_eager("cfg5", "dx", dx, leaves[0].grad, t_dx)
    no_worse_than_eager("cfg5", "dscale", ds, leaves[1].grad, t_ds)
    no_worse_than_eager("cfg5", "dshift", dh, leaves[2].grad, t_dh)
    no_worse_than_eager("cfg5", "dweight", dw, leaves[3].grad, t_dw)
    for name, got, want in (("dweight", dw, leaves[3].grad), ("dscale", ds, leaves[1].grad),
                            ("dshift", dh, leaves[2].grad)):
        grad_bar("cfg5", name, got, want, allow=3e-3)
    grad_bar("cfg5", "dx", dx, leaves[0].grad, allow=1e-4)


# ---------------------------------------------------------------- gated op

def test_gated_residual_adaln_against_the_truth(capi, gpu_device):
    h, a, q, sc, sh, go, g2 = O.make_gated_inputs(2, 4099, 3072, torch.bfloat16, seed=5)
    want = O.eager_gated_residual_adaln_fwd_bwd(h, a, q, sc, sh, go, g2)
    truth = O.truth_gated_residual_adaln_fwd_bwd(h, a, q, sc, sh, go, g2)
    H, A, Q, SC, SH, GO, G2 = (t.to(gpu_device) for t in (h, a, q, sc, sh, go, g2))
    h2, out, mean, rstd = capi.gated_residual_adaln_forward(H, A, Q, SC, SH, EPS)
    grads = capi.gated_residual_adaln_backward(GO, G2, h2, A, Q, SC, mean, rstd)
    assert torch.equal(h2.cpu(), want[0])
    got = (h2, out) + tuple(grads)
    for name, gt, w, t in zip(("h2", "out", "dh", "dattn", "dgate", "dscale", "dshift"), got, want, truth):
        no_worse_than_eager("gated", name, gt, w, t)


# ------------------------------------------- rows that stress the row sums

def _stress_rows(B, S, C, dtype, kind, seed):
    d = O.make_adaln_inputs(B, S, C, dtype, seed=seed)
    x = d["x"].float()
    if kind == "mean":          # mean 30 sigma: sum(gx*x) - mu*sum(gx) cancels 30:1
        x = x + 30.0
    else:                       # a few +-200 channels per row on top of N(0, 1)
        gen = torch.Generator().manual_seed(seed + 1)
        idx = torch.randint(0, C, (B, S, 3), generator=gen)
        sign = torch.randint(0, 2, (B, S, 3), generator=gen).float() * 2 - 1
        x.scatter_(2, idx, 200.0 * sign)
    d["x"] = x.to(dtype)
    return d


@pytest.mark.parametrize("C,dtype", [(3072, torch.bfloat16), (1536, torch.bfloat16), (3072, torch.float16),
                                     (256, torch.bfloat16), (64, torch.bfloat16), (3072, torch.float32)])
@pytest.mark.parametrize("kind", ["mean", "outliers"])
def test_adaln_rows_with_large_mean_or_outliers(capi, gpu_device, C, dtype, kind):
    """The backward forms sum(gx * xhat) as r * (sum(gx * x) - mu * sum(gx)): with a large mean the two sums
    cancel, with outlier channels single terms dominate.  Judged against the truth (eager on the CPU keeps
    the statistics of a 16-bit row in 16 bits and is itself far from the truth here), and against eager
    with the bound scaled by the terms the backward adds."""
    B, S = 2, 515
    d = _stress_rows(B, S, C, dtype, kind, seed=300 + C)
    want = O.eager_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], d["grad"])
    truth = O.truth_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], d["grad"])
    g = dev(d, gpu_device)
    out, mean, rstd = capi.adaln_forward(g["x"], g["scale"], g["shift"], EPS)
    dx, ds, dh = capi.adaln_backward(g["grad"], g["x"], g["scale"], mean, rstd)
    case = f"stress_{kind}_{C}_{str(dtype).split('.')[-1]}"
    mu64 = d["x"].double().mean(-1).reshape(-1)
    torch.testing.assert_close(mean.double().cpu(), mu64, rtol=1e-5, atol=1e-5)
    f32 = dtype == torch.float32
    for name, got, w, t in zip(("out", "dx", "dscale", "dshift"), (out, dx, ds, dh), want, truth):
        # fp32: both sit at the noise floor of the input itself (an fp32 value near 30 is known to 2e-6) and
        # differ in the order of summation only; no bar against eager was widened for fp32
        no_worse_than_eager(case, name, got, w, t, slack=1.5 if f32 else 1.05, slack_max=3.0 if f32 else 1.25)
    if f32:
        torch.testing.assert_close(out.cpu(), want[0], rtol=1e-5, atol=1e-5)
        torch.testing.assert_close(dx.cpu(), want[1], rtol=1e-3, atol=1e-4)
        return
    terms = O.adaln_dx_terms(d["x"], d["scale"], d["grad"])
    frac = O.frac_outside(dx.cpu(), want[1], 1e-2, 1e-3, magnitude=terms)
    REPORT[case]["dx_vs_eager"] = {"frac_outside_term_scaled": frac}
    if kind == "outliers":
        assert frac <= 1e-4, (case, frac)
    # kind == "mean": no bar against eager for dx.  Eager's CPU LayerNorm backward rounds the saved mean of a
    # 16-bit row to 16 bits (30 +- 0.06 in bf16), which moves its xhat by up to 0.1 r; its dx is then 1.2-2.6x
    # further from the truth (RMS) than the kernel's, and the two differ on up to 16 % of elements of narrow
    # rows.  The truth bar above is the one that binds.


def test_rmsnorm_rows_with_outliers(capi, gpu_device):
    d = O.make_rmsnorm_inputs((1031,), 3072, torch.bfloat16, seed=77)
    x = d["x"].float()
    x[:, 5] = 200.0
    x[:, 1700] = -150.0
    d["x"] = x.bfloat16()
    want = O.eager_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
    truth = O.truth_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
    g = dev(d, gpu_device)
    out, rstd = capi.rmsnorm_forward(g["x"], g["weight"], EPS)
    dx, dw = capi.rmsnorm_backward(g["grad"], g["x"], g["weight"], rstd)
    forward_bar("rms_outliers", "out", out, want[0], O.rmsnorm_excuse(want[0]))
    for name, got, w, t in zip(("out", "dx", "dweight"), (out, dx, dw), want, truth):
        no_worse_than_eager("rms_outliers", name, got, w, t)
