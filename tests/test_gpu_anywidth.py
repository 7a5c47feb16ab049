"""GPU parity of the any-width kernels (rows of any whole number of 16-byte pieces, bf16 / fp16 /
fp32) through the C ABI, against the eager oracle.  Same bars as tests/test_gpu_parity.py:
forward 16-bit: >= 99.9 % bit-identical, <= 1 ulp except excused cancellation cases; forward fp32
rel 1e-5; gradients 16-bit |got - want| <= 1e-3 + 1e-2 |want|; gradients fp32 rel 1e-4."""
import pytest
import torch

from oracle import norm_oracle as O

pytestmark = pytest.mark.gpu
EPS = 1e-6

BF, HF, F32 = torch.bfloat16, torch.float16, torch.float32
# (cols, rows, dtype): every kernel geometry (8 / 16 / 32 lanes; 1, 2, 3, 4, 6, 8, 12, 16 accesses per lane),
# full and ragged last accesses, row counts that do not fill the last wavefront
RMS_CASES = [
    (8, 5, BF), (40, 300, HF), (64, 1001, BF), (96, 130, BF), (128, 77, HF), (200, 513, BF), (256, 4099, BF), (512, 300, BF),
    (768, 257, BF), (1000, 50, BF), (1024, 1000, BF), (1536, 333, HF), (2048, 77, BF), (2560, 65, BF),
    (3072, 300, HF), (3080, 33, BF), (4096, 129, BF), (5120, 130, BF), (6144, 70, HF), (8192, 66, BF),
    (8192, 9, HF), (4, 3, F32), (64, 100, F32), (256, 1000, F32), (1000, 77, F32), (2048, 129, F32), (4096, 40, F32),
]
ADALN_CASES = [
    (1, 5, 8, BF), (2, 301, 56, HF), (3, 333, 64, BF), (2, 65, 96, HF), (2, 1001, 256, BF), (4, 100, 512, BF), (1, 257, 1000, BF),
    (2, 130, 1024, HF), (3, 77, 1536, BF), (2, 300, 2048, BF), (5, 33, 3072, HF), (2, 65, 4096, BF),
    (2, 130, 5120, BF), (3, 40, 6144, BF), (2, 35, 6144, HF), (2, 66, 8192, BF), (1, 9, 8192, HF),
    (2, 50, 64, F32), (3, 100, 1000, F32), (2, 40, 4096, F32),
    # wide rows with more samples than the persistent grid has workgroups (one workgroup per sample), with fewer rows
    # per sample than a sample's share of the grid, and a single row
    (700, 3, 4096, BF), (3, 2, 8192, BF), (1, 1, 5120, HF), (600, 1, 2048, F32),
]


@pytest.fixture(scope="module")
def capi(gpu_device):
    from teletron_amd import capi as c
    c.lib()
    return c


def fwd_16bit_ok(got, want, excuse, what):
    rep = O.compare_bf16_ulp(got.cpu(), want, excuse_abs=excuse)
    assert rep.n_gt1 == 0, (what, rep)
    assert rep.n_excused <= max(2, 1e-4 * rep.n), (what, rep)
    assert rep.frac_exact >= 0.999 or rep.n - rep.n_exact <= 2, (what, rep)


def grad_ok(got, want, what, allow=0.0):
    if want.dtype == F32:
        torch.testing.assert_close(got.cpu(), want, rtol=1e-4, atol=1e-5, msg=what)
    else:
        assert O.frac_outside(got.cpu(), want, 1e-2, 1e-3) <= allow, what


def colsum_ok(got, want, terms, dim, what):
    """Column sums.  fp32: within 1e-4 of the column's L1 mass.  16-bit: the gradient bar on all but
    1e-4 of columns, and every column within 1e-2 |want| + 2^-8 * L2 mass (a term that flips by one ulp
    in one implementation moves a cancelling column by more than the absolute part of the bar)."""
    if want.dtype == F32:
        l1 = terms.abs().sum(dim).reshape(want.shape)
        assert ((got.cpu() - want).abs() <= 1e-4 * l1 + 1e-5).all(), what
    else:
        assert O.frac_outside(got.cpu(), want, 1e-2, 1e-3) <= 1e-4, what
        assert O.colsum_outside(got.cpu(), want, terms, dim, ulp=2.0 ** -8) == 0, what


@pytest.mark.parametrize("cols,rows,dtype", RMS_CASES)
def test_rmsnorm_any_width_vs_eager(capi, gpu_device, cols, rows, dtype):
    d = O.make_rmsnorm_inputs((rows,), cols, dtype, seed=500 + cols % 101 + rows % 7)
    want_out, want_dx, want_dw = O.eager_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
    x, w, g = (d[k].to(gpu_device) for k in ("x", "weight", "grad"))
    out, rstd = capi.rmsnorm_forward(x, w, EPS)
    if dtype == F32:
        torch.testing.assert_close(out.cpu(), want_out, rtol=1e-5, atol=1e-6)
    else:
        fwd_16bit_ok(out, want_out, O.rmsnorm_excuse(want_out), "out")
    _, want_r = O.staged_rmsnorm_fwd(d["x"], d["weight"])
    torch.testing.assert_close(rstd.cpu(), want_r.reshape(-1), rtol=2e-6, atol=0)
    dx, dw = capi.rmsnorm_backward(g, x, w, rstd)
    grad_ok(dx, want_dx, "dx")
    colsum_ok(dw, want_dw, d["grad"].float() * want_out.float(), 0, "dweight")
    dx2, dw2 = capi.rmsnorm_backward(g, x, w, rstd)
    assert torch.equal(dx, dx2) and torch.equal(dw, dw2)      # fixed-order reduction


@pytest.mark.parametrize("batch,seq,cols,dtype", ADALN_CASES)
def test_adaln_any_width_vs_eager(capi, gpu_device, batch, seq, cols, dtype):
    d = O.make_adaln_inputs(batch, seq, cols, dtype, seed=600 + cols % 103 + seq % 5, sigma=1.5)
    want_out, want_dx, want_ds, want_dh = O.eager_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], d["grad"])
    x, sc, sh, g = (d[k].to(gpu_device) for k in ("x", "scale", "shift", "grad"))
    out, mean, rstd = capi.adaln_forward(x, sc, sh, EPS)
    if dtype == F32:
        torch.testing.assert_close(out.cpu(), want_out, rtol=1e-5, atol=1e-5)
    else:
        fwd_16bit_ok(out, want_out, O.adaln_excuse(d["x"], d["scale"], d["shift"], want_out), "out")
    _, want_mu, want_r = O.staged_adaln_fwd(d["x"], d["scale"], d["shift"])
    torch.testing.assert_close(rstd.cpu(), want_r.reshape(-1), rtol=4e-6, atol=0)
    torch.testing.assert_close(mean.cpu(), want_mu.reshape(-1), rtol=0, atol=2e-6)
    dx, ds, dh = capi.adaln_backward(g, x, sc, mean, rstd)
    if dtype == F32:
        grad_ok(dx, want_dx, "dx")
    else:  # narrow rows: the bound scales with the terms the backward adds (see adaln_dx_terms)
        terms = O.adaln_dx_terms(d["x"], d["scale"], d["grad"])
        assert O.frac_outside(dx.cpu(), want_dx, 1e-2, 1e-3, magnitude=terms) <= 1e-4, "dx"
    xn = torch.nn.functional.layer_norm(d["x"].float(), (cols,), None, None, EPS)
    colsum_ok(ds, want_ds, d["grad"].float() * xn, 1, "dscale")
    colsum_ok(dh, want_dh, d["grad"].float(), 1, "dshift")
    again = capi.adaln_backward(g, x, sc, mean, rstd)
    assert all(torch.equal(a, b) for a, b in zip((dx, ds, dh), again))


def test_fp16_and_bf16_kernels_agree_on_statistics(capi, gpu_device):
    """The same values held in fp16 and in bf16 (where both are exact) give the same row statistics."""
    d = O.make_adaln_inputs(2, 131, 3072, BF, seed=7)
    x = d["x"].to(gpu_device)
    sc, sh = d["scale"].to(gpu_device), d["shift"].to(gpu_device)
    _, mean_t, rstd_t = capi.adaln_forward(x, sc, sh, EPS)
    _, mean_a, rstd_a = capi.adaln_forward(x.half(), sc.half(), sh.half(), EPS)   # N(0, 1.5): exact in fp16 too
    exact = (x.half().float() == x.float()).all(dim=-1).reshape(-1)
    assert exact.float().mean() > 0.5
    torch.testing.assert_close(mean_a[exact], mean_t[exact], rtol=0, atol=1e-6)
    torch.testing.assert_close(rstd_a[exact], rstd_t[exact], rtol=2e-6, atol=0)


def test_unsupported_widths_and_entry_points(capi, gpu_device):
    mk = lambda *shape, dt=BF: torch.zeros(*shape, device=gpu_device, dtype=dt)
    for cols, dt in ((100, BF), (8200, BF), (4100, F32), (6, F32)):
        with pytest.raises(capi.NormError) as e:
            capi.rmsnorm_forward(mk(4, cols, dt=dt), mk(cols, dt=dt), EPS)
        assert e.value.status == 2
    # reference-contract entry points exist for the tuned shapes only
    with pytest.raises(capi.NormError) as e:
        capi.rmsnorm_backward(mk(4, 256), mk(4, 256), mk(256), torch.zeros(4, device=gpu_device), from_out=True)
    assert e.value.status == 2
    with pytest.raises(capi.NormError) as e:
        capi.adaln_forward(mk(1, 4, 256), mk(1, 256), mk(1, 256), EPS, want_xnorm=True)
    assert e.value.status == 2
    # zero rows at a non-tuned width: no-op forward, zero parameter gradients
    out, rstd = capi.rmsnorm_forward(mk(0, 512, dt=HF), mk(512, dt=HF), EPS)
    dx, dw = capi.rmsnorm_backward(mk(0, 512, dt=HF), mk(0, 512, dt=HF), mk(512, dt=HF), rstd)
    assert dw.shape == (512,) and not dw.any()


def test_functions_take_other_widths_and_fp16(gpu_device):
    """The autograd Functions and modules on a smaller model's shapes: hidden 1536 in fp16, head dim 64."""
    from teletron_amd import fusedlayers as FL
    d = O.make_adaln_inputs(2, 97, 1536, HF, seed=71)
    want_out, want_dx, want_ds, want_dh = O.eager_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], d["grad"])
    x, sc, sh = (d[k].to(gpu_device).requires_grad_(True) for k in ("x", "scale", "shift"))
    out = FL.AdaLNCustom(1536)(x, sc, sh)
    out.backward(d["grad"].to(gpu_device))
    fwd_16bit_ok(out.detach(), want_out, O.adaln_excuse(d["x"], d["scale"], d["shift"], want_out), "out")
    grad_ok(x.grad, want_dx, "dx", allow=1e-4)
    grad_ok(sc.grad, want_ds, "dscale")
    grad_ok(sh.grad, want_dh, "dshift")
    # QK-norm with head dim 64 on the transposed view: falls back to a contiguous copy, then any-width kernels
    q = O.make_rmsnorm_inputs((2, 50, 6), 64, BF, seed=72)
    want_q, want_dq, want_dw = O.eager_rmsnorm_fwd_bwd(q["x"].transpose(1, 2), q["weight"], q["grad"].transpose(1, 2))
    xq = q["x"].to(gpu_device).requires_grad_(True)
    wq = q["weight"].to(gpu_device).requires_grad_(True)
    got = FL.RMSNormModelFunction.apply(xq.transpose(1, 2), wq, EPS, 64)
    got.backward(q["grad"].to(gpu_device).transpose(1, 2))
    fwd_16bit_ok(got.detach(), want_q, O.rmsnorm_excuse(want_q), "q")
    assert xq.grad.shape == q["x"].shape
    grad_ok(xq.grad.transpose(1, 2), want_dq, "dq")
    grad_ok(wq.grad, want_dw, "dw")


def test_geometry_boundaries_forward_and_backward(capi, gpu_device):
    """Row widths on both sides of every geometry switch (8, 16, 32, 64 lanes; 1, 2, 3, 4, 6, 8, 12, 16 accesses
    per lane), with row counts that leave the last wavefront partly empty."""
    pieces = [1, 7, 8, 9, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 191, 192, 193, 255, 256, 257, 383, 384, 385,
              511, 512, 513, 767, 768, 769, 1023, 1024]
    for i, p in enumerate(pieces):
        cols = p * 8
        rows = 3 + (i * 7) % 11
        d = O.make_rmsnorm_inputs((rows,), cols, BF, seed=800 + i)
        want_out, want_dx, want_dw = O.eager_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
        x, w, g = (d[k].to(gpu_device) for k in ("x", "weight", "grad"))
        out, rstd = capi.rmsnorm_forward(x, w, EPS)
        fwd_16bit_ok(out, want_out, O.rmsnorm_excuse(want_out), f"rms out cols={cols}")
        dx, dw = capi.rmsnorm_backward(g, x, w, rstd)
        grad_ok(dx, want_dx, f"rms dx cols={cols}")
        colsum_ok(dw, want_dw, d["grad"].float() * want_out.float(), 0, f"rms dw cols={cols}")
        a = O.make_adaln_inputs(2, rows, cols, BF, seed=900 + i)
        a_out, a_dx, a_ds, a_dh = O.eager_adaln_fwd_bwd(a["x"], a["scale"], a["shift"], a["grad"])
        ax, asc, ash, ag = (a[k].to(gpu_device) for k in ("x", "scale", "shift", "grad"))
        out, mean, rstd = capi.adaln_forward(ax, asc, ash, EPS)
        if cols >= 64:   # a row of 8 or 56 elements has no meaningful 1-ulp statistics (xn is O(1) with 3 bits of x)
            fwd_16bit_ok(out, a_out, O.adaln_excuse(a["x"], a["scale"], a["shift"], a_out), f"adaln out cols={cols}")
        dx, ds, dh = capi.adaln_backward(ag, ax, asc, mean, rstd)
        terms = O.adaln_dx_terms(a["x"], a["scale"], a["grad"])
        # eager on the CPU keeps mean and rstd of a 16-bit row in 16 bits: a stray element of these tiny
        # tensors may sit just outside the bar; none may be far outside
        assert O.frac_outside(dx.cpu(), a_dx, 1e-2, 1e-3, magnitude=terms) * a_dx.numel() <= max(2, 2e-4 * a_dx.numel()), \
            f"adaln dx cols={cols}"
        assert O.frac_outside(dx.cpu(), a_dx, 3e-2, 3e-3, magnitude=terms) == 0.0, f"adaln dx cols={cols}"
        colsum_ok(dh, a_dh, a["grad"].float(), 1, f"adaln dshift cols={cols}")
        xn = torch.nn.functional.layer_norm(a["x"].float(), (cols,), None, None, EPS)
        colsum_ok(ds, a_ds, a["grad"].float() * xn, 1, f"adaln dscale cols={cols}")


def test_fp16_through_the_tuned_only_entry_points(capi, gpu_device):
    """fp16 at 128 / 3072 columns runs the tuned kernels, so the strided, gated and residual forms take it too."""
    from teletron_amd import fusedlayers as FL
    # strided QK-norm on the fused projection, forward and backward through the Function
    B, S, H, D = 1, 203, 6, 128
    gen = torch.Generator().manual_seed(91)
    mixed = torch.randn(B, S, H, 3 * D, generator=gen).half()
    wq, wk = (1 + 0.02 * torch.randn(D, generator=gen)).half(), (1 + 0.02 * torch.randn(D, generator=gen)).half()
    gq, gk, gv = (torch.randn(B, H, S, D, generator=gen).half() for _ in range(3))
    m_c = mixed.clone().requires_grad_(True)
    q_c, k_c, v_c = torch.split(m_c, [D, D, D], dim=3)
    q_c, k_c = O.eager_rmsnorm(q_c.transpose(1, 2), wq), O.eager_rmsnorm(k_c.transpose(1, 2), wk)
    torch.autograd.backward([q_c, k_c, v_c.transpose(1, 2)], [gq, gk, gv])
    m_g = mixed.to(gpu_device).requires_grad_(True)
    q_g, k_g, v_g = FL.QKVSplitNormFunction.apply(m_g, wq.to(gpu_device), wk.to(gpu_device), EPS)
    fwd_16bit_ok(q_g.detach(), q_c.detach(), O.rmsnorm_excuse(q_c.detach()), "q")
    fwd_16bit_ok(k_g.detach(), k_c.detach(), O.rmsnorm_excuse(k_c.detach()), "k")
    torch.autograd.backward([q_g, k_g, v_g], [gq.to(gpu_device), gk.to(gpu_device), gv.to(gpu_device)])
    grad_ok(m_g.grad, m_c.grad, "d mixed")
    # gated residual + AdaLN
    h, a, q, sc, sh, go, g2 = O.make_gated_inputs(2, 257, 3072, HF, seed=92)
    want = O.eager_gated_residual_adaln_fwd_bwd(h, a, q, sc, sh, go, g2)
    dev_ = lambda t: t.to(gpu_device)
    h2, out, mean, rstd = capi.gated_residual_adaln_forward(dev_(h), dev_(a), dev_(q), dev_(sc), dev_(sh), EPS)
    assert torch.equal(h2.cpu(), want[0])
    fwd_16bit_ok(out, want[1], O.adaln_excuse(want[0], sc, sh, want[1]), "gated out")
    dh, da, dq, dsc, dsh = capi.gated_residual_adaln_backward(dev_(go), dev_(g2), h2, dev_(a), dev_(q), dev_(sc), mean, rstd)
    terms = want[2].float().abs() + g2.float().abs()
    assert O.frac_outside(dh.cpu(), want[2], 1e-2, 1e-3, magnitude=terms) <= 1e-4
    assert O.frac_outside(da.cpu(), want[3], 1e-2, 1e-3, magnitude=terms * q.float().abs()[:, None]) <= 1e-4
    assert O.colsum_outside(dq.cpu(), want[4], terms * a.float(), dim=1) == 0
    grad_ok(dsc, want[5], "dscale")
    grad_ok(dsh, want[6], "dshift")
    # residual form == plain backward, then the addition
    x, gr, other = dev_(h), dev_(go), dev_(g2)
    _, mean, rstd = capi.adaln_forward(x, dev_(sc), dev_(sh), EPS)
    dx, _, _ = capi.adaln_backward(gr, x, dev_(sc), mean, rstd)
    dxr, _, _ = capi.adaln_backward_residual(gr, other, x, dev_(sc), mean, rstd)
    assert torch.equal(dxr, dx + other)


# ------------------------- the call-site forms at other widths (strided, gated, residual, sequence-first)

@pytest.mark.parametrize("D,dtype,B,S,H", [(64, BF, 2, 203, 5), (256, HF, 1, 77, 3), (96, F32, 1, 130, 2), (40, BF, 1, 9, 1)])
def test_strided_qk_norm_at_other_head_dims(capi, gpu_device, D, dtype, B, S, H):
    """The transposed [B, H, S, D] views into a fused [B, S, H, 3D] projection, read in place, for head
    dimensions the tuned kernels are not built for: equal to the dense kernels on a contiguous copy bit for
    bit, and to eager within the bars."""
    gen = torch.Generator().manual_seed(D)
    mixed = torch.randn(B, S, H, 3 * D, generator=gen).to(dtype)
    w = (1 + 0.02 * torch.randn(D, generator=gen)).to(dtype)
    grad = torch.randn(B, H, S, D, generator=gen).to(dtype)
    mixed_g, w_g, grad_g = mixed.to(gpu_device), w.to(gpu_device), grad.to(gpu_device)
    for i in range(2):
        x_cpu = mixed[..., i * D:(i + 1) * D].transpose(1, 2)
        x_g = mixed_g[..., i * D:(i + 1) * D].transpose(1, 2)
        assert not x_g.is_contiguous()
        want_out, want_dx, want_dw = O.eager_rmsnorm_fwd_bwd(x_cpu, w, grad)
        out, rstd = capi.rmsnorm_forward_strided(x_g, w_g, EPS)
        dx, dw = capi.rmsnorm_backward_strided(grad_g, x_g, w_g, rstd)
        out_d, rstd_d = capi.rmsnorm_forward(x_g.contiguous(), w_g, EPS)
        dx_d, dw_d = capi.rmsnorm_backward(grad_g, x_g.contiguous(), w_g, rstd_d)
        assert torch.equal(out, out_d) and torch.equal(rstd, rstd_d)
        assert torch.equal(dx.contiguous(), dx_d)
        # (the strided traversal hands rows to wavefronts in another order, so dweight's fp32 partial sums
        # associate differently: equal after rounding to a 16-bit type, a few fp32 ulps apart otherwise)
        torch.testing.assert_close(dw.float(), dw_d.float(), rtol=1e-5, atol=1e-4)
        if dtype == F32:
            torch.testing.assert_close(out.cpu(), want_out, rtol=1e-5, atol=1e-6)
            torch.testing.assert_close(dx.cpu(), want_dx, rtol=1e-4, atol=1e-5)
        else:
            fwd_16bit_ok(out, want_out, O.rmsnorm_excuse(want_out), "out")
            grad_ok(dx, want_dx, "dx")
            grad_ok(dw, want_dw, "dweight")
    # dx written through strides into a slice of one gradient tensor (what QKVSplitNormFunction does)
    d_mixed = torch.zeros_like(mixed_g)
    x_g = mixed_g[..., :D].transpose(1, 2)
    out, rstd = capi.rmsnorm_forward_strided(x_g, w_g, EPS)
    dx, _ = capi.rmsnorm_backward_strided(grad_g, x_g, w_g, rstd)
    capi.rmsnorm_backward_strided(grad_g, x_g, w_g, rstd, dx=d_mixed[..., :D].transpose(1, 2))
    assert torch.equal(d_mixed[..., :D].transpose(1, 2), dx) and not d_mixed[..., D:].any()


@pytest.mark.parametrize("C,dtype,B,S,with_h2", [(1536, BF, 2, 515, True), (1024, HF, 3, 130, False), (512, F32, 2, 77, True),
                                                 (2048, BF, 1, 300, True), (64, BF, 2, 1001, True), (1536, F32, 1, 65, False),
                                                 # rows of more than 384 pieces: four wavefronts per row
                                                 (4096, BF, 2, 515, True), (5120, HF, 1, 130, False), (8192, BF, 3, 67, True),
                                                 (3080, BF, 1, 1100, True), (2048, F32, 2, 77, True), (4096, F32, 1, 33, False)])
def test_gated_residual_adaln_at_other_widths(capi, gpu_device, C, dtype, B, S, with_h2):
    h, a, q, sc, sh, go, g2 = O.make_gated_inputs(B, S, C, dtype, seed=C + S, with_grad_h2=with_h2)
    want = O.eager_gated_residual_adaln_fwd_bwd(h, a, q, sc, sh, go, g2)
    to = lambda t: None if t is None else t.to(gpu_device)
    H, A, Q, SC, SH, GO, G2 = (to(t) for t in (h, a, q, sc, sh, go, g2))
    h2, out, mean, rstd = capi.gated_residual_adaln_forward(H, A, Q, SC, SH, EPS)
    dh, da, dq, dsc, dsh = capi.gated_residual_adaln_backward(GO, G2, h2, A, Q, SC, mean, rstd)
    # bit-identical to its parts run one after the other: elementwise update, plain AdaLN, plain backward + add
    h2_parts = H + A * Q[:, None]
    assert torch.equal(h2, h2_parts)
    out_p, mean_p, rstd_p = capi.adaln_forward(h2_parts, SC, SH, EPS)
    assert torch.equal(out, out_p) and torch.equal(mean, mean_p) and torch.equal(rstd, rstd_p)
    dxn, dsc_p, dsh_p = capi.adaln_backward(GO, h2_parts, SC, mean_p, rstd_p)
    dh_parts = dxn + G2 if with_h2 else dxn
    assert torch.equal(dh, dh_parts) and torch.equal(da, dh_parts * Q[:, None])
    assert torch.equal(dsc, dsc_p) and torch.equal(dsh, dsh_p)
    if dtype == F32:
        torch.testing.assert_close(out.cpu(), want[1], rtol=1e-5, atol=1e-5)
        torch.testing.assert_close(dh.cpu(), want[2], rtol=1e-3, atol=1e-4)
        l1 = (want[2].abs() * a.abs()).sum(1)
        assert ((dq.cpu() - want[4]).abs() <= 1e-4 * l1 + 1e-5).all()
    else:
        assert torch.equal(h2.cpu(), want[0])
        fwd_16bit_ok(out, want[1], O.adaln_excuse(want[0], sc, sh, want[1]), "out")
        terms = O.adaln_dx_terms(want[0], sc, go) + (g2.float().abs() if with_h2 else 0)
        assert O.frac_outside(dh.cpu(), want[2], 1e-2, 1e-3, magnitude=terms) <= 1e-4
        assert O.colsum_outside(dq.cpu(), want[4], terms * a.float(), dim=1) == 0
        colsum_ok(dsc, want[5], go.float() * 3, 1, "dscale")
        colsum_ok(dsh, want[6], go.float(), 1, "dshift")


@pytest.mark.parametrize("C,dtype", [(1536, BF), (1024, HF), (768, F32), (128, BF), (4096, BF), (6152, HF), (1540, F32),
                                     (8192, BF)])
def test_adaln_backward_residual_at_other_widths(capi, gpu_device, C, dtype):
    d = O.make_adaln_inputs(2, 301, C, dtype, seed=C)
    other = O.make_adaln_inputs(2, 301, C, dtype, seed=C + 1)["grad"]
    g = {k: v.to(gpu_device) for k, v in d.items()}
    _, mean, rstd = capi.adaln_forward(g["x"], g["scale"], g["shift"], EPS)
    dx, ds, dh = capi.adaln_backward(g["grad"], g["x"], g["scale"], mean, rstd)
    dxr, dsr, dhr = capi.adaln_backward_residual(g["grad"], other.to(gpu_device), g["x"], g["scale"], mean, rstd)
    assert torch.equal(dxr, dx + other.to(gpu_device)) and torch.equal(dsr, ds) and torch.equal(dhr, dh)


@pytest.mark.parametrize("C,dtype,B,S", [(3072, BF, 3, 129), (3072, F32, 2, 33), (1536, HF, 4, 65), (128, BF, 3, 1001),
                                         (64, BF, 5, 77), (3072, BF, 1, 100), (4096, BF, 2, 40)])
def test_adaln_on_sequence_first_rows(capi, gpu_device, C, dtype, B, S):
    """x [S, B, C] with one modulation row per sample (the output norm's layout, dit_layerspec.py:72-78),
    normalised where it lies: bit-identical to the sample-major call on the regrouped rows, statistics
    included (they are indexed by the same row numbers as x)."""
    d = O.make_adaln_inputs(B, S, C, dtype, seed=7 * C + B)
    g = {k: v.to(gpu_device) for k, v in d.items()}
    x_sf, grad_sf = g["x"].transpose(0, 1).contiguous(), g["grad"].transpose(0, 1).contiguous()   # [S, B, C]
    out, mean, rstd = capi.adaln_forward(g["x"], g["scale"], g["shift"], EPS)
    dx, ds, dh = capi.adaln_backward(g["grad"], g["x"], g["scale"], mean, rstd)
    out_sf, mean_sf, rstd_sf = capi.adaln_forward(x_sf, g["scale"], g["shift"], EPS, seq_first=True)
    dx_sf, ds_sf, dh_sf = capi.adaln_backward(grad_sf, x_sf, g["scale"], mean_sf, rstd_sf, seq_first=True)
    assert torch.equal(out_sf.transpose(0, 1), out) and torch.equal(dx_sf.transpose(0, 1), dx)
    assert torch.equal(mean_sf.reshape(S, B).t(), mean.reshape(B, S))
    assert torch.equal(rstd_sf.reshape(S, B).t(), rstd.reshape(B, S))
    assert torch.equal(ds_sf, ds) and torch.equal(dh_sf, dh)
    # and the eager formula as the caller writes it: norm(x) * (1 + scale) + shift broadcast over S
    if dtype != F32:
        want = torch.nn.functional.layer_norm(d["x"].transpose(0, 1), (C,), None, None, EPS) * (1 + d["scale"]) + d["shift"]
        assert O.frac_outside(out_sf.cpu(), want, 1e-2, 1e-2) <= 1e-4


def test_functions_take_the_wide_forms_at_other_widths(gpu_device):
    """The autograd Functions at hidden 1536: gated residual + AdaLN and the stream-keeping AdaLN, and
    QKVSplitNormFunction at head dimension 64."""
    from teletron_amd import fusedlayers as FL
    h, a, q, sc, sh, go, g2 = O.make_gated_inputs(2, 130, 1536, BF, seed=5)
    want = O.eager_gated_residual_adaln_fwd_bwd(h, a, q, sc, sh, go, g2)
    leaves = [t.to(gpu_device).requires_grad_(True) for t in (h, a, q, sc, sh)]
    h2, out = FL.gated_residual_layer_norm(*leaves, eps=EPS)
    torch.autograd.backward([out, h2], [go.to(gpu_device), g2.to(gpu_device)])
    assert torch.equal(h2.detach().cpu(), want[0])
    fwd_16bit_ok(out.detach(), want[1], O.adaln_excuse(want[0], sc, sh, want[1]), "out")
    grad_ok(leaves[3].grad, want[5], "dscale")
    grad_ok(leaves[4].grad, want[6], "dshift")
    x = h.to(gpu_device).requires_grad_(True)
    same, out2 = FL.modulated_layer_norm_keeping_stream(x, sc.to(gpu_device), sh.to(gpu_device), EPS)
    torch.autograd.backward([out2, same * 1.0], [go.to(gpu_device), g2.to(gpu_device)])
    assert x.grad is not None and x.grad.shape == h.shape
    with pytest.raises(ValueError, match="unsupported cols|rows of at most"):
        FL.gated_residual_layer_norm(torch.zeros(1, 4, 4100, dtype=BF, device=gpu_device),
                                     torch.zeros(1, 4, 4100, dtype=BF, device=gpu_device),
                                     *(torch.zeros(1, 4100, dtype=BF, device=gpu_device) for _ in range(3)), eps=EPS)
    B, S, H, D = 1, 101, 4, 64
    gen = torch.Generator().manual_seed(64)
    mixed = torch.randn(B, S, H, 3 * D, generator=gen).bfloat16()
    wq, wk = (1 + 0.02 * torch.randn(D, generator=gen)).bfloat16(), (1 + 0.02 * torch.randn(D, generator=gen)).bfloat16()
    gq, gk, gv = (torch.randn(B, H, S, D, generator=gen).bfloat16() for _ in range(3))
    m_c = mixed.clone().requires_grad_(True)
    q_c, k_c, v_c = torch.split(m_c, [D, D, D], dim=3)
    q_c, k_c = O.eager_rmsnorm(q_c.transpose(1, 2), wq), O.eager_rmsnorm(k_c.transpose(1, 2), wk)
    torch.autograd.backward([q_c, k_c, v_c.transpose(1, 2)], [gq, gk, gv])
    m_g = mixed.to(gpu_device).requires_grad_(True)
    q_g, k_g, v_g = FL.QKVSplitNormFunction.apply(m_g, wq.to(gpu_device), wk.to(gpu_device), EPS)
    fwd_16bit_ok(q_g.detach(), q_c.detach(), O.rmsnorm_excuse(q_c.detach()), "q")
    torch.autograd.backward([q_g, k_g, v_g], [gq.to(gpu_device), gk.to(gpu_device), gv.to(gpu_device)])
    grad_ok(m_g.grad, m_c.grad, "d mixed")
