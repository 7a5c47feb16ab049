"""CPU oracle for the fused normalization path.  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import
this module; the shipped operators never do.

It restates, in plain PyTorch CPU ops, the eager formulas the reference uses
when its fused kernels are off -- the behaviour the fused kernels must match:

  * RMSNorm  -- teletron/models/dit/dit_fusedlayers.py:360-370
        out = (x.float() * rsqrt(x.float().pow(2).mean(-1, keepdim=True) + eps)).type_as(x) * weight
  * AdaLN    -- teletron/models/dit/dit_fusedlayers.py:198,223 (and :251,271)
        out = LayerNorm(C, elementwise_affine=False, eps)(x) * (1 + scale[:, None]) + shift[:, None]

  * gated residual + AdaLN -- teletron/models/dit/dit_layerspec.py:152,158,161-163
        h2  = h + attn * gate.unsqueeze(1)
        out = LayerNorm(C, elementwise_affine=False, eps)(h2) * (1 + scale[:, None]) + shift[:, None]
    (h2 also continues as the residual stream, :180-182)

Three layers of the same math live here, each one a check on the others:

  eager_*     the formulas above, verbatim in behaviour, differentiated by
              torch.autograd (this is what "parity with eager" means);
  staged_*    the same arithmetic written out by hand with every rounding
              point explicit (the order a fused kernel has to follow);
  truth_*     float64 closed forms with no intermediate rounding.

What pins the arithmetic (see tests/test_oracle.py): library routines
(F.rms_norm, F.layer_norm with weight=1+scale, bias=shift), closed forms on
constant / unit-weight rows, scale and affine invariances, the orthogonality
invariants of the backward (sum_c dx = 0, sum_c dx*xhat = 0), brute-force
float64 loops on tiny inputs, torch.autograd.gradcheck, and an independent
scalar C restatement (oracle/norm_oracle_c.c) that models the bf16 rounding
points bit by bit.  The reference's own tests hold no vectors for this path.

One function restates a third-party routine: apply_rotary_emb_real follows the
published diffusers.models.embeddings.apply_rotary_emb (diffusers==0.32.1,
not installed here).  It is pinned by mathematical properties only; its parity
with the library itself is UNPINNED (see the section comment below).
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch
import torch.nn.functional as F

EPS = 1e-6  # teletron/models/hunyuanvideo/model.py:109 (layernorm_epsilon)


# --------------------------------------------------------------------------
# eager: the reference's fallback formulas, differentiated by autograd
# --------------------------------------------------------------------------

def eager_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = EPS) -> torch.Tensor:
    """dit_fusedlayers.py:360-361,369-370."""
    xf = x.float()
    normed = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return normed.type_as(x) * weight


def eager_adaln(x: torch.Tensor, scale: torch.Tensor, shift: torch.Tensor,
                eps: float = EPS) -> torch.Tensor:
    """dit_fusedlayers.py:198 + :223.  x [B,S,C]; scale, shift [B,C]."""
    xn = F.layer_norm(x, (x.shape[-1],), None, None, eps)
    return xn * (1 + scale[:, None]) + shift[:, None]


def eager_rmsnorm_fwd_bwd(x, weight, grad, eps: float = EPS):
    """Returns (out, dx, dweight) exactly as autograd produces them."""
    x = x.detach().clone().requires_grad_(True)
    weight = weight.detach().clone().requires_grad_(True)
    out = eager_rmsnorm(x, weight, eps)
    out.backward(grad)
    return out.detach(), x.grad, weight.grad


def eager_adaln_fwd_bwd(x, scale, shift, grad, eps: float = EPS):
    """Returns (out, dx, dscale, dshift) exactly as autograd produces them."""
    x = x.detach().clone().requires_grad_(True)
    scale = scale.detach().clone().requires_grad_(True)
    shift = shift.detach().clone().requires_grad_(True)
    out = eager_adaln(x, scale, shift, eps)
    out.backward(grad)
    return out.detach(), x.grad, scale.grad, shift.grad


def eager_gated_residual_adaln(h, attn, gate, scale, shift, eps: float = EPS):
    """dit_layerspec.py:152 then :158,:161-163.  h, attn [B,S,C]; gate, scale, shift [B,C].
    Returns (h2, out): the updated residual stream and its modulated norm."""
    h2 = h + attn * gate.unsqueeze(1)
    return h2, eager_adaln(h2, scale, shift, eps)


def eager_gated_residual_adaln_fwd_bwd(h, attn, gate, scale, shift, grad_out, grad_h2=None,
                                       eps: float = EPS):
    """Returns (h2, out, dh, dattn, dgate, dscale, dshift) as autograd produces them;
    grad_h2 is the gradient h2 receives from its later uses (None: it has none)."""
    leaves = [t.detach().clone().requires_grad_(True) for t in (h, attn, gate, scale, shift)]
    h2, out = eager_gated_residual_adaln(*leaves, eps)
    if grad_h2 is None:
        out.backward(grad_out)
    else:
        torch.autograd.backward([out, h2], [grad_out, grad_h2])
    return (h2.detach(), out.detach()) + tuple(t.grad for t in leaves)


# --------------------------------------------------------------------------
# rotary embedding behind the per-head norm
# --------------------------------------------------------------------------
# The callers (teletron/models/dit/dit_attention.py:266-273 and :435-443) rotate the normalised query and
# key with diffusers.models.embeddings.apply_rotary_emb(x, (freqs_cos, freqs_sin)).  diffusers is a
# third-party dependency (requirements.txt:3 pins diffusers==0.32.1) and is not installed here, so its
# published algorithm is restated below (defaults use_real=True, use_real_unbind_dim=-1) and pinned in
# tests/test_oracle.py by what the mathematics fixes: identity at angle 0, preservation of each pair's norm,
# composition of angles, a brute-force complex multiplication, the inverse rotation as its gradient, and
# negative controls for the other pairing conventions.  PARITY AGAINST THE LIBRARY ITSELF IS UNPINNED: no
# file of the reference holds an input/output vector of this function.

def apply_rotary_emb_real(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x [B, H, S, D]; cos, sin [S, D] (each angle's value repeated for the two elements of its pair, as
    get_1d_rotary_pos_embed(use_real=True) builds them, hunyuanvideo/layers.py:245-252)."""
    cos, sin = cos[None, None], sin[None, None]
    x_real, x_imag = x.reshape(*x.shape[:-1], -1, 2).unbind(-1)
    x_rotated = torch.stack([-x_imag, x_real], dim=-1).flatten(3)
    return (x.float() * cos + x_rotated.float() * sin).to(x.dtype)


def eager_qk_norm_rope(x, weight, cos, sin, eps: float = EPS):
    """q_layernorm / k_layernorm on the [B, H, S, D] view, then the rotary embedding on the first
    cos.shape[0] tokens (all tokens in the double-stream block, dit_attention.py:266-273; the image tokens
    in the single-stream block, :435-443)."""
    y = eager_rmsnorm(x, weight, eps)
    n = cos.shape[0]
    if n == 0:
        return y
    if n == y.shape[2]:
        return apply_rotary_emb_real(y, cos, sin)
    return torch.cat([apply_rotary_emb_real(y[:, :, :n], cos, sin), y[:, :, n:]], dim=2)


def eager_qk_norm_rope_fwd_bwd(x, weight, cos, sin, grad, eps: float = EPS):
    """Returns (out, dx, dweight) as autograd produces them."""
    xr = x.detach().clone().requires_grad_(True)
    wr = weight.detach().clone().requires_grad_(True)
    out = eager_qk_norm_rope(xr, wr, cos, sin, eps)
    out.backward(grad)
    return out.detach(), xr.grad, wr.grad


def truth_qk_norm_rope_fwd_bwd(x, weight, cos, sin, grad, eps: float = EPS):
    """float64, no intermediate rounding: the rotation is linear and orthogonal per pair when both elements
    of a pair share an angle, but the general (per-element table) form is kept."""
    n = cos.shape[0]
    c, s = cos.double()[None, None], sin.double()[None, None]

    def rot(v):
        a, b = v[..., 0::2], v[..., 1::2]
        out = torch.empty_like(v)
        out[..., 0::2] = a * c[..., 0::2] - b * s[..., 0::2]
        out[..., 1::2] = b * c[..., 1::2] + a * s[..., 1::2]
        return out

    def rot_t(g):   # transpose of rot
        a, b = g[..., 0::2], g[..., 1::2]
        out = torch.empty_like(g)
        out[..., 0::2] = a * c[..., 0::2] + b * s[..., 1::2]
        out[..., 1::2] = b * c[..., 1::2] - a * s[..., 0::2]
        return out

    y, _, _ = truth_rmsnorm_fwd_bwd(x, weight, grad, eps)
    out = y.clone()
    out[:, :, :n] = rot(y[:, :, :n])
    gy = grad.double().clone()
    gy[:, :, :n] = rot_t(gy[:, :, :n])
    _, dx, dw = truth_rmsnorm_fwd_bwd(x, weight, gy, eps)
    return out, dx, dw


def make_rope_tables(tokens: int, cols: int, seed: int = 0, theta: float = 256.0):
    """cos, sin [tokens, cols] fp32 in the layout get_1d_rotary_pos_embed(use_real=True) produces: one angle
    per pair, repeated for both elements; angles position * theta^(-2i/cols) over a shuffled position list."""
    g = _gen(seed + 1234)
    pos = torch.randperm(tokens, generator=g).float()
    inv = 1.0 / (theta ** (torch.arange(0, cols, 2).float() / cols))
    ang = torch.outer(pos, inv)
    return ang.cos().repeat_interleave(2, dim=1).contiguous(), ang.sin().repeat_interleave(2, dim=1).contiguous()


# --------------------------------------------------------------------------
# staged: every rounding point written out (what a fused kernel must follow)
# --------------------------------------------------------------------------

def staged_rmsnorm_fwd(x, weight, eps: float = EPS):
    """Returns (out, rstd[rows] fp32).  Rounding points for low-precision x:
    y -> dtype(x); y*w -> promoted dtype."""
    xf = x.float()
    rstd = torch.rsqrt((xf * xf).mean(-1, keepdim=True) + eps)
    y = (xf * rstd).to(x.dtype)
    return y * weight, rstd.squeeze(-1)


def staged_rmsnorm_bwd(x, weight, rstd, grad):
    """dx = r*(gy - xhat*mean_c(gy*xhat)), dw = sum_rows round(g*y).
    gy = g*w is rounded to the promoted dtype first (that is how autograd
    materialises it); y is the dtype(x)-rounded normalised row."""
    C = x.shape[-1]
    xf = x.float()
    r = rstd.reshape(*x.shape[:-1], 1)
    xhat = xf * r
    y = xhat.to(x.dtype)
    gy = (grad * weight).float()
    m = (gy * xhat).sum(-1, keepdim=True) / C
    dx = (r * (gy - xhat * m)).to(x.dtype)
    prod = grad * y                                   # rounded to the promoted dtype
    dw = prod.reshape(-1, C).sum(0).to(weight.dtype)  # fp32 accumulation inside sum
    return dx, dw


def staged_adaln_fwd(x, scale, shift, eps: float = EPS):
    """Returns (out, mean[rows], rstd[rows]).  Rounding points (bf16 case):
    xn; t = 1+scale; p = xn*t; out = p+shift."""
    xf = x.float()
    mean = xf.mean(-1, keepdim=True)
    var = ((xf - mean) ** 2).mean(-1, keepdim=True)
    rstd = torch.rsqrt(var + eps)
    xn = ((xf - mean) * rstd).to(x.dtype)
    t = 1 + scale[:, None]
    p = xn * t
    out = p + shift[:, None]
    return out, mean.squeeze(-1), rstd.squeeze(-1)


def staged_adaln_bwd(x, scale, mean, rstd, grad):
    """dshift = sum_s g; dscale = sum_s round(g*xn); gx = round(g*t);
    dx = r*(gx - mean_c(gx) - xhat*mean_c(gx*xhat))."""
    B, S, C = x.shape
    xf = x.float()
    mu = mean.reshape(B, S, 1)
    r = rstd.reshape(B, S, 1)
    xhat = (xf - mu) * r
    xn = xhat.to(x.dtype)
    t = 1 + scale[:, None]
    gx = (grad * t).float()
    m1 = gx.sum(-1, keepdim=True) / C
    m2 = (gx * xhat).sum(-1, keepdim=True) / C
    dx = (r * (gx - m1 - xhat * m2)).to(x.dtype)
    dshift = grad.sum(1).to(scale.dtype)
    dscale = (grad * xn).sum(1).to(scale.dtype)
    return dx, dscale, dshift


def staged_gated_residual_adaln_fwd(h, attn, gate, scale, shift, eps: float = EPS):
    """Returns (h2, out, mean, rstd).  Rounding points: m = attn*gate; h2 = h+m; then the AdaLN chain."""
    m = attn * gate[:, None]
    h2 = h + m
    out, mean, rstd = staged_adaln_fwd(h2, scale, shift, eps)
    return h2, out, mean, rstd


def staged_gated_residual_adaln_bwd(h2, attn, gate, scale, mean, rstd, grad_out, grad_h2=None):
    """dxl = AdaLN dx (rounded); dh = round(dxl + grad_h2); dattn = round(dh*gate);
    dgate = sum_s round(dh*attn).  Returns (dh, dattn, dgate, dscale, dshift)."""
    dxl, dscale, dshift = staged_adaln_bwd(h2, scale, mean, rstd, grad_out)
    dh = dxl if grad_h2 is None else dxl + grad_h2
    dattn = dh * gate[:, None]
    dgate = (dh * attn).sum(1).to(gate.dtype)
    return dh, dattn, dgate, dscale, dshift


# --------------------------------------------------------------------------
# truth: float64 closed forms, no intermediate rounding
# --------------------------------------------------------------------------

def truth_gated_residual_adaln_fwd_bwd(h, attn, gate, scale, shift, grad_out, grad_h2=None,
                                       eps: float = EPS):
    """Returns (h2, out, dh, dattn, dgate, dscale, dshift) in float64."""
    hd, ad, qd = h.double(), attn.double(), gate.double()
    h2 = hd + ad * qd[:, None]
    out, dxl, dscale, dshift = truth_adaln_fwd_bwd(h2, scale, shift, grad_out, eps)
    dh = dxl if grad_h2 is None else dxl + grad_h2.double()
    return h2, out, dh, dh * qd[:, None], (dh * ad).sum(1), dscale, dshift


def truth_rmsnorm_fwd_bwd(x, weight, grad, eps: float = EPS):
    C = x.shape[-1]
    xd, wd, gd = x.double(), weight.double(), grad.double()
    r = 1.0 / torch.sqrt((xd * xd).mean(-1, keepdim=True) + eps)
    xhat = xd * r
    out = xhat * wd
    gy = gd * wd
    dx = r * (gy - xhat * (gy * xhat).sum(-1, keepdim=True) / C)
    dw = (gd * xhat).reshape(-1, C).sum(0)
    return out, dx, dw


def truth_adaln_fwd_bwd(x, scale, shift, grad, eps: float = EPS):
    B, S, C = x.shape
    xd, sd, hd, gd = x.double(), scale.double(), shift.double(), grad.double()
    mu = xd.mean(-1, keepdim=True)
    var = ((xd - mu) ** 2).mean(-1, keepdim=True)
    r = 1.0 / torch.sqrt(var + eps)
    xhat = (xd - mu) * r
    t = 1 + sd[:, None]
    out = xhat * t + hd[:, None]
    gx = gd * t
    dx = r * (gx - gx.mean(-1, keepdim=True) - xhat * (gx * xhat).mean(-1, keepdim=True))
    return out, dx, (gd * xhat).sum(1), gd.sum(1)


# --------------------------------------------------------------------------
# comparators
# --------------------------------------------------------------------------

def bf16_ordinal(t: torch.Tensor) -> torch.Tensor:
    """Monotone integer index of each bf16 value (adjacent values differ by 1;
    +0 and -0 share index 0)."""
    assert t.dtype in (torch.bfloat16, torch.float16)  # both are 16-bit sign-magnitude patterns
    bits = t.contiguous().view(torch.int16).to(torch.int32)
    return torch.where(bits >= 0, bits, -(bits & 0x7FFF))


def bf16_ulp_distance(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    return (bf16_ordinal(a) - bf16_ordinal(b)).abs()


@dataclass
class UlpReport:
    n: int
    n_exact: int
    n_gt1: int          # > 1 ulp and not excused
    n_excused: int      # > 1 ulp but within excuse_abs
    max_ulp: int

    @property
    def frac_exact(self) -> float:
        return self.n_exact / max(self.n, 1)


def compare_bf16_ulp(got: torch.Tensor, want: torch.Tensor,
                     excuse_abs: Optional[torch.Tensor] = None) -> UlpReport:
    """Element-wise bf16 ulp comparison.

    Two correct implementations of the eager chain sum a row in different
    orders (and may form (x-mu)*r differently), so the normalised value (y for
    RMSNorm, xn for AdaLN) can land on the other side of a rounding boundary:
    a step of one ulp, up to 2^-7 relative.  Eager then multiplies it, rounds,
    (AdaLN:) adds shift and rounds again, and each of those roundings can add
    half an ulp in either implementation.  The result can therefore differ by
    2-3 of its own ulp, or by many when p + shift cancels.  `excuse_abs` is the
    per-element absolute bound that chain allows; an element more than 1 ulp
    off is excused iff |got - want| <= excuse_abs.  Use rmsnorm_excuse() /
    adaln_excuse(); callers also bound how many elements are excused.
    """
    got, want = got.cpu(), want.cpu()
    d = bf16_ulp_distance(got, want)
    nan_both = torch.isnan(got) & torch.isnan(want)
    d = torch.where(nan_both, torch.zeros_like(d), d)
    bad = d > 1
    excused = torch.zeros_like(bad)
    if excuse_abs is not None and bad.any():
        diff = (got.float() - want.float()).abs()
        excused = bad & (diff <= excuse_abs.float().cpu())
    return UlpReport(n=d.numel(), n_exact=int((d == 0).sum()),
                     n_gt1=int((bad & ~excused).sum()), n_excused=int(excused.sum()),
                     max_ulp=int(d.max()) if d.numel() else 0)


def _ulp_rel(dtype: torch.dtype) -> float:
    """Largest relative size of one ulp: 2^-7 for bf16 (8 significant bits), 2^-10 for fp16 (11)."""
    return 2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7


def rmsnorm_excuse(want_out: torch.Tensor) -> torch.Tensor:
    """out = rnd(y*w): one-ulp step of y (<= u |y*w|) plus one ulp of out; u = 2^-7 for bf16."""
    return want_out.float().abs() * (2 * _ulp_rel(want_out.dtype))


def adaln_excuse(x, scale, shift, want_out, eps: float = EPS) -> torch.Tensor:
    """out = rnd(rnd(xn*t) + shift): one-ulp step of xn carried through t
    (<= u |p|), one ulp of p (<= u |p|), one ulp of out (<= u |out|); u = 2^-7 for bf16."""
    B, C = scale.shape
    x3 = x.reshape(B, -1, C)
    xn = F.layer_norm(x3, (C,), None, None, eps)
    p = (xn * (1 + scale[:, None])).float().abs().reshape(want_out.shape)
    u = _ulp_rel(want_out.dtype)
    return p * (2 * u) + want_out.float().abs() * u


def rope_excuse(y: torch.Tensor, want_out: torch.Tensor) -> torch.Tensor:
    """Rotated norm output: a one-ulp step of either element of a pair of y moves both rotated elements by up
    to u*(|y_even| + |y_odd|) (|cos|, |sin| <= 1), on top of the norm's own excuse and one ulp of the result."""
    u = _ulp_rel(want_out.dtype)
    yf = y.float().abs()
    pair = (yf[..., 0::2] + yf[..., 1::2]).repeat_interleave(2, dim=-1)
    return pair * (3 * u) + want_out.float().abs() * u


def frac_outside(got: torch.Tensor, want: torch.Tensor, rtol: float, atol: float,
                 magnitude: Optional[torch.Tensor] = None) -> float:
    """Fraction of elements with |got-want| > atol + rtol*|want| (allclose's rule).
    `magnitude`, when given, replaces |want| in the bound: for a result that is a sum of
    separately rounded terms (h2's gradient = the norm's dx + the upstream gradient) the honest
    scale of a one-ulp disagreement is the size of the terms, not of a sum that may cancel."""
    g, w = got.double().cpu(), want.double().cpu()
    if g.numel() == 0:
        return 0.0
    m = w.abs() if magnitude is None else magnitude.double().cpu().abs()
    return float(((g - w).abs() > atol + rtol * m).double().mean())


def adaln_dx_terms(x, scale, grad, eps: float = EPS) -> torch.Tensor:
    """Size of the three terms LayerNorm's backward adds, r*(|gx| + |mean gx| + |xhat * mean(gx*xhat)|).
    For short rows the two means are not small and the terms cancel; eager on the CPU moreover keeps
    mean and rstd of a 16-bit input in 16 bits, so its dx carries that rounding times the terms.
    Used as `magnitude` of frac_outside for dx of narrow rows."""
    xf = x.float()
    mu = xf.mean(-1, keepdim=True)
    r = torch.rsqrt(((xf - mu) ** 2).mean(-1, keepdim=True) + eps)
    xhat = (xf - mu) * r
    gx = (grad * (1 + scale[:, None])).float()
    return r * (gx.abs() + gx.mean(-1, keepdim=True).abs() + (xhat * (gx * xhat).mean(-1, keepdim=True)).abs())


def colsum_outside(got: torch.Tensor, want: torch.Tensor, terms: torch.Tensor, dim: int,
                   rtol: float = 1e-2, ulp: float = 2.0 ** -5) -> int:
    """Number of column sums with |got-want| > rtol*|want| + ulp*||terms||_2, the L2 norm taken over
    the summed dimension.  For a column sum whose TERMS are known to one rounding of the element
    type only (each may differ by an ulp between two correct implementations): such errors add
    like a random walk, so the column's L2 mass is their natural scale: a per-term error uniform
    within one ulp (2^-8 relative) gives a sum error of about 2^-8 * 0.8 * L2 at one sigma, and
    the eager result itself sits up to 2^-6 * L2 from the float64 truth over thousands of columns.
    A dropped or misplaced term moves a column by the order of L2 itself."""
    l2 = terms.double().cpu().pow(2).sum(dim).sqrt().reshape(want.shape)
    g, w = got.double().cpu().reshape(want.shape), want.double().cpu()
    return int(((g - w).abs() > rtol * w.abs() + ulp * l2).sum())


# --------------------------------------------------------------------------
# seeded inputs for the benchmark configurations
# --------------------------------------------------------------------------

def _gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def make_rmsnorm_inputs(lead_shape: Tuple[int, ...], cols: int, dtype: torch.dtype,
                        seed: int = 0, sigma: float = 1.0) -> Dict[str, torch.Tensor]:
    """x ~ N(0, sigma), weight ~ N(1, 0.02), upstream grad ~ N(0, 1)."""
    g = _gen(seed)
    x = (sigma * torch.randn(*lead_shape, cols, generator=g)).to(dtype)
    w = (1 + 0.02 * torch.randn(cols, generator=g)).to(dtype)
    grad = torch.randn(*lead_shape, cols, generator=g).to(dtype)
    return {"x": x, "weight": w, "grad": grad}


def make_adaln_inputs(batch: int, seq: int, cols: int, dtype: torch.dtype,
                      seed: int = 0, sigma: float = 1.0) -> Dict[str, torch.Tensor]:
    """x ~ N(0, sigma); per-sample scale, shift ~ N(0, 0.1); grad ~ N(0, 1)."""
    g = _gen(seed)
    x = (sigma * torch.randn(batch, seq, cols, generator=g)).to(dtype)
    scale = (0.1 * torch.randn(batch, cols, generator=g)).to(dtype)
    shift = (0.1 * torch.randn(batch, cols, generator=g)).to(dtype)
    grad = torch.randn(batch, seq, cols, generator=g).to(dtype)
    return {"x": x, "scale": scale, "shift": shift, "grad": grad}


CONFIGS = {
    # name: (op, kwargs) -- the five workloads of the benchmark definition
    "cfg1_rms_fp32": ("rmsnorm", dict(lead_shape=(2, 4096), cols=3072, dtype=torch.float32)),
    "cfg2_qk_rms_bf16": ("rmsnorm", dict(lead_shape=(1, 29700, 24), cols=128, dtype=torch.bfloat16)),
    "cfg3_adaln_bf16": ("adaln", dict(batch=1, seq=29700, cols=3072, dtype=torch.bfloat16)),
    "cfg4_rms_bf16": ("rmsnorm", dict(lead_shape=(1, 118800), cols=3072, dtype=torch.bfloat16)),
    "cfg4_adaln_bf16": ("adaln", dict(batch=1, seq=118800, cols=3072, dtype=torch.bfloat16)),
    "cfg5_adaln_bf16": ("adaln", dict(batch=4, seq=11056, cols=3072, dtype=torch.bfloat16, sigma=2.0)),
}


def make_gated_inputs(batch: int, seq: int, cols: int, dtype: torch.dtype, seed: int = 0,
                      with_grad_h2: bool = True):
    """(h, attn, gate, scale, shift, grad_out, grad_h2): a residual stream of O(1) entries with a
    per-row offset, attention output of O(1), gates and modulation of the size an adaLN-Zero linear
    produces after some training (|.| ~ 0.3)."""
    g = _gen(seed + 77)
    h = torch.randn(batch, seq, cols, generator=g) * (0.5 + torch.rand(batch, seq, 1, generator=g) * 1.5) \
        + torch.randn(batch, seq, 1, generator=g) * 0.3
    attn = torch.randn(batch, seq, cols, generator=g)
    gate = torch.randn(batch, cols, generator=g) * 0.3
    scale = torch.randn(batch, cols, generator=g) * 0.3
    shift = torch.randn(batch, cols, generator=g) * 0.3
    grad_out = torch.randn(batch, seq, cols, generator=g) * 0.1
    grad_h2 = torch.randn(batch, seq, cols, generator=g) * 0.1 if with_grad_h2 else None
    cast = lambda t: None if t is None else t.to(dtype)
    return tuple(cast(t) for t in (h, attn, gate, scale, shift, grad_out, grad_h2))


def make_config_inputs(name: str, seed: int = 0, rows_limit: Optional[int] = None):
    """Seeded inputs for one named configuration.  `rows_limit` shrinks the
    token dimension (for quick checks) without changing anything else."""
    op, kw = CONFIGS[name]
    kw = dict(kw)
    if op == "rmsnorm":
        if rows_limit is not None:
            lead = list(kw["lead_shape"])
            lead[1] = min(lead[1], rows_limit)
            kw["lead_shape"] = tuple(lead)
        return op, make_rmsnorm_inputs(seed=seed, **kw)
    if rows_limit is not None:
        kw["seq"] = min(kw["seq"], rows_limit)
    return op, make_adaln_inputs(seed=seed, **kw)
