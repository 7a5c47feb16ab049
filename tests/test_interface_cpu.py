"""CPU-side checks of the boundary: the C ABI library exports what the header
declares, the extension modules expose the reference's function names, host
argument checking works, and the module-level selection logic follows the
reference (eager math when FUSED_KERNELS is off).  No kernel is launched."""
import os
import re

import pytest
import torch

from oracle import norm_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions(header="teletron_norm.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tt_\w+)\s*\(", text)))


def test_c_abi_exports_every_declared_symbol():
    from teletron_amd import capi
    L = capi.lib()
    names = _declared_functions()
    assert len(names) >= 14
    for n in names:
        assert hasattr(L, n), f"{n} declared in teletron_norm.h but not exported"
    assert sorted(capi.EXPORTS) == names
    assert L.tt_norm_abi_version() == 3
    assert L.tt_norm_status_string(0) == b"ok"
    assert L.tt_norm_status_string(4).startswith(b"workspace")
    assert L.tt_norm_supported(3072, capi.BF16) == 1 and L.tt_norm_supported(128, capi.F32) == 1
    assert L.tt_norm_supported(3072, 5) == 0
    # every row of whole 16-byte pieces up to 1024 of them, in bf16 / fp16 / fp32
    assert L.tt_norm_supported(1024, capi.BF16) == 1 and L.tt_norm_supported(8192, capi.F16) == 1
    assert L.tt_norm_supported(4096, capi.F32) == 1 and L.tt_norm_supported(4100, capi.F32) == 0
    assert L.tt_norm_supported(1000, capi.F32) == 1 and L.tt_norm_supported(1004, capi.BF16) == 0
    assert L.tt_norm_supported(8200, capi.BF16) == 0
    # the tuned shapes: the only ones the reference-contract, strided and gated entry points take
    assert L.tt_norm_tuned(3072, capi.BF16) == 1 and L.tt_norm_tuned(128, capi.F32) == 1
    assert L.tt_norm_tuned(3072, capi.F16) == 1 and L.tt_norm_tuned(256, capi.BF16) == 0
    assert L.tt_rmsnorm_backward_from_out(None, None, None, None, None, None, 4, 256, 0, None, 0, None) == 2
    assert L.tt_adaln_forward_xnorm(None, None, None, None, None, None, 1, 4, 1536, 1e-6, capi.F16, None) == 2


def test_c_abi_argument_errors_need_no_gpu():
    from teletron_amd import capi
    L = capi.lib()
    assert L.tt_rmsnorm_forward(None, None, None, None, 4, 3072, 1e-6, 0, None) == 1      # null pointers
    assert L.tt_rmsnorm_forward(None, None, None, None, 4, 1004, 1e-6, 0, None) == 2      # unsupported cols
    assert b"cols=1004" in L.tt_norm_last_error()
    assert L.tt_rmsnorm_forward(None, None, None, None, 4, 1000, 1e-6, 0, None) == 1      # supported; null pointers
    assert L.tt_adaln_forward(None, None, None, None, None, None, 0, 4, 3072, 1e-6, 0, None) == 1


def test_probe_library_is_separate_and_exports_its_header():
    """The measurement kernels live in a library of their own: its header's symbols are exported there, none of
    them by the operator library, and its argument checks answer before anything is launched."""
    from teletron_amd import capi, probe
    P, L = probe.lib(), capi.lib()
    names = _declared_functions("teletron_probe.h")
    assert sorted(probe.EXPORTS) == names and len(names) == 4
    for n in names:
        assert hasattr(P, n), f"{n} declared in teletron_probe.h but not exported"
        assert not hasattr(L, n)
    for gone in ("tt_norm_stream_copy", "tt_norm_stream_probe"):
        assert not hasattr(L, gone)
    assert P.tt_probe_abi_version() == 1
    assert P.tt_probe_stream_copy(None, None, 32, None) == 1
    assert P.tt_probe_stream_copy(16, 16, 24, None) == 1                                  # not whole 16-byte pieces
    # allocation lengths are part of the call: the third and fourth tensor read and the second written
    # follow the first ones in the same allocations, and a call that would step outside is refused
    KiB = 1024
    ok = (0x10000, 8 * KiB, 0x20000, 8 * KiB, 0x30000, 8 * KiB)                          # (dst, len, a, len, b, len)
    assert P.tt_probe_stream(*ok, 4 * KiB, 3, 1, 1, 0, 0, None) != 1 or b"need" not in P.tt_probe_last_error()
    short = (0x10000, 4 * KiB, 0x20000, 4 * KiB, 0x30000, 4 * KiB)
    for reads, writes in ((3, 1), (4, 2), (2, 2)):
        assert P.tt_probe_stream(*short, 4 * KiB, reads, writes, 1, 0, 0, None) == 1
        assert b"need allocations" in P.tt_probe_last_error()
    assert P.tt_probe_stream(*short, 4 * KiB, 2, 1, 3, 0, 0, None) == 2                   # shape not built
    assert P.tt_probe_stream(*short, 4 * KiB + 16, 2, 1, 1, 0, 0, None) == 1              # not whole runs
    assert P.tt_probe_stream(*short, 4 * KiB, 0, 0, 1, 0, 0, None) == 1                   # no stream at all


def test_wide_forms_query_matches_the_python_gate():
    """tt_norm_wide_forms_supported: every supported row (whole 16-byte pieces, at most 1024 of them); the
    Python-side gate of the gated / residual Functions says the same for every width."""
    from teletron_amd import capi
    from teletron_amd import fusedlayers as FL
    L = capi.lib()
    for dt, code in ((torch.bfloat16, capi.BF16), (torch.float16, capi.F16), (torch.float32, capi.F32)):
        for cols in list(range(0, 8200, 4)) + [3072, 3080, 1536, 1540, 8192]:
            assert bool(L.tt_norm_wide_forms_supported(cols, code)) == FL.wide_forms_supported(cols, dt), (cols, dt)
    assert L.tt_norm_wide_forms_supported(3072, capi.F32) == 1 and L.tt_norm_wide_forms_supported(1540, capi.F32) == 1
    assert L.tt_norm_wide_forms_supported(3080, capi.BF16) == 1 and L.tt_norm_wide_forms_supported(8192, capi.BF16) == 1
    assert L.tt_norm_wide_forms_supported(4100, capi.F32) == 0 and L.tt_norm_wide_forms_supported(3076, capi.BF16) == 0
    assert L.tt_norm_wide_forms_supported(3072, 7) == 0
    # other rows: the three entry points answer TT_NORM_EUNSUPPORTED before touching a pointer
    assert L.tt_gated_residual_adaln_forward(*([None] * 9), 1, 4, 3076, 1e-6, capi.BF16, None) == 2
    assert L.tt_gated_residual_adaln_backward(*([None] * 13), 1, 4, 8200, capi.BF16, None, 0, None) == 2
    assert L.tt_adaln_backward_residual(*([None] * 9), 1, 4, 4100, capi.F32, None, 0, None) == 2
    assert L.tt_gated_residual_adaln_backward_workspace_bytes(1, 4, 3076, capi.BF16) == 0


def test_extension_modules_expose_reference_names():
    from teletron_amd import fusedlayers as FL
    assert FL.fused_kernels_available()
    for fn in ("torch_launch_rms_forward", "torch_launch_rms_backward", "torch_launch_rms_backward_x"):
        assert callable(getattr(FL.fused_rmsnorm, fn))
    for fn in ("torch_launch_adaln_forward", "torch_launch_adaln_backward",
               "torch_launch_adaln_forward_stats", "torch_launch_adaln_backward_x"):
        assert callable(getattr(FL.fused_adaln, fn))
    # operator-library registrations under the reference's namespaces
    assert hasattr(torch.ops.Fused_RMSNorm, "torch_launch_rms_forward")
    assert hasattr(torch.ops.layernorm_block_smem, "torch_launch_adaln_backward")
    FL.install_as_teletron_op()
    import fused_adaln
    import fused_rmsnorm
    assert fused_adaln is FL.fused_adaln and fused_rmsnorm is FL.fused_rmsnorm


def test_extension_rejects_cpu_tensors_loudly():
    from teletron_amd import fusedlayers as FL
    x = torch.zeros(2, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        FL.fused_rmsnorm.torch_launch_rms_forward(torch.empty_like(x), x, torch.ones(128, dtype=torch.bfloat16),
                                                  2, 128, 1e-6, torch.empty(2))
    with pytest.raises(ValueError, match="GPU tensor"):
        FL.RMSNormModelFunction.apply(x, torch.ones(128, dtype=torch.bfloat16), 1e-6, 128)
    with pytest.raises(ValueError, match="GPU tensor"):
        FL.AdaLNModelFunction.apply(torch.zeros(1, 2, 3072), torch.zeros(1, 3072), torch.zeros(1, 3072), 1e-6, 3072)


def test_adaln_custom_shape_errors():
    from teletron_amd import fusedlayers as FL
    m = FL.AdaLNCustom(3072)
    with pytest.raises(ValueError, match="input x"):
        m(torch.zeros(1, 2, 128), torch.zeros(1, 3072), torch.zeros(1, 3072))
    with pytest.raises(ValueError, match="scale"):
        m(torch.zeros(1, 2, 3072), torch.zeros(1, 128), torch.zeros(1, 3072))
    with pytest.raises(ValueError, match="shift"):
        m(torch.zeros(1, 2, 3072), torch.zeros(1, 3072), torch.zeros(1, 128))


def test_rmsnorm_module_env_gate_and_eager_branch(monkeypatch):
    from teletron_amd import fusedlayers as FL
    RMSNorm = FL.Get_RMSNorm()
    assert RMSNorm is FL.RMSNorm
    m = RMSNorm(128, config=None)
    assert m.weight.shape == (128,) and m.eps == 1e-6 and m.hidden_size == 128
    d = O.make_rmsnorm_inputs((5, 7), 128, torch.bfloat16, seed=1)
    with torch.no_grad():
        m.weight.copy_(d["weight"].float())
    m = m.bfloat16()
    monkeypatch.delenv("FUSED_KERNELS", raising=False)
    assert not FL.fused_kernels_requested()
    assert torch.equal(m(d["x"]), O.eager_rmsnorm(d["x"], d["weight"]))
    monkeypatch.setenv("FUSED_KERNELS", "0")
    assert not FL.fused_kernels_requested()
    assert torch.equal(m(d["x"]), O.eager_rmsnorm(d["x"], d["weight"]))
    monkeypatch.setenv("FUSED_KERNELS", "1")
    assert FL.fused_kernels_requested()
    with pytest.raises(ValueError, match="GPU tensor"):   # fused requested: no quiet CPU fallback
        m(d["x"])
    other = RMSNorm(98, config=None)                        # a width the kernels are not built for
    assert other(torch.ones(2, 98)).shape == (2, 98)        # (rows must be whole 16-byte pieces): eager
    assert FL.cols_supported(96, torch.float32) and FL.cols_supported(96, torch.float16)
    assert not FL.cols_supported(100, torch.bfloat16) and not FL.cols_supported(8200, torch.bfloat16)
    assert not FL.cols_supported(128, torch.float64)


def test_adaln_zero_modules_eager_branch_matches_oracle():
    from teletron_amd import fusedlayers as FL
    torch.manual_seed(0)
    B, S, C = 2, 5, 64
    x = torch.randn(B, S, C)
    temb = torch.randn(B, C)
    m6 = FL.FusedAdaLayerNormZero(C, linear_parallel=False)
    out, gate_msa, shift_mlp, scale_mlp, gate_mlp = m6(x, emb=temb)
    chunks = m6.linear(torch.nn.functional.silu(temb)).chunk(6, dim=1)
    torch.testing.assert_close(out, O.eager_adaln(x, chunks[1], chunks[0]))
    for got, want in zip((gate_msa, shift_mlp, scale_mlp, gate_mlp), chunks[2:]):
        assert torch.equal(got, want)
    m3 = FL.FusedAdaLayerNormZeroSingle(C, linear_parallel=False, norm_type="fp32_layer_norm")
    out3, gate3 = m3(x, emb=temb)
    c3 = m3.linear(torch.nn.functional.silu(temb)).chunk(3, dim=1)
    # the reference builds FP32LayerNorm without eps, i.e. with nn.LayerNorm's default 1e-5
    torch.testing.assert_close(out3, O.eager_adaln(x, c3[1], c3[0], eps=1e-5))
    assert torch.equal(gate3, c3[2])
    with pytest.raises(ValueError, match="norm_type"):
        FL.FusedAdaLayerNormZeroSingle(C, linear_parallel=False, norm_type="nope")
    with pytest.raises(ValueError, match="unsupported cols 66"):   # not whole 16-byte pieces
        FL.FusedAdaLayerNormZero(66, linear_parallel=False, fused_kernels=True)
    fused = FL.FusedAdaLayerNormZero(C, linear_parallel=False, fused_kernels=True)   # 64 columns: any-width kernels
    with pytest.raises(ValueError, match="GPU tensor"):                               # and no quiet CPU fallback
        fused(x, emb=temb)


def test_adaln_continuous_eager_branch():
    """dit_layerspec.py:72-78: x is sequence-first [S, B, C]; scale/shift [B, C] broadcast along dim -2."""
    from types import SimpleNamespace
    from teletron_amd import fusedlayers as FL
    torch.manual_seed(1)
    S, B, C, E = 7, 3, 64, 32
    m = FL.AdaLNContinuous(SimpleNamespace(hidden_size=C), E)
    x, cond = torch.randn(S, B, C), torch.randn(B, E)
    emb = m.adaLN_modulation(cond)
    scale, shift = emb[:, :C], emb[:, C:]
    want = O.eager_adaln(x.transpose(0, 1), scale, shift, 1e-6).transpose(0, 1)   # per-sample modulation
    torch.testing.assert_close(m(x, cond), want)
    r = FL.AdaLNContinuous(SimpleNamespace(hidden_size=C), E, norm_type="rms_norm")
    assert r(x, cond).shape == x.shape
    with pytest.raises(ValueError, match="Unknown normalization"):
        FL.AdaLNContinuous(SimpleNamespace(hidden_size=C), E, norm_type="nope")
    f = FL.AdaLNContinuous(SimpleNamespace(hidden_size=C), E, fused_kernels=True)
    with pytest.raises(ValueError, match="GPU tensor"):
        f(x, cond)


def test_fp32_layer_norm():
    from teletron_amd import fusedlayers as FL
    x = torch.randn(3, 64, generator=torch.Generator().manual_seed(0)).bfloat16()
    ln = FL.FP32LayerNorm(64, elementwise_affine=False, bias=False)
    want = torch.nn.functional.layer_norm(x.float(), (64,), None, None, ln.eps).bfloat16()
    assert torch.equal(ln(x), want)


def test_c_abi_accepts_zero_rows_without_a_gpu_launch():
    from teletron_amd import capi
    L = capi.lib()
    # forward over zero rows is a no-op: returns OK without touching any pointer
    assert L.tt_rmsnorm_forward(None, None, None, None, 0, 3072, 1e-6, 0, None) == 0
    assert L.tt_adaln_forward(None, None, None, None, None, None, 3, 0, 3072, 1e-6, 0, None) == 0
    assert L.tt_rmsnorm_forward(None, None, None, None, -1, 3072, 1e-6, 0, None) == 1
    assert L.tt_rmsnorm_backward_workspace_bytes(0, 3072, 0) == 0


def test_eager_fallback_switch_restores_the_reference_gating(monkeypatch):
    """TELETRON_AMD_FALLBACK=eager: with FUSED_KERNELS on, a tensor the fused path cannot take (here: on the CPU;
    also a weight of another dtype, or a missing extension) is computed by the eager formula, silently, as
    the reference does (dit_fusedlayers.py:194-204, 364-370).  Without the switch the same call raises."""
    from teletron_amd import fusedlayers as FL
    monkeypatch.setenv("FUSED_KERNELS", "1")
    monkeypatch.delenv("TELETRON_AMD_FALLBACK", raising=False)
    x = torch.randn(3, 5, 128).bfloat16()
    norm = FL.RMSNorm(128).bfloat16()
    with pytest.raises(ValueError, match="GPU tensor"):
        norm(x)
    ada = FL.FusedAdaLayerNormZeroSingle(256, fused_kernels=True, linear_parallel=False)
    h, temb = torch.randn(2, 7, 256), torch.randn(2, 256)
    with pytest.raises(ValueError, match="GPU tensor"):
        ada(h, emb=temb)
    monkeypatch.setenv("TELETRON_AMD_FALLBACK", "eager")
    assert FL.eager_fallback_enabled()
    assert torch.equal(norm(x), O.eager_rmsnorm(x, norm.weight))
    out, gate = ada(h, emb=temb)
    c = ada.linear(torch.nn.functional.silu(temb)).chunk(3, dim=1)
    torch.testing.assert_close(out, O.eager_adaln(h, c[1], c[0]))
    # an fp32 weight with a bf16 input: eager promotes to fp32, and so does the fallback
    mixed = FL.RMSNorm(128)
    assert mixed(x).dtype == torch.float32
    # the constructor gate: a width the kernels do not take builds the eager norm instead of raising
    odd = FL.FusedAdaLayerNormZero(66, fused_kernels=True, linear_parallel=False)
    assert odd.fused_kernels is False and isinstance(odd.norm, torch.nn.LayerNorm)
    monkeypatch.setenv("TELETRON_AMD_FALLBACK", "")
    with pytest.raises(ValueError, match="unsupported cols 66"):
        FL.FusedAdaLayerNormZero(66, fused_kernels=True, linear_parallel=False)
