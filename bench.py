#!/usr/bin/env python3
"""Benchmark of the fused normalization hot path on one MI355X.

One step = fused RMSNorm(3072) forward + backward and fused AdaLN(3072) forward
+ backward over 118 800 x 3072 bf16 tokens (a full 129-frame 720p sequence),
through the C ABI, inputs resident in HBM.  Reports whole-step algorithmic
GB/s (5 * N * C * 2 bytes per operator: forward reads x and writes out,
backward reads grad and x and writes dx), the roofline fraction of the slowest
call measured with HIP events, and the reference's eager path timed on the
host CPU on a bounded sample of the same workload.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

`--workload` selects one of the other configurations (cfg1, cfg2, cfg2-strided, cfg3, cfg5) or
the gated residual + AdaLN call site instead; same timing method, same JSON line, no CPU leg.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

ROWS, COLS = 118800, 3072
EPS = 1e-6
HBM_PEAK_GBS = 8000.0

def measured_cfg4_profile():
    """profiles/cfg4_traffic.json: per C-ABI call the row kernel's symbol and its HBM bytes per launch from
    rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by the same counters on the plain copy kernel), written
    by `python -m teletron_amd.profile_summary cfg4` together with profiles/bench_cfg4_all_kernels.md.  Returns
    ({call: record}, valid): valid only while the kernel sources are the ones that were profiled."""
    from teletron_amd.build import kernel_source_digest
    path = os.path.join(ROOT, "profiles", "cfg4_traffic.json")
    if not os.path.exists(path):
        return {}, False
    with open(path) as f:
        rec = json.load(f)
    return rec.get("calls", {}), rec.get("source_digest") == kernel_source_digest()


WORKLOADS = {
    "cfg4": "cfg4: 118800 tokens x 3072 bf16; fused RMSNorm(3072) fwd+bwd + fused AdaLN fwd+bwd "
            "per step (4 C-ABI calls), eps 1e-6, one modulation row",
    "cfg1": "cfg1: 8192 x 3072 fp32; fused RMSNorm fwd+bwd (2 C-ABI calls)",
    "cfg2": "cfg2: q and k of one CP=4 rank, [1, 29700, 24, 128] bf16 each, contiguous; per-head RMSNorm(128) "
            "fwd+bwd on both (4 C-ABI calls)",
    "cfg2-strided": "cfg2 on the call site's own layout: q and k are transposed [B, H, S, D] views into the fused "
                    "[1, 29700, 24, 384] QKV projection, read in place; outputs and dx contiguous (4 C-ABI calls)",
    "cfg2-strided-rope": "cfg2-strided with the rotary embedding applied behind each norm (fp32 cos/sin tables "
                         "[29700, 128], every token rotated), forward and backward (4 C-ABI calls; the tables' bytes "
                         "are not counted)",
    "cfg3": "cfg3: 29700 tokens x 3072 bf16; fused AdaLN fwd+bwd (2 C-ABI calls)",
    "cfg5": "cfg5: batch 4 x 11056 tokens x 3072 bf16, one modulation row per sample; AdaLN then RMSNorm(3072), "
            "forward and backward of the chain (4 C-ABI calls)",
    "w1536-f16": "237600 tokens x 1536 fp16 (a smaller model's hidden size, the any-width kernels); fused RMSNorm "
                 "fwd+bwd + fused AdaLN fwd+bwd per step (4 C-ABI calls)",
    "w4096-bf16": "89100 tokens x 4096 bf16 (a wider model's hidden size; rows of 512 16-byte pieces, four wavefronts "
                  "per row); fused RMSNorm fwd+bwd + fused AdaLN fwd+bwd per step (4 C-ABI calls)",
    "w5120-bf16": "71280 tokens x 5120 bf16 (640 pieces per row); the same step",
    "w8192-bf16": "44550 tokens x 8192 bf16 (1024 pieces per row, the widest supported); the same step",
    "w4096-bf16-gated": "89100 tokens x 4096 bf16; gated residual update fused with the AdaLN that follows it, forward "
                        "+ backward with a gradient on h2, on the wide-row kernels (2 C-ABI calls)",
    "cfg4-eager-gpu": "cfg4's step computed by the reference's eager formulas as PyTorch ops on the same GPU "
                      "(what the reference runs with FUSED_KERNELS off): a baseline, not this library",
    "qkv-site": "the QK-norm call site through the autograd Function: [1, 29700, 24, 384] bf16 fused projection -> "
                "q, k normalised [B, H, S, 128] + v view, forward + backward with the projection's gradient "
                "assembled in place (QKVSplitNormFunction); traffic counted as 12 slice-sized tensors",
    "qkv-site-reference": "the same call site the reference's way with these kernels: torch.split, transpose, "
                          "contiguous copy, dense RMSNorm Function per tensor, torch.split's backward; same "
                          "traffic accounting as qkv-site (12 slice-sized tensors of useful work)",
    "stream-ceiling": "plain streams over 729.9 MB tensors: 0-2 tensors read, 0-1 written, 1/2/6 KiB per wavefront per "
                      "tensor, one-shot and persistent grids, streaming and write-through stores; the 3+1, 2+2 and 4+2 "
                      "mixes of the residual and gated kernels; plus the runtime's "
                      "and PyTorch's copies (no normalization arithmetic: the bandwidth envelope the kernels live in)",
    "qkv-site-rope": "the QK-norm call site including the rotary embedding the attention forward applies to q and k "
                     "behind the norms (fp32 cos/sin tables [29700, 128]): QKVSplitNormFunction with the tables, "
                     "forward + backward; traffic counted as 12 slice-sized tensors plus the two tables once per "
                     "kernel launch (4 launches)",
    "qkv-site-rope-reference": "the same call site the reference's way with these kernels: torch.split, transpose, "
                               "contiguous copy, dense RMSNorm Function per tensor, then the rotary embedding as "
                               "PyTorch ops (the published apply_rotary_emb formula), torch.split's backward; same "
                               "traffic accounting as qkv-site-rope",
    "cached-set": "the four cfg4 kernels on working sets that stay in the 256 MB last-level cache (4096 and 8192 rows x "
                  "3072 bf16, the same buffers launch after launch): what the kernels' own instruction streams "
                  "allow when memory is not the limit, as the per-row slope between the two sizes",
    "timeline-cfg3": "cfg3's step (AdaLN forward, backward, column reducer; 29700 x 3072 bf16, three rotating buffer "
                     "sets, back to back) seen from inside: every wavefront's start and end on the constant 100 MHz "
                     "clock, from a measurement build of the library (python -m teletron_amd.build --variant LIB "
                     "--flag=-DTTN_WAVE_CLOCK=1, loaded with TELETRON_AMD_LIB=LIB); --steps = timelines collected",
    "timeline-cfg4": "the same view of cfg4's step (118800 x 3072 bf16, one buffer set): the AdaLN forward and backward "
                     "kernels and the last column reducer of the step carry the clocks",
    "gated": "118800 tokens x 3072 bf16; gated residual update fused with the AdaLN that follows it, forward "
             "(2 reads, 2 writes) + backward with a gradient on h2 (4 reads, 2 writes) (2 C-ABI calls)",
}


# The HIP stream every call is enqueued on (looked up at call time: graph capture swaps it).
_LAUNCH_STREAM = [None]


def build_workload(name, torch, capi, dev):
    """Allocates the inputs of one workload in HBM and returns (calls, tensor_bytes, tokens_per_step, dtype)
    with calls = [(call name, closure, algorithmic traffic in tensors)]."""
    L = capi.lib()
    gen = torch.Generator(device=dev).manual_seed(0)
    p = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())
    _LAUNCH_STREAM[0] = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)

    def ck(st, what):
        if st != 0:
            raise RuntimeError(f"{what}: {L.tt_norm_last_error().decode()}")

    def rnd(*shape, dtype, k=1.0, bias=0.0):
        return (bias + k * torch.randn(*shape, device=dev, generator=gen)).to(dtype)

    f32 = lambda n: torch.empty(n, device=dev, dtype=torch.float32)
    scratch = lambda n: torch.empty(max(int(n), 16), device=dev, dtype=torch.uint8)

    def rms_pair(x, grad, w, tag=""):
        rows, cols = x.numel() // x.shape[-1], x.shape[-1]
        dt = capi._DTYPES[x.dtype]
        out, dx, rstd, dw = torch.empty_like(x), torch.empty_like(x), f32(rows), torch.empty_like(w)
        n = L.tt_rmsnorm_backward_workspace_bytes(rows, cols, dt)
        ws = scratch(n)
        fwd = lambda: ck(L.tt_rmsnorm_forward(p(out), p(rstd), p(x), p(w), rows, cols, EPS, dt, _LAUNCH_STREAM[0]), "rms fwd")
        bwd = lambda: ck(L.tt_rmsnorm_backward(p(dx), p(dw), p(grad), p(x), p(w), p(rstd), rows, cols, dt, p(ws), n,
                                               _LAUNCH_STREAM[0]), "rms bwd")
        return [("rmsnorm_forward" + tag, fwd, 2), ("rmsnorm_backward" + tag, bwd, 3)], out

    def adaln_pair(x, grad, scale, shift):
        batch, cols = scale.shape
        rps = x.numel() // cols // batch
        dt = capi._DTYPES[x.dtype]
        out, dx = torch.empty_like(x), torch.empty_like(x)
        mean, rstd = f32(batch * rps), f32(batch * rps)
        dsc, dsh = torch.empty_like(scale), torch.empty_like(scale)
        n = L.tt_adaln_backward_workspace_bytes(batch, rps, cols, dt)
        ws = scratch(n)
        fwd = lambda: ck(L.tt_adaln_forward(p(out), p(mean), p(rstd), p(x), p(scale), p(shift), batch, rps, cols,
                                            EPS, dt, _LAUNCH_STREAM[0]), "adaln fwd")
        bwd = lambda: ck(L.tt_adaln_backward(p(dx), p(dsc), p(dsh), p(grad), p(x), p(scale), p(mean), p(rstd), batch,
                                             rps, cols, dt, p(ws), n, _LAUNCH_STREAM[0]), "adaln bwd")
        return [("adaln_forward", fwd, 2), ("adaln_backward", bwd, 3)], out

    bf = torch.bfloat16
    if name in ("cfg4", "cfg3", "w1536-f16", "w4096-bf16", "w5120-bf16", "w8192-bf16"):
        rows, cols, dt = {"cfg4": (ROWS, COLS, bf), "cfg3": (29700, COLS, bf),
                          "w1536-f16": (2 * ROWS, 1536, torch.float16), "w4096-bf16": (89100, 4096, bf),
                          "w5120-bf16": (71280, 5120, bf), "w8192-bf16": (44550, 8192, bf)}[name]
        x, grad = rnd(rows, cols, dtype=dt), rnd(rows, cols, dtype=dt)
        scale, shift = rnd(1, cols, dtype=dt, k=0.1), rnd(1, cols, dtype=dt, k=0.1)
        calls = []
        if name != "cfg3":
            calls += rms_pair(x, grad, rnd(cols, dtype=dt, k=0.02, bias=1.0))[0]
        calls += adaln_pair(x, grad, scale, shift)[0]
        return calls, rows * cols * 2, rows * (1 if name == "cfg3" else 2), "f16" if dt != bf else "bf16", x
    if name == "cfg1":
        x, grad = rnd(8192, COLS, dtype=torch.float32), rnd(8192, COLS, dtype=torch.float32)
        calls, _ = rms_pair(x, grad, rnd(COLS, dtype=torch.float32, k=0.02, bias=1.0))
        return calls, 8192 * COLS * 4, 8192, "f32", x
    if name == "cfg2":
        calls = []
        for tag in ("_q", "_k"):
            x, grad = rnd(712800, 128, dtype=bf), rnd(712800, 128, dtype=bf)
            calls += rms_pair(x, grad, rnd(128, dtype=bf, k=0.02, bias=1.0), tag)[0]
        return calls, 712800 * 128 * 2, 29700, "bf16", x
    if name in ("cfg2-strided", "cfg2-strided-rope"):
        B, S, H, D = 1, 29700, 24, 128
        mixed = rnd(B, S, H, 3 * D, dtype=bf)
        calls = []
        rope = name.endswith("-rope")
        if rope:   # any fp32 tables do for timing; [S, D] as get_1d_rotary_pos_embed(use_real=True) lays them out
            ang = torch.rand(S, D // 2, device=dev, generator=gen) * 6.28
            cos, sin = (t.repeat_interleave(2, dim=1).contiguous() for t in (ang.cos(), ang.sin()))
        for i, tag in enumerate(("_q", "_k")):
            view = mixed[..., i * D:(i + 1) * D].transpose(1, 2)          # [B, H, S, D], strides (S*H*3D, 3D, H*3D, 1)
            grad = rnd(B, H, S, D, dtype=bf)
            w = rnd(D, dtype=bf, k=0.02, bias=1.0)
            out, dx, rstd, dw = torch.empty_like(grad), torch.empty_like(grad), f32(B * H * S), torch.empty_like(w)
            xs, ds = view.stride(), dx.stride()
            n = L.tt_rmsnorm_backward_workspace_bytes(B * H * S, D, capi.BF16)
            ws = scratch(n)
            fwd = (lambda out=out, rstd=rstd, view=view, w=w, xs=xs:
                   ck(L.tt_rmsnorm_forward_strided(p(out), p(rstd), p(view), p(w), B, H, S, xs[0], xs[1], xs[2], D,
                                                   EPS, capi.BF16, _LAUNCH_STREAM[0]), "rms fwd strided"))
            bwd = (lambda dx=dx, dw=dw, grad=grad, view=view, w=w, rstd=rstd, xs=xs, ds=ds, ws=ws, n=n:
                   ck(L.tt_rmsnorm_backward_strided(p(dx), p(dw), p(grad), p(view), p(w), p(rstd), B, H, S, xs[0],
                                                    xs[1], xs[2], ds[0], ds[1], ds[2], D, capi.BF16, p(ws), n,
                                                    _LAUNCH_STREAM[0]), "rms bwd strided"))
            if rope:
                fwd = (lambda out=out, rstd=rstd, view=view, w=w, xs=xs:
                       ck(L.tt_rmsnorm_rope_forward_strided(p(out), p(rstd), p(view), p(w), p(cos), p(sin), S, B, H, S,
                                                            xs[0], xs[1], xs[2], D, EPS, capi.BF16, _LAUNCH_STREAM[0]),
                          "rms rope fwd strided"))
                bwd = (lambda dx=dx, dw=dw, grad=grad, view=view, w=w, rstd=rstd, xs=xs, ds=ds, ws=ws, n=n:
                       ck(L.tt_rmsnorm_rope_backward_strided(p(dx), p(dw), p(grad), p(view), p(w), p(rstd), p(cos), p(sin),
                                                             S, B, H, S, xs[0], xs[1], xs[2], ds[0], ds[1], ds[2], D,
                                                             capi.BF16, p(ws), n, _LAUNCH_STREAM[0]), "rms rope bwd strided"))
            calls += [("rmsnorm_forward_strided" + tag, fwd, 2), ("rmsnorm_backward_strided" + tag, bwd, 3)]
        return calls, B * H * S * D * 2, S, "bf16", mixed
    if name == "cfg5":
        B, S = 4, 11056
        x, grad = rnd(B, S, COLS, dtype=bf, k=2.0), rnd(B, S, COLS, dtype=bf)
        scale, shift = rnd(B, COLS, dtype=bf, k=0.1), rnd(B, COLS, dtype=bf, k=0.1)
        ada, y = adaln_pair(x, grad, scale, shift)
        ada[0][1]()                                                         # y = AdaLN(x) feeds the RMSNorm
        rms, _ = rms_pair(y, grad, rnd(COLS, dtype=bf, k=0.02, bias=1.0))
        # chain order: AdaLN fwd, RMSNorm fwd, RMSNorm bwd, AdaLN bwd (the gradient buffers are stand-ins of the
        # right size: timing does not depend on their values)
        return [ada[0], rms[0], rms[1], ada[1]], B * S * COLS * 2, B * S, "bf16", x
    if name == "cfg4-eager-gpu":
        x = rnd(1, ROWS, COLS, dtype=bf).requires_grad_(True)
        grad = rnd(1, ROWS, COLS, dtype=bf)
        w = rnd(COLS, dtype=bf, k=0.02, bias=1.0).requires_grad_(True)
        scale, shift = (rnd(1, COLS, dtype=bf, k=0.1).requires_grad_(True) for _ in range(2))

        def eager_rmsnorm():     # teletron/models/dit/dit_fusedlayers.py:360-370
            y = (x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + EPS)).type_as(x) * w
            y.backward(grad)
            x.grad = None

        def eager_adaln():       # teletron/models/dit/dit_fusedlayers.py:198,223
            y = torch.nn.functional.layer_norm(x, (COLS,), None, None, EPS) * (1 + scale[:, None]) + shift[:, None]
            y.backward(grad)
            x.grad = None

        return [("eager_rmsnorm_fwd_bwd", eager_rmsnorm, 5), ("eager_adaln_fwd_bwd", eager_adaln, 5)], \
            ROWS * COLS * 2, 2 * ROWS, "bf16", grad
    if name in ("qkv-site-rope", "qkv-site-rope-reference"):
        from teletron_amd import fusedlayers as FL
        B, S, H, D = 1, 29700, 24, 128
        mixed = rnd(B, S, H, 3 * D, dtype=bf).requires_grad_(True)
        wq = rnd(D, dtype=bf, k=0.02, bias=1.0).requires_grad_(True)
        wk = rnd(D, dtype=bf, k=0.02, bias=1.0).requires_grad_(True)
        gq, gk, gv = (rnd(B, H, S, D, dtype=bf) for _ in range(3))
        ang = torch.outer(torch.arange(S, device=dev, dtype=torch.float32),
                          1.0 / (256.0 ** (torch.arange(0, D, 2, device=dev, dtype=torch.float32) / D)))
        cos, sin = ang.cos().repeat_interleave(2, dim=1).contiguous(), ang.sin().repeat_interleave(2, dim=1).contiguous()

        def fused():
            q, k, v = FL.QKVSplitNormFunction.apply(mixed, wq, wk, EPS, cos, sin)
            torch.autograd.backward([q, k, v], [gq, gk, gv])
            mixed.grad = None

        def reference_way():
            q, k, v = torch.split(mixed, [D, D, D], dim=3)
            q, k, v = q.transpose(1, 2).contiguous(), k.transpose(1, 2).contiguous(), v.transpose(1, 2)
            q = FL.rotate_pairs_eager(FL.RMSNormModelFunction.apply(q, wq, EPS, D), cos, sin)
            k = FL.rotate_pairs_eager(FL.RMSNormModelFunction.apply(k, wk, EPS, D), cos, sin)
            torch.autograd.backward([q, k, v], [gq, gk, gv])
            mixed.grad = None

        fn = fused if name == "qkv-site-rope" else reference_way
        slice_bytes = B * H * S * D * 2
        tensors = 12 + 4 * (2 * S * D * 4) / slice_bytes
        return [(name.replace("-", "_") + "_fwd_bwd", fn, tensors)], slice_bytes, S, "bf16", gq
    if name in ("qkv-site", "qkv-site-reference"):
        from teletron_amd import fusedlayers as FL
        B, S, H, D = 1, 29700, 24, 128
        mixed = rnd(B, S, H, 3 * D, dtype=bf).requires_grad_(True)
        wq = rnd(D, dtype=bf, k=0.02, bias=1.0).requires_grad_(True)
        wk = rnd(D, dtype=bf, k=0.02, bias=1.0).requires_grad_(True)
        gq, gk, gv = (rnd(B, H, S, D, dtype=bf) for _ in range(3))

        def fused():
            q, k, v = FL.QKVSplitNormFunction.apply(mixed, wq, wk, EPS)
            torch.autograd.backward([q, k, v], [gq, gk, gv])
            mixed.grad = None

        def reference_way():
            q, k, v = torch.split(mixed, [D, D, D], dim=3)
            q, k, v = q.transpose(1, 2).contiguous(), k.transpose(1, 2).contiguous(), v.transpose(1, 2)
            q = FL.RMSNormModelFunction.apply(q, wq, EPS, D)
            k = FL.RMSNormModelFunction.apply(k, wk, EPS, D)
            torch.autograd.backward([q, k, v], [gq, gk, gv])
            mixed.grad = None

        fn = fused if name == "qkv-site" else reference_way
        return [(name.replace("-", "_") + "_fwd_bwd", fn, 12)], B * H * S * D * 2, S, "bf16", gq
    if name in ("gated", "w4096-bf16-gated"):
        B, S, W = (1, ROWS, COLS) if name == "gated" else (1, 89100, 4096)
        h, a = rnd(B, S, W, dtype=bf), rnd(B, S, W, dtype=bf)
        go, g2 = rnd(B, S, W, dtype=bf, k=0.1), rnd(B, S, W, dtype=bf, k=0.1)
        gate, scale, shift = (rnd(B, W, dtype=bf, k=0.3) for _ in range(3))
        h2, out, dh, da = (torch.empty_like(h) for _ in range(4))
        mean, rstd = f32(B * S), f32(B * S)
        dq, dsc, dsh = (torch.empty_like(gate) for _ in range(3))
        n = L.tt_gated_residual_adaln_backward_workspace_bytes(B, S, W, capi.BF16)
        ws = scratch(n)
        fwd = lambda: ck(L.tt_gated_residual_adaln_forward(p(h2), p(out), p(mean), p(rstd), p(h), p(a), p(gate),
                                                           p(scale), p(shift), B, S, W, EPS, capi.BF16, _LAUNCH_STREAM[0]),
                         "gated fwd")
        bwd = lambda: ck(L.tt_gated_residual_adaln_backward(p(dh), p(da), p(dq), p(dsc), p(dsh), p(go), p(g2), p(h2),
                                                            p(a), p(gate), p(scale), p(mean), p(rstd), B, S, W,
                                                            capi.BF16, p(ws), n, _LAUNCH_STREAM[0]), "gated bwd")
        return [("gated_residual_adaln_forward", fwd, 4), ("gated_residual_adaln_backward", bwd, 6)], \
            S * W * 2, S, "bf16", h
    raise ValueError(name)


def stream_ceiling(args, torch, capi, dev):
    """What the memory system gives plain streams of each read/write mix and access shape (the probe
    library's kernels over cfg4-sized tensors), next to two copies not written here: the runtime's
    device-to-device copy and a PyTorch elementwise copy.  Every figure is back-to-back launches between
    two events."""
    from teletron_amd import probe as P
    nbytes = ROWS * COLS * 2
    # two tensors per allocation: the probe's third and fourth read and its second write follow the first
    a = torch.empty(2 * nbytes, dtype=torch.uint8, device=dev).random_(0, 255)
    b = torch.empty(2 * nbytes, dtype=torch.uint8, device=dev).random_(0, 255)
    d = torch.empty(2 * nbytes, dtype=torch.uint8, device=dev)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    hip = ctypes.CDLL("libamdhip64.so")

    def timed(fn, n_streams):
        for _ in range(max(3, args.warmup // 4)):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) / args.steps * 1e3
        return {"us": round(us, 1), "GB/s": round(n_streams * nbytes / us / 1e3, 1),
                "frac_of_peak": round(n_streams * nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}

    def probe(reads, writes, per_lane, blocks, through):
        return timed(lambda: P.stream(d, a, b, nbytes, reads, writes, per_lane, blocks, through), reads + writes)

    rows = []
    for reads, writes in ((1, 0), (2, 0), (0, 1), (1, 1), (2, 1)):
        for per_lane in (1, 2, 6):
            for blocks in (0, 256, 1024):
                for through in ((0, 1) if writes and per_lane == 6 else (0,)):
                    r = probe(reads, writes, per_lane, blocks, through)
                    r.update({"reads": reads, "writes": writes, "KiB_per_wavefront_per_tensor": per_lane,
                              "grid": "one-shot" if blocks == 0 else f"persistent {blocks} workgroups",
                              "store": "write-through" if through else ("streaming" if writes else "-")})
                    rows.append(r)
    # the mixes of the residual (3 + 1) and gated kernels (forward 2 + 2, backward 4 + 2)
    for reads, writes in ((3, 1), (2, 2), (4, 2)):
        for per_lane in (1, 6):
            for blocks in (0, 256, 1024):
                for through in (0, 1):
                    r = probe(reads, writes, per_lane, blocks, through)
                    r.update({"reads": reads, "writes": writes, "KiB_per_wavefront_per_tensor": per_lane,
                              "grid": "one-shot" if blocks == 0 else f"persistent {blocks} workgroups",
                              "store": "write-through" if through else "streaming"})
                    rows.append(r)
    d1, a1 = d[:nbytes], a[:nbytes]
    others = {
        "hipMemcpyDtoDAsync": timed(lambda: hip.hipMemcpyDtoDAsync(p(d), p(a), ctypes.c_size_t(nbytes), stream), 2),
        "torch copy_ (bf16)": timed(lambda: d1.view(torch.bfloat16).copy_(a1.view(torch.bfloat16)), 2),
        "torch zero_ (write only)": timed(lambda: d1.view(torch.bfloat16).zero_(), 1),
        "tt_probe_stream_copy": timed(lambda: P.stream_copy(d1, a1), 2),
    }
    best = lambda r_, w_: max((r for r in rows if r["reads"] == r_ and r["writes"] == w_), key=lambda r: r["GB/s"])
    two_one = best(2, 1)
    print(json.dumps({
        "metric": "plain-stream HBM GB/s per read/write mix (ceiling probe), 729.9 MB per tensor",
        "value": two_one["GB/s"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(two_one["us"] / 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": WORKLOADS["stream-ceiling"], "tensor_bytes": nbytes},
        "best": {"read_only": best(1, 0), "two_reads": best(2, 0), "write_only": best(0, 1),
                 "copy_1R_1W": best(1, 1), "2R_1W": two_one, "3R_1W": best(3, 1), "2R_2W": best(2, 2),
                 "4R_2W": best(4, 2)},
        "probes": rows, "other_copies": others,
    }))


def cached_set(args, torch, capi, dev):
    """The cfg4 kernels with memory taken out of the picture as far as this part allows: 4096 and 8192 rows (25 and
    50 MB per tensor; a backward call touches three of them), the same buffers launch after launch, so every
    launch after the first finds its working set in the 256 MB last-level cache.  Both sizes give every one of the
    1024 wavefronts of a backward grid whole rows (4 and 8), so the difference between them is the steady-state
    cost of 4 rows per wavefront without the launch, the parameter loads and the final reduction; scaled to the
    116 rows per wavefront of the full problem it says how fast the kernel's own instruction stream could go."""
    L = capi.lib()
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    bf = torch.bfloat16
    gen = torch.Generator(device=dev).manual_seed(0)
    big = 8192
    x = torch.randn(big, COLS, device=dev, generator=gen).to(bf)
    g = torch.randn(big, COLS, device=dev, generator=gen).to(bf)
    w = (1 + 0.02 * torch.randn(COLS, device=dev, generator=gen)).to(bf)
    sc, sh = ((0.1 * torch.randn(1, COLS, device=dev, generator=gen)).to(bf) for _ in range(2))
    out, dx = torch.empty_like(x), torch.empty_like(x)
    rstd, mean = (torch.empty(big, device=dev, dtype=torch.float32) for _ in range(2))
    dw, dsc, dsh = torch.empty_like(w), torch.empty_like(sc), torch.empty_like(sc)
    n = max(L.tt_rmsnorm_backward_workspace_bytes(big, COLS, capi.BF16),
            L.tt_adaln_backward_workspace_bytes(1, big, COLS, capi.BF16))
    ws = torch.empty(n, device=dev, dtype=torch.uint8)

    def calls(rows):
        return {
            "rmsnorm_forward": (2, lambda: L.tt_rmsnorm_forward(p(out), p(rstd), p(x), p(w), rows, COLS, EPS, capi.BF16, stream)),
            "rmsnorm_backward": (3, lambda: L.tt_rmsnorm_backward(p(dx), p(dw), p(g), p(x), p(w), p(rstd), rows, COLS,
                                                                  capi.BF16, p(ws), n, stream)),
            "adaln_forward": (2, lambda: L.tt_adaln_forward(p(out), p(mean), p(rstd), p(x), p(sc), p(sh), 1, rows, COLS, EPS,
                                                            capi.BF16, stream)),
            "adaln_backward": (3, lambda: L.tt_adaln_backward(p(dx), p(dsc), p(dsh), p(g), p(x), p(sc), p(mean), p(rstd), 1,
                                                              rows, COLS, capi.BF16, p(ws), n, stream)),
        }

    def timed(fn):
        for _ in range(max(5, args.warmup)):
            if fn() != 0:
                raise RuntimeError(L.tt_norm_last_error().decode())
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps * 1e3

    # forward calls first so that rstd / mean hold real statistics for the backward ones
    small, large = calls(big // 2), calls(big)
    res = {}
    for name in ("rmsnorm_forward", "adaln_forward", "rmsnorm_backward", "adaln_backward"):
        mult = large[name][0]
        t_large = timed(large[name][1])
        t_small = timed(small[name][1])
        slope = (t_large - t_small) / (big // 2)                    # us per row, all wavefronts working
        full = slope * ROWS
        res[name] = {"us_4096_rows": round(t_small, 2), "us_8192_rows": round(t_large, 2),
                     "us_per_1024_rows": round(slope * 1024, 3),
                     "cfg4_us_at_this_rate": round(full, 1),
                     "GB/s_at_this_rate": round(mult * ROWS * COLS * 2 / full / 1e3, 0),
                     "frac_of_hbm_peak_at_this_rate": round(mult * ROWS * COLS * 2 / full / 1e3 / HBM_PEAK_GBS, 3)}
    worst = min(res.values(), key=lambda r: r["GB/s_at_this_rate"])
    print(json.dumps({
        "metric": "rate of the cfg4 kernels on a cache-resident working set (instruction-stream ceiling), GB/s equivalent",
        "value": worst["GB/s_at_this_rate"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sum(r["us_8192_rows"] for r in res.values()) / 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": WORKLOADS["cached-set"], "rows": [big // 2, big], "cols": COLS},
        "kernels": res,
    }))


def wave_timeline(args, torch, capi, dev):
    """Where a short step spends its time: the ramp of each kernel (first to last wavefront start), its tail (first
    to last wavefront end), the gaps between kernels, and in the persistent backward the wavefronts that carry one
    row more than the others.  Needs the measurement build (see WORKLOADS); figures are medians over the collected
    timelines, in microseconds from the first wavefront start of the forward kernel."""
    import numpy as np

    L = capi.lib()
    try:
        set_clock, clock_bytes = L.tt_norm_debug_wave_clock, L.tt_norm_debug_wave_clock_bytes
    except AttributeError:
        print("timeline-cfg3 needs a library built with -DTTN_WAVE_CLOCK=1 (python -m teletron_amd.build --variant "
              "LIB.so --flag=-DTTN_WAVE_CLOCK=1; TELETRON_AMD_LIB=LIB.so)", file=sys.stderr)
        sys.exit(2)
    set_clock.argtypes, set_clock.restype = [ctypes.c_void_p], ctypes.c_int
    clock_bytes.argtypes, clock_bytes.restype = [], ctypes.c_size_t
    base = args.workload[len("timeline-"):]
    sets = [build_workload(base, torch, capi, dev)[0] for _ in range(3 if base == "cfg3" else 1)]
    rows = 29700 if base == "cfg3" else ROWS
    buf = torch.zeros(clock_bytes() // 8, dtype=torch.int64, device=dev)
    torch.cuda.synchronize()
    if set_clock(ctypes.c_void_p(buf.data_ptr())) != 0:
        raise RuntimeError("tt_norm_debug_wave_clock failed")
    slots = buf.numel() // (3 * 4)
    kinds = ("adaln_forward", "adaln_backward", "column_reducer")
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    collected = []
    turn = 0
    for _ in range(max(1, min(args.steps, 25))):
        buf.zero_()
        torch.cuda.synchronize()
        for i in range(args.warmup + 1):      # back to back; the last step's marks are the ones that survive
            if i == args.warmup:
                e0.record()
            turn += 1
            for _, fn, _ in sets[turn % len(sets)]:
                fn()
        e1.record()
        torch.cuda.synchronize()
        t = buf.view(3, slots, 4).cpu().numpy().astype(np.float64)
        rec = {"step_us_by_events": e0.elapsed_time(e1) * 1e3}
        origin = None
        for k, name in enumerate(kinds):
            a = t[k][t[k][:, 0] != 0]
            if origin is None:
                origin = a[:, 0].min()
            st, en = (a[:, 0] - origin) / 100.0, (a[:, 1] - origin) / 100.0     # 100 MHz ticks -> us
            r = {"wavefronts": int(len(a)), "first_start": st.min(), "last_start": st.max(), "first_end": en.min(),
                 "last_end": en.max(), "median_wavefront_life": float(np.median(en - st))}
            lo, hi = st.min(), en.max()
            r["active_at_tenths"] = [int(((st <= x) & (en > x)).sum()) for x in np.linspace(lo, hi, 11)[:-1] + (hi - lo) / 20]
            if name == "adaln_backward":
                done = (a[:, 2] - origin) / 100.0
                w = np.nonzero(t[k][:, 0] != 0)[0]
                per_wave = rows // len(a)
                extra = w < rows - per_wave * len(a)      # these wavefronts own one row more
                r.update({"rows_per_wavefront": per_wave, "wavefronts_with_one_more": int(extra.sum()),
                          "rows_done_first": done.min(), "rows_done_median": float(np.median(done)),
                          "rows_done_last_without_extra": done[~extra].max(),
                          "rows_done_last_with_extra": done[extra].max() if extra.any() else None,
                          "us_per_row_median": float(np.median((done - st) / (per_wave + extra))),
                          # workgroups are dealt to the eight XCDs in turn
                          "rows_done_median_by_xcd": [round(float(np.median(done[(w // 4) % 8 == x])), 2) for x in range(8)]})
                if len(a) % 4 == 0:      # per workgroup: its slowest wavefront's last row -> its partial row written
                    wg_done, wg_end = done.reshape(-1, 4), en.reshape(-1, 4)
                    r["partial_row_flush_median"] = float(np.median(wg_end.max(axis=1) - wg_done.max(axis=1)))
                    r["rows_done_spread_inside_workgroup_median"] = float(np.median(wg_done.max(axis=1) - wg_done.min(axis=1)))
            rec[name] = r
        rec["gap_forward_to_backward"] = rec["adaln_backward"]["first_start"] - rec["adaln_forward"]["last_end"]
        rec["gap_backward_to_reducer"] = rec["column_reducer"]["first_start"] - rec["adaln_backward"]["last_end"]
        rec["span"] = rec["column_reducer"]["last_end"]
        collected.append(rec)

    def med(path):
        vals = []
        for rec in collected:
            v = rec
            for key in path:
                v = v[key]
            vals.append(v)
        if vals[0] is None:
            return None
        if isinstance(vals[0], list):
            return [round(float(np.median([v[i] for v in vals])), 2) for i in range(len(vals[0]))]
        return round(float(np.median(vals)), 2)

    out = {}
    for key, v in collected[0].items():
        out[key] = {k2: med((key, k2)) for k2 in v} if isinstance(v, dict) else med((key,))
    set_clock(None)
    step_us = out["step_us_by_events"]
    algo = (5 if base == "cfg3" else 10) * rows * COLS * 2
    print(json.dumps({
        "metric": "timeline of %s's step from per-wavefront clocks (medians, us)" % base, "value": round(algo / step_us / 1e3, 1),
        "unit": "GB/s", "n_gpus": 1, "steps": len(collected), "warmup": args.warmup, "ms_per_step": round(step_us / 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": WORKLOADS[args.workload], "rows": rows, "cols": COLS}, "timeline_us": out,
    }))


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-CPU eager timing")
    ap.add_argument("--hip-graph", action="store_true",
                    help="capture one step per buffer set into a HIP graph and replay it in the timed region "
                         "(what a launch-bound caller would do; matters for the small workloads only)")
    ap.add_argument("--workload", default="cfg4", choices=sorted(WORKLOADS),
                    help="cfg4 (default) is the headline step; the others measure the remaining "
                         "configurations and the call sites around the path with the same method")
    return ap.parse_args()


def cpu_eager_baseline(sample_rows: int = ROWS, reps: int = 5):
    """The reference's eager formulas (oracle restatement) on the host cores, over the rows of the
    same workload (all of them by default: about ten seconds of CPU work); returns GB/s in the same
    algorithmic-bytes accounting."""
    import torch
    from oracle import norm_oracle as O

    # every core the box gives this process (its CPU share), as intra-op threads
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    limit = os.environ.get("OMP_NUM_THREADS")
    threads = min(cores, int(limit)) if limit and limit.isdigit() else cores
    torch.set_num_threads(threads)
    threads = torch.get_num_threads()
    cpu_model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            cpu_model = next((l.split(":", 1)[1].strip() for l in f if l.startswith("model name")), "unknown")
    except OSError:
        pass
    r = O.make_rmsnorm_inputs((1, sample_rows), COLS, torch.bfloat16, seed=0)
    a = O.make_adaln_inputs(1, sample_rows, COLS, torch.bfloat16, seed=0)

    def step():
        O.eager_rmsnorm_fwd_bwd(r["x"], r["weight"], r["grad"])
        O.eager_adaln_fwd_bwd(a["x"], a["scale"], a["shift"], a["grad"])

    step()  # warm
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    t = sorted(times)[len(times) // 2]
    nbytes = 2 * 5 * sample_rows * COLS * 2

    # BASELINE config 1, the reference's own CPU-runnable case: RMSNorm fwd+bwd on x [2, 4096, 3072] fp32,
    # 3 warm-up passes, 10 timed, median
    c1 = O.make_rmsnorm_inputs((2, 4096), COLS, torch.float32, seed=0)
    t1 = []
    for k in range(13):
        t0 = time.perf_counter()
        O.eager_rmsnorm_fwd_bwd(c1["x"], c1["weight"], c1["grad"])
        if k >= 3:
            t1.append(time.perf_counter() - t0)
    m1 = sorted(t1)[len(t1) // 2]
    cfg1 = {"value": round(5 * 8192 * COLS * 4 / m1 / 1e9, 3), "unit": "GB/s", "cores": threads, "threads": threads,
            "cpu_model": cpu_model, "kind": "port",
            "ms_per_pass": round(m1 * 1e3, 2),
            "sample": "config 1 in full: RMSNorm fwd+bwd, x [2, 4096, 3072] fp32, PyTorch CPU eager (oracle "
                      "restatement), 3 warm-up + 10 timed passes, median"}
    return {
        "value": round(nbytes / t / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "threads": threads,
        "cpu_model": cpu_model,
        "host_cpus": os.cpu_count(),
        "kind": "port",
        "sample": f"{sample_rows} of {ROWS} rows x {COLS} bf16, RMSNorm + AdaLN fwd+bwd via PyTorch CPU eager "
                  f"(oracle restatement), median of {reps}, {t * 1e3:.1f} ms per pass",
        "config1": cfg1,
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported in this build "
              "(rows shard trivially across GPUs; nothing here uses a second one)", file=sys.stderr)
        sys.exit(2)

    import torch
    from teletron_amd import capi

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L = capi.lib()
    if args.workload == "stream-ceiling":
        stream_ceiling(args, torch, capi, dev)
        return
    if args.workload == "cached-set":
        cached_set(args, torch, capi, dev)
        return
    if args.workload.startswith("timeline-"):
        wave_timeline(args, torch, capi, dev)
        return
    calls, tensor_bytes, tokens_per_step, dtype_name, a_tensor = build_workload(args.workload, torch, capi, dev)
    headline = args.workload == "cfg4"
    # A step streams every tensor once.  When a tensor is smaller than twice the 256 MB last-level
    # cache, successive steps rotate through three separately allocated buffer sets so that no step
    # finds its inputs cached by the one before; the large workloads evict themselves.
    buffer_sets = [calls]
    if tensor_bytes < 512 * 2 ** 20:
        buffer_sets += [build_workload(args.workload, torch, capi, dev)[0] for _ in range(2)]
    turn = [0]

    def next_set():
        turn[0] += 1
        return buffer_sets[turn[0] % len(buffer_sets)]

    names = [n for n, _, _ in calls]
    mults = dict((n, m) for n, _, m in calls)

    def step():
        """One pass of the hot path."""
        for _, fn, _ in next_set():
            fn()

    def per_call_profile(n_steps):
        """HIP-event duration of every call over n_steps untimed steps (events recorded on the
        launch stream); used for the breakdown and to find the slowest call."""
        evs = [{n: (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for n in names}
               for _ in range(n_steps)]
        for k in range(n_steps):
            for name, fn, _ in next_set():
                evs[k][name][0].record()
                fn()
                evs[k][name][1].record()
        torch.cuda.synchronize()
        return {n: sorted(evs[k][n][0].elapsed_time(evs[k][n][1]) for k in range(n_steps)) for n in names}

    # warm-up: W untimed steps, then (still untimed) a few more with per-call events for the breakdown
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    samples = per_call_profile(30)
    avg_ms = {n: sum(v) / len(v) for n, v in samples.items()}
    pct = lambda v, q: v[min(len(v) - 1, int(round(q * (len(v) - 1))))]
    per_call = {n: {"avg_us": round(avg_ms[n] * 1e3, 1),
                    "p10_us": round(pct(samples[n], 0.1) * 1e3, 1),
                    "median_us": round(pct(samples[n], 0.5) * 1e3, 1),
                    "p90_us": round(pct(samples[n], 0.9) * 1e3, 1),
                    "GB/s": round(mults[n] * tensor_bytes / avg_ms[n] / 1e6, 1),
                    "frac_of_peak": round(mults[n] * tensor_bytes / avg_ms[n] / 1e6 / HBM_PEAK_GBS, 4)}
                for n in names}
    dom = max(names, key=lambda n: avg_ms[n])

    # timed region: exactly K steps back to back, wall clock between two synchronisations.  The row
    # kernel of the slowest call is bracketed by a pair of HIP events recorded by the library itself on
    # the launch stream (immediately before and after that kernel, before the column reducer), so the
    # figure is the duration of exactly the kernel a profiler reports.
    hip = ctypes.CDLL("libamdhip64.so")

    def hip_event():
        e = ctypes.c_void_p()
        if hip.hipEventCreate(ctypes.byref(e)) != 0:
            raise RuntimeError("hipEventCreate failed")
        return e

    # a call that is a whole autograd forward + backward launches several row kernels: no single one to bracket
    composite = args.workload.startswith("qkv-site") or args.workload == "cfg4-eager-gpu"
    pairs = [] if (args.hip_graph or composite) else [(hip_event(), hip_event()) for _ in range(args.steps)]
    arm = L.tt_norm_profile_next_row_kernel
    graphs = []
    if args.hip_graph:
        # the entry points only launch kernels, so a step captures as is; one graph per buffer set
        for cs in buffer_sets:
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                eager_stream = _LAUNCH_STREAM[0]
                _LAUNCH_STREAM[0] = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
                for _, fn, _ in cs:
                    fn()
                _LAUNCH_STREAM[0] = eager_stream
            graphs.append(g)
        for g in graphs:
            g.replay()

    def timed_step(k):
        if graphs:
            graphs[k % len(graphs)].replay()
            return
        for name, fn, _ in next_set():
            if name == dom and pairs:
                arm(pairs[k][0], pairs[k][1])
            fn()

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        timed_step(k)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    ms_per_step = wall / args.steps * 1e3
    step_bytes = sum(m for _, _, m in calls) * tensor_bytes
    dom_ms = 0.0
    for a, b in pairs:
        ms = ctypes.c_float()
        if hip.hipEventElapsedTime(ctypes.byref(ms), a, b) != 0:
            raise RuntimeError("hipEventElapsedTime failed")
        dom_ms += ms.value
        hip.hipEventDestroy(a)
        hip.hipEventDestroy(b)
    # under graph replay, and for composite calls, no event pair is armed: the call's untimed HIP-event average stands in
    dom_ms = dom_ms / args.steps if pairs else avg_ms[dom]
    achieved = mults[dom] * tensor_bytes / (dom_ms * 1e-3) / 1e9

    # streaming-copy yardstick (read one tensor, write one tensor) with the same access pattern
    src = a_tensor.reshape(-1)[:tensor_bytes // a_tensor.element_size()]
    dst = torch.empty_like(src)
    from teletron_amd import probe as P
    for _ in range(3):
        P.stream_copy(dst, src)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(10):
        P.stream_copy(dst, src)
    e1.record()
    torch.cuda.synchronize()
    copy_gbs = 2 * tensor_bytes / (e0.elapsed_time(e1) / 10) / 1e6

    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    dom_call = "tt_" + dom.removesuffix("_q").removesuffix("_k")
    prof_calls, prof_valid = measured_cfg4_profile() if headline else ({}, False)
    prof_rec = prof_calls.get(dom_call, {})
    result = {
        "metric": "fwd+bwd HBM GB/s and % of peak for RMSNorm/AdaLN at 118800x3072 bf16" if headline
                  else "fwd+bwd HBM GB/s and % of peak, workload " + args.workload,
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype_name,
        "data": "synthetic",
        "config": {"workload": WORKLOADS[args.workload], "tensor_bytes": tensor_bytes,
                   "buffer_sets": len(buffer_sets), "hip_graph": bool(args.hip_graph),
                   "algorithmic_bytes_per_step": step_bytes},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "tokens_per_s": round(tokens_per_step / (ms_per_step * 1e-3), 1),
        "per_call_untimed": per_call,
        "stream_copy_GB/s": round(copy_gbs, 1),
        "roofline": {"bound": "hbm", "kernel": prof_rec.get("symbol") if headline else None, "call": dom_call,
                     "avg_us": round(dom_ms * 1e3, 1),
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": prof_rec.get("traffic_bytes") if (headline and prof_valid) else None,
                     "traffic_source": ("profiles/cfg4_traffic.json" if prof_valid else
                                        "none: kernel sources differ from the profiled ones") if headline else None},
    }
    if headline:
        result["config"].update({"rows": ROWS, "cols": COLS})
    if headline and not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_eager_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
