"""Writes tests/golden/norm_golden.npz: small seeded inputs and the outputs the
PyTorch-eager restatement (oracle/norm_oracle.py) gives for them on CPU.

The reference repository holds no vectors for this path and its Python module
cannot be imported here (its top-level imports need diffusers and megatron),
so these vectors come from the restatement, whose arithmetic is pinned by the
checks in tests/test_oracle.py.  bf16 tensors are stored as their uint16 bit
patterns, fp16 tensors as numpy float16.  Run from the repo root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import norm_oracle as O  # noqa: E402

CASES = {
    # name: (op, generator kwargs)
    "rms_bf16_c128": ("rmsnorm", dict(lead_shape=(2, 19, 3), cols=128, dtype=torch.bfloat16, seed=11)),
    "rms_bf16_c3072": ("rmsnorm", dict(lead_shape=(1, 7), cols=3072, dtype=torch.bfloat16, seed=12)),
    "rms_f32_c3072": ("rmsnorm", dict(lead_shape=(5,), cols=3072, dtype=torch.float32, seed=13)),
    "rms_f32_c128": ("rmsnorm", dict(lead_shape=(33,), cols=128, dtype=torch.float32, seed=14)),
    "adaln_bf16_b1": ("adaln", dict(batch=1, seq=9, cols=3072, dtype=torch.bfloat16, seed=15)),
    "adaln_bf16_b3": ("adaln", dict(batch=3, seq=5, cols=3072, dtype=torch.bfloat16, seed=16, sigma=2.0)),
    "adaln_f32_b2": ("adaln", dict(batch=2, seq=4, cols=3072, dtype=torch.float32, seed=17)),
    # other widths and fp16 (the any-width kernels)
    "rms_f16_c1000": ("rmsnorm", dict(lead_shape=(6,), cols=1000, dtype=torch.float16, seed=18)),
    "rms_bf16_c5120": ("rmsnorm", dict(lead_shape=(3,), cols=5120, dtype=torch.bfloat16, seed=19)),
    "adaln_f16_c64": ("adaln", dict(batch=2, seq=9, cols=64, dtype=torch.float16, seed=20)),
    # gated residual update + AdaLN, with a gradient arriving at h2
    "gated_bf16_b2": ("gated", dict(batch=2, seq=4, cols=3072, dtype=torch.bfloat16, seed=21)),
}


def to_np(t: torch.Tensor) -> np.ndarray:
    t = t.detach().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def main():
    torch.set_num_threads(1)
    blob = {}
    for name, (op, kw) in CASES.items():
        if op == "rmsnorm":
            d = O.make_rmsnorm_inputs(**kw)
            out, dx, dw = O.eager_rmsnorm_fwd_bwd(d["x"], d["weight"], d["grad"])
            res = {"out": out, "dx": dx, "dweight": dw}
        elif op == "adaln":
            d = O.make_adaln_inputs(**kw)
            out, dx, ds, dh = O.eager_adaln_fwd_bwd(d["x"], d["scale"], d["shift"], d["grad"])
            res = {"out": out, "dx": dx, "dscale": ds, "dshift": dh}
        else:
            names = ("h", "attn", "gate", "scale", "shift", "grad", "grad_h2")
            d = dict(zip(names, O.make_gated_inputs(**kw)))
            got = O.eager_gated_residual_adaln_fwd_bwd(d["h"], d["attn"], d["gate"], d["scale"], d["shift"],
                                                       d["grad"], d["grad_h2"])
            res = dict(zip(("h2", "out", "dh", "dattn", "dgate", "dscale", "dshift"), got))
        for k, v in {**d, **res}.items():
            blob[f"{name}/{k}"] = to_np(v)
        blob[f"{name}/is_16bit"] = np.array(kw["dtype"] != torch.float32)
    np.savez_compressed(os.path.join(HERE, "norm_golden.npz"), **blob)
    print("wrote", len(blob), "arrays")


if __name__ == "__main__":
    main()
