"""Loader for tests/golden/norm_golden.npz (bf16 stored as uint16 bit patterns, fp16 as float16)."""
import os

import numpy as np
import torch

_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "norm_golden.npz")


def load_golden():
    z = np.load(_PATH, allow_pickle=False)
    cases = {}
    for key in z.files:
        name, field = key.split("/")
        cases.setdefault(name, {})[field] = z[key]
    out = {}
    for name, fields in cases.items():
        is_16bit = bool(fields.pop("is_16bit"))
        d = {}
        for k, a in fields.items():
            if a.dtype == np.uint16:
                d[k] = torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
            else:
                d[k] = torch.from_numpy(a.copy())
        d["is_16bit"] = is_16bit
        out[name] = d
    return out
