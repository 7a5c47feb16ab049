"""Runs inside a Python started with the AddressSanitizer runtime preloaded: imports the sanitised builds of the
two extension modules from the directory given on the command line and drives their argument checking with
tensors that live on the CPU (every call must raise before anything reaches a GPU)."""
import importlib.util
import sys

import torch


def load(name, directory):
    spec = importlib.util.spec_from_file_location(name, f"{directory}/{name}.so")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def raises(fn, *args):
    try:
        fn(*args)
    except (RuntimeError, TypeError) as exc:
        return str(exc)
    raise AssertionError(f"{fn.__name__} accepted CPU tensors")


def main(directory):
    rms, ada = load("fused_rmsnorm", directory), load("fused_adaln", directory)
    bf = torch.bfloat16
    x, w = torch.zeros(4, 128, dtype=bf), torch.ones(128, dtype=bf)
    r, e = torch.empty(4), torch.empty(0)
    views = [x, x.view(2, 2, 128), x.view(1, 2, 2, 128), x.view(1, 1, 2, 2, 128), x.t(), x[:, ::2], torch.Tensor()]
    n = 0
    for v in views:   # shapes the view decoding must survive: 2 to 5 dimensions, transposed, strided last dim, undefined
        for call in ((rms.torch_launch_rms_forward, (torch.empty_like(x), v, w, 4, 128, 1e-6, r)),
                     (rms.torch_launch_rms_backward, (torch.empty_like(x), torch.empty_like(w), v, x, w, r, 4, 128)),
                     (rms.torch_launch_rms_backward_x, (torch.empty_like(x), torch.empty_like(w), x, v, w, r, 4, 128)),
                     (rms.torch_launch_rms_forward_strided, (torch.empty_like(x), v, w, 1e-6, r)),
                     (rms.torch_launch_rms_backward_strided, (torch.empty_like(x), torch.empty_like(w), x, v, w, r)),
                     (rms.torch_launch_copy_rows_strided, (v, x)),
                     (rms.torch_launch_rms_rope_forward_strided, (torch.empty_like(x), v, w, 1e-6, r, e, e)),
                     (rms.torch_launch_rms_rope_backward_strided, (torch.empty_like(x), torch.empty_like(w), x, v, w, r, e, e))):
            raises(*call[:1], *call[1])
            n += 1
    h = torch.zeros(2, 4, 3072, dtype=bf)
    s = torch.zeros(2, 3072, dtype=bf)
    st = torch.empty(8)
    for name in dir(ada):
        fn = getattr(ada, name)
        if not name.startswith("torch_launch_") or not callable(fn):
            continue
        # every launcher takes tensors first: feed it CPU tensors in every position, with too few and too many arguments
        for args in ((h, h, h, s, s, 8, 3072, 1e-6, st), (h,) * 3, (h, h, s, s, h, h, s, st, st, 8, 3072), ()):
            raises(fn, *args)
            n += 1
    assert rms.supported(128, x) and rms.supported(3072, torch.zeros(1)) and not rms.supported(3071, x)
    assert not rms.supported(128, torch.zeros(1, dtype=torch.int32))
    print(f"sanitised extensions ok: {n} refused calls")


if __name__ == "__main__":
    main(sys.argv[1])
