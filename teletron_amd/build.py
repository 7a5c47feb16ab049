"""Build recipe for the native parts, all compiled for gfx950 and kept in-tree:

  teletron_amd/lib/libteletron_norm.so   HIP kernels + C ABI (include/teletron_norm.h)
  teletron_amd/lib/libteletron_probe.so  measurement only: plain streaming kernels (include/teletron_probe.h),
                                         loaded by bench.py and the tests of the probes, never by the operators
  teletron_amd/ext/fused_rmsnorm*.so     PyTorch extension modules with the reference's
  teletron_amd/ext/fused_adaln*.so       module names and torch_launch_* signatures

Run `python -m teletron_amd.build` (hipcc cross-compiles; no GPU needed).
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
import sysconfig

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIB_DIR = os.path.join(PKG, "lib")
EXT_DIR = os.path.join(PKG, "ext")
LIB_PATH = os.path.join(LIB_DIR, "libteletron_norm.so")
PROBE_LIB_PATH = os.path.join(LIB_DIR, "libteletron_probe.so")

HIPCC = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
ARCH = "gfx950"
# -packed-fp32-ops off: scalar fp32 VALU only (packed fp32 forms are not trusted on this fleet).
# -ffp-contract=off: the kernels reproduce the eager graph's rounding points, so a multiply and a
# later add must stay two roundings unless the source says fmaf; with contraction allowed the
# compiler narrows fp16 chains to half arithmetic and then fuses across a rounding point.
HIP_FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-result",
             "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
KERNEL_SOURCES = ["norm_host.hip", "rmsnorm.hip", "adaln.hip", "anywidth.hip", "widerow.hip"]
EXT_MODULES = {"fused_rmsnorm": "fused_rmsnorm_ext.cpp", "fused_adaln": "fused_adaln_ext.cpp"}


def kernel_source_digest() -> str:
    """First 16 hex digits of a sha256 over the kernel sources (names and contents of csrc/*.hip and
    csrc/*.h): what a measurement of the kernels is tied to."""
    import hashlib

    h = hashlib.sha256()
    for name in sorted(os.listdir(CSRC)):
        if name.endswith((".hip", ".h")):
            h.update(name.encode())
            with open(os.path.join(CSRC, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()[:16]


def _run(cmd, cwd=None):
    proc = subprocess.run(cmd, cwd=cwd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass says it does not know the packed-fp32 feature; that is expected
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_kernels(verbose: bool = True, out: str = None, extra_flags=()) -> str:
    """Each source is compiled to an object of its own (in parallel), then linked.  `out` and
    `extra_flags` build a tuning variant beside the shipped library (the TTN_* macros at the top of
    the kernel sources); load it with TELETRON_AMD_LIB=<out>."""
    from concurrent.futures import ThreadPoolExecutor

    out = os.path.abspath(out) if out else LIB_PATH
    obj_dir = os.path.join(LIB_DIR, "obj") if out == LIB_PATH else out + ".obj"
    os.makedirs(obj_dir, exist_ok=True)
    objs = [os.path.join(obj_dir, os.path.splitext(src)[0] + ".o") for src in KERNEL_SOURCES]
    with ThreadPoolExecutor(max_workers=min(4, len(KERNEL_SOURCES))) as pool:
        logs = list(pool.map(lambda so: _run([HIPCC, *HIP_FLAGS, *extra_flags, "-c", so[0], "-o", so[1]], cwd=CSRC),
                             zip(KERNEL_SOURCES, objs)))
    logs.append(_run([HIPCC, "--offload-arch=" + ARCH, "-fPIC", "-shared", "-o", out] + objs))
    if verbose:
        print("built", os.path.relpath(out, ROOT), "\n".join(l for l in logs if l.strip()).strip())
    return out


def build_probe(verbose: bool = True) -> str:
    """The measurement library: one source, nothing of the operator library linked in."""
    os.makedirs(LIB_DIR, exist_ok=True)
    log = _run([HIPCC, *HIP_FLAGS, "-shared", "probe.hip", "-o", PROBE_LIB_PATH], cwd=CSRC)
    if verbose:
        print("built", os.path.relpath(PROBE_LIB_PATH, ROOT), log.strip())
    return PROBE_LIB_PATH


def ext_path(name: str) -> str:
    suffix = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
    return os.path.join(EXT_DIR, name + suffix)


def build_extensions(verbose: bool = True):
    """The two PyTorch extension modules: host-only C++ (argument checks, current
    stream, workspace from the caching allocator) linked against the C ABI."""
    from torch.utils import cpp_extension as ce
    import torch

    os.makedirs(EXT_DIR, exist_ok=True)
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = [f"-I{p}" for p in ce.include_paths()]
    inc += ["-I" + sysconfig.get_paths()["include"], "-I" + os.path.join(ROOT, "include"),
            "-I/opt/rocm/include"]
    paths = []
    for name, src in EXT_MODULES.items():
        out = ext_path(name)
        cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
               f"-DTORCH_EXTENSION_NAME={name}", "-DTORCH_API_INCLUDE_EXTENSION_H",
               *inc, os.path.join(CSRC, src), "-o", out,
               f"-L{torch_lib}", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip", "-ltorch_python",
               f"-L{LIB_DIR}", "-lteletron_norm",
               "-Wl,-rpath,$ORIGIN/../lib", f"-Wl,-rpath,{torch_lib}"]
        log = _run(cmd)
        if verbose:
            print("built", os.path.relpath(out, ROOT), log.strip())
        paths.append(out)
    return paths


def build_all(verbose: bool = True):
    build_kernels(verbose)
    build_probe(verbose)
    build_extensions(verbose)


if __name__ == "__main__":
    import argparse

    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--variant", metavar="LIB.so", help="build only the kernel library, to this path")
    ap.add_argument("--flag", action="append", default=[], metavar="-DTTN_...=V",
                    help="extra hipcc flag for the variant (repeatable)")
    a = ap.parse_args()
    if a.variant:
        build_kernels(out=a.variant, extra_flags=a.flag)
    else:
        build_all()
