"""Builds the host passes of the kernel sources (no device code) and host_driver.cpp with AddressSanitizer and
UndefinedBehaviorSanitizer, into `out_dir`; returns the path of the driver executable.

    python tests/host_sanitize/build_host_sanitized.py [out_dir]
"""
import os
import re
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "teletron_amd", "csrc")
SOURCES = ["norm_host.hip", "rmsnorm.hip", "adaln.hip", "anywidth.hip", "widerow.hip", "probe.hip"]
HIPCC = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
SAN = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined", "-Xarch_host",
       "-fno-sanitize-recover=undefined", "-Xarch_host", "-fno-omit-frame-pointer"]


def _run(cmd, **kw):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, **kw)
    if p.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), p.stdout))
    return p.stdout


def build(out_dir: str) -> str:
    os.makedirs(out_dir, exist_ok=True)
    objs = []
    for src in SOURCES:   # host pass only: seconds per file, and nothing of the device side is needed here
        obj = os.path.join(out_dir, src.replace(".hip", ".host.o"))
        _run([HIPCC, "--offload-arch=gfx950", "--cuda-host-only", "-O1", "-g", "-std=c++17", "-ffp-contract=off", *SAN,
              "-c", os.path.join(CSRC, src), "-o", obj])
        objs.append(obj)
    # each host object refers to the device code object that a full build embeds next to it; give those
    # references something to point at (the driver replaces the registration calls, so it is never read)
    names = set()
    for obj in objs:
        names.update(re.findall(r"\bU (__hip_fatbin_\w+)", _run(["nm", obj])))
    stub = os.path.join(out_dir, "fatbin_stubs.c")
    with open(stub, "w") as f:
        for n in sorted(names):
            f.write("const char %s[16] = {0};\n" % n)
    stub_obj = os.path.join(out_dir, "fatbin_stubs.o")
    _run(["gcc", "-c", stub, "-o", stub_obj])
    drv_obj = os.path.join(out_dir, "host_driver.o")
    _run([HIPCC, "--offload-arch=gfx950", "--cuda-host-only", "-O1", "-g", "-std=c++17", *SAN, "-x", "hip",
          "-c", os.path.join(HERE, "host_driver.cpp"), "-o", drv_obj])
    exe = os.path.join(out_dir, "host_driver")
    _run([HIPCC, "--offload-arch=gfx950", "--cuda-host-only", drv_obj, stub_obj, *objs, "-o", exe,
          "-fsanitize=address", "-fsanitize=undefined"])
    return exe


if __name__ == "__main__":
    print(build(sys.argv[1] if len(sys.argv) > 1 else os.path.join(HERE, "_build")))
