"""The host layer under AddressSanitizer + UndefinedBehaviorSanitizer, on the CPU: a sanitised build of the host
passes of the kernel sources driven through the C ABI (tests/host_sanitize/host_driver.cpp), and sanitised
builds of the two extension modules driven from Python (tests/host_sanitize/exercise_extensions.py).  No
device code is built or run; the product libraries are untouched (everything goes to a temporary directory)."""
import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HERE = os.path.join(ROOT, "tests", "host_sanitize")
# leak checking is off: the interpreter and the HIP runtime keep memory until exit by design
SAN_ENV = {"ASAN_OPTIONS": "detect_leaks=0:abort_on_error=0", "UBSAN_OPTIONS": "print_stacktrace=1:halt_on_error=1"}


def test_c_abi_host_layer_under_asan_ubsan(tmp_path):
    sys.path.insert(0, HERE)
    try:
        import build_host_sanitized
    finally:
        sys.path.remove(HERE)
    exe = build_host_sanitized.build(str(tmp_path))
    syms = subprocess.run(["nm", exe], capture_output=True, text=True).stdout
    assert "__asan_init" in syms and "__ubsan_handle" in syms, "the driver was not built with the sanitizers"
    run = subprocess.run([exe], capture_output=True, text=True, env={**os.environ, **SAN_ENV}, timeout=300)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "host sanitize driver ok" in run.stdout
    assert "runtime error" not in run.stderr and "AddressSanitizer" not in run.stderr, run.stderr


def _gcc_file(name):
    return subprocess.run(["gcc", "-print-file-name=" + name], capture_output=True, text=True).stdout.strip()


def test_extension_argument_checks_under_asan_ubsan(tmp_path):
    import torch
    from torch.utils import cpp_extension as ce
    from teletron_amd import build as B

    asan, stdcxx = _gcc_file("libasan.so"), _gcc_file("libstdc++.so")
    if not (os.path.isabs(asan) and os.path.isabs(stdcxx)):
        pytest.skip("gcc's sanitizer runtime is not installed")
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = [f"-I{p}" for p in ce.include_paths()] + ["-I" + sysconfig.get_paths()["include"],
                                                    "-I" + os.path.join(ROOT, "include"), "-I/opt/rocm/include"]

    def build(item):
        name, src = item
        cmd = ["g++", "-O1", "-g", "-std=c++17", "-fPIC", "-shared", "-fsanitize=address,undefined",
               "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
               f"-DTORCH_EXTENSION_NAME={name}", "-DTORCH_API_INCLUDE_EXTENSION_H", *inc,
               os.path.join(B.CSRC, src), "-o", str(tmp_path / (name + ".so")),
               f"-L{torch_lib}", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip", "-ltorch_python",
               f"-L{B.LIB_DIR}", "-lteletron_norm", f"-Wl,-rpath,{B.LIB_DIR}", f"-Wl,-rpath,{torch_lib}"]
        return subprocess.run(cmd, capture_output=True, text=True)

    with ThreadPoolExecutor(max_workers=2) as pool:
        for res in pool.map(build, B.EXT_MODULES.items()):
            assert res.returncode == 0, res.stderr[-2000:]
    # the sanitizer runtime has to be the first library of the process; libstdc++ with it, so that the
    # runtime finds the C++ exception entry points it wraps (the interpreter itself does not link libstdc++)
    preload = " ".join(p for p in (asan, stdcxx, os.environ.get("LD_PRELOAD", "")) if p)
    env = {**os.environ, **SAN_ENV, "LD_PRELOAD": preload, "PYTHONPATH": ROOT}
    run = subprocess.run([sys.executable, os.path.join(HERE, "exercise_extensions.py"), str(tmp_path)],
                         capture_output=True, text=True, env=env, timeout=600)
    assert run.returncode == 0, run.stdout[-2000:] + run.stderr[-4000:]
    assert "sanitised extensions ok" in run.stdout
    assert "runtime error" not in run.stderr and "ERROR: AddressSanitizer" not in run.stderr, run.stderr[-4000:]
