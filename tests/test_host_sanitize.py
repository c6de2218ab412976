"""The host side of the C ABI under AddressSanitizer and UndefinedBehaviorSanitizer (host code only; the device
code of the same files is compiled without them): tests/host_sanitize/driver.cpp runs every entry point that works
without a GPU, the error paths of those that do not, and the clean-up of a model whose construction fails."""
import os
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "llama2.rs_amd"))

SAN = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined", "-Xarch_host",
       "-fno-sanitize-recover=undefined", "-Xarch_host", "-fno-omit-frame-pointer", "-g"]


def test_host_code_under_asan_and_ubsan(tmp_path):
    import build as b     # llama2.rs_amd/build.py: the flags of the product build
    hipcc = b.hipcc()
    kernels = [os.path.join(b.OBJ, os.path.splitext(n)[0] + ".o") for n in b.SOURCES if n.endswith(".hip")]
    if not all(os.path.exists(k) for k in kernels):
        b.build()
    objs = []
    for name in ("host.cpp", "textgen.cpp"):
        obj = str(tmp_path / (name + ".o"))
        cmd = [hipcc, *b.COMMON, *b.DEVICE_FLAGS, *b.SOURCES[name], *SAN, "-c", os.path.join(b.CSRC, name), "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-4000:]
        objs.append(obj)
    drv = str(tmp_path / "driver.o")
    r = subprocess.run(["g++", "-O1", "-g", "-std=c++17", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
                        "-c", os.path.join(ROOT, "tests", "host_sanitize", "driver.cpp"), "-o", drv],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-4000:]
    exe = str(tmp_path / "driver")
    r = subprocess.run([hipcc, f"--offload-arch={b.ARCH}", "-fsanitize=address", "-fsanitize=undefined", "-fno-gpu-sanitize",
                        "-o", exe, drv, *objs, *kernels, "-lpthread"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-4000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    r = subprocess.run([exe, os.path.join(ROOT, "tests", "golden", "tokenizer.bin")], capture_output=True, text=True,
                       env=env, timeout=300)
    assert r.returncode == 0 and r.stdout.strip().endswith("ok"), (r.stdout[-2000:], r.stderr[-6000:])
