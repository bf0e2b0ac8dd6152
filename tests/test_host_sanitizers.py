"""Host code of the C ABI under AddressSanitizer + UndefinedBehaviorSanitizer (no GPU needed).

The library is rebuilt with the sanitizers on its HOST pass only (``-Xarch_host -fsanitize=...``; the device code is built as
always) and linked into ``tests/host_sanitizers/driver.cpp``, which calls every entry point of ``include/alto_mxfp4.h`` a few
thousand times with argument sets that are valid up to three replaced values (extreme sizes, negative strides, null and
misaligned pointers, bad modes).  Without a device every call must end in an error code with a message -- at an argument
check or at the launch -- and no sanitizer may report: no signed overflow in the size arithmetic, no access outside the
host-side tables, no write through a pointer that stands for device memory.
"""
import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

from alto_amd import build as B

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "host_sanitizers", "driver.cpp")
OUT = os.path.join(HERE, "host_sanitizers", "_build")
SAN = ["-fsanitize=address", "-fsanitize=undefined", "-fno-sanitize-recover=undefined"]


def _rocm_llvm_clang():
    exe = os.path.join(os.path.dirname(os.path.realpath(B._hipcc())), "..", "lib", "llvm", "bin", "clang++")
    return exe if os.path.exists(exe) else None


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="needs hipcc")
def test_c_abi_host_code_under_asan_and_ubsan():
    clang = _rocm_llvm_clang()
    if clang is None:
        pytest.skip("ROCm's clang++ not found next to hipcc")
    os.makedirs(OUT, exist_ok=True)
    host_san = [f for s in SAN for f in ("-Xarch_host", s)]
    flags = [f for f in B.HIPCC_FLAGS if f != "-O3"] + ["-O1", "-g"] + host_san

    def comp(src):
        obj = os.path.join(OUT, os.path.splitext(src)[0] + ".o")
        r = subprocess.run([B._hipcc(), *flags, "-c", os.path.join(B.CSRC, src), "-o", obj], capture_output=True, text=True)
        assert r.returncode == 0, f"{src}:\n{r.stderr[-3000:]}"
        return obj

    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        objs = list(pool.map(comp, B.SOURCES))
    exe = os.path.join(OUT, "driver")
    rocm_lib = os.path.join(os.path.dirname(os.path.realpath(B._hipcc())), "..", "lib")
    r = subprocess.run([clang, "-std=c++17", "-O1", "-g", *SAN, "-I", os.path.join(HERE, "..", "include"), SRC, *objs, "-o", exe,
                        "-L", rocm_lib, "-lamdhip64", f"-Wl,-rpath,{rocm_lib}"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    # leak checking is off: the HIP runtime keeps its own allocations until the process ends
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    # HIP_VISIBLE_DEVICES hides a GPU if there is one: with a device the valid calls would launch kernels on host memory
    env["HIP_VISIBLE_DEVICES"] = ""
    env["ROCR_VISIBLE_DEVICES"] = ""
    r = subprocess.run([exe, "2000"], capture_output=True, text=True, env=env, timeout=600)
    tail = (r.stdout[-2500:] + "\n" + r.stderr[-4000:])
    assert r.returncode == 0, tail
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr, tail
    # every entry point got past its argument checks with its valid set (the driver exits 4 otherwise) and the run is complete
    assert f"calls {2000 * 30}" in r.stdout, tail
