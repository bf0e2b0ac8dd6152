"""Builds libalto_mxfp4.so (hand-written HIP for gfx950) in-tree with hipcc.

Usage: ``python -m alto_amd.build [--force]``.  The library lands in ``alto_amd/lib/`` next to the
sources so that it travels with the tree; nothing is installed outside the repository.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(HERE, "lib", "obj")
LIBNAME = "libalto_mxfp4.so"

SOURCES = ["capi.hip", "quantize.hip", "dequantize.hip", "gemm.hip", "gemm_tiled.hip", "grouped_gemm.hip", "probe.hip", "qdq.hip", "attention.hip", "quantize_dynamic.hip", "random.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    # packed-FP32 VALU forms are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def lib_path() -> str:
    return os.path.join(LIBDIR, LIBNAME)


def stamp_path() -> str:
    return lib_path() + ".srchash"


def source_hash() -> str:
    """Digest of every file the library is built from (kernels, their headers, the C ABI header, the compiler flags)."""
    import hashlib
    h = hashlib.sha256(" ".join(HIPCC_FLAGS).encode())
    files = sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hip", ".h")))
    files.append(os.path.join(HERE, "..", "include", "alto_mxfp4.h"))
    for f in files:
        h.update(os.path.basename(f).encode())
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def is_stale() -> bool:
    """True when the built library does not come from the sources in the tree (or carries no record of its sources)."""
    try:
        with open(stamp_path()) as f:
            return f.read().strip() != source_hash()
    except OSError:
        return True


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the MXFP4 kernels need the ROCm toolchain to build")
    return exe


def _compile(src: str) -> str:
    obj = os.path.join(OBJDIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stdout}\n{res.stderr}")
    return obj


def build(verbose: bool = True) -> str:
    """Compile every HIP source and link the shared library; always rebuilds."""
    os.makedirs(OBJDIR, exist_ok=True)
    digest = source_hash()   # taken before compiling: an edit made during the build leaves the library marked stale
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(_compile, SOURCES))
    out = lib_path()
    tmp = out + ".tmp"
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, out)
    with open(stamp_path(), "w") as f:
        f.write(digest + "\n")
    if verbose:
        print(f"built {out} ({os.path.getsize(out)} bytes)")
    return out


if __name__ == "__main__":
    build()
    sys.exit(0)
