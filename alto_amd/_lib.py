"""ctypes binding of libalto_mxfp4.so (the C ABI declared in include/alto_mxfp4.h).

The product path has no CPU fallback: if the library is missing or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes
import os
import threading

from . import build as _build

_lock = threading.Lock()
_lib = None

c_i64 = ctypes.c_int64
c_int = ctypes.c_int
c_vp = ctypes.c_void_p
c_f32 = ctypes.c_float

# name -> (restype, argtypes); mirrors include/alto_mxfp4.h
SIGNATURES = {
    "alto_mxfp4_version": (c_int, []),
    "alto_mxfp4_last_error": (ctypes.c_char_p, []),
    "alto_mxfp4_init": (c_int, []),
    "alto_mxfp4_quantize": (c_int, [c_vp, c_int, c_i64, c_i64, c_i64, c_i64, c_i64,
                                    c_vp, c_vp, c_vp, c_vp,
                                    c_int, c_int, c_vp, c_i64, c_i64,
                                    c_int, c_vp, c_vp, c_int, c_int, c_vp]),
    "alto_mxfp4_quantize_pitched": (c_int, [c_vp, c_int, c_i64, c_i64, c_i64, c_i64, c_i64,
                                            c_vp, c_vp, c_vp, c_vp, c_i64, c_i64,
                                            c_int, c_int, c_vp, c_i64, c_i64,
                                            c_int, c_vp, c_vp, c_int, c_int, c_vp]),
    "alto_mxfp4_quantize_sr_philox": (c_int, [c_vp, c_int, c_i64, c_i64, c_i64, c_i64, c_i64,
                                              c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_int,
                                              ctypes.c_uint64, ctypes.c_uint64, c_vp,
                                              c_int, c_vp, c_vp, c_int, c_int, c_vp]),
    "alto_mxfp4_quantize_sr_hw": (c_int, [c_vp, c_int, c_i64, c_i64, c_i64, c_i64, c_i64,
                                          c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_int,
                                          ctypes.c_uint64, ctypes.c_uint64, c_vp,
                                          c_int, c_vp, c_vp, c_int, c_int, c_vp]),
    "alto_mxfp4_quantize_sr_hw_words": (c_i64, [c_int, c_i64, c_i64, c_i64]),
    "alto_mxfp4_quantize_ex": (c_int, [c_vp, c_int, c_i64, c_i64, c_i64, c_i64, c_i64,
                                       c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_int, c_int,
                                       c_vp, c_i64, c_i64, ctypes.c_uint64, ctypes.c_uint64, c_vp,
                                       c_int, c_vp, c_vp, c_int, c_int, c_int, c_vp]),
    "alto_mxfp4_philox_advance": (c_int, [c_vp, ctypes.c_uint64, c_vp]),
    "alto_mxfp4_hadamard": (c_int, [c_vp, c_int, c_i64, c_i64, c_i64, c_vp, c_i64, c_vp, c_vp, c_vp]),
    "alto_mxfp4_hadamard_apply": (c_int, [c_vp, c_int, c_i64, c_i64, c_i64, c_vp, c_i64, c_vp, c_vp, c_int, c_int, c_vp]),
    "alto_mxfp4_dequantize": (c_int, [c_vp, c_vp, c_i64, c_i64, c_int, c_vp, c_int, c_i64, c_i64, c_int, c_vp]),
    "alto_mxfp4_transpose_codes": (c_int, [c_vp, c_i64, c_i64, c_vp, c_vp]),
    "alto_mxfp4_gemm": (c_int, [c_vp, c_i64, c_vp, c_i64, c_i64, c_int,
                                c_vp, c_i64, c_vp, c_i64, c_i64, c_int,
                                c_i64, c_i64, c_i64, c_vp, c_int, c_i64, c_f32, c_vp]),
    "alto_mxfp4_packed_scales_bytes": (c_i64, [c_i64, c_i64]),
    "alto_mxfp4_pack_scales": (c_int, [c_vp, c_i64, c_i64, c_int, c_i64, c_i64, c_vp, c_vp]),
    "alto_mxfp4_gemm_ps": (c_int, [c_vp, c_i64, c_vp, c_vp, c_i64, c_vp, c_i64, c_i64, c_i64, c_vp, c_i64, c_f32, c_vp]),
    "alto_mxfp4_grouped_gemm_ps": (c_int, [c_vp, c_i64, c_vp, c_vp, c_i64, c_i64, c_vp, c_i64, c_vp, c_vp, c_int, c_int, c_i64, c_i64, c_i64, c_vp, c_i64,
                                          c_vp, c_i64, c_int, c_vp]),
    "alto_mxfp4_grouped_gemm": (c_int, [c_vp, c_i64, c_vp, c_i64, c_i64, c_int,
                                        c_vp, c_i64, c_i64, c_vp, c_i64, c_i64, c_i64, c_int,
                                        c_vp, c_vp, c_int, c_int, c_i64, c_i64, c_i64, c_vp, c_int, c_i64, c_vp, c_i64, c_vp]),
    "alto_mxfp4_grouped_gemm_planned": (c_int, [c_vp, c_i64, c_vp, c_i64, c_i64, c_int,
                                        c_vp, c_i64, c_i64, c_vp, c_i64, c_i64, c_i64, c_int,
                                        c_vp, c_vp, c_int, c_int, c_i64, c_i64, c_i64, c_vp, c_int, c_i64, c_vp, c_i64, c_vp]),
    "alto_mxfp4_grouped_gemm_plan": (c_int, [c_vp, c_vp, c_int, c_int, c_i64, c_vp, c_i64, c_vp]),
    "alto_mxfp4_grouped_gemm_noalloc": (c_int, [c_vp, c_i64, c_vp, c_i64, c_i64, c_int,
                                                c_vp, c_i64, c_i64, c_vp, c_i64, c_i64, c_i64, c_int,
                                                c_vp, c_vp, c_int, c_int, c_i64, c_i64, c_i64, c_vp, c_int, c_i64, c_vp]),
    "alto_mxfp4_grouped_gemm_workspace_bytes": (c_i64, [c_i64, c_int]),
    "alto_mxfp4_grouped_gemm_dw": (c_int, [c_vp, c_i64, c_vp, c_i64, c_i64, c_int,
                                           c_vp, c_i64, c_vp, c_i64, c_i64, c_int,
                                           c_vp, c_vp, c_int, c_int, c_i64, c_i64, c_i64,
                                           c_vp, c_int, c_i64, c_i64, c_i64, c_f32, c_vp]),
    "alto_mxfp4_grouped_gemm_dw_ps": (c_int, [c_vp, c_i64, c_vp, c_vp, c_i64, c_vp, c_vp, c_vp, c_int, c_int, c_i64, c_i64, c_i64,
                                              c_vp, c_i64, c_i64, c_i64, c_f32, c_vp]),
    "alto_mxfp4_probe_mfma": (c_int, [c_int, c_int, c_int, c_vp, c_vp, c_vp]),
    "alto_mxfp4_attention_fwd": (c_int, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
                                         c_f32, c_int, c_vp]),
    "alto_mxfp4_attention_fwd_ex": (c_int, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64,
                                            c_f32, c_int, c_vp, c_i64, c_i64, c_i64, c_vp, c_i64, c_i64, c_vp]),
    "alto_mxfp4_random_bits": (c_int, [c_vp, c_i64, ctypes.c_uint64, ctypes.c_uint64, c_vp]),
    "alto_mxfp4_qdq": (c_int, [c_vp, c_int, c_i64, c_i64, c_i64, c_i64, c_i64, c_vp, c_i64, c_i64, c_int, c_int, c_vp]),
}


class AltoMxfp4Error(RuntimeError):
    pass


def load():
    """Load the in-tree shared library.  It is built first when it does not exist, and rebuilt when it was made from
    other sources than the tree holds now (a digest of the sources is recorded beside it), so that an edited kernel is
    never tested through a stale binary; ``ALTO_MXFP4_NO_REBUILD=1`` turns a stale library into an error instead."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = os.environ.get("ALTO_MXFP4_LIB")   # an explicit library (a build with other options) is loaded as it is
        if path:
            lib = ctypes.CDLL(path)
            for name, (res, args) in SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = res
                fn.argtypes = args
            _lib = lib
            return lib
        path = _build.lib_path()
        if not os.path.exists(path):
            _build.build(verbose=False)
        elif _build.is_stale():
            if os.environ.get("ALTO_MXFP4_NO_REBUILD") == "1":
                raise AltoMxfp4Error(f"{path} was not built from the sources in this tree: run `python -m alto_amd.build`")
            import sys
            print(f"alto_amd: {path} is older than its sources, rebuilding", file=sys.stderr, flush=True)
            _build.build(verbose=False)
        lib = ctypes.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the ABI and the header drifted apart
            fn.restype = res
            fn.argtypes = args
        _lib = lib
        return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().alto_mxfp4_last_error().decode("utf-8", "replace")
        if rc == -1:
            raise AssertionError(f"{what}: {msg}")
        if rc == -3:
            raise NotImplementedError(f"{what}: {msg}")
        raise AltoMxfp4Error(f"{what} failed with code {rc}: {msg}")
