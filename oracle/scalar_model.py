"""Second, scalar model of the per-element MXFP4 arithmetic in pure Python integers (TEST INFRASTRUCTURE ONLY).

Written independently of ``mxfp4_oracle`` (no torch, no vector ops) so that the
two can be checked against each other; used on small inputs only.  Follows
alto/kernels/fp4/fp4_common/triton_fp4_ops.py:24-95 (encode), :98-134 (decode)
and alto/kernels/fp4/mxfp4/mxfp_quantization.py:73-94 (scale).
"""
from __future__ import annotations

import struct


def f32_bits(f: float) -> int:
    return struct.unpack("<I", struct.pack("<f", f))[0]


def bits_f32(b: int) -> float:
    return struct.unpack("<f", struct.pack("<I", b & 0xFFFFFFFF))[0]


def bf16_bits_to_float(b: int) -> float:
    return bits_f32((b & 0xFFFF) << 16)


def to_f32(x: float) -> float:
    """Round a Python float (double) to the nearest fp32 (RNE), as a double."""
    return struct.unpack("<f", struct.pack("<f", x))[0]


def scale_from_absmax_bits(bits: int, mbits: int) -> int:
    """absmax bit pattern (bf16: mbits=7, fp32: mbits=23) -> E8M0 byte. mxfp_quantization.py:80-94."""
    e = ((bits + (1 << (mbits - 2))) & (0x1FF << mbits)) >> mbits
    return max(e - 2, 1)


def encode_rne(q: float) -> int:
    """q is an fp32 value (given as a double that is exactly representable in fp32)."""
    b = f32_bits(q)
    sign = b & 0x80000000
    mb = b ^ sign
    m = bits_f32(mb)
    if m >= 6.0:
        code = 7
    elif m < 1.0:
        t = to_f32(m + 4194304.0)  # fp32 add, RNE
        code = (f32_bits(t) - 0x4A800000) & 0xFF
    else:
        odd = (mb >> 22) & 1
        code = (((mb + (((1 - 127) << 23) & 0xFFFFFFFF) + 0x1FFFFF + odd) & 0xFFFFFFFF) >> 22) & 0xFF
    return code | (sign >> 28)


def encode_sr(q: float, r: int) -> int:
    """Stochastic rounding with 32 random bits ``r``. triton_fp4_ops.py:49-61,79-80."""
    b = f32_bits(q)
    sign = b & 0x80000000
    mb = b ^ sign
    m = bits_f32(mb)
    r &= 0xFFFFFFFF
    if m >= 6.0:
        code = 7
    elif m < 0.5:
        t = int(to_f32(m * 8589934592.0))  # 2**33 - 2 rounds to 2^33 in fp32; product exact up to fp32 range
        code = 1 if r <= t else 0
    elif m < 1.0:
        t = int(to_f32(to_f32(to_f32(m * 2.0) - 1.0) * 4294967296.0))
        code = 2 if r <= t else 1
    else:
        code = (((mb + (((1 - 127) << 23) & 0xFFFFFFFF) + (r & 0x3FFFFF)) & 0xFFFFFFFF) >> 22) & 0xFF
    return code | (sign >> 28)


GRID = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)


def decode(code: int) -> float:
    v = GRID[code & 7]
    return -v if code & 8 else v


def quantize_row_1d(vals_bits, mbits, rne=True, rand=None):
    """One row of bf16/fp32 bit patterns (length multiple of 32) -> (bytes, scales). Pure-int reference for small tests."""
    to_float = bf16_bits_to_float if mbits == 7 else bits_f32
    absmask = 0x7FFF if mbits == 7 else 0x7FFFFFFF
    out, scales = [], []
    for b0 in range(0, len(vals_bits), 32):
        blk = vals_bits[b0:b0 + 32]
        amax = max(v & absmask for v in blk)  # same ordering as float magnitudes for finite values
        s = scale_from_absmax_bits(amax, mbits)
        scales.append(s)
        sc = bits_f32(s << 23)
        codes = []
        for i, v in enumerate(blk):
            q = to_f32(to_float(v) / sc)
            codes.append(encode_rne(q) if rne else encode_sr(q, rand[b0 + i]))
        for i in range(0, 32, 2):
            out.append(codes[i] | (codes[i + 1] << 4))
    return out, scales
