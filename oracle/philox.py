"""Philox4x32-10 in numpy (TEST INFRASTRUCTURE ONLY): the checker of ``alto_mxfp4_random_bits``.

The algorithm is the published one (Salmon, Moraes, Dror, Shaw, "Parallel random numbers: as easy as 1, 2, 3", SC'11);
it is pinned by the known-answer vectors of the authors' Random123 library (tests/test_oracle_pins.py).  The reference
uses the same generator family inside its Triton kernels (``tl.randint4x``,
alto/kernels/fp4/fp4_common/triton_fp4_ops.py:15-18) with tile-local offsets that this build does not reproduce: the
random words are an explicit input of the quantizer here.
"""
from __future__ import annotations

import numpy as np

M0, M1 = 0xD2511F53, 0xCD9E8D57
W0, W1 = 0x9E3779B9, 0xBB67AE85
MASK = 0xFFFFFFFF


def philox4x32_10(counter: np.ndarray, key: np.ndarray) -> np.ndarray:
    """counter [..., 4] uint32 (little end first), key [..., 2] uint32 -> [..., 4] uint32."""
    c = [counter[..., i].astype(np.uint64) for i in range(4)]
    k0 = key[..., 0].astype(np.uint64)
    k1 = key[..., 1].astype(np.uint64)
    for _ in range(10):
        p0 = np.uint64(M0) * c[0]
        p1 = np.uint64(M1) * c[2]
        hi0, lo0 = p0 >> np.uint64(32), p0 & np.uint64(MASK)
        hi1, lo1 = p1 >> np.uint64(32), p1 & np.uint64(MASK)
        c = [(hi1 ^ c[1] ^ k0) & np.uint64(MASK), lo1, (hi0 ^ c[3] ^ k1) & np.uint64(MASK), lo0]
        k0 = (k0 + np.uint64(W0)) & np.uint64(MASK)
        k1 = (k1 + np.uint64(W1)) & np.uint64(MASK)
    return np.stack(c, axis=-1).astype(np.uint32)


def random_bits(n: int, seed: int, offset: int = 0) -> np.ndarray:
    """The n words ``alto_mxfp4_random_bits(out, n, seed, offset)`` writes: word 4 c + j = word j of the block with the
    128-bit counter c + offset and the key ``seed``."""
    quads = (n + 3) // 4
    ctr = [(q + offset) & ((1 << 128) - 1) for q in range(quads)] if quads < 1024 else None
    if ctr is None:
        lo = (np.arange(quads, dtype=np.uint64) + np.uint64(offset & 0xFFFFFFFFFFFFFFFF))
        carry = (lo < np.uint64(offset & 0xFFFFFFFFFFFFFFFF)).astype(np.uint64)
        counter = np.stack([lo & np.uint64(MASK), lo >> np.uint64(32), carry, np.zeros_like(carry)], axis=-1).astype(np.uint32)
    else:
        counter = np.array([[(v >> (32 * i)) & MASK for i in range(4)] for v in ctr], dtype=np.uint32).reshape(quads, 4)
    key = np.broadcast_to(np.array([seed & MASK, (seed >> 32) & MASK], dtype=np.uint32), (quads, 2))
    return philox4x32_10(counter, key).reshape(-1)[:n]
