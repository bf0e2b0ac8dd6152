"""Randomized 32-point Hadamard transform: host-side description of the matrix the kernels apply.

Mirrors ``HadamardFactory`` / ``HadamardTransform`` of the reference
(alto/kernels/hadamard_transform/transform.py:15-142): ``W = W0[perm][:, perm]`` with ``W0 = diag(Q) @ H32``
(H32 in Sylvester order, alto/kernels/hadamard_transform/hadamard.py:63-87,130-161).  Instead of a dense 32x32
matrix the transform carries ``signs`` (Q, 32 values of +-1) and ``perm``; the HIP kernels run the equivalent
butterfly.  Random draws use the same torch CPU generator calls in the same order as the reference
(``randint(0, 2, (32,))`` then ``randperm(32)``), so a given seed yields the same (Q, perm).
"""
from __future__ import annotations

from typing import Optional

import torch

BLOCK = 32


class HadamardTransform:
    def __init__(self, signs: torch.Tensor, perm: Optional[torch.Tensor]):
        signs = signs.detach().to("cpu", torch.int8).contiguous()
        assert signs.shape == (BLOCK,) and bool(((signs == 1) | (signs == -1)).all())
        self.signs = signs
        if perm is not None:
            perm = perm.detach().to("cpu", torch.uint8).contiguous()
            assert perm.shape == (BLOCK,) and sorted(perm.tolist()) == list(range(BLOCK))
        self.perm = perm

    @property
    def weight(self) -> torch.Tensor:
        """The dense 32x32 fp32 matrix (for inspection/tests; the kernels never materialise it)."""
        idx = torch.arange(BLOCK)
        v = idx[:, None] & idx[None, :]
        pc = sum(((v >> b) & 1) for b in range(5))
        w0 = self.signs.float().reshape(BLOCK, 1) * (1 - 2 * (pc & 1)).float()
        if self.perm is None:
            return w0
        p = self.perm.long()
        return w0[p][:, p]

    def __call__(self, value: torch.Tensor, inverse: bool = False, left_mul: bool = False) -> torch.Tensor:
        """``W @ value`` (``left_mul``) or ``value @ W`` over blocks of 32, divided by ``sqrt(32)``, in the input dtype;
        ``inverse`` uses ``W.T`` (transform.py:115-142).  The MXFP4 path itself only uses ``left_mul=True``."""
        from .quantization import hadamard_apply  # local import: quantization imports this module
        return hadamard_apply(value, self, inverse=inverse, left_mul=left_mul)


class HadamardFactory:
    block_size: int = BLOCK
    randomized: bool = True
    dtype: torch.dtype = torch.float32
    seed: Optional[int] = None
    generator: torch.Generator = torch.Generator()

    @classmethod
    def configure(cls, block_size=None, randomized=None, dtype=None, seed=None) -> None:
        if block_size is not None:
            if block_size != BLOCK:
                raise ValueError("the HIP kernels implement the 32-point transform only")
            cls.block_size = block_size
        if randomized is not None:
            cls.randomized = randomized
        if dtype is not None:
            cls.dtype = dtype
        if seed is not None:
            cls.seed = seed
            cls.generator.manual_seed(seed)

    @classmethod
    def create_transform(cls, device=None) -> HadamardTransform:
        if not cls.randomized:
            return HadamardTransform(torch.ones(BLOCK, dtype=torch.int8), None)
        q = torch.randint(low=0, high=2, size=(BLOCK,), generator=cls.generator, dtype=cls.dtype)
        q = q * 2 - 1
        perm = torch.randperm(BLOCK, generator=cls.generator)
        return HadamardTransform(q.to(torch.int8), perm)
