"""Shared helpers of the GPU parity tests (inputs are generated on the CPU with fixed seeds, then copied)."""
import numpy as np
import torch

import oracle as O


def gen(seed):
    return torch.Generator().manual_seed(seed)


def randn_outliers(shape, dtype, seed, p=0.005, mag=100.0):
    """N(0,1) plus sparse large outliers, the data shape of the reference's tests (tests/unittest/mxfp4/utils.py:16-22)."""
    g = gen(seed)
    x = torch.randn(shape, generator=g)
    mask = torch.bernoulli(torch.full(shape, p), generator=g)
    x = x + mag * torch.randn(shape, generator=g) * mask
    return x.to(dtype)


def laplace(shape, scale, dtype, seed):
    g = gen(seed)
    u = (torch.rand(shape, generator=g) - 0.5).clamp(-0.4999999, 0.4999999)  # keep log1p finite
    x = -scale * torch.sign(u) * torch.log1p(-2 * u.abs())
    return x.to(dtype)


def rand_bits(shape, seed):
    """int32 tensor carrying 32 uniform random bits per element."""
    g = gen(seed)
    return torch.randint(-2 ** 31, 2 ** 31, shape, generator=g, dtype=torch.int64).to(torch.int32)


def hadamard_from_seed(seed):
    """(signs int8[32], perm uint8[32]) drawn the way HadamardFactory does: randint then randperm on one CPU generator."""
    g = gen(seed)
    q = torch.randint(0, 2, (32,), generator=g, dtype=torch.float32) * 2 - 1
    perm = torch.randperm(32, generator=g)
    return q.to(torch.int8), perm


def assert_bytes_equal(got: torch.Tensor, exp: torch.Tensor, what: str):
    got = got.cpu()
    assert got.shape == exp.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(exp.shape)}"
    if not torch.equal(got, exp):
        bad = (got != exp).nonzero()
        i = tuple(bad[0].tolist())
        raise AssertionError(f"{what}: {bad.shape[0]} of {exp.numel()} bytes differ; first at {i}: got {int(got[i]):#x}, expected {int(exp[i]):#x}")


def snr_db(ref: torch.Tensor, got: torch.Tensor) -> float:
    r, g = ref.double().cpu(), got.double().cpu()
    noise = ((r - g) ** 2).sum()
    return float("inf") if noise == 0 else float(10 * torch.log10((r ** 2).sum() / noise))
