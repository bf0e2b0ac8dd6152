"""Differentiable-gradient-estimator multiplier of the weight gradient (``alto/kernels/dge/dge.py:80-93``).

The reference multiplies dW by ``dge_bwd(w_fp4_values)`` where ``w_fp4_values`` are the E2M1 grid values of the quantised
weight (decoded with unit scales, ``mxfp_linear.py:549-568``, ``cg_backward.py:911-928``).  Every grid value is a break
point of the piecewise estimator, i.e. it sits exactly half an interval away from the interval's mid point, where the
derivative ``half_delta^(1-1/k) * |x - mid|^(1/k-1) / k`` collapses to ``1/k`` for all sixteen codes (up to the last bit of ``pow``).  The product is
therefore a constant and rides in the wgrad GEMM's output scale instead of a second pass over dW.
"""
from __future__ import annotations

import numpy as np

DGE_K = 5

_BREAK_POINTS = np.array([-6, -4, -3, -2, -1.5, -1, -0.5, 0, 0.5, 1, 1.5, 2, 3, 4, 6], dtype=np.float32)
_E2M1_GRID = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6], dtype=np.float32)


def dge_bwd_e2m1_grid() -> np.ndarray:
    """``dge_bwd`` evaluated in fp32 at the sixteen E2M1 values (code order), following dge.py:80-93."""
    bp = _BREAK_POINTS
    idx = np.searchsorted(bp, _E2M1_GRID, side="left").astype(np.int32) - 1
    idx = np.clip(idx, 0, len(bp) - 2)
    half = (bp[idx + 1] - bp[idx]) / np.float32(2.0)
    mid = bp[idx] + half
    k = DGE_K
    out = np.power(half, np.float32(1 - 1 / k)) * np.power(np.abs(_E2M1_GRID - mid), np.float32(1 / k - 1)) / np.float32(k)
    return np.clip(out, 0, 3.0).astype(np.float32)


def dge_weight_grad_factor() -> float:
    """fp32(1/k): the value all sixteen codes share.  The two ``pow`` calls of the formula cancel only up to the last
    bit of the math library in use, so the table above is checked to lie within two fp32 ulps of this constant."""
    f = np.float32(1.0 / DGE_K)
    t = dge_bwd_e2m1_grid()
    if not np.all(np.abs(t - f) <= 2 * np.spacing(f)):
        raise RuntimeError(f"DGE factors are not 1/k on the E2M1 grid: {t}")
    return float(f)


DGE_FACTOR = dge_weight_grad_factor()
