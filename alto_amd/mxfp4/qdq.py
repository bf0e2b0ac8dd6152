"""Fused quantize -> dequantize for the weight de-oscillation hook.

``_make_qdq_fn_for(cfg)`` mirrors ``alto/components/optimizer.py:123-158``: it returns ``qdq(w, axis)`` equal to
``convert_from_mxfp4(*convert_to_mxfp4(w, axis=axis, is_2d_block=cfg.use_2dblock_w, use_uos=cfg.use_uos), output_dtype=w.dtype,
axis=axis, is_2d_block=cfg.use_2dblock_w)``, including the reference's padding of a 2D weight whose row count is not a
multiple of 32.  2D blocks and 1D blocks along the last dim run as ONE launch; a 1D quantisation along another axis
falls back to the two calls.
"""
from __future__ import annotations

from typing import Callable

import torch

from . import _runtime as rt
from .._lib import check
from .config import TrainingOpConfig
from .quantization import _aligned, _batched_view, convert_from_mxfp4, convert_to_mxfp4


def quantize_dequantize(w: torch.Tensor, axis: int = -1, is_2d_block: bool = False, use_uos: bool = False) -> torch.Tensor:
    assert w.dtype in (torch.float32, torch.bfloat16)
    rt.require_gpu(w)
    ax = axis % w.dim()
    fused = w.dim() >= 2 and (is_2d_block or ax == w.dim() - 1) and w.shape[-1] % 32 == 0 and (not is_2d_block or w.shape[-2] % 32 == 0)
    if is_2d_block and ax not in (w.dim() - 1, w.dim() - 2):
        fused = False
    if not fused:
        q, s = convert_to_mxfp4(w, axis=axis, is_2d_block=is_2d_block, use_uos=use_uos)
        return convert_from_mxfp4(q, s, output_dtype=w.dtype, axis=axis, is_2d_block=is_2d_block)
    x3 = _batched_view(w)
    if x3 is None or not _aligned(x3):
        x3 = _batched_view(w.contiguous())
    out = torch.empty(w.shape, dtype=w.dtype, device=w.device)
    if w.numel() == 0:
        return out
    y3 = _batched_view(out)
    B, M, C = x3.shape
    ld_x = x3.stride(1) if M > 1 else C
    bs_x = x3.stride(0) if B > 1 else M * ld_x
    rc = rt.lib().alto_mxfp4_qdq(x3.data_ptr(), rt.dtype_code(w.dtype), B, M, C, ld_x, bs_x, y3.data_ptr(), C, M * C,
                                 int(is_2d_block), int(use_uos), rt.stream_ptr(w.device))
    check(rc, "alto_mxfp4_qdq")
    return out


QdqFn = Callable[[torch.Tensor, int], torch.Tensor]


def _make_qdq_fn_for(cfg: TrainingOpConfig) -> QdqFn:
    """``dequant(quant(., axis))`` matching the forward path's weight quantisation (optimizer.py:123-176)."""
    if cfg.precision != "mxfp4":
        raise ValueError(f"this build implements precision='mxfp4' only, got {cfg.precision!r}")
    is_2d_block = cfg.use_2dblock_w

    def qdq(w: torch.Tensor, axis: int) -> torch.Tensor:
        original_rows = -1
        if w.dim() == 2 and w.shape[0] % 32 != 0:   # the reference pads such a weight to whole blocks and cuts the result
            original_rows = w.shape[0]
            w = torch.nn.functional.pad(w, (0, 0, 0, 32 - original_rows % 32))
        out = quantize_dequantize(w, axis=axis, is_2d_block=is_2d_block, use_uos=cfg.use_uos)
        if original_rows >= 0:
            out = out[:original_rows]
        return out

    return qdq
