"""Block-scaled MXFP4 GEMM and the linear autograd function on the HIP kernels.

Mirrors ``alto/kernels/fp4/mxfp4/mxfp_linear.py``: ``blockwise_mxfp4_gemm`` (:142-255), ``MXFP4LinearFunction``
(:258-570) and ``_to_mxfp4_then_scaled_mm`` (:573-602), same argument order and meaning.
"""
from __future__ import annotations

import os
import weakref
from typing import Optional

import torch

from . import _runtime as rt
from .._lib import check
from .dge import DGE_FACTOR
from .hadamard import HadamardFactory, HadamardTransform
from .quantization import BLOCK_SIZE_DEFAULT, convert_to_mxfp4, quantize_rowcol


def unwrap_weight_wrapper(weight: torch.Tensor) -> torch.Tensor:
    """Plain local tensor behind a training-time weight wrapper (alto/kernels/fp4/fp4_common/tensor_wrappers.py:8-30)."""
    if type(weight) is torch.Tensor:
        return weight
    if hasattr(weight, "_data"):
        return weight._data
    return weight.as_subclass(torch.Tensor)


# ----------------------------------------------------------------------------------------------- quantized-weight cache
# The reference re-quantizes the weight in every forward (mxfp_linear.py:317-322).  Between two optimizer steps the
# weight does not change (gradient accumulation, activation recomputation), so the four tensors of its 2D-block
# quantisation can be kept.  An entry belongs to one tensor OBJECT (held through a weak reference, so a new tensor that
# the allocator places at a freed weight's address never matches) and is valid while that object's storage address,
# shape, strides, dtype and autograd version counter are the ones it was made from: any in-place update (optimizer
# step, copy_) bumps the counter and the entry is rebuilt.  The entry dies with the weight.  Writes that bypass the
# version counter (``weight.data.copy_(...)``, some sharded-optimizer paths) are invisible to it: call
# ``clear_weight_cache()`` after them.
_WEIGHT_CACHE_ENABLED = False
_WEIGHT_CACHE: dict = {}
_WEIGHT_CACHE_STATS = {"hits": 0, "misses": 0}


def enable_weight_cache(enabled: bool = True) -> None:
    """Keep the quantized form of 2D-block weights across forwards until the weight is modified in place."""
    global _WEIGHT_CACHE_ENABLED
    _WEIGHT_CACHE_ENABLED = bool(enabled)
    if not enabled:
        clear_weight_cache()


def clear_weight_cache() -> None:
    _WEIGHT_CACHE.clear()
    _WEIGHT_CACHE_STATS["hits"] = _WEIGHT_CACHE_STATS["misses"] = 0


def weight_cache_stats() -> dict:
    return dict(_WEIGHT_CACHE_STATS, entries=len(_WEIGHT_CACHE))


def cached_weight_quantisation(weight: torch.Tensor, tag, make):
    """``make()`` or, with the cache enabled and the tensor object ``weight`` unchanged since, what it returned last time."""
    if not _WEIGHT_CACHE_ENABLED:
        return make()
    key = (id(weight), tag)
    inner = getattr(weight, "_data", weight)   # a wrapper subclass keeps the tensor that in-place updates touch in _data
    stamp = (inner._version, inner.data_ptr(), tuple(inner.shape), tuple(inner.stride()), inner.dtype, inner.device)
    hit = _WEIGHT_CACHE.get(key)
    if hit is not None and hit[0]() is weight and hit[1] == stamp:
        _WEIGHT_CACHE_STATS["hits"] += 1
        return hit[2]
    _WEIGHT_CACHE_STATS["misses"] += 1
    out = make()
    if hit is None or hit[0]() is not weight:   # first entry of this object: drop it when the object goes away
        weakref.finalize(weight, _WEIGHT_CACHE.pop, key, None)
    _WEIGHT_CACHE[key] = (weakref.ref(weight), stamp, out)
    return out


def _quantize_weight_2d(weight: torch.Tensor, use_uos: bool, owner: Optional[torch.Tensor] = None,
                        pack_fprop: bool = False, pack_dgrad: bool = False):
    """(w_q, w_s, w_qt, w_st) of a 2D-block quantisation, from the cache when the weight is unchanged.  ``owner`` is the
    object the CALLER keeps alive (the ``nn.Parameter`` or wrapper tensor): ``weight`` itself may be a plain-tensor alias
    made for this call only (``unwrap_weight_wrapper`` of a Parameter is a new object every time), on which an entry
    would never be found again.  The alias shares the owner's storage and version counter.

    ``pack_fprop`` / ``pack_dgrad``: ``w_s`` / ``w_st`` come in the packed form of :func:`pack_scales` (rows N, reduction K
    resp. rows K, reduction N), written by the quantizer."""
    return cached_weight_quantisation(weight if owner is None else owner, ("linear2d", bool(use_uos), bool(pack_fprop), bool(pack_dgrad)),
                                      lambda: quantize_rowcol(weight, True, use_uos=use_uos, pad_codes=True,
                                                              pack_row_scales=pack_fprop, pack_col_scales=pack_dgrad))


def transpose_codes(codes: torch.Tensor) -> torch.Tensor:
    """[R, C/2] bytes packed along C -> [C, R/2] bytes packed along R (same 4-bit codes)."""
    assert codes.dim() == 2 and codes.dtype == torch.uint8
    rt.require_gpu(codes)
    c = codes.contiguous()
    R, C = c.shape[0], c.shape[1] * 2
    assert R % 2 == 0
    out = torch.empty((C, R // 2), dtype=torch.uint8, device=codes.device)
    check(rt.lib().alto_mxfp4_transpose_codes(c.data_ptr(), R, C, out.data_ptr(), rt.stream_ptr(codes.device)), "alto_mxfp4_transpose_codes")
    return out


def _canonical_operand(t: torch.Tensor, s: torch.Tensor, rows_first: bool, k_pack: bool):
    """Bring one GEMM operand to the form the kernel consumes: codes [rows, K/2] with unit stride along K.

    ``t`` is the 2D code tensor in the orientation the caller holds (rows x K if ``rows_first`` else K x rows, the
    packed dim halved); ``s`` the scales in the same orientation.  Returns (codes, scales_view[rows(/32), K/32]).
    """
    tv = t if rows_first else t.transpose(0, 1)   # [rows', K'] with one of the dims halved
    sv = s if rows_first else s.transpose(0, 1)   # [rows or rows/32, K/32]
    if k_pack:
        if tv.stride(1) != 1 or tv.stride(0) % 16 != 0 or tv.data_ptr() % 16 != 0:
            tv = tv.contiguous()
        return tv, sv
    # packed along the row dim: memory must be [K][rows/2]; nibble-transpose into [rows][K/2]
    return transpose_codes(tv.transpose(0, 1)), sv


def pack_scales(scales: torch.Tensor, rows: int, K: int, is_2d_block: bool = False) -> torch.Tensor:
    """Scales of one GEMM operand ([rows or rows/32, K/32], any strides) -> the packed form the tile kernels read without a
    detour through registers: uint8 ``[ceil(K/512), rows, 16]``, the 16 bytes of a row and 512-K block in the order the MFMA
    loop uses them, bytes beyond K = 127.  An internal operand layout (no counterpart in the reference)."""
    rt.require_gpu(scales)
    assert scales.dim() == 2 and scales.dtype == torch.uint8
    out = torch.empty((-(-(K // 32) // 16), rows, 16), dtype=torch.uint8, device=scales.device)
    if out.numel():
        rc = rt.lib().alto_mxfp4_pack_scales(scales.data_ptr(), scales.stride(0), scales.stride(1), int(is_2d_block), rows, K, out.data_ptr(),
                                             rt.stream_ptr(scales.device))
        check(rc, "alto_mxfp4_pack_scales")
    return out


def packed_gemm_supported(M: int, N: int, K: int) -> bool:
    """Shapes the packed-scale kernel serves (the 256x256 tile kernel's conditions; anything else takes plain scales)."""
    return M >= 128 and N >= 128 and K >= 512 and N % 8 == 0 and M * (K // 2) < 2 ** 31 and N * (K // 2) < 2 ** 31


_PACKED_SCALES = os.environ.get("ALTO_MXFP4_PACKED_SCALES", "1") != "0"   # the process-wide default; see use_packed_scales


def use_packed_scales(enabled: bool = True) -> None:
    """The linear and grouped autograd functions hand scales to their GEMMs in the packed form wherever the tile kernel
    serves the shape (default), or always in the reference's plain form.  Results are the same bit for bit."""
    global _PACKED_SCALES
    _PACKED_SCALES = bool(enabled)


def packed_scales_enabled() -> bool:
    return _PACKED_SCALES


def _k_major(codes: torch.Tensor) -> torch.Tensor:
    """Codes [rows, K/2] with unit stride along K and 16-byte aligned rows (a copy only when the view is not)."""
    if codes.stride(1) != 1 or codes.stride(0) % 16 != 0 or codes.data_ptr() % 16 != 0:
        return codes.contiguous()
    return codes


def gemm_packed(a_q: torch.Tensor, a_ps: torch.Tensor, b_q: torch.Tensor, b_ps: torch.Tensor, out_scale: float = 1.0) -> torch.Tensor:
    """C [M, N] (bf16) = A [M, K] . B [N, K]^T with codes packed along K and scales in the form of :func:`pack_scales`."""
    M, N, K = a_q.shape[0], b_q.shape[0], a_q.shape[1] * 2
    assert b_q.shape[1] * 2 == K and a_q.stride(1) == 1 and b_q.stride(1) == 1
    assert a_ps.shape == (-(-(K // 32) // 16), M, 16) and b_ps.shape == (-(-(K // 32) // 16), N, 16) and a_ps.is_contiguous() and b_ps.is_contiguous()
    c = torch.empty((M, N), dtype=torch.bfloat16, device=a_q.device)
    rc = rt.lib().alto_mxfp4_gemm_ps(a_q.data_ptr(), a_q.stride(0), a_ps.data_ptr(), b_q.data_ptr(), b_q.stride(0), b_ps.data_ptr(), M, N, K,
                                     c.data_ptr(), c.stride(0), float(out_scale), rt.stream_ptr(a_q.device))
    check(rc, "alto_mxfp4_gemm_ps")
    return c


def blockwise_mxfp4_gemm(
    a: torch.Tensor,
    a_s: torch.Tensor,
    b: torch.Tensor,
    b_s: torch.Tensor,
    use_2dblock_a: bool = False,
    use_2dblock_b: bool = False,
    k_pack_a: bool = True,
    k_pack_b: bool = True,
    trans_a: bool = False,
    trans_b: bool = False,
    block_size: int = BLOCK_SIZE_DEFAULT,
    output_dtype: torch.dtype = torch.float32,
    out_scale: float = 1.0,
) -> torch.Tensor:
    """C = op(A) @ op(B) on FP4 codes with E8M0 scales per 32 along K, fp32 accumulation (mxfp_linear.py:142-255).

    M, N, K refer to unpacked FP4 element counts.  ``a`` is ``[M, K]`` (``[K, M]`` if ``trans_a``), ``b`` is
    ``[K, N]`` (``[N, K]`` if ``trans_b``), each with its packed dim halved: packed along K when ``k_pack_*``.
    """
    assert a.dim() == 2 and b.dim() == 2
    assert block_size == BLOCK_SIZE_DEFAULT
    rt.require_gpu(a, a_s, b, b_s)
    if trans_a:
        K, M = a.shape
    else:
        M, K = a.shape
    if k_pack_a:
        K *= 2
    else:
        M *= 2
    a_rows_s = M // block_size if use_2dblock_a else M
    exp_as = (K // block_size, a_rows_s) if trans_a else (a_rows_s, K // block_size)
    assert a_s.shape == torch.Size(exp_as), f"A scale has shape {a_s.shape}, but {exp_as} is expected."
    if trans_b:
        N, KB = b.shape
    else:
        KB, N = b.shape
    if k_pack_b:
        KB *= 2
    else:
        N *= 2
    assert KB == K, f"Input B has unpacked reduction shape ({KB}) but {(K)} is expected."
    b_rows_s = N // block_size if use_2dblock_b else N
    exp_bs = (b_rows_s, K // block_size) if trans_b else (K // block_size, b_rows_s)
    assert b_s.shape == torch.Size(exp_bs)
    assert output_dtype in (torch.float32, torch.bfloat16)

    ac, asv = _canonical_operand(a, a_s, rows_first=not trans_a, k_pack=k_pack_a)
    bc, bsv = _canonical_operand(b, b_s, rows_first=trans_b, k_pack=k_pack_b)
    c = torch.empty((M, N), dtype=output_dtype, device=a.device)
    if M == 0 or N == 0:
        return c
    if K == 0:
        return c.zero_()
    rc = rt.lib().alto_mxfp4_gemm(
        ac.data_ptr(), ac.stride(0), asv.data_ptr(), asv.stride(0), asv.stride(1), int(use_2dblock_a),
        bc.data_ptr(), bc.stride(0), bsv.data_ptr(), bsv.stride(0), bsv.stride(1), int(use_2dblock_b),
        M, N, K, c.data_ptr(), rt.dtype_code(output_dtype), c.stride(0), float(out_scale), rt.stream_ptr(a.device))
    check(rc, "alto_mxfp4_gemm")
    return c


def _wgrad_scale(clip_mode: str, use_dge: bool) -> float:
    """Constant multiplier of dW: 16/9 undoes the two 3/4 clips (mxfp_linear.py:543-544), the estimator's factor follows
    mxfp_linear.py:549-568 (constant on the E2M1 grid, see dge.py)."""
    s = 16.0 / 9.0 if clip_mode == "static" else 1.0
    return s * DGE_FACTOR if use_dge else s


@torch.compiler.allow_in_graph
class MXFP4LinearFunction(torch.autograd.Function):
    """``y = x @ W^T`` with MXFP4 operands in forward and in both backward GEMMs (mxfp_linear.py:258-570).

    Recipe branch ``use_2dblock_x=False, use_2dblock_w=True`` runs on three fused launches per direction:
    forward = one pass over x (row codes for fprop + Hadamard/column codes saved for wgrad), one pass over W
    (both packings of its 2D-block codes), one GEMM; backward = one pass over dY (row + Hadamard/column codes,
    stochastic rounding) and two GEMMs.  Other flag combinations follow the reference's call sequence with the
    same kernels.
    """

    @staticmethod
    def forward(ctx, x, weight, use_2dblock_x, use_2dblock_w, use_sr_grad, use_dge, clip_mode,
                use_macro_block_scaling, hadamard_transform: Optional[HadamardTransform] = None, use_uos: bool = False):
        assert not use_macro_block_scaling, "Macro block scaling is not supported in real MXFP4 kernels"
        weight_owner = weight
        weight = unwrap_weight_wrapper(weight)
        original_shape = x.shape
        original_dtype = x.dtype
        x2 = x.reshape(-1, original_shape[-1])
        M = x2.shape[0]

        fuse_x = (not use_2dblock_x) and M % 32 == 0
        # Packed scales: each of the three GEMMs takes them when the tile kernel serves its shape; the quantizers then
        # write that layout directly, so nothing is converted on the way.
        N, K = weight.shape
        can_pack = (_PACKED_SCALES and fuse_x and clip_mode != "dynamic" and original_dtype == torch.bfloat16
                    and weight.dtype in (torch.bfloat16, torch.float32) and M * max(N, K) < 2 ** 36 and N * K < 2 ** 36)
        pk_f = can_pack and packed_gemm_supported(M, N, K)   # fprop: y [M, N], reduction K
        pk_d = can_pack and packed_gemm_supported(M, K, N)   # dgrad: dx [M, K], reduction N
        pk_w = can_pack and packed_gemm_supported(N, K, M)   # wgrad: dw [N, K], reduction M
        if fuse_x:
            x_q, x_s, x_qm, x_sm = quantize_rowcol(x2, False, hadamard=hadamard_transform, clip_mode=clip_mode, use_uos=use_uos, pad_codes=True,
                                                   pack_row_scales=pk_f, pack_col_scales=pk_w)
        else:
            x_q, x_s = convert_to_mxfp4(x2, axis=-1, is_2d_block=use_2dblock_x, use_uos=use_uos)
            if use_2dblock_x:
                x_qm, x_sm = x_q, x_s
            else:  # token count not a multiple of 32: the reference fails in its axis=0 quantisation as well
                x_qm, x_sm = convert_to_mxfp4(x2, axis=0, clip_mode=clip_mode, use_uos=use_uos, hadamard=hadamard_transform)

        if use_2dblock_w:
            w_q, w_s, w_qt, w_st = _quantize_weight_2d(weight, use_uos, owner=weight_owner, pack_fprop=pk_f, pack_dgrad=pk_d)
            # [N/2, K] view over [K][N/2] memory; scales [N/32, K/32] as a view over [K/32][N/32] memory (same values as
            # w_s, stored so that the dgrad GEMM reads them with unit stride along its reduction dim N), or packed
            w_bwd, w_bwd_s = w_qt, w_st
        else:
            w_q, w_s = convert_to_mxfp4(weight, axis=-1, is_2d_block=False, use_uos=use_uos)
            w_bwd, w_bwd_s = convert_to_mxfp4(weight, axis=0, is_2d_block=False, use_uos=use_uos)
            if pk_f:
                w_s = pack_scales(w_s, N, K)
            if pk_d:
                w_bwd_s = pack_scales(w_bwd_s.transpose(0, 1), K, N)

        if pk_f:
            y = gemm_packed(_k_major(x_q), x_s, _k_major(w_q), w_s)
        else:
            y = blockwise_mxfp4_gemm(x_q, x_s, w_q, w_s, use_2dblock_a=use_2dblock_x, use_2dblock_b=use_2dblock_w,
                                     trans_b=True, output_dtype=original_dtype)
        ctx.save_for_backward(x_qm, x_sm, w_bwd, w_bwd_s)
        ctx.packed = (pk_d, pk_w)
        ctx.use_2dblock_x = use_2dblock_x
        ctx.use_2dblock_w = use_2dblock_w
        ctx.original_dtype = original_dtype
        ctx.use_sr_grad = use_sr_grad
        ctx.hadamard_transform = hadamard_transform
        ctx.clip_mode = clip_mode
        ctx.use_uos = use_uos
        ctx.use_dge = bool(use_dge)
        return y.view(*original_shape[:-1], -1)

    @staticmethod
    def backward(ctx, grad_output):
        original_shape = grad_output.shape
        go = grad_output.reshape(-1, original_shape[-1])
        x_qm, x_sm, w_bwd, w_bwd_s = ctx.saved_tensors
        pk_d, pk_w = ctx.packed
        sr = bool(ctx.use_sr_grad)
        # random words: made inside the quantizer (Philox) unless a source of explicit words is installed
        rand = rt.draw_rand_bits(go.shape, go.device) if (sr and not rt.philox_in_kernel()) else None
        if ctx.use_2dblock_x:
            go_q, go_s = convert_to_mxfp4(go, axis=-1, is_2d_block=True, use_sr=sr, rand_bits=rand, use_uos=ctx.use_uos)
            go_qm, go_sm = go_q, go_s
        else:
            go_q, go_s, go_qm, go_sm = quantize_rowcol(go, False, use_sr=sr, rand_bits=rand, hadamard=ctx.hadamard_transform,
                                                       clip_mode=ctx.clip_mode, use_uos=ctx.use_uos, pad_codes=True,
                                                       pack_row_scales=pk_d, pack_col_scales=pk_w)
        # dgrad: reduction over N.  The saved weight operand is already packed along N (both layouts of a 2D-block
        # quantisation hold the same codes), so no k_pack=False repack is needed here.
        if pk_d:
            grad_inputs = gemm_packed(_k_major(go_q), go_s, _k_major(w_bwd.transpose(0, 1)), w_bwd_s)
        else:
            grad_inputs = blockwise_mxfp4_gemm(go_q, go_s, w_bwd, w_bwd_s, use_2dblock_a=ctx.use_2dblock_x,
                                               use_2dblock_b=ctx.use_2dblock_w, k_pack_b=True, output_dtype=ctx.original_dtype)
        # wgrad: reduction over tokens
        if pk_w:
            grad_weights = gemm_packed(_k_major(go_qm.transpose(0, 1)), go_sm, _k_major(x_qm.transpose(0, 1)), x_sm,
                                       out_scale=_wgrad_scale(ctx.clip_mode, ctx.use_dge))
        else:
            grad_weights = blockwise_mxfp4_gemm(go_qm, go_sm, x_qm, x_sm, use_2dblock_a=ctx.use_2dblock_x,
                                                use_2dblock_b=ctx.use_2dblock_x, trans_a=True,
                                                k_pack_a=not ctx.use_2dblock_x, k_pack_b=not ctx.use_2dblock_x,
                                                output_dtype=ctx.original_dtype,
                                                out_scale=_wgrad_scale(ctx.clip_mode, ctx.use_dge))
        return grad_inputs.view(*original_shape[:-1], -1), grad_weights, None, None, None, None, None, None, None, None


def _to_mxfp4_then_scaled_mm(
    a: torch.Tensor,
    b: torch.Tensor,
    use_2dblock_x: bool,
    use_2dblock_w: bool,
    use_sr_grad: int,
    use_dge: bool,
    clip_mode: str,
    use_hadamard: bool,
    use_macro_block_scaling: bool = False,
    use_uos: bool = False,
) -> torch.Tensor:
    """``a @ b.T`` through ``MXFP4LinearFunction`` with a fresh random Hadamard per call (mxfp_linear.py:573-602)."""
    hadamard_transform = HadamardFactory.create_transform(device=b.device) if use_hadamard else None
    return MXFP4LinearFunction.apply(a, b, use_2dblock_x, use_2dblock_w, use_sr_grad, use_dge, clip_mode,
                                     use_macro_block_scaling, hadamard_transform, use_uos)
