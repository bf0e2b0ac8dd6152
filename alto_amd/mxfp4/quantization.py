"""MXFP4 quantize / dequantize entry points backed by the HIP kernels.

Same names, argument meaning and error behaviour as the reference's
``alto/kernels/fp4/mxfp4/mxfp_quantization.py:410-545`` (``convert_to_mxfp4`` / ``convert_from_mxfp4``), plus two
explicit inputs the reference draws from hidden state: ``rand_bits`` (the 32 random bits per element that
stochastic rounding consumes) and ``hadamard`` (a ``HadamardTransform`` fused in front of an ``axis=-2``
quantisation).  ``quantize_rowcol`` exposes the fused row + column quantizer the linear layer uses.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

from . import _runtime as rt
from .._lib import check
from .hadamard import HadamardTransform

BLOCK_SIZE_DEFAULT = 32


def _clip_code(clip_mode: str) -> int:
    if clip_mode not in rt.CLIP:
        raise ValueError(f"Invalid clip mode: {clip_mode}")
    return rt.CLIP[clip_mode]


def _as_i32(r: torch.Tensor) -> torch.Tensor:
    if r.dtype == torch.uint32:
        return r.view(torch.int32)
    assert r.dtype == torch.int32, f"rand_bits must be int32/uint32, got {r.dtype}"
    return r


def _signs_perm_ptrs(h: Optional[HadamardTransform]):
    if h is None:
        return 0, None, None
    return 1, h.signs.data_ptr(), (None if h.perm is None else h.perm.data_ptr())


def _code_buffer(B: int, R: int, nbytes: int, dev, pad: bool) -> torch.Tensor:
    """[B, R, nbytes] code tensor; with ``pad`` its rows start on 128-byte boundaries (a view over padded storage)."""
    pitch = (nbytes + 127) // 128 * 128 if pad else nbytes
    if pitch == nbytes:
        return torch.empty((B, R, nbytes), dtype=torch.uint8, device=dev)
    return torch.empty((B, R, pitch), dtype=torch.uint8, device=dev)[:, :, :nbytes]


def _quantize_call(x3: torch.Tensor, want_row: bool, want_col: bool, is_2d: bool, use_sr: bool,
                   rand3: Optional[torch.Tensor], hadamard: Optional[HadamardTransform], clip: int, use_uos: bool,
                   pad_codes: bool = False, philox: Optional[Tuple[int, int]] = None, hw_sr: bool = False,
                   pack_row_scales: bool = False, pack_col_scales: bool = False):
    """x3: [B, M, C] with unit stride along C and uniform row / batch strides. Returns the outputs (or None): dense, or
    with ``pad_codes`` code tensors whose rows are padded to whole 128-byte cache lines (for GEMM operands).
    ``philox = (seed, offset)`` with ``use_sr`` and no ``rand3``: the kernel makes the random words itself, element
    (b, i, j) taking word (b M + i) C + j of the stream ``alto_mxfp4_random_bits(.., seed, offset)`` writes.
    ``philox`` = an int64[2] device tensor {key, counter}: the same, with key and counter read on the device and the
    counter moved past the B M C words afterwards (nothing about the draw is a kernel argument: safe under graph capture).
    ``hw_sr``: round with the hardware's stochastic converts (``alto_mxfp4_quantize_sr_hw``; needs ``philox``).
    ``pack_row_scales`` / ``pack_col_scales``: that scale output comes in the packed form of ``linear.pack_scales`` --
    [B, ceil(C/512), M, 16] resp. [B, ceil(M/512), C, 16] -- written by the kernel itself."""
    B, M, C = x3.shape
    dev = x3.device
    packed = pack_row_scales or pack_col_scales
    row_codes = row_scales = col_codes = col_scales = None
    if want_row:
        row_codes = _code_buffer(B, M, C // 2, dev, pad_codes)
        if pack_row_scales:
            row_scales = torch.empty((B, -(-(C // 32) // 16), M, 16), dtype=torch.uint8, device=dev)
        else:
            row_scales = torch.empty((B, M // 32, C // 32) if is_2d else (B, M, C // 32), dtype=torch.uint8, device=dev)
    if want_col:
        col_codes = _code_buffer(B, C, M // 2, dev, pad_codes)
        if pack_col_scales:
            col_scales = torch.empty((B, -(-(M // 32) // 16), C, 16), dtype=torch.uint8, device=dev)
        else:
            col_scales = torch.empty((B, C // 32, M // 32) if is_2d else (B, C, M // 32), dtype=torch.uint8, device=dev)
    had, sp, pp = _signs_perm_ptrs(hadamard)
    ld_x = x3.stride(1) if M > 1 else C
    bs_x = x3.stride(0) if B > 1 else M * ld_x
    ld_r = bs_r = 0
    if use_sr and rand3 is not None:
        ld_r = rand3.stride(1) if M > 1 else C
        bs_r = rand3.stride(0) if B > 1 else M * ld_r
    if packed:   # the general entry point: every rounding mode plus the layout flags
        state, seed, offset, sr_mode = None, 0, 0, 0
        if use_sr and rand3 is not None:
            sr_mode = 1
        elif use_sr:
            assert philox is not None, "stochastic rounding needs rand_bits or a Philox (seed, offset)"
            state = philox if isinstance(philox, torch.Tensor) else None
            seed, offset = (0, 0) if state is not None else (philox[0] & (2 ** 64 - 1), philox[1] & (2 ** 64 - 1))
            sr_mode = 3 if hw_sr else 2
        rc = rt.lib().alto_mxfp4_quantize_ex(
            x3.data_ptr(), rt.dtype_code(x3.dtype), B, M, C, ld_x, bs_x,
            rt.ptr(row_codes), rt.ptr(row_scales), rt.ptr(col_codes), rt.ptr(col_scales),
            row_codes.stride(1) if want_row else 0, col_codes.stride(1) if want_col else 0,
            int(is_2d), sr_mode, rt.ptr(rand3) if sr_mode == 1 else None, ld_r, bs_r, seed, offset, rt.ptr(state),
            had, sp, pp, clip, int(use_uos), int(pack_row_scales) | (int(pack_col_scales) << 1), rt.stream_ptr(dev))
        check(rc, "alto_mxfp4_quantize_ex")
        if state is not None:
            rt.philox_advance(state, rt.lib().alto_mxfp4_quantize_sr_hw_words(rt.dtype_code(x3.dtype), B, M, C) if hw_sr else B * M * C)
        return row_codes, row_scales, col_codes, col_scales
    if use_sr and rand3 is None:
        assert philox is not None, "stochastic rounding needs rand_bits or a Philox (seed, offset)"
        state = philox if isinstance(philox, torch.Tensor) else None
        seed, offset = (0, 0) if state is not None else (philox[0] & (2 ** 64 - 1), philox[1] & (2 ** 64 - 1))
        if hw_sr:
            rc = rt.lib().alto_mxfp4_quantize_sr_hw(
                x3.data_ptr(), rt.dtype_code(x3.dtype), B, M, C, ld_x, bs_x,
                rt.ptr(row_codes), rt.ptr(row_scales), rt.ptr(col_codes), rt.ptr(col_scales),
                row_codes.stride(1) if want_row else 0, col_codes.stride(1) if want_col else 0,
                int(is_2d), seed, offset, rt.ptr(state),
                had, sp, pp, clip, int(use_uos), rt.stream_ptr(dev))
            check(rc, "alto_mxfp4_quantize_sr_hw")
            if state is not None:
                rt.philox_advance(state, rt.lib().alto_mxfp4_quantize_sr_hw_words(rt.dtype_code(x3.dtype), B, M, C))
            return row_codes, row_scales, col_codes, col_scales
        rc = rt.lib().alto_mxfp4_quantize_sr_philox(
            x3.data_ptr(), rt.dtype_code(x3.dtype), B, M, C, ld_x, bs_x,
            rt.ptr(row_codes), rt.ptr(row_scales), rt.ptr(col_codes), rt.ptr(col_scales),
            row_codes.stride(1) if want_row else 0, col_codes.stride(1) if want_col else 0,
            int(is_2d), seed, offset, rt.ptr(state),
            had, sp, pp, clip, int(use_uos), rt.stream_ptr(dev))
        check(rc, "alto_mxfp4_quantize_sr_philox")
        if state is not None:
            rt.philox_advance(state, B * M * C)
        return row_codes, row_scales, col_codes, col_scales
    rc = rt.lib().alto_mxfp4_quantize_pitched(
        x3.data_ptr(), rt.dtype_code(x3.dtype), B, M, C, ld_x, bs_x,
        rt.ptr(row_codes), rt.ptr(row_scales), rt.ptr(col_codes), rt.ptr(col_scales),
        row_codes.stride(1) if want_row else 0, col_codes.stride(1) if want_col else 0,
        int(is_2d), rt.ROUND_SR if use_sr else rt.ROUND_RNE, rt.ptr(rand3), ld_r, bs_r,
        had, sp, pp, clip, int(use_uos), rt.stream_ptr(dev))
    check(rc, "alto_mxfp4_quantize_pitched")
    return row_codes, row_scales, col_codes, col_scales


def _batched_view(t: torch.Tensor) -> Optional[torch.Tensor]:
    """[..., M, C] -> [B, M, C] view with unit stride along C and uniform strides, or None if a copy is needed."""
    if t.dim() < 2 or (t.shape[-1] != 1 and t.stride(-1) != 1):
        return None
    if t.dim() == 2:
        return t.unsqueeze(0)
    for d in range(t.dim() - 3):  # leading dims must collapse into a single batch stride
        if t.shape[d] != 1 and t.stride(d) != t.stride(d + 1) * t.shape[d + 1]:
            return None
    batch = int(math.prod(t.shape[:-2]))
    return t.as_strided((batch, t.shape[-2], t.shape[-1]), (t.stride(-3), t.stride(-2), 1))


def _aligned(t: torch.Tensor) -> bool:
    vec = 8 if t.dtype == torch.bfloat16 else 4
    return t.data_ptr() % 16 == 0 and all(s % vec == 0 for s in t.stride()[:-1])


def _prep(t: torch.Tensor) -> torch.Tensor:
    """Return a [B, M, C] view the kernel accepts (copying only when the strides force it)."""
    v = _batched_view(t)
    if v is None or not _aligned(v):
        v = _batched_view(t.contiguous())
    return v


def convert_to_mxfp4(
    data_hp: torch.Tensor,
    block_size: int = BLOCK_SIZE_DEFAULT,
    axis: int = -1,
    is_2d_block: bool = False,
    use_sr: bool = False,
    use_asm: Optional[bool] = None,
    philox_seed: Optional[int] = None,
    philox_offset: Optional[int] = None,
    clip_mode: str = "none",
    use_uos: bool = False,
    *,
    rand_bits: Optional[torch.Tensor] = None,
    hadamard: Optional[HadamardTransform] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """bf16/fp32 tensor -> (packed E2M1 codes uint8, E8M0 scales uint8).

    Layout contract of the reference (mxfp_quantization.py:439-448,484): the quantisation axis is moved last,
    the results are computed densely in that orientation and returned transposed back, so ``axis=-2`` on
    ``[M, C]`` yields logical ``[M/2, C]`` codes backed by ``[C][M/2]`` memory.

    ``use_asm`` selects the rounding hardware of ``use_sr`` (round-to-nearest always runs on the hardware convert, whose
    results equal the software rule bit for bit): ``True`` rounds with ``v_cvt_scalef32_sr_pk_fp4_{bf16,f32}``, one random
    dword per pair of neighbouring elements, cut from the Philox stream ``(philox_seed, philox_offset)`` inside the kernel
    (mxfp_quantization.py:133-182; ``rand_bits`` cannot be given, ``clip_mode="dynamic"`` is not offered); ``False`` runs
    the software rule of triton_fp4_ops.py:49-61 with 32 random bits per element; ``None`` means the hardware converts, as in the
    reference on gfx950 (``USE_ASM = is_cdna4()``, mxfp_quantization.py:426-427), unless ``rand_bits`` are given, the clip is
    dynamic, or ``use_hardware_stochastic_rounding(False)`` / ``ALTO_MXFP4_HW_SR=0`` moved the default to the software rule.
    ``use_sr`` (software rule) consumes ``rand_bits`` (int32/uint32, same shape as ``data_hp``; element ``[i, j]`` uses
    ``rand_bits[i, j]``); when omitted they come from the library's Philox4x32-10 fill kernel (key and
    counter start ``philox_seed``/``philox_offset`` if given, else a draw from torch's CPU generator).  ``hadamard`` fuses ``hadamard(x, left_mul=True)`` in front of
    an ``axis=-2`` quantisation of a 2D tensor.
    """
    assert block_size == BLOCK_SIZE_DEFAULT, "only block_size=32 is implemented"
    torch._check(data_hp.shape[axis] % block_size == 0)
    assert not is_2d_block or data_hp.size(-2) % block_size == 0
    assert data_hp.dtype in [torch.float32, torch.bfloat16]
    clip = _clip_code(clip_mode)
    rt.require_gpu(data_hp)
    nd = data_hp.dim()
    ax = axis % nd
    philox = None
    hw_sr = bool(use_sr) and rt.hardware_stochastic_rounding(use_asm)
    if hw_sr and (clip_mode == "dynamic" or rand_bits is not None):
        # the hardware path has neither; an explicit use_asm=True says so, the session-wide default steps aside
        if use_asm and clip_mode == "dynamic":
            raise NotImplementedError("clip_mode='dynamic' with the hardware stochastic rounding is not implemented")
        if use_asm:
            raise ValueError("the hardware stochastic rounding draws its random dwords from the Philox stream: pass philox_seed/offset, not rand_bits")
        hw_sr = False
    if hw_sr:
        state = rt.philox_device_state(data_hp.device) if philox_seed is None else None
        philox = state if state is not None else rt.philox_seed_offset(philox_seed, philox_offset)
    elif use_sr:
        if rand_bits is None and ax >= nd - 2 and clip_mode != "dynamic" and data_hp.shape[-1] < 2 ** 26 and rt.philox_in_kernel():
            # the kernel makes the words itself: same bytes as rand_bits = draw_rand_bits(shape, seed, offset), no tensor
            state = rt.philox_device_state(data_hp.device) if philox_seed is None else None
            direct = ax == nd - 1 or data_hp.shape[-1] % 8 == 0   # the paths that hand the stream to the kernel
            philox = state if (state is not None and direct) else rt.philox_seed_offset(philox_seed, philox_offset)
        else:
            if rand_bits is None:
                rand_bits = rt.draw_rand_bits(data_hp.shape, data_hp.device, philox_seed, philox_offset)
            assert rand_bits.shape == data_hp.shape, "rand_bits must have the shape of data_hp"
            rt.require_gpu(rand_bits)
            rand_bits = _as_i32(rand_bits)
    if hadamard is not None:
        assert nd == 2 and ax == 0 and not is_2d_block, "hadamard fuses with a 1D axis=-2 quantisation of a 2D tensor"
    if clip_mode == "dynamic" and data_hp.numel() != 0:
        return _convert_dynamic(data_hp, ax, is_2d_block, use_sr, rand_bits, hadamard, use_uos)

    if data_hp.numel() == 0:
        xt = data_hp.transpose(ax, -1)
        shp = xt.shape
        codes = torch.empty((*shp[:-1], shp[-1] // 2), dtype=torch.uint8, device=data_hp.device)
        ss = (*shp[:-2], shp[-2] // 32, shp[-1] // 32) if is_2d_block else (*shp[:-1], shp[-1] // 32)
        return codes.transpose(ax, -1), torch.empty(ss, dtype=torch.uint8, device=data_hp.device).transpose(ax, -1)

    if nd >= 2 and ax == nd - 2 and data_hp.shape[-1] % 8 == 0:
        # quantise along the second-to-last dim: column output of the [.., M, C] matrices
        x3 = _prep(data_hp)
        r3 = None
        if use_sr and philox is None:
            r3 = rand_bits.expand_as(data_hp)
            r3 = _batched_view(r3 if r3.is_contiguous() else r3.contiguous())
        _, _, cc, cs = _quantize_call(x3, False, True, is_2d_block, use_sr, r3, hadamard, clip, use_uos, philox=philox, hw_sr=hw_sr)
        lead = data_hp.shape[:-2]
        M, C = data_hp.shape[-2], data_hp.shape[-1]
        codes = cc.reshape(*lead, C, M // 2).transpose(-1, -2)
        scales = cs.reshape(*lead, C // 32 if is_2d_block else C, M // 32).transpose(-1, -2)
        return codes, scales

    # general case: move the axis last (view), then quantise along the contiguous dim
    xt = data_hp.transpose(ax, -1)
    shp = xt.shape
    if philox is not None and ax != nd - 1 and not hw_sr:   # (only the last-axis case reaches here with Philox; other axes take a tensor)
        rand_bits = _as_i32(rt.draw_rand_bits(data_hp.shape, data_hp.device, philox[0], philox[1]))
        philox = None
    rtens = rand_bits.transpose(ax, -1) if (use_sr and philox is None) else None
    if is_2d_block:
        x3 = _prep(xt)
        r3 = None
        if use_sr and philox is None:
            r3 = _batched_view(rtens.contiguous())
        rcodes, rscales, _, _ = _quantize_call(x3, True, False, True, use_sr, r3, None, clip, use_uos, philox=philox, hw_sr=hw_sr)
        codes = rcodes.reshape(*shp[:-1], shp[-1] // 2)
        scales = rscales.reshape(*shp[:-2], shp[-2] // 32, shp[-1] // 32)
    else:
        x2 = xt.reshape(-1, shp[-1])
        if x2.stride(-1) != 1 or not _aligned(x2):
            x2 = x2.contiguous()
        r3 = None
        if use_sr and philox is None:
            r3 = rtens.reshape(-1, shp[-1]).contiguous().unsqueeze(0)
        rcodes, rscales, _, _ = _quantize_call(x2.unsqueeze(0), True, False, False, use_sr, r3, None, clip, use_uos, philox=philox, hw_sr=hw_sr)
        codes = rcodes.reshape(*shp[:-1], shp[-1] // 2)
        scales = rscales.reshape(*shp[:-1], shp[-1] // 32)
    return codes.transpose(ax, -1), scales.transpose(ax, -1)


def _convert_dynamic(x: torch.Tensor, ax: int, is_2d_block: bool, use_sr: bool, rand_bits: Optional[torch.Tensor],
                     hadamard: Optional[HadamardTransform], use_uos: bool):
    """``clip_mode="dynamic"`` (std-based scale, mxfp_quantization.py:54-59,65-70): an optional knob served by a plain
    kernel that quantises along the contiguous dim; other axes are brought there with a copy, a Hadamard transform runs
    as its own launch first."""
    if hadamard is not None:
        x = hadamard_left(x, hadamard)
    xt = x.transpose(ax, -1)
    shp = xt.shape
    rows = shp[-2] if (is_2d_block and len(shp) >= 2) else 1
    x3 = xt.contiguous().reshape(-1, rows, shp[-1]) if is_2d_block else xt.contiguous().reshape(1, -1, shp[-1])
    r3 = None
    if use_sr:
        r3 = rand_bits.transpose(ax, -1).contiguous().reshape(x3.shape)
    codes, scales, _, _ = _quantize_call(x3, True, False, is_2d_block, use_sr, r3, None, rt.CLIP["dynamic"], use_uos)
    codes = codes.reshape(*shp[:-1], shp[-1] // 2)
    scales = scales.reshape(*shp[:-2], shp[-2] // 32, shp[-1] // 32) if is_2d_block else scales.reshape(*shp[:-1], shp[-1] // 32)
    return codes.transpose(ax, -1), scales.transpose(ax, -1)


def quantize_rowcol(
    x: torch.Tensor,
    is_2d_block: bool = False,
    use_sr: bool = False,
    rand_bits: Optional[torch.Tensor] = None,
    hadamard: Optional[HadamardTransform] = None,
    clip_mode: str = "none",
    use_uos: bool = False,
    pad_codes: bool = False,
    use_asm: Optional[bool] = None,
    pack_row_scales: bool = False,
    pack_col_scales: bool = False,
):
    """One pass over a 2D ``x [M, C]`` producing BOTH quantisations the linear layer needs.

    Returns ``(row_codes [M, C/2], row_scales, col_codes, col_scales)`` where the column pair equals
    ``convert_to_mxfp4(hadamard(x) if hadamard else x, axis=0, ...)`` (transposed views over ``[C][M/2]`` memory,
    ``clip_mode`` applied there) and the row pair equals ``convert_to_mxfp4(x, axis=-1, ...)`` (no transform, no
    clipping).  Fuses mxfp_linear.py:310-315 with :383-396 (forward, x) and
    :466-494 (backward, dY); for 2D blocks it yields both packings of a weight from one read.

    ``pack_row_scales`` / ``pack_col_scales`` (no dynamic clip): that scale output is the packed tensor
    ``linear.pack_scales`` would make of it -- ``[ceil(C/512), M, 16]`` resp. ``[ceil(M/512), C, 16]`` -- written by the
    quantizer itself, for ``linear.gemm_packed`` / ``grouped_gemm.grouped_forward_packed``.
    """
    assert x.dim() == 2 and x.dtype in (torch.float32, torch.bfloat16)
    rt.require_gpu(x)
    M, C = x.shape
    torch._check(M % 32 == 0 and C % 32 == 0)
    clip = _clip_code(clip_mode)
    philox = None
    hw_sr = bool(use_sr) and rand_bits is None and clip_mode != "dynamic" and rt.hardware_stochastic_rounding(use_asm)
    if hw_sr:
        philox = rt.philox_device_state(x.device)
        if philox is None:
            philox = rt.philox_seed_offset(None, None)
    elif use_sr and rand_bits is None:
        if clip_mode != "dynamic" and C < 2 ** 26 and rt.philox_in_kernel():
            # the kernel makes the words: no tensor, no fill launch
            philox = rt.philox_device_state(x.device)
            if philox is None:
                philox = rt.philox_seed_offset(None, None)
        else:
            rand_bits = rt.draw_rand_bits(x.shape, x.device)
    torch._check(not (pack_row_scales or pack_col_scales) or clip_mode != "dynamic", lambda: "packed scales come without the dynamic clip")
    if clip_mode == "dynamic":   # the row pair is never clipped; the column pair takes the plain path
        rc, rs = convert_to_mxfp4(x, axis=-1, is_2d_block=is_2d_block, use_sr=use_sr, use_uos=use_uos, rand_bits=rand_bits)
        cc, cs = convert_to_mxfp4(x, axis=0, is_2d_block=is_2d_block, use_sr=use_sr, clip_mode="dynamic", use_uos=use_uos,
                                  rand_bits=rand_bits, hadamard=hadamard)
        return rc, rs, cc, cs
    x3 = _prep(x)
    r3 = None
    if use_sr and philox is None:
        assert rand_bits.shape == x.shape
        r3 = _as_i32(rand_bits)
        r3 = _batched_view(r3 if r3.stride(-1) == 1 and r3.stride(0) % 4 == 0 and r3.data_ptr() % 16 == 0 else r3.contiguous())
    rc, rs, cc, cs = _quantize_call(x3, True, True, is_2d_block, use_sr, r3, hadamard, clip, use_uos, pad_codes, philox=philox, hw_sr=hw_sr,
                                    pack_row_scales=pack_row_scales, pack_col_scales=pack_col_scales)
    return rc[0], rs[0], cc[0].transpose(0, 1), cs[0] if pack_col_scales else cs[0].transpose(0, 1)


def hadamard_apply(x: torch.Tensor, h: HadamardTransform, inverse: bool = False, left_mul: bool = False) -> torch.Tensor:
    """``h(x, inverse, left_mul)`` of the reference (transform.py:115-142) in the dtype of ``x``.

    ``left_mul``: ``W @ x`` over the last two dims in blocks of 32 rows; otherwise ``x @ W`` in blocks of 32 along the
    last dim.  ``inverse`` multiplies with ``W.T`` instead.  Leading dims are batch dims.
    """
    assert x.dtype in (torch.float32, torch.bfloat16)
    rt.require_gpu(x)
    if left_mul:
        torch._check(x.dim() >= 2 and x.shape[-2] % 32 == 0, lambda: f"left_mul needs a row count that is a multiple of 32, got {tuple(x.shape)}")
    else:
        torch._check(x.dim() >= 1 and x.shape[-1] % 32 == 0, lambda: f"the last dim must be a multiple of 32, got {tuple(x.shape)}")
    C = x.shape[-1]
    x2 = x.reshape(-1, C)   # whole blocks of 32 rows stay whole: every matrix has a multiple of 32 rows
    if x2.stride(-1) != 1 and x2.numel():
        x2 = x2.contiguous()
    y = torch.empty(x2.shape, dtype=x.dtype, device=x.device)
    M = x2.shape[0]
    if M and C:
        rc = rt.lib().alto_mxfp4_hadamard_apply(x2.data_ptr(), rt.dtype_code(x.dtype), M, C, x2.stride(0) if M > 1 else C, y.data_ptr(), C,
                                                h.signs.data_ptr(), None if h.perm is None else h.perm.data_ptr(),
                                                int(bool(inverse)), int(bool(left_mul)), rt.stream_ptr(x.device))
        check(rc, "alto_mxfp4_hadamard_apply")
    return y.reshape(x.shape)


def hadamard_left(x: torch.Tensor, h: HadamardTransform) -> torch.Tensor:
    """``h(x, left_mul=True)``: the transform along dim 0 in blocks of 32 rows, output in the dtype of ``x``."""
    assert x.dim() == 2
    return hadamard_apply(x, h, inverse=False, left_mul=True)


def convert_from_mxfp4(
    data_lp: torch.Tensor,
    scales: torch.Tensor,
    output_dtype: torch.dtype = torch.float32,
    block_size: int = BLOCK_SIZE_DEFAULT,
    axis: int = -1,
    is_2d_block: bool = False,
    use_asm: Optional[bool] = None,
    clip_mode: str = "none",
) -> torch.Tensor:
    """(packed codes, scales) -> tensor of ``output_dtype`` (mxfp_quantization.py:487-545)."""
    assert output_dtype in [torch.float32, torch.bfloat16]
    assert block_size == BLOCK_SIZE_DEFAULT
    clip = _clip_code(clip_mode)
    rt.require_gpu(data_lp, scales)
    lt = data_lp.transpose(axis, -1)
    st = scales.transpose(axis, -1)
    orig = (*lt.shape[:-1], lt.shape[-1] * 2)
    l2 = lt.reshape(-1, lt.shape[-1]).contiguous()
    R, C = l2.shape[0], l2.shape[1] * 2
    s2 = st.reshape(-1, C // 32).contiguous()
    out = torch.empty((R, C), dtype=output_dtype, device=data_lp.device)
    if R and C:
        if is_2d_block:
            assert orig[-2] % 32 == 0
        rc = rt.lib().alto_mxfp4_dequantize(l2.data_ptr(), s2.data_ptr(), R, C, int(is_2d_block), out.data_ptr(),
                                            rt.dtype_code(output_dtype), C, 1, clip, rt.stream_ptr(data_lp.device))
        check(rc, "alto_mxfp4_dequantize")
    return out.reshape(orig).transpose(axis, -1)
