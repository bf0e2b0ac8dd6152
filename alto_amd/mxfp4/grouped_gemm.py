"""Contiguous grouped (MoE) MXFP4 GEMM on the HIP kernels.

Mirrors ``alto/kernels/fp4/mxfp4/mxfp_grouped_gemm``: ``mxfp4_grouped_gemm_forward`` (cg_forward.py:200-303),
``mxfp4_grouped_gemm_backward_inputs`` / ``_weights`` (cg_backward.py:398-593), ``MXFP4GroupedGEMM`` (:599-930),
``mxfp4_grouped_gemm`` (:933-991) and ``_quantize_then_mxfp_scaled_grouped_mm`` (functional.py:11-38).

The kernels consume expert row ranges (``offs``: E+1 int32 offsets on the device) instead of a per-row expert
index; the index form of the reference API is converted on the device without a host sync.  Groups may be ragged
for 1D activation scales; the weight gradient (and 2D activation blocks) need every boundary between two experts at a
multiple of 32 rows, since one MX block along the token dim cannot be split between experts: the kernel checks this on
the device and writes NaN into the weight gradient of an expert with a misaligned boundary (the reference asks for 128).
"""
from __future__ import annotations

from typing import NamedTuple, Optional

import torch

from . import _runtime as rt
from .._lib import check
from .hadamard import HadamardFactory, HadamardTransform
from .linear import _wgrad_scale, cached_weight_quantisation, packed_scales_enabled, transpose_codes, unwrap_weight_wrapper
from .quantization import quantize_rowcol

ALIGN_SIZE_M = 128


def create_indices_from_offsets_nosync(m_offsets: torch.Tensor) -> torch.Tensor:
    """Cumulative group ends -> per-row expert index, no host sync beyond the size read the reference also does
    (alto/kernels/dsgemm_utils.py:96-112)."""
    total_size = m_offsets[-1]
    all_indices = torch.arange(total_size, device=m_offsets.device, dtype=torch.int32)
    return torch.bucketize(all_indices, m_offsets, right=True, out_int32=True)


class Groups(NamedTuple):
    """Row groups of a grouped GEMM: group g = rows [offs[g], offs[g+1]) served by expert ``expert[g]`` (or g)."""
    offs: torch.Tensor                # int32 [n + 1] on the device
    expert: Optional[torch.Tensor]    # int32 [n] on the device, None: expert id == group index
    n: int


def groups_from_indices(expert_indices: torch.Tensor) -> Groups:
    """Per-row expert ids with one expert per aligned 128-row group (the reference's contract, cg_forward.py:135-136)."""
    M_total = expert_indices.shape[0]
    n = M_total // ALIGN_SIZE_M
    offs = torch.arange(n + 1, device=expert_indices.device, dtype=torch.int32) * ALIGN_SIZE_M
    return Groups(offs, expert_indices[::ALIGN_SIZE_M].to(torch.int32).contiguous(), n)


def groups_from_offsets(offsets: torch.Tensor) -> Groups:
    """int32 [E+1] offsets with a leading 0: rows sorted by expert, group g == expert g, ragged sizes allowed."""
    assert offsets.dtype == torch.int32 and offsets.dim() == 1
    return Groups(offsets.contiguous(), None, offsets.shape[0] - 1)


def offsets_from_ends(offs: torch.Tensor) -> torch.Tensor:
    """Cumulative group ends [E] (torch._grouped_mm convention) -> offsets [E+1] with a leading 0."""
    return torch.cat([torch.zeros(1, dtype=torch.int32, device=offs.device), offs.to(torch.int32)])


def _scale_strides(s: torch.Tensor):
    return s.stride(0), s.stride(1), s.stride(2)


def grouped_forward(a_q, a_s, w_q, w_s, groups: Groups, use_2dblock_x, use_2dblock_w, output_dtype, plan=None, return_plan=False):
    """out[r] = A[r] . W[e(r)]^T with w_q [E, N, K/2] (unit stride along K) and w_s [E, N or N/32, K/32].

    ``plan``: the pass list an earlier call over the same ``groups`` and row count wrote (``return_plan=True`` hands it
    out): the one-workgroup kernel that builds it is then not launched again (the input gradient reuses the forward's)."""
    E, N = w_q.shape[0], w_q.shape[1]
    K = a_q.shape[1] * 2
    assert w_q.shape[2] * 2 == K, f"Input K ({K}) must match weight K ({w_q.shape[2] * 2})"
    if a_q.stride(1) != 1 or a_q.stride(0) % 16:
        a_q = a_q.contiguous()
    if w_q.stride(2) != 1 or w_q.stride(1) % 16 or w_q.stride(0) % 16:
        w_q = w_q.contiguous()
    out = torch.empty((a_q.shape[0], N), dtype=output_dtype, device=a_q.device)
    if out.numel() == 0:
        return (out, plan) if return_plan else out
    # the pass list the kernels exchange (a few KB; torch's caching allocator hands it out without a device call)
    ws_bytes = rt.lib().alto_mxfp4_grouped_gemm_workspace_bytes(a_q.shape[0], groups.n)
    if plan is not None:
        assert plan.dtype == torch.uint8 and plan.numel() >= ws_bytes and plan.device == a_q.device
        ws, fn, name = plan, rt.lib().alto_mxfp4_grouped_gemm_planned, "alto_mxfp4_grouped_gemm_planned"
    else:
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a_q.device)
        fn, name = rt.lib().alto_mxfp4_grouped_gemm, "alto_mxfp4_grouped_gemm"
    rc = fn(
        a_q.data_ptr(), a_q.stride(0), a_s.data_ptr(), a_s.stride(0), a_s.stride(1), int(use_2dblock_x),
        w_q.data_ptr(), w_q.stride(0), w_q.stride(1), w_s.data_ptr(), w_s.stride(0), w_s.stride(1), w_s.stride(2), int(use_2dblock_w),
        groups.offs.data_ptr(), rt.ptr(groups.expert), groups.n, E, a_q.shape[0], N, K, out.data_ptr(), rt.dtype_code(output_dtype), out.stride(0),
        ws.data_ptr(), ws.numel(), rt.stream_ptr(a_q.device))
    check(rc, name)
    return (out, ws) if return_plan else out


def pack_expert_scales(w_s: torch.Tensor, N: int, K: int, is_2d_block: bool) -> torch.Tensor:
    """Weight scales [E, N or N/32, K/32] -> packed [E, ceil(K/512), N, 16] (see ``linear.pack_scales``)."""
    from .linear import pack_scales
    return torch.stack([pack_scales(w_s[e], N, K, is_2d_block) for e in range(w_s.shape[0])])


def grouped_forward_packed(a_q, a_ps, w_q, w_ps, groups: Groups, plan=None, return_plan=False):
    """:func:`grouped_forward` on packed scales (bf16 output): ``a_ps`` [ceil(K/512), M, 16], ``w_ps`` [E, ceil(K/512), N, 16]."""
    E, N = w_q.shape[0], w_q.shape[1]
    M, K = a_q.shape[0], a_q.shape[1] * 2
    assert w_q.shape[2] * 2 == K and a_q.stride(1) == 1 and w_q.stride(2) == 1
    KB = -(-(K // 32) // 16)
    assert a_ps.shape == (KB, M, 16) and w_ps.shape == (E, KB, N, 16) and a_ps.is_contiguous() and w_ps.is_contiguous()
    out = torch.empty((M, N), dtype=torch.bfloat16, device=a_q.device)
    ws_bytes = rt.lib().alto_mxfp4_grouped_gemm_workspace_bytes(M, groups.n)
    ws = plan if plan is not None else torch.empty(ws_bytes, dtype=torch.uint8, device=a_q.device)
    rc = rt.lib().alto_mxfp4_grouped_gemm_ps(
        a_q.data_ptr(), a_q.stride(0), a_ps.data_ptr(), w_q.data_ptr(), w_q.stride(0), w_q.stride(1), w_ps.data_ptr(), w_ps.stride(0),
        groups.offs.data_ptr(), rt.ptr(groups.expert), groups.n, E, M, N, K, out.data_ptr(), out.stride(0),
        ws.data_ptr(), ws.numel(), int(plan is not None), rt.stream_ptr(a_q.device))
    check(rc, "alto_mxfp4_grouped_gemm_ps")
    return (out, ws) if return_plan else out


def grouped_packed_supported(M: int, N: int, K: int, num_groups: int, lda: Optional[int] = None, ldw: Optional[int] = None) -> bool:
    """Shapes :func:`grouped_forward_packed` serves (the conditions of the grouped 256x256 tile kernel); ``lda`` / ``ldw`` are
    the row pitches of the codes in bytes (default: K/2 rounded up to 16)."""
    pitch = -(-(K // 2) // 16) * 16
    lda = pitch if lda is None else lda
    ldw = pitch if ldw is None else ldw
    return (M >= 128 and N >= 128 and K >= 512 and N % 8 == 0 and M * lda < 2 ** 31 and N * ldw < 2 ** 31
            and -(-(K // 32) // 16) * max(M, N) * 16 < 2 ** 31 and (-(-M // 256) + num_groups + 2) * -(-N // 256) < 2 ** 28)


def grouped_plan(groups: Groups, num_experts: int, m_total: int) -> torch.Tensor:
    """The pass list of ``groups`` over ``m_total`` rows, for ``grouped_forward(..., plan=...)``."""
    dev = groups.offs.device
    ws_bytes = rt.lib().alto_mxfp4_grouped_gemm_workspace_bytes(m_total, groups.n)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    rc = rt.lib().alto_mxfp4_grouped_gemm_plan(groups.offs.data_ptr(), rt.ptr(groups.expert), groups.n, num_experts, m_total, ws.data_ptr(), ws_bytes,
                                               rt.stream_ptr(dev))
    check(rc, "alto_mxfp4_grouped_gemm_plan")
    return ws


def mxfp4_grouped_gemm_forward(inputs, expert_weights, expert_indices, input_scales, weight_scales, trans_weights=True,
                               use_2dblock_x=False, use_2dblock_w=True, output_dtype=torch.bfloat16):
    """cg_forward.py:200-303.  inputs [M_buf, K/2]; expert_weights [E, N, K/2] if trans_weights else [E, K/2, N]."""
    assert expert_indices.is_contiguous(), "Expert indices tensor must be contiguous"
    M_total = expert_indices.shape[0]
    torch._check(M_total > 0)
    torch._check(M_total % ALIGN_SIZE_M == 0)
    rt.require_gpu(inputs, expert_weights, expert_indices, input_scales, weight_scales)
    E = expert_weights.shape[0]
    w_q = expert_weights if trans_weights else expert_weights.transpose(1, 2)
    w_s = weight_scales if trans_weights else weight_scales.transpose(1, 2)
    return grouped_forward(inputs, input_scales, w_q, w_s, groups_from_indices(expert_indices), use_2dblock_x, use_2dblock_w, output_dtype)


def mxfp4_grouped_gemm_backward_inputs(grad_output, expert_weights, expert_indices, go_scales, expert_weight_scales,
                                       trans_weights=True, use_2dblock_x=False, use_2dblock_w=True, k_pack_w=True,
                                       output_dtype=torch.bfloat16):
    """dX[r] = dY[r] . W[e(r)] (cg_backward.py:500-593).  Reduction over N; W packed along N iff ``k_pack_w``."""
    assert expert_indices.is_contiguous(), "Expert indices tensor must be contiguous"
    M_total = expert_indices.shape[0]
    torch._check(M_total > 0)
    torch._check(M_total % ALIGN_SIZE_M == 0)
    rt.require_gpu(grad_output, expert_weights, expert_indices, go_scales, expert_weight_scales)
    E = expert_weights.shape[0]
    # bring the weights to [E, K_out, N/2] packed along N
    wv = expert_weights if trans_weights else expert_weights.transpose(1, 2)          # [E, N', K'] one dim halved
    sv = expert_weight_scales if trans_weights else expert_weight_scales.transpose(1, 2)
    if k_pack_w:
        w_can = wv.transpose(1, 2)                                                    # [E, K, N/2] view
    else:
        w_can = torch.stack([transpose_codes(wv[e]) for e in range(E)])               # [E, N, K/2] -> [E, K, N/2]
    s_can = sv.transpose(1, 2)                                                        # [E, K(/32), N/32]
    return grouped_forward(grad_output, go_scales, w_can, s_can, groups_from_indices(expert_indices), use_2dblock_x, use_2dblock_w, output_dtype)


def grouped_dw(go_qm, go_sm, x_qm, x_sm, groups: Groups, num_experts, output_dtype, trans_weights=True, out_scale=1.0, is_2d=False):
    """dW[e] = sum_{rows of e} dY^T X with token-packed operands: go_qm [N, M/2], x_qm [K, M/2] (unit stride along tokens),
    scales [N, M/32] / [K, M/32], or with ``is_2d`` one scale per 32 x 32 block: [N/32, M/32] / [K/32, M/32]."""
    N, K = go_qm.shape[0], x_qm.shape[0]
    M_total = go_qm.shape[1] * 2
    assert x_qm.shape[1] * 2 == M_total
    if go_qm.stride(1) != 1 or go_qm.stride(0) % 16:
        go_qm = go_qm.contiguous()
    if x_qm.stride(1) != 1 or x_qm.stride(0) % 16:
        x_qm = x_qm.contiguous()
    if go_sm.stride(1) != 1:   # the tiled kernel reads scale rows with unit stride along the tokens
        go_sm = go_sm.contiguous()
    if x_sm.stride(1) != 1:
        x_sm = x_sm.contiguous()
    shape = (num_experts, N, K) if trans_weights else (num_experts, K, N)
    dw = torch.empty(shape, dtype=output_dtype, device=go_qm.device)
    s_e, s_n, s_k = (dw.stride(0), dw.stride(1), dw.stride(2)) if trans_weights else (dw.stride(0), dw.stride(2), dw.stride(1))
    rc = rt.lib().alto_mxfp4_grouped_gemm_dw(
        go_qm.data_ptr(), go_qm.stride(0), go_sm.data_ptr(), go_sm.stride(0), go_sm.stride(1), int(is_2d),
        x_qm.data_ptr(), x_qm.stride(0), x_sm.data_ptr(), x_sm.stride(0), x_sm.stride(1), int(is_2d),
        groups.offs.data_ptr(), rt.ptr(groups.expert), groups.n, num_experts, M_total, N, K, dw.data_ptr(), rt.dtype_code(output_dtype), s_e, s_n, s_k,
        float(out_scale), rt.stream_ptr(go_qm.device))
    check(rc, "alto_mxfp4_grouped_gemm_dw")
    return dw


def grouped_dw_packed_supported(M_total: int, N: int, K: int, num_groups: int, num_experts: int) -> bool:
    """Shapes :func:`grouped_dw_packed` serves (the conditions of the 256x256 dW tile kernel, dW stored [E, N, K] or [E, K, N]
    contiguous, code rows of M_total / 2 bytes rounded up to 16)."""
    pitch = -(-(M_total // 2) // 16) * 16
    return (M_total >= 512 and M_total % 32 == 0 and N >= 128 and K >= 128 and N % 8 == 0 and K % 8 == 0 and N * pitch < 2 ** 31 and K * pitch < 2 ** 31
            and num_groups <= 32768 and num_experts <= 65535 and -(-M_total // 512) * max(N, K) * 16 < 2 ** 31)


def grouped_dw_packed(go_qm, go_ps, x_qm, x_ps, groups: Groups, num_experts, trans_weights=True, out_scale=1.0):
    """:func:`grouped_dw` on scales packed along the tokens (bf16 dW): ``go_ps`` [ceil(M/512), N, 16], ``x_ps`` [ceil(M/512), K, 16]
    -- the column scales ``quantize_rowcol(..., pack_col_scales=True)`` writes."""
    N, K = go_qm.shape[0], x_qm.shape[0]
    M_total = go_qm.shape[1] * 2
    assert x_qm.shape[1] * 2 == M_total
    if go_qm.stride(1) != 1 or go_qm.stride(0) % 16:
        go_qm = go_qm.contiguous()
    if x_qm.stride(1) != 1 or x_qm.stride(0) % 16:
        x_qm = x_qm.contiguous()
    KB = -(-M_total // 512)
    assert go_ps.shape == (KB, N, 16) and x_ps.shape == (KB, K, 16) and go_ps.is_contiguous() and x_ps.is_contiguous()
    shape = (num_experts, N, K) if trans_weights else (num_experts, K, N)
    dw = torch.empty(shape, dtype=torch.bfloat16, device=go_qm.device)
    s_e, s_n, s_k = (dw.stride(0), dw.stride(1), dw.stride(2)) if trans_weights else (dw.stride(0), dw.stride(2), dw.stride(1))
    rc = rt.lib().alto_mxfp4_grouped_gemm_dw_ps(
        go_qm.data_ptr(), go_qm.stride(0), go_ps.data_ptr(), x_qm.data_ptr(), x_qm.stride(0), x_ps.data_ptr(),
        groups.offs.data_ptr(), rt.ptr(groups.expert), groups.n, num_experts, M_total, N, K, dw.data_ptr(), s_e, s_n, s_k,
        float(out_scale), rt.stream_ptr(go_qm.device))
    check(rc, "alto_mxfp4_grouped_gemm_dw_ps")
    return dw


def _token_packed(codes: torch.Tensor, k_pack: bool) -> torch.Tensor:
    """An operand of the weight gradient as [features, M/2] codes with unit stride along the tokens: a transposed view
    when it arrives packed along the tokens ([M/2, features], ``k_pack``), a nibble transpose when it arrives packed along
    the features ([M, features/2])."""
    return codes.transpose(0, 1) if k_pack else transpose_codes(codes)


def mxfp4_grouped_gemm_backward_weights(grad_output, inputs, expert_indices, num_experts, go_scales, input_scales,
                                        trans_weights=True, use_2dblock_go=False, use_2dblock_x=True, k_pack_go=True,
                                        k_pack_x=True, output_dtype=torch.bfloat16):
    """cg_backward.py:398-497.  With ``k_pack_*`` the operands are [M/2, N] / [M/2, K] packed along the tokens, otherwise
    [M, N/2] / [M, K/2]; the scales are [M/32, N] / [M/32, K] (1D along the tokens) or [M/32, N/32] / [M/32, K/32] (2D)."""
    assert expert_indices.is_contiguous(), "Expert indices tensor must be contiguous"
    M_total = expert_indices.shape[0]
    torch._check(M_total > 0)
    torch._check(M_total % ALIGN_SIZE_M == 0)
    assert bool(use_2dblock_go) == bool(use_2dblock_x), "the two operands of the weight gradient share their block layout (cg_backward.py:880-893)"
    rt.require_gpu(grad_output, inputs, expert_indices, go_scales, input_scales)
    return grouped_dw(_token_packed(grad_output, k_pack_go), go_scales.transpose(0, 1), _token_packed(inputs, k_pack_x), input_scales.transpose(0, 1),
                      groups_from_indices(expert_indices), num_experts, output_dtype, trans_weights, is_2d=bool(use_2dblock_x))


@torch.compiler.allow_in_graph
class MXFP4GroupedGEMM(torch.autograd.Function):
    """Grouped GEMM with full backward (cg_backward.py:599-930), every block-layout combination of the reference:
    activations and gradients with 1D blocks (then the weight-gradient operands are separate token-axis quantisations, with
    the Hadamard transform and the clip mode) or 2D blocks (one quantisation serves all three GEMMs); weights with 2D
    blocks (one quantisation, both packings) or 1D blocks (one quantisation along K for the forward, one along N for dX)."""

    @staticmethod
    def forward(ctx, inputs, expert_weights, expert_indices, trans_weights=True, use_2dblock_x=False, use_2dblock_w=True,
                use_sr_grad=False, use_dge=False, clip_mode="none", use_macro_block_scaling=False,
                hadamard_transform: Optional[HadamardTransform] = None, use_uos: bool = False, offsets: Optional[torch.Tensor] = None):
        assert not use_macro_block_scaling, "Macro block scaling is not supported in real MXFP4 kernels"
        original_dtype = inputs.dtype
        weights_owner = expert_weights   # the object the caller keeps: cache entries belong to it, not to the alias below
        expert_weights = unwrap_weight_wrapper(expert_weights)
        E = expert_weights.shape[0]
        M_buf = inputs.shape[0]
        if offsets is None:
            M_total = expert_indices.shape[0]
            torch._check(M_total > 0)
            torch._check(M_total % ALIGN_SIZE_M == 0)
            groups = groups_from_indices(expert_indices)
        else:
            groups = groups_from_offsets(offsets)
        torch._check(M_buf % 32 == 0)
        x = inputs if inputs.is_contiguous() else inputs.contiguous()
        w = expert_weights if trans_weights else expert_weights.transpose(1, 2)   # logical [E, N, K]
        N, K = w.shape[1], w.shape[2]
        # Packed scales for the three grouped GEMMs where their tile kernels serve the shape: the quantizers write that
        # layout themselves.
        can_pack = (packed_scales_enabled() and original_dtype == torch.bfloat16 and clip_mode != "dynamic"
                    and M_buf * max(N, K) < 2 ** 36 and N * K < 2 ** 36)
        pk_f = can_pack and grouped_packed_supported(M_buf, N, K, groups.n)
        pk_d = can_pack and grouped_packed_supported(M_buf, K, N, groups.n)
        pk_w = can_pack and grouped_dw_packed_supported(M_buf, N, K, groups.n, E)
        if use_2dblock_x:   # one 2D-block quantisation, both packings: K-packed for the forward, token-packed for dW
            a_q, a_s, a_qm, a_sm = quantize_rowcol(x, True, use_uos=use_uos, pad_codes=True, pack_row_scales=pk_f, pack_col_scales=pk_w)
        else:               # row copy for the forward; Hadamard + clip on the token-axis copy saved for dW
            a_q, a_s, a_qm, a_sm = quantize_rowcol(x, False, hadamard=hadamard_transform, clip_mode=clip_mode, use_uos=use_uos, pad_codes=True,
                                                   pack_row_scales=pk_f, pack_col_scales=pk_w)
        # weights: codes packed along K [E, N, K/2] for the forward, packed along N [E, K, N/2] for dX
        if w.stride(2) == 1:
            wq_nk, ws_nk, wq_kn, ws_kn = _quantize_experts(weights_owner, w, use_2dblock_w, use_uos, pk_f, pk_d)
        else:                                                                     # stored [E, K, N]: same pass, roles swapped
            wq_kn, ws_kn, wq_nk, ws_nk = _quantize_experts(weights_owner, w.transpose(1, 2), use_2dblock_w, use_uos, pk_d, pk_f)
        if pk_f:
            out, plan = grouped_forward_packed(a_q, a_s, wq_nk, ws_nk, groups, return_plan=True)
        else:
            out, plan = grouped_forward(a_q, a_s, wq_nk, ws_nk, groups, use_2dblock_x, use_2dblock_w, original_dtype, return_plan=True)
        ctx.save_for_backward(a_qm, a_sm, wq_kn, ws_kn, groups.offs, groups.expert, plan)   # (plan: the pass list, reused by dX)
        ctx.packed_dx = pk_d
        ctx.packed_dw = pk_w
        ctx.num_groups = groups.n
        ctx.trans_weights = trans_weights
        ctx.original_dtype = original_dtype
        ctx.use_2dblock_x = bool(use_2dblock_x)
        ctx.use_2dblock_w = bool(use_2dblock_w)
        ctx.use_sr_grad = use_sr_grad
        ctx.hadamard_transform = hadamard_transform
        ctx.clip_mode = clip_mode
        ctx.use_uos = use_uos
        ctx.num_experts = E
        ctx.use_dge = bool(use_dge)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        a_qm, a_sm, wq_kn, ws_kn, g_offs, g_expert, plan = ctx.saved_tensors
        groups = Groups(g_offs, g_expert, ctx.num_groups)
        go = grad_output if grad_output.is_contiguous() else grad_output.contiguous()
        sr = bool(ctx.use_sr_grad)
        # random words: made inside the quantizer (Philox) unless a source of explicit words is installed
        rand = rt.draw_rand_bits(go.shape, go.device) if (sr and not rt.philox_in_kernel()) else None
        pk_d, pk_w = ctx.packed_dx, ctx.packed_dw
        if ctx.use_2dblock_x:
            go_q, go_s, go_qm, go_sm = quantize_rowcol(go, True, use_sr=sr, rand_bits=rand, use_uos=ctx.use_uos, pad_codes=True, pack_row_scales=pk_d,
                                                       pack_col_scales=pk_w)
        else:
            go_q, go_s, go_qm, go_sm = quantize_rowcol(go, False, use_sr=sr, rand_bits=rand, hadamard=ctx.hadamard_transform,
                                                       clip_mode=ctx.clip_mode, use_uos=ctx.use_uos, pad_codes=True, pack_row_scales=pk_d, pack_col_scales=pk_w)
        if pk_d:
            grad_inputs = grouped_forward_packed(go_q, go_s, wq_kn, ws_kn, groups, plan=plan)
        else:
            grad_inputs = grouped_forward(go_q, go_s, wq_kn, ws_kn, groups, ctx.use_2dblock_x, ctx.use_2dblock_w, ctx.original_dtype, plan=plan)
        if pk_w:
            grad_weights = grouped_dw_packed(go_qm.transpose(0, 1), go_sm, a_qm.transpose(0, 1), a_sm, groups, ctx.num_experts, ctx.trans_weights,
                                             _wgrad_scale(ctx.clip_mode, ctx.use_dge))
        else:
            grad_weights = grouped_dw(go_qm.transpose(0, 1), go_sm.transpose(0, 1), a_qm.transpose(0, 1), a_sm.transpose(0, 1),
                                      groups, ctx.num_experts, ctx.original_dtype, ctx.trans_weights,
                                      _wgrad_scale(ctx.clip_mode, ctx.use_dge), is_2d=ctx.use_2dblock_x)
        return (grad_inputs, grad_weights) + (None,) * 11


def _quantize_experts(owner: torch.Tensor, w: torch.Tensor, is_2d: bool, use_uos: bool, pack_rows: bool = False, pack_cols: bool = False):
    """w [E, R, C] (unit stride along C; ``owner`` or a transposed view of it) -> codes packed along C [E,R,C/2] with
    their scales, and codes packed along R [E,C,R/2] with theirs (each operand of a GEMM wants unit stride along its
    reduction dim).  2D blocks: one quantisation, scales [E,R/32,C/32] and the same values stored transposed
    [E,C/32,R/32].  1D blocks: two quantisations (blocks along C: scales [E,R,C/32]; blocks along R: [E,C,R/32]), still one
    pass over the weights.  ``pack_rows`` / ``pack_cols``: the first / second scale tensor comes packed, [E, ceil(C/512), R, 16]
    / [E, ceil(R/512), C, 16].  The cache entry belongs to ``owner``, the tensor object the caller keeps."""
    from .quantization import _prep, _quantize_call
    return cached_weight_quantisation(owner, ("experts", bool(is_2d), bool(use_uos), tuple(w.shape), tuple(w.stride()), bool(pack_rows), bool(pack_cols)),
                                      lambda: _quantize_call(_prep(w), True, True, bool(is_2d), False, None, None, 0, use_uos, True,
                                                             pack_row_scales=pack_rows, pack_col_scales=pack_cols))


def mxfp4_grouped_gemm(inputs, expert_weights, expert_indices, *, trans_weights=True, use_2dblock_x=False, use_2dblock_w=True,
                       use_sr_grad=False, use_dge=False, use_hadamard=False, clip_mode="none", use_macro_block_scaling=False,
                       use_uos=False, offsets: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Grouped GEMM with full backward support (cg_backward.py:933-991).

    ``offsets`` (int32 [E+1], leading 0) may be given instead of ``expert_indices`` to describe ragged groups.
    """
    if use_hadamard:
        assert not use_2dblock_x, "Hadamard transform can only be applied if 2D block is not used for activations."
    if expert_indices is not None and expert_indices.dtype != torch.int32:
        expert_indices = expert_indices.to(torch.int32)
    hadamard_transform = HadamardFactory.create_transform(device=expert_weights.device) if use_hadamard else None
    return MXFP4GroupedGEMM.apply(inputs, expert_weights, expert_indices, trans_weights, use_2dblock_x, use_2dblock_w, use_sr_grad,
                                  use_dge, clip_mode, use_macro_block_scaling, hadamard_transform, use_uos, offsets)


def _quantize_then_mxfp_scaled_grouped_mm(A, B, offs, use_2dblock_x, use_2dblock_w, use_sr_grad, use_dge, use_hadamard, clip_mode,
                                          use_macro_block_scaling, use_uos=False) -> torch.Tensor:
    """``torch._grouped_mm(A, B, offs=offs)`` replacement (functional.py:11-38): B is [E, K, N], offs are group ends."""
    return mxfp4_grouped_gemm(A, B, None, trans_weights=False, use_2dblock_x=use_2dblock_x, use_2dblock_w=use_2dblock_w,
                              use_sr_grad=use_sr_grad, use_dge=use_dge, use_hadamard=use_hadamard, clip_mode=clip_mode,
                              use_macro_block_scaling=use_macro_block_scaling, use_uos=use_uos, offsets=offsets_from_ends(offs))
