"""MXFP4 flash-attention forward, named as in ``alto/kernels/fp4/mxfp4/triton_flash_attention_mxfp4.py``.

``triton_attention_mxfp4`` keeps the reference's name and argument list (:1206-1239) so that
``alto/kernels/dispatch/attention.py:22`` can point at it; here it quantises Q, K, V with the fused HIP quantizer
(2D blocks along the head dim, :1105-1107; V also packed along the keys by the same pass) and runs one HIP kernel.
Like the reference (:1143-1145) it has no backward.  Options outside the path ALTO's dispatch layer uses
(``alto/kernels/dispatch/attention.py:61-77``: layout "bhsd", no bias, no alibi, no dropout, fixed lengths) raise.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _runtime as rt
from .._lib import check
from .config import TrainingOpConfig
from .quantization import _prep, _quantize_call


def attention_mxfp4_forward(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q_scale: torch.Tensor, k_scale: torch.Tensor,
                            v_scale: torch.Tensor, sm_scale: float, causal: bool, seqlen_k: Optional[int] = None,
                            bias: Optional[torch.Tensor] = None, alibi_slopes: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Pre-quantised operands -> (out bf16 [B,Hq,Sq,Dv], lse fp32 [B,Hq,Sq]).

    q [B,Hq,Sq,D/2], q_scale [B,Hq,Sq/32,D/32]; k [B,Hk,Sk,D/2], k_scale [B,Hk,Sk/32,D/32]; v packed along the keys:
    [B,Hk,Dv,Sk/2] with v_scale [B,Hk,Sk/32,Dv/32] (the reference's kernel takes V packed along Dv and unpacks it inside
    ``tl.dot_scaled(..., rhs_k_pack=False)``, :393; same codes, other byte order).  The key dim of k / v is a multiple of
    64; ``seqlen_k`` (default: all of it) says how many keys exist when the caller padded a sequence of 32 (mod 64) keys.
    ``bias`` (broadcastable to [B, Hq, Sq, seqlen_k]) is added to the scaled scores, ``alibi_slopes`` ([Hq] or [B, Hq]) give
    the ALiBi term ``-slope * |row + Sk - Sq - key|`` (:135-164,288-299).
    """
    rt.require_gpu(q, k, v, q_scale, k_scale, v_scale)
    for t in (q, k, v, q_scale, k_scale, v_scale):
        assert t.is_contiguous() and t.dtype == torch.uint8
    B, Hq, Sq, D = q.shape[0], q.shape[1], q.shape[2], q.shape[3] * 2
    Hk, Sk = k.shape[1], k.shape[2]
    Dv = v.shape[2]
    assert k.shape == (B, Hk, Sk, D // 2) and v.shape == (B, Hk, Dv, Sk // 2)
    assert q_scale.shape == (B, Hq, Sq // 32, D // 32) and k_scale.shape == (B, Hk, Sk // 32, D // 32)
    assert v_scale.shape == (B, Hk, Sk // 32, Dv // 32)
    out = torch.empty((B, Hq, Sq, Dv), dtype=torch.bfloat16, device=q.device)
    lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=q.device)
    sk_used = Sk if seqlen_k is None else int(seqlen_k)
    b4 = sl = None
    if bias is not None:
        rt.require_gpu(bias)
        b4 = bias.to(torch.float32)
        while b4.dim() < 4:
            b4 = b4.unsqueeze(0)
        torch._check(b4.shape[-2] == Sq and b4.shape[-1] == sk_used and b4.shape[0] in (1, B) and b4.shape[1] in (1, Hq),
                     lambda: f"bias of shape {tuple(bias.shape)} does not broadcast to {(B, Hq, Sq, sk_used)}")
        if b4.stride(3) != 1 or b4.stride(2) % 4 or b4.data_ptr() % 16 or (b4.shape[0] > 1 and b4.stride(0) < 0) or (b4.shape[1] > 1 and b4.stride(1) < 0):
            b4 = b4.contiguous()
    if alibi_slopes is not None:
        rt.require_gpu(alibi_slopes)
        sl = alibi_slopes.to(torch.float32)
        if sl.dim() == 1:
            sl = sl.unsqueeze(0)
        torch._check(sl.dim() == 2 and sl.shape[1] == Hq and sl.shape[0] in (1, B), lambda: f"alibi_slopes of shape {tuple(alibi_slopes.shape)}: [Hq] or [B, Hq]")
        sl = sl.contiguous()
    if b4 is None and sl is None:
        check(rt.lib().alto_mxfp4_attention_fwd(q.data_ptr(), q_scale.data_ptr(), k.data_ptr(), k_scale.data_ptr(), v.data_ptr(),
                                                v_scale.data_ptr(), out.data_ptr(), lse.data_ptr(), B, Hq, Hk, Sq, Sk, sk_used, D, Dv,
                                                float(sm_scale), int(bool(causal)), rt.stream_ptr(q.device)), "alto_mxfp4_attention_fwd")
        return out, lse
    check(rt.lib().alto_mxfp4_attention_fwd_ex(
        q.data_ptr(), q_scale.data_ptr(), k.data_ptr(), k_scale.data_ptr(), v.data_ptr(), v_scale.data_ptr(), out.data_ptr(), lse.data_ptr(),
        B, Hq, Hk, Sq, Sk, sk_used, D, Dv, float(sm_scale), int(bool(causal)),
        rt.ptr(b4), 0 if b4 is None or b4.shape[0] == 1 else b4.stride(0), 0 if b4 is None or b4.shape[1] == 1 else b4.stride(1),
        0 if b4 is None else b4.stride(2),
        rt.ptr(sl), 0 if sl is None or sl.shape[0] == 1 else sl.stride(0), 0 if sl is None else sl.stride(1),
        rt.stream_ptr(q.device)), "alto_mxfp4_attention_fwd_ex")
    return out, lse


def quantize_qkv(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor):
    """bf16/fp32 [B,H,S,D] tensors -> (q, q_scale, k, k_scale, v packed along keys, v_scale): three quantizer launches."""
    def rows(t):
        t3 = _prep(t.reshape(-1, t.shape[-2], t.shape[-1]))
        codes, scales, _, _ = _quantize_call(t3, True, False, True, False, None, None, 0, False)
        return codes.view(*t.shape[:-1], t.shape[-1] // 2), scales.view(*t.shape[:-2], t.shape[-2] // 32, t.shape[-1] // 32)

    def cols(t):
        t3 = _prep(t.reshape(-1, t.shape[-2], t.shape[-1]))
        _, _, codes, scales = _quantize_call(t3, False, True, True, False, None, None, 0, False)
        # the block scales go back to the [S/32, D/32] order of the tensor itself (a few KB; 2D-block scales are symmetric)
        scales = scales.view(*t.shape[:-2], t.shape[-1] // 32, t.shape[-2] // 32).transpose(-1, -2).contiguous()
        return codes.view(*t.shape[:-2], t.shape[-1], t.shape[-2] // 2), scales

    qq, qs = rows(q)
    kq, ks = rows(k)
    vq, vs = cols(v)
    return qq, qs, kq, ks, vq, vs


def triton_attention_mxfp4(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, alibi_slopes: Optional[torch.Tensor] = None,
                           bias: Optional[torch.Tensor] = None, sm_scale: Optional[float] = None, dropout_p: float = 0.0,
                           cu_seqlens_q=0, cu_seqlens_k=0, max_seqlens_q: Optional[int] = None, max_seqlens_k: Optional[int] = None,
                           causal: bool = True, return_scores: bool = False, use_exp2: bool = True, layout: str = "bhsd"):
    """(q, k, v) [B,H,S,D] (or [B,S,H,D] with ``layout="bshd"``, or packed [T,H,D] with ``layout="thd"`` and ``cu_seqlens_*``)
    -> (out bf16 in the layout of q, softmax_lse fp32 [B,H,S] ([T,H] for 'thd'), exp_scores placeholder), as :1206-1239.

    ``use_exp2`` is accepted either way: both settings evaluate exp(x) as exp2(x * log2 e) on the GPU's exp unit.
    """
    if layout == "bshd":
        # [B, S, H, D] tensors: the same attention on the permuted views, result back in [B, S, H, D].  (The reference's
        # wrapper has no consistent behaviour to reproduce here: it takes 2D blocks over (heads, head dim) of the tensor as
        # given and then reads those scales with strides permuted as if they were per (32 rows, 32 of head dim),
        # triton_flash_attention_mxfp4.py:68-77,1023-1025,1105-1107.)
        out, lse, scores = triton_attention_mxfp4(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), alibi_slopes, bias, sm_scale,
                                                  dropout_p, cu_seqlens_q, cu_seqlens_k, max_seqlens_q, max_seqlens_k, causal, return_scores,
                                                  use_exp2, "bhsd")
        return out.transpose(1, 2), lse, scores
    if layout == "thd":
        # Variable-length sequences packed along the tokens: q [Tq, Hq, D], k / v [Tk, Hk, D], boundaries cu_seqlens_q /
        # cu_seqlens_k (int [n + 1], leading 0); out [Tq, Hq, Dv], softmax_lse [Tq, Hq] (the shapes of :1199-1203).  Every
        # sequence is the 'bhsd' attention of its own rows: its 32 x 32 quantisation blocks start at its first token, so the
        # boundaries must be multiples of 32 (no block may belong to two sequences), and a causal mask is aligned to the
        # bottom-right corner of each sequence's own score matrix.  One launch per sequence.
        cq = [int(c) for c in (cu_seqlens_q.tolist() if isinstance(cu_seqlens_q, torch.Tensor) else cu_seqlens_q)]
        ck = [int(c) for c in (cu_seqlens_k.tolist() if isinstance(cu_seqlens_k, torch.Tensor) else cu_seqlens_k)]
        torch._check(q.dim() == 3 and k.dim() == 3 and v.dim() == 3, lambda: "layout 'thd' takes [tokens, heads, head dim] tensors")
        if bias is not None:
            raise NotImplementedError("a bias tensor with layout 'thd' is not implemented (ALiBi slopes are)")
        if alibi_slopes is not None and alibi_slopes.dim() == 2:
            raise NotImplementedError("layout 'thd' takes one ALiBi slope per head")
        torch._check(len(cq) == len(ck) and len(cq) >= 2 and cq[0] == 0 and ck[0] == 0 and cq[-1] == q.shape[0] and ck[-1] == k.shape[0],
                     lambda: "cu_seqlens_q / cu_seqlens_k must start at 0, end at the token counts and describe the same number of sequences")
        torch._check(all(c % 32 == 0 for c in cq) and all(c % 32 == 0 for c in ck), lambda: "sequence boundaries must be multiples of 32 tokens")
        out = torch.empty((q.shape[0], q.shape[1], v.shape[2]), dtype=torch.bfloat16, device=q.device)
        lse = torch.empty((q.shape[0], q.shape[1]), dtype=torch.float32, device=q.device)
        for i in range(len(cq) - 1):
            q0, q1, k0, k1 = cq[i], cq[i + 1], ck[i], ck[i + 1]
            torch._check(q1 > q0 and k1 > k0, lambda: "empty sequences are not supported")
            o_i, l_i, _ = triton_attention_mxfp4(q[q0:q1].transpose(0, 1).unsqueeze(0), k[k0:k1].transpose(0, 1).unsqueeze(0),
                                                 v[k0:k1].transpose(0, 1).unsqueeze(0), alibi_slopes, bias, sm_scale, dropout_p, 0, 0,
                                                 q1 - q0, k1 - k0, causal, return_scores, use_exp2, "bhsd")
            out[q0:q1] = o_i[0].transpose(0, 1)
            lse[q0:q1] = l_i[0].transpose(0, 1)
        return out, lse, torch.empty([], device=q.device, dtype=torch.float32)
    if layout != "bhsd":
        raise NotImplementedError(f"layout {layout!r}: 'bhsd', 'bshd' and 'thd' are implemented")
    if dropout_p != 0.0:
        raise NotImplementedError("dropout is not implemented (the reference's own dropout is a no-op after PNQ, :357-360)")
    if return_scores:
        raise NotImplementedError("return_scores is a debugging output of the reference and is not implemented")
    rt.require_gpu(q, k, v)
    assert q.dim() == 4 and k.dim() == 4 and v.dim() == 4
    assert max_seqlens_q in (None, q.shape[2]) and max_seqlens_k in (None, k.shape[2]), "variable lengths are not implemented"
    if sm_scale is None:
        sm_scale = q.shape[-1] ** -0.5
    seqlen_k = k.shape[2]
    if seqlen_k % 64 == 32:   # one 32-row block of zeros: quantises to zero codes, the kernel masks those keys out
        k = torch.nn.functional.pad(k, (0, 0, 0, 32))
        v = torch.nn.functional.pad(v, (0, 0, 0, 32))
    qq, qs, kq, ks, vq, vs = quantize_qkv(q, k, v)
    out, lse = attention_mxfp4_forward(qq, kq, vq, qs, ks, vs, sm_scale=sm_scale, causal=causal, seqlen_k=seqlen_k, bias=bias, alibi_slopes=alibi_slopes)
    return out, lse, torch.empty([], device=q.device, dtype=torch.float32)


class LPScaledDotProductAttention(torch.nn.Module):
    """Module form used by ALTO's model converter (``alto/kernels/dispatch/attention.py:14-80``): inputs [B, L, N, H]."""

    def __init__(self, config: TrainingOpConfig):
        super().__init__()
        if not (isinstance(config, TrainingOpConfig) and config.precision == "mxfp4"):
            raise ValueError(f"Unsupported SDPA config: {config}")
        self.config = config

    def forward(self, q_BLNH, k_BLNH, v_BLNH, *, attention_masks=None, scale: Optional[float] = None, enable_gqa: bool = False,
                is_causal: bool = True, **kwargs):
        if attention_masks is not None:
            raise ValueError("ScaledDotProductAttention does not support attention_masks; it only supports causal/non-causal "
                             "attention via is_causal.")
        q, k, v = (t.transpose(1, 2).contiguous() for t in (q_BLNH, k_BLNH, v_BLNH))
        assert q.shape[0] == k.shape[0] == v.shape[0] and k.shape[1] == v.shape[1]
        assert q.shape[3] == k.shape[3] and k.shape[2] == v.shape[2]
        sm_scale = q.shape[3] ** -0.5 if scale is None else scale
        o = triton_attention_mxfp4(q, k, v, sm_scale=sm_scale, causal=is_causal, max_seqlens_q=q.shape[2], max_seqlens_k=k.shape[2])[0]
        return o.transpose(1, 2)
