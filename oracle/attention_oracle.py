"""CPU restatement (torch, CPU tensors only) of ALTO's MXFP4 flash-attention forward.

THIS IS TEST INFRASTRUCTURE: the checker of the HIP kernel, never a code path of the product.  Only ``tests/``,
``__graft_entry__.smoke`` and the ``cpu_baseline`` leg of ``bench.py`` import it.

It follows, block of 64 keys by block of 64 keys,

* the kernel's recurrence      alto/kernels/fp4/mxfp4/triton_flash_attention_mxfp4.py:227-398 (inner loop),
                               :667-669 (initial state), :817-851 (normalisation, log-sum-exp), :1031-1080 (BLOCK_N = 64)
* the quantisation of Q, K, V  the same file :1105-1107 (2D-block MXFP4 along the head dim)
* and the reference's own CPU model of it   tests/unittest/mxfp4/test_mxfp_pnq.py:87-149

What pins it (the reference stores no vectors for this path; tests/test_oracle_attention.py):
* the reference's own assertion (test_mxfp_pnq.py:163-174): with V = 1 the output is exactly 1 when the row sum is
  taken from the quantised probabilities, and is visibly not 1 when it is taken from the unquantised ones;
* a brute-force per-row Python-float evaluation of the same recurrence on a tiny case;
* agreement with fp32 softmax attention within the error MXFP4 operands allow (relative L2 below 0.3, cosine above 0.97 for N(0,1) inputs);
* invariances the recurrence must have: a fully masked key block changes nothing; grouped-query heads equal repeated
  K/V heads.
* the additive terms (``bias``, ``alibi_slopes``; the reference's CPU model has neither): a bias that is constant along
  every row changes nothing beyond rounding (softmax is shift-invariant), a bias of -inf on a set of keys equals attention
  without those keys, and ALiBi slopes equal the explicit bias tensor -slope |row + Sk - Sq - key|.
The exponentials differ between CPU libm and the GPU's v_exp_f32 in the last bit, which can move a probability across
an E2M1 rounding boundary: parity of the HIP kernel with this model is therefore a tolerance, not bit equality.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .mxfp4_oracle import dequantize, quantize

RCP_LN2 = 1.4426950408889634
LN2 = 0.6931471824645996
BLOCK_N = 64


def _qdq(x: torch.Tensor, is_2d_block: bool) -> torch.Tensor:
    codes, scales = quantize(x, axis=-1, is_2d_block=is_2d_block)
    return dequantize(codes, scales, torch.float32, axis=-1, is_2d_block=is_2d_block)


def attention_fwd_ref(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, *, causal: bool, sm_scale: Optional[float] = None,
                      pnq: bool = True, use_exp2: bool = True, block_n: int = BLOCK_N, bias: Optional[torch.Tensor] = None,
                      alibi_slopes: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """q [B, Hq, Sq, D], k [B, Hk, Sk, D], v [B, Hk, Sk, Dv] (bf16) -> (out bf16 [B, Hq, Sq, Dv], lse fp32 [B, Hq, Sq]).

    ``pnq=False`` takes the row sum from the unquantised probabilities (the behaviour the reference replaced; kept for
    the V = 1 test).  Rows are independent, so the query-block size of the kernel does not enter.
    """
    assert q.dim() == 4 and k.dim() == 4 and v.dim() == 4
    B, Hq, Sq, D = q.shape
    _, Hk, Sk, Dv = v.shape
    assert k.shape == (B, Hk, Sk, D) and Hq % Hk == 0
    assert Sq % 32 == 0 and Sk % 32 == 0 and D % 32 == 0 and Dv % 32 == 0
    if sm_scale is None:
        sm_scale = D ** -0.5
    qd = _qdq(q, True)
    kd = _qdq(k, True).repeat_interleave(Hq // Hk, dim=1)
    vd = _qdq(v, True).repeat_interleave(Hq // Hk, dim=1)

    m_i = torch.full((B, Hq, Sq), float("-inf"), dtype=torch.float32)
    l_i = torch.ones((B, Hq, Sq), dtype=torch.float32)          # :668 (the first block's alpha = 0 wipes it)
    acc = torch.zeros((B, Hq, Sq, Dv), dtype=torch.float32)
    q_pos = torch.arange(Sq) + (Sk - Sq)                         # bottom-right aligned causal mask (:291-294, :754)
    sm = torch.tensor(sm_scale, dtype=torch.float32)
    for key0 in range(0, Sk, block_n):
        key1 = min(key0 + block_n, Sk)
        if causal and key0 > int(q_pos[-1]):
            break
        s = (qd @ kd[:, :, key0:key1].transpose(-1, -2)) * sm                      # :275-277
        if causal:
            masked = torch.arange(key0, key1)[None, :] > q_pos[:, None]
            s = s.masked_fill(masked, float("-inf"))
        if bias is not None:                                                       # :288-291 (broadcast over batch / heads)
            s = s + bias.float()[..., key0:key1]
        if alibi_slopes is not None:                                               # :135-164,293-299
            rel = (q_pos[:, None] - torch.arange(key0, key1)[None, :]).abs().float()
            sl = alibi_slopes.float()
            sl = sl[None, :] if sl.dim() == 1 else sl
            s = s - sl[..., None, None] * rel
        m_ij = torch.maximum(m_i, s.amax(dim=-1))                                  # :308
        shifted = s - m_ij[..., None]
        p = torch.exp2(shifted * RCP_LN2) if use_exp2 else torch.exp(shifted)      # :318-322
        p = torch.nan_to_num(p, nan=0.0)                                           # rows with nothing visible yet
        p_dq = _qdq(p, False)                                                      # :324-353, one scale per (row, 32 keys)
        l_ij = (p_dq if pnq else p).sum(dim=-1)                                    # :356
        diff = m_i - m_ij
        alpha = torch.exp2(diff * RCP_LN2) if use_exp2 else torch.exp(diff)        # :378-382
        alpha = torch.nan_to_num(alpha, nan=0.0)
        acc = acc * alpha[..., None] + p_dq @ vd[:, :, key0:key1]                  # :383,393
        l_i = l_i * alpha + l_ij                                                   # :388
        m_i = m_ij
    out = (acc * (1.0 / l_i)[..., None]).to(torch.bfloat16)                        # :817-818,825
    lse = (m_i * RCP_LN2 + torch.log2(l_i)) * LN2 if use_exp2 else m_i + torch.log(l_i)   # :840-847
    return out, lse


def attention_fp32_ref(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, *, causal: bool, sm_scale: Optional[float] = None) -> torch.Tensor:
    """Plain fp32 softmax attention with the same bottom-right aligned mask (what MXFP4 attention approximates)."""
    B, Hq, Sq, D = q.shape
    Hk, Sk = k.shape[1], k.shape[2]
    if sm_scale is None:
        sm_scale = D ** -0.5
    kf = k.float().repeat_interleave(Hq // Hk, dim=1)
    vf = v.float().repeat_interleave(Hq // Hk, dim=1)
    s = (q.float() @ kf.transpose(-1, -2)) * sm_scale
    if causal:
        masked = torch.arange(Sk)[None, :] > (torch.arange(Sq) + (Sk - Sq))[:, None]
        s = s.masked_fill(masked, float("-inf"))
    return torch.softmax(s, dim=-1) @ vf
