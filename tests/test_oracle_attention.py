"""Pins of the CPU model of MXFP4 flash attention (oracle/attention_oracle.py); no GPU.

The reference stores no vectors for this path; what it holds is one exact assertion on its own CPU model
(tests/unittest/mxfp4/test_mxfp_pnq.py:163-174), reproduced first.  The rest are checks a wrong term, sign or index fails.
"""
import math

import numpy as np
import torch

from oracle import scalar_model as sm
from oracle.attention_oracle import BLOCK_N, LN2, RCP_LN2, attention_fp32_ref, attention_fwd_ref


def test_constant_value_attention_is_preserved_exactly():
    """test_mxfp_pnq.py:163-174: same seed, shapes and assertions."""
    torch.manual_seed(1234)
    q = torch.randn(1, 32, 64, 64, dtype=torch.bfloat16)
    k = torch.randn(1, 8, 64, 64, dtype=torch.bfloat16)
    v = torch.ones(1, 8, 64, 64, dtype=torch.bfloat16)
    out_pnq, _ = attention_fwd_ref(q, k, v, causal=True, pnq=True)
    out_plain, _ = attention_fwd_ref(q, k, v, causal=True, pnq=False)
    assert torch.allclose(out_pnq, torch.ones_like(out_pnq), atol=0.0, rtol=0.0)
    assert not torch.allclose(out_plain, torch.ones_like(out_plain), atol=1e-2, rtol=0.0)


def _f32(x):
    return float(np.float32(x))


def _scalar_row(qd, kd, vd, row, causal, shift, sm_scale):
    """One query row of the recurrence in scalar Python (fp32 roundings made explicit), quantisation by the integer
    scalar model.  qd/kd/vd are the dequantised operands as nested lists."""
    Sk, Dv = len(kd), len(vd[0])
    m_i, l_i, acc = -math.inf, 1.0, [0.0] * Dv
    for key0 in range(0, Sk, BLOCK_N):
        keys = list(range(key0, min(key0 + BLOCK_N, Sk)))
        if causal and key0 > row + shift:
            break
        s = []
        for j in keys:
            dot = float(np.dot(np.asarray(qd[row], dtype=np.float32), np.asarray(kd[j], dtype=np.float32)))
            x = _f32(_f32(dot) * _f32(sm_scale))
            s.append(-math.inf if causal and j > row + shift else x)
        m_ij = max(m_i, max(s))
        p = [_f32(2.0 ** _f32(_f32(x - m_ij) * _f32(RCP_LN2))) if x != -math.inf else 0.0 for x in s]
        p_dq = []
        for b0 in range(0, len(p), 32):
            bits = [sm.f32_bits(x) for x in p[b0:b0 + 32]]
            packed, scales = sm.quantize_row_1d(bits, 23)
            sc = sm.bits_f32(scales[0] << 23)
            for byte in packed:
                p_dq.append(sm.decode(byte & 0xF) * sc)
                p_dq.append(sm.decode(byte >> 4) * sc)
        alpha = 0.0 if m_i == -math.inf else _f32(2.0 ** _f32(_f32(m_i - m_ij) * _f32(RCP_LN2)))
        for d in range(Dv):
            acc[d] = _f32(acc[d] * alpha + sum(p_dq[i] * vd[keys[i]][d] for i in range(len(keys))))
        l_i = _f32(l_i * alpha + sum(p_dq))
        m_i = m_ij
    return [a / l_i for a in acc], (m_i * RCP_LN2 + math.log2(l_i)) * LN2


def test_matches_a_scalar_evaluation_of_the_recurrence():
    from oracle.mxfp4_oracle import dequantize, quantize
    torch.manual_seed(5)
    B, Hq, Hk, Sq, Sk, D, Dv = 1, 2, 1, 32, 128, 32, 32
    q = torch.randn(B, Hq, Sq, D, dtype=torch.bfloat16)
    k = torch.randn(B, Hk, Sk, D, dtype=torch.bfloat16)
    v = torch.randn(B, Hk, Sk, Dv, dtype=torch.bfloat16)
    for causal in (False, True):
        out, lse = attention_fwd_ref(q, k, v, causal=causal)
        dq = lambda t: dequantize(*quantize(t, axis=-1, is_2d_block=True), torch.float32, axis=-1, is_2d_block=True)
        qd, kd, vd = dq(q), dq(k), dq(v)
        for head in range(Hq):
            for row in (0, 7, 31):
                o_row, lse_row = _scalar_row(qd[0, head].tolist(), kd[0, 0].tolist(), vd[0, 0].tolist(), row, causal, Sk - Sq, D ** -0.5)
                got = out[0, head, row].float().tolist()
                # bf16 output: half an ulp is 2^-9 relative; sums are ordered differently in the two evaluations
                assert max(abs(a - b) for a, b in zip(got, o_row)) <= 2 ** -7 * max(1.0, max(abs(x) for x in o_row))
                assert abs(float(lse[0, head, row]) - lse_row) < 1e-4


def test_close_to_fp32_attention():
    torch.manual_seed(0)
    q = torch.randn(2, 8, 256, 128, dtype=torch.bfloat16)
    k = torch.randn(2, 2, 256, 128, dtype=torch.bfloat16)
    v = torch.randn(2, 2, 256, 128, dtype=torch.bfloat16)
    for causal in (True, False):
        out, lse = attention_fwd_ref(q, k, v, causal=causal)
        ref = attention_fp32_ref(q, k, v, causal=causal)
        rel = float((out.float() - ref).norm() / ref.norm())
        cos = float(torch.nn.functional.cosine_similarity(out.float().flatten(), ref.flatten(), dim=0))
        assert rel < 0.3 and cos > 0.97, (rel, cos)
        # the log-sum-exp of the quantised scores stays near the exact one (Q and K carry ~10 % quantisation noise)
        s = (q.float() @ k.float().repeat_interleave(4, 1).transpose(-1, -2)) * 128 ** -0.5
        if causal:
            s = s.masked_fill(torch.arange(256)[None, :] > torch.arange(256)[:, None], float("-inf"))
        assert float((lse - torch.logsumexp(s, -1)).abs().max()) < 1.0


def test_grouped_query_heads_equal_repeated_kv_heads():
    torch.manual_seed(1)
    q = torch.randn(1, 4, 64, 64, dtype=torch.bfloat16)
    k = torch.randn(1, 2, 128, 64, dtype=torch.bfloat16)
    v = torch.randn(1, 2, 128, 64, dtype=torch.bfloat16)
    a, la = attention_fwd_ref(q, k, v, causal=True)
    b, lb = attention_fwd_ref(q, k.repeat_interleave(2, 1), v.repeat_interleave(2, 1), causal=True)
    assert torch.equal(a, b) and torch.equal(la, lb)


def test_masked_future_keys_do_not_matter():
    """Causal, Sq < Sk: keys beyond the last visible one may hold anything (whole masked blocks and a masked tail)."""
    torch.manual_seed(2)
    q = torch.randn(1, 2, 64, 64, dtype=torch.bfloat16)
    k = torch.randn(1, 2, 192, 64, dtype=torch.bfloat16)
    v = torch.randn(1, 2, 192, 64, dtype=torch.bfloat16)
    a, la = attention_fwd_ref(q, k, v, causal=True)
    # bottom-right alignment: query i sees keys 0 .. i + 128; shrink to Sk = 64 + 128 and compare the first rows instead:
    # row 0 sees keys 0..128 -> equals non-causal attention of that row over keys 0..128 padded to a block multiple
    row0, _ = attention_fwd_ref(q[:, :, :32], k[:, :, :192], v[:, :, :192], causal=False)
    full, _ = attention_fwd_ref(q, k, v, causal=False)
    assert torch.equal(row0, full[:, :, :32])            # rows are independent
    assert not torch.equal(a, full)                       # the mask does something
    last = a[:, :, 63]                                    # the last row sees every key
    assert torch.equal(last, full[:, :, 63]) and torch.equal(la[:, :, 63], attention_fwd_ref(q, k, v, causal=False)[1][:, :, 63])


def test_exp_and_exp2_forms_agree():
    torch.manual_seed(3)
    q = torch.randn(1, 2, 64, 64, dtype=torch.bfloat16)
    k = torch.randn(1, 1, 128, 64, dtype=torch.bfloat16)
    v = torch.randn(1, 1, 128, 64, dtype=torch.bfloat16)
    a, la = attention_fwd_ref(q, k, v, causal=True, use_exp2=True)
    b, lb = attention_fwd_ref(q, k, v, causal=True, use_exp2=False)
    assert float((a.float() - b.float()).norm() / b.float().norm()) < 2e-2
    assert float((la - lb).abs().max()) < 1e-3


def test_additive_terms_of_the_scores():
    """bias and ALiBi (triton_flash_attention_mxfp4.py:135-164,288-299), which the reference's CPU model does not have:
    a bias constant along each row only shifts the row (same probabilities, lse moves by the constant), a -inf bias on a
    set of keys is attention without them, and ALiBi slopes are the bias -slope |row + Sk - Sq - key|."""
    torch.manual_seed(5)
    B, H, Sq, Sk, D = 1, 2, 64, 128, 64
    q = torch.randn(B, H, Sq, D, dtype=torch.bfloat16)
    k = torch.randn(B, H, Sk, D, dtype=torch.bfloat16)
    v = torch.randn(B, H, Sk, D, dtype=torch.bfloat16)
    base, lse0 = attention_fwd_ref(q, k, v, causal=True)
    # (1) per-row constant: powers of two times the natural-log unit would be exact; a general constant moves the fractional
    # part of the maximum in the base-2 domain, so only closeness is claimed
    c = torch.randn(B, H, Sq, 1)
    shifted, lse1 = attention_fwd_ref(q, k, v, causal=True, bias=c.expand(B, H, Sq, Sk))
    assert float((shifted.float() - base.float()).norm() / base.float().norm()) < 0.05
    assert float((lse1 - lse0 - c[..., 0]).abs().max()) < 0.05
    # (2) -inf on the second half of the keys == attention over the first half (whole blocks: nothing else changes)
    hide = torch.zeros(1, 1, Sq, Sk)
    hide[..., 64:] = float("-inf")
    a, la = attention_fwd_ref(q, k, v, causal=False, bias=hide)
    b, lb = attention_fwd_ref(q, k[:, :, :64], v[:, :, :64], causal=False)
    assert torch.equal(a, b) and torch.equal(la, lb)
    # (3) ALiBi slopes == the explicit bias (bottom-right aligned positions), per head
    slopes = torch.tensor([0.25, 0.0625])
    rel = ((torch.arange(Sq) + (Sk - Sq))[:, None] - torch.arange(Sk)[None, :]).abs().float()
    explicit = -slopes[None, :, None, None] * rel[None, None]
    a, la = attention_fwd_ref(q, k, v, causal=True, alibi_slopes=slopes)
    b, lb = attention_fwd_ref(q, k, v, causal=True, bias=explicit)
    assert torch.equal(a, b) and torch.equal(la, lb)
    assert not torch.equal(a, base)
    # and a slope of zero is no ALiBi at all
    z, lz = attention_fwd_ref(q, k, v, causal=True, alibi_slopes=torch.zeros(2))
    assert torch.equal(z, base) and torch.equal(lz, lse0)
