"""HIP MXFP4 flash attention (through the C ABI) against the CPU model of
alto/kernels/fp4/mxfp4/triton_flash_attention_mxfp4.py.

Tolerance: Q/K/V operands are compared bit for bit; the output is floating point and passes through v_exp_f32 on the GPU
and libm on the CPU, so a probability can land on the other side of an E2M1 rounding boundary now and then.  Bound used:
relative L2 error <= 2e-3 of the bf16 output (observed: 0 to 2e-8), log-sum-exp within 1e-4 absolute.
"""
import pytest
import torch

from oracle import mxfp4_oracle as O
from oracle.attention_oracle import attention_fp32_ref, attention_fwd_ref

pytestmark = pytest.mark.gpu
DEV = "cuda"
REL_L2 = 2e-3


@pytest.fixture(scope="module")
def m():
    import alto_amd.mxfp4 as mod
    return mod


def _qkv(B, Hq, Hk, Sq, Sk, D, Dv, seed, v_mode="randn"):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, Sq, D, generator=g).to(torch.bfloat16)
    k = torch.randn(B, Hk, Sk, D, generator=g).to(torch.bfloat16)
    v = torch.randn(B, Hk, Sk, Dv, generator=g).to(torch.bfloat16)
    if v_mode == "ones":
        v = torch.ones_like(v)
    elif v_mode == "biased":
        v = v + 2.0
    return q, k, v


def _rel(a, b):
    return float((a.float() - b.float()).norm() / b.float().norm().clamp_min(1e-12))


CASES = [
    # B, Hq, Hk, Sq, Sk, D, Dv, causal
    (1, 4, 2, 128, 128, 64, 64, True),
    (2, 4, 4, 256, 256, 128, 128, True),
    (1, 8, 1, 256, 256, 128, 128, False),
    (1, 2, 1, 128, 256, 128, 64, True),       # Sq < Sk: mask aligned to the bottom-right corner
    (1, 2, 2, 96, 128, 192, 128, False),      # Sq not a multiple of the 128 rows a workgroup covers
    (1, 2, 1, 64, 192, 256, 128, False),
    (1, 2, 1, 32, 64, 64, 128, True),
    (1, 3, 3, 160, 320, 192, 64, True),
    (1, 2, 1, 96, 96, 128, 128, True),        # 96 keys: the second block is half there
    (2, 2, 2, 64, 224, 64, 64, False),
    (1, 4, 2, 32, 32, 128, 64, True),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(map(str, c)))
def test_attention_matches_cpu_model(m, case):
    B, Hq, Hk, Sq, Sk, D, Dv, causal = case
    q, k, v = _qkv(B, Hq, Hk, Sq, Sk, D, Dv, seed=sum(case))
    out, lse, _ = m.triton_attention_mxfp4(q.to(DEV), k.to(DEV), v.to(DEV), None, None, D ** -0.5, 0.0, 0, 0, Sq, Sk, causal, False, True, "bhsd")
    ref, ref_lse = attention_fwd_ref(q, k, v, causal=causal)
    assert out.dtype == torch.bfloat16 and out.shape == (B, Hq, Sq, Dv) and lse.shape == (B, Hq, Sq)
    assert _rel(out.cpu(), ref) <= REL_L2
    assert float((lse.cpu() - ref_lse).abs().max()) <= 1e-4
    # and it is attention: close to the fp32 result within what 4-bit operands allow
    assert _rel(out.cpu(), attention_fp32_ref(q, k, v, causal=causal)) < 0.35


def test_long_sequence_matches_cpu_model(m):
    """The bench shape per (batch, KV head): 2048 tokens, 8 query heads on one KV head, head dim 128, causal."""
    q, k, v = _qkv(1, 8, 1, 2048, 2048, 128, 128, seed=77)
    out, lse, _ = m.triton_attention_mxfp4(q.to(DEV), k.to(DEV), v.to(DEV), causal=True)
    ref, ref_lse = attention_fwd_ref(q, k, v, causal=True)
    assert _rel(out.cpu(), ref) <= REL_L2
    assert float((lse.cpu() - ref_lse).abs().max()) <= 1e-4
    # size-independent property: every output row is a convex combination of the (quantised) value rows it may see
    vq = O.dequantize(*O.quantize(v, axis=-1, is_2d_block=True), torch.float32, axis=-1, is_2d_block=True)[0, 0]
    hi = torch.cummax(vq, dim=0).values
    lo = -torch.cummax(-vq, dim=0).values
    o = out.cpu().float()[0]                                   # [8, 2048, 128]; row i sees keys 0..i
    tol = 2 ** -7 * vq.abs().max()
    assert bool(((o <= hi[None] + tol) & (o >= lo[None] - tol)).all())


def test_operands_are_the_reference_quantisations(m):
    """Q, K: 2D-block codes/scales along the head dim; V: the same 2D-block quantisation, packed along the keys."""
    q, k, v = _qkv(2, 2, 1, 64, 128, 128, 64, seed=3)
    qq, qs, kq, ks, vq, vs = m.quantize_qkv(q.to(DEV), k.to(DEV), v.to(DEV))
    for got, got_s, src in ((qq, qs, q), (kq, ks, k)):
        c, s = O.quantize(src, axis=-1, is_2d_block=True)
        assert torch.equal(got.cpu(), c) and torch.equal(got_s.cpu(), s)
    c, s = O.quantize(v.transpose(-1, -2).contiguous(), axis=-1, is_2d_block=True)
    assert torch.equal(vq.cpu(), c) and torch.equal(vs.cpu(), s.transpose(-1, -2))
    # same codes as quantising V along Dv (2D blocks are symmetric), only packed the other way
    c2, s2 = O.quantize(v, axis=-1, is_2d_block=True)
    assert torch.equal(O.unpack_nibbles(c.reshape(-1, c.shape[-1])).reshape(2, 1, 64, 128).transpose(-1, -2),
                       O.unpack_nibbles(c2.reshape(-1, c2.shape[-1])).reshape(2, 1, 128, 64))
    assert torch.equal(s.transpose(-1, -2), s2)


@pytest.mark.parametrize("v_mode", ["ones", "biased"])
def test_constant_value_attention(m, v_mode):
    """test_mxfp_pnq.py:163-174 on the GPU: with V = 1 the output is exactly 1 (row sums come from the quantised P)."""
    torch.manual_seed(1234)
    q = torch.randn(1, 32, 64, 64, dtype=torch.bfloat16)
    k = torch.randn(1, 8, 64, 64, dtype=torch.bfloat16)
    v = torch.ones(1, 8, 64, 64, dtype=torch.bfloat16)
    if v_mode == "biased":
        v = torch.randn(1, 8, 64, 64, dtype=torch.bfloat16) + 2.0
    out, lse, _ = m.triton_attention_mxfp4(q.to(DEV), k.to(DEV), v.to(DEV), causal=True)
    if v_mode == "ones":
        assert torch.equal(out.cpu(), torch.ones_like(out.cpu()))
    else:
        ref, _ = attention_fwd_ref(q, k, v, causal=True)
        assert _rel(out.cpu(), ref) <= REL_L2


def test_module_form_and_prequantised_entry(m):
    cfg = m.TrainingOpConfig()
    B, L, Hq, Hk, D = 1, 128, 4, 2, 128
    q, k, v = _qkv(B, Hq, Hk, L, L, D, D, seed=9)
    attn = m.LPScaledDotProductAttention(cfg)
    o = attn(q.transpose(1, 2).to(DEV), k.transpose(1, 2).to(DEV), v.transpose(1, 2).to(DEV), is_causal=True)   # [B, L, N, H]
    assert o.shape == (B, L, Hq, D)
    ref, _ = attention_fwd_ref(q, k, v, causal=True)
    assert _rel(o.transpose(1, 2).cpu(), ref) <= REL_L2
    qq, qs, kq, ks, vq, vs = m.quantize_qkv(q.to(DEV), k.to(DEV), v.to(DEV))
    o2, _ = m.attention_mxfp4_forward(qq, kq, vq, qs, ks, vs, D ** -0.5, True)
    assert torch.equal(o2, o.transpose(1, 2))
    with pytest.raises(ValueError):
        attn(q.to(DEV), k.to(DEV), v.to(DEV), attention_masks=object())


def test_layout_bshd_is_the_same_attention_on_permuted_views(m):
    q, k, v = (t.to(DEV) for t in _qkv(2, 4, 2, 128, 192, 64, 64, seed=9))      # [B, H, S, D]
    o, lse, _ = m.triton_attention_mxfp4(q, k, v, causal=True)
    qs, ks, vs = (t.transpose(1, 2).contiguous() for t in (q, k, v))            # [B, S, H, D]
    o2, lse2, _ = m.triton_attention_mxfp4(qs, ks, vs, causal=True, layout="bshd")
    assert o2.shape == qs.shape[:3] + (v.shape[-1],)
    assert torch.equal(o2.transpose(1, 2), o) and torch.equal(lse2, lse)


@pytest.mark.parametrize("causal", [True, False])
def test_layout_thd_is_the_attention_of_every_sequence(m, causal):
    """Packed variable-length sequences (layout 'thd', cu_seqlens): each sequence's rows equal the 'bhsd' attention of that
    sequence alone and match the CPU model; lengths of 32, 96 (half a key block), 256 and 160 / 192 (Sq < Sk)."""
    Hq, Hk, D, Dv = 4, 2, 128, 128
    lens_q, lens_k = [32, 96, 256, 160], [32, 96, 256, 192]
    cq = [0] + list(torch.tensor(lens_q).cumsum(0).tolist())
    ck = [0] + list(torch.tensor(lens_k).cumsum(0).tolist())
    g = torch.Generator().manual_seed(17)
    q = torch.randn(cq[-1], Hq, D, generator=g).to(torch.bfloat16)
    k = torch.randn(ck[-1], Hk, D, generator=g).to(torch.bfloat16)
    v = torch.randn(ck[-1], Hk, Dv, generator=g).to(torch.bfloat16)
    out, lse, _ = m.triton_attention_mxfp4(q.to(DEV), k.to(DEV), v.to(DEV), sm_scale=D ** -0.5, cu_seqlens_q=torch.tensor(cq, dtype=torch.int32),
                                           cu_seqlens_k=ck, max_seqlens_q=max(lens_q), max_seqlens_k=max(lens_k), causal=causal, layout="thd")
    assert out.shape == (cq[-1], Hq, Dv) and out.dtype == torch.bfloat16 and lse.shape == (cq[-1], Hq)
    for i in range(len(lens_q)):
        qi, ki, vi = (t.transpose(0, 1).unsqueeze(0) for t in (q[cq[i]:cq[i + 1]], k[ck[i]:ck[i + 1]], v[ck[i]:ck[i + 1]]))
        o1, l1, _ = m.triton_attention_mxfp4(qi.to(DEV), ki.to(DEV), vi.to(DEV), sm_scale=D ** -0.5, causal=causal)
        assert torch.equal(out[cq[i]:cq[i + 1]].transpose(0, 1), o1[0]) and torch.equal(lse[cq[i]:cq[i + 1]].transpose(0, 1), l1[0])
        ref, ref_lse = attention_fwd_ref(qi, ki, vi, causal=causal)
        assert _rel(o1.cpu(), ref) <= REL_L2 and float((l1.cpu() - ref_lse).abs().max()) <= 1e-4


@pytest.mark.parametrize("case", [(2, 4, 2, 128, 256, 128, 128, True), (1, 2, 2, 96, 96, 64, 64, False), (1, 4, 1, 64, 192, 192, 128, True)],
                         ids=lambda c: "x".join(map(str, c)))
@pytest.mark.parametrize("terms", ["bias", "alibi", "both", "bias_per_head", "hide_keys"])
def test_bias_and_alibi_match_the_cpu_model(m, case, terms):
    """The additive score terms of the reference's kernel (:288-299): a full bias tensor, a bias broadcast over the batch,
    ALiBi slopes per head, both together, and a bias of -inf that hides the second half of the keys of some rows."""
    B, Hq, Hk, Sq, Sk, D, Dv, causal = case
    q, k, v = _qkv(B, Hq, Hk, Sq, Sk, D, Dv, seed=sum(case) + len(terms))
    g = torch.Generator().manual_seed(3)
    bias = slopes = None
    if terms in ("bias", "both"):
        bias = torch.randn(B, Hq, Sq, Sk, generator=g)
    if terms == "bias_per_head":
        bias = torch.randn(1, Hq, Sq, Sk, generator=g)
    if terms == "hide_keys":
        bias = torch.zeros(1, 1, Sq, Sk)
        bias[..., : Sq // 2, Sk // 2:] = float("-inf")     # (causal rows keep key 0 at least)
    if terms in ("alibi", "both"):
        slopes = 2.0 ** -(1 + torch.arange(Hq).float() % 4)
    out, lse, _ = m.triton_attention_mxfp4(q.to(DEV), k.to(DEV), v.to(DEV), None if slopes is None else slopes.to(DEV),
                                           None if bias is None else bias.to(DEV), D ** -0.5, 0.0, 0, 0, Sq, Sk, causal, False, True, "bhsd")
    ref, ref_lse = attention_fwd_ref(q, k, v, causal=causal, bias=bias, alibi_slopes=slopes)
    assert _rel(out.cpu(), ref) <= REL_L2
    assert float((lse.cpu() - ref_lse).abs().max()) <= 1e-4
    plain, _, _ = m.triton_attention_mxfp4(q.to(DEV), k.to(DEV), v.to(DEV), sm_scale=D ** -0.5, causal=causal)
    assert not torch.equal(plain, out)


def test_alibi_with_packed_sequences(m):
    Hq, D = 2, 64
    g = torch.Generator().manual_seed(4)
    q = torch.randn(160, Hq, D, generator=g).to(torch.bfloat16)
    k = torch.randn(160, Hq, D, generator=g).to(torch.bfloat16)
    v = torch.randn(160, Hq, D, generator=g).to(torch.bfloat16)
    slopes = torch.tensor([0.5, 0.125])
    out, lse, _ = m.triton_attention_mxfp4(q.to(DEV), k.to(DEV), v.to(DEV), slopes.to(DEV), None, D ** -0.5, cu_seqlens_q=[0, 64, 160],
                                           cu_seqlens_k=[0, 64, 160], causal=True, layout="thd")
    for lo, hi in ((0, 64), (64, 160)):
        ref, _ = attention_fwd_ref(*(t[lo:hi].transpose(0, 1).unsqueeze(0) for t in (q, k, v)), causal=True, alibi_slopes=slopes)
        assert _rel(out[lo:hi].transpose(0, 1).unsqueeze(0).cpu(), ref) <= REL_L2


def test_rejected_arguments(m):
    q, k, v = (t.to(DEV) for t in _qkv(1, 2, 2, 64, 64, 64, 64, seed=1))
    with pytest.raises(NotImplementedError):
        m.triton_attention_mxfp4(q, k, v, layout="hsd")
    with pytest.raises(RuntimeError, match="multiples of 32"):
        m.triton_attention_mxfp4(q[0].transpose(0, 1), k[0].transpose(0, 1), v[0].transpose(0, 1), cu_seqlens_q=[0, 40, 64], cu_seqlens_k=[0, 32, 64],
                                 layout="thd")
    with pytest.raises(RuntimeError, match="same number of sequences"):
        m.triton_attention_mxfp4(q[0].transpose(0, 1), k[0].transpose(0, 1), v[0].transpose(0, 1), cu_seqlens_q=[0, 64], cu_seqlens_k=[0, 32, 64],
                                 layout="thd")
    with pytest.raises(NotImplementedError):
        m.triton_attention_mxfp4(q, k, v, dropout_p=0.1)
    with pytest.raises(RuntimeError, match="does not broadcast"):
        m.triton_attention_mxfp4(q, k, v, bias=torch.zeros(3, 64, 64, device=DEV))
    with pytest.raises(AssertionError, match="Sq <= Sk"):
        m.triton_attention_mxfp4(q.repeat(1, 1, 2, 1), k, v, causal=True)
    qb, kb, vb = (t.to(DEV) for t in _qkv(1, 2, 2, 64, 80, 64, 64, seed=1))
    with pytest.raises(Exception):      # 80 keys: not a multiple of the 32-row quantisation blocks
        m.triton_attention_mxfp4(qb, kb, vb, causal=False)
    q3, k3, v3 = (t.to(DEV) for t in _qkv(1, 2, 2, 64, 64, 96, 64, seed=1))
    with pytest.raises(AssertionError, match="head dim"):
        m.triton_attention_mxfp4(q3, k3, v3, causal=False)
    with pytest.raises(RuntimeError):
        m.triton_attention_mxfp4(q.cpu(), k.cpu(), v.cpu())


# the configurations of the reference's own attention test (tests/unittest/mxfp4/test_mxfp_attention.py:51-70, batch 4,
# causal, bhsd): seqlen, query heads, key/value heads, head dim of Q/K, head dim of V
REFERENCE_CONFIGS = [
    (1024, 32, 32, 128, 128),
    (1024, 64, 8, 128, 128),
    (1024, 32, 8, 128, 128),
    (1024, 16, 16, 192, 128),
    (1024, 128, 128, 192, 128),
    (1024, 48, 8, 128, 128),
    (2048, 64, 8, 128, 128),
]


@pytest.mark.parametrize("cfg", REFERENCE_CONFIGS, ids=lambda c: "x".join(map(str, c)))
def test_reference_attention_configs(m, cfg):
    """The reference's test runs these shapes against bf16 scaled_dot_product_attention and reports SNR and cosine
    similarity without a threshold (test_mxfp_attention.py:122-128).  Here the same comparison carries floors chosen
    below what MXFP4 operands and probabilities give on this data (observed 12.1 to 12.3 dB, cosine 0.970 to 0.972): a wrong mask
    offset, head mapping or scale block would fall far below them."""
    from tests.helpers import snr_db
    S, Hq, Hk, D, Dv = cfg
    B = 4
    g = torch.Generator(device=DEV).manual_seed(1234)
    q = torch.randn(B, Hq, S, D, device=DEV, generator=g).bfloat16()
    k = torch.randn(B, Hk, S, D, device=DEV, generator=g).bfloat16()
    v = torch.randn(B, Hk, S, Dv, device=DEV, generator=g).bfloat16()
    sm_scale = D ** -0.5
    print(f"attention {cfg}", flush=True)
    out = m.triton_attention_mxfp4(q, k, v, bias=None, alibi_slopes=None, sm_scale=sm_scale, dropout_p=0.0, cu_seqlens_q=0, cu_seqlens_k=0,
                                   max_seqlens_q=S, max_seqlens_k=S, causal=True, return_scores=False, use_exp2=True, layout="bhsd")[0]
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, scale=sm_scale, enable_gqa=Hq != Hk)
    assert out.shape == ref.shape and out.dtype == torch.bfloat16
    snr = snr_db(ref.float().cpu(), out.float().cpu())
    cos = float(torch.nn.functional.cosine_similarity(ref.float().flatten(), out.float().flatten(), dim=0))
    print(f"  SNR {snr:.2f} dB, cosine {cos:.5f}", flush=True)
    assert snr > 11.0 and cos > 0.96
