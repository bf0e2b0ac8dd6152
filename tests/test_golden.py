"""Committed vectors (tests/golden/mxfp4_vectors.npz, written by tests/golden/make_vectors.py): the oracle and the HIP
path must both reproduce every byte.  The reference holds no stored vectors for this path; these freeze the pinned
oracle's outputs on small inputs."""
import os

import numpy as np
import pytest
import torch

import oracle as O
from tests.helpers import assert_bytes_equal

V = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mxfp4_vectors.npz"))


def t(name):
    return torch.from_numpy(V[name])


def bf16(name):
    return t(name).view(torch.bfloat16)


# ----------------------------------------------------------------------------------------------- oracle (CPU)
def test_oracle_attention_and_dynamic_clip_vectors():
    from oracle.attention_oracle import attention_fwd_ref
    o, lse = attention_fwd_ref(bf16("attn_q_bf16bits"), bf16("attn_k_bf16bits"), bf16("attn_v_bf16bits"), causal=True)
    assert_bytes_equal(o.view(torch.int16), t("attn_out_bf16bits"), "attention output")
    assert torch.equal(lse, t("attn_lse_f32"))
    q, s = O.quantize(bf16("rne_x_bf16bits"), clip_mode="dynamic")
    assert_bytes_equal(q, t("dyn_codes"), "dynamic-clip codes")
    assert_bytes_equal(s, t("dyn_scales"), "dynamic-clip scales")


def test_oracle_rne_vectors():
    q, s = O.quantize(bf16("rne_x_bf16bits"))
    assert_bytes_equal(q, t("rne_codes"), "codes")
    assert_bytes_equal(s, t("rne_scales"), "scales")
    dq = O.dequantize(q, s, torch.bfloat16)
    assert_bytes_equal(dq.view(torch.int16), t("rne_dequant_bf16bits"), "dequantised bf16 bits")
    q, s = O.quantize(t("w2d_x_f32"), is_2d_block=True)
    assert_bytes_equal(q, t("w2d_codes"), "2D codes")
    assert_bytes_equal(s, t("w2d_scales"), "2D scales")


def test_oracle_sr_rht_vectors():
    g, r = bf16("sr_x_bf16bits"), t("sr_rand")
    q, s = O.quantize(g, use_sr=True, rand_bits=r)
    assert_bytes_equal(q, t("sr_row_codes"), "row codes")
    assert_bytes_equal(s, t("sr_row_scales"), "row scales")
    gh = O.rht_left(g, t("had_signs"), t("had_perm"))
    assert_bytes_equal(gh.view(torch.int16), t("sr_rht_bf16bits"), "transformed bf16 bits")
    qc, sc = O.quantize(gh, axis=0, use_sr=True, rand_bits=r)
    assert_bytes_equal(qc.contiguous(), t("sr_col_codes"), "column codes")
    assert_bytes_equal(sc.contiguous(), t("sr_col_scales"), "column scales")


def test_oracle_gemm_vector():
    c = O.gemm_ref(t("gemm_a_codes"), t("gemm_a_scales"), t("gemm_b_codes"), t("gemm_b_scales"), use_2dblock_b=True, trans_b=True)
    assert torch.equal(c.float(), t("gemm_c_f32"))


# ----------------------------------------------------------------------------------------------- HIP path (GPU)
@pytest.fixture(scope="module")
def m():
    import alto_amd.mxfp4 as mod
    return mod


@pytest.mark.gpu
def test_hip_rne_vectors(m):
    q, s = m.convert_to_mxfp4(bf16("rne_x_bf16bits").cuda())
    assert_bytes_equal(q, t("rne_codes"), "codes")
    assert_bytes_equal(s, t("rne_scales"), "scales")
    dq = m.convert_from_mxfp4(q, s, torch.bfloat16)
    assert_bytes_equal(dq.view(torch.int16), t("rne_dequant_bf16bits"), "dequantised bf16 bits")
    q, s = m.convert_to_mxfp4(t("w2d_x_f32").cuda(), is_2d_block=True)
    assert_bytes_equal(q, t("w2d_codes"), "2D codes")
    assert_bytes_equal(s, t("w2d_scales"), "2D scales")


@pytest.mark.gpu
def test_hip_sr_rht_vectors(m):
    g, r = bf16("sr_x_bf16bits").cuda(), t("sr_rand").cuda()
    h = m.HadamardTransform(t("had_signs"), t("had_perm"))
    rq, rs, cq, cs = m.quantize_rowcol(g, False, use_sr=True, rand_bits=r, hadamard=h)
    assert_bytes_equal(rq, t("sr_row_codes"), "row codes")
    assert_bytes_equal(rs, t("sr_row_scales"), "row scales")
    assert_bytes_equal(cq.contiguous(), t("sr_col_codes"), "column codes")
    assert_bytes_equal(cs.contiguous(), t("sr_col_scales"), "column scales")
    gh = m.hadamard_left(g, h)
    assert_bytes_equal(gh.view(torch.int16), t("sr_rht_bf16bits"), "transformed bf16 bits")


@pytest.mark.gpu
def test_hip_gemm_vector(m):
    c = m.blockwise_mxfp4_gemm(t("gemm_a_codes").cuda(), t("gemm_a_scales").cuda(), t("gemm_b_codes").cuda(), t("gemm_b_scales").cuda(),
                               use_2dblock_b=True, trans_b=True, output_dtype=torch.float32)
    ref = t("gemm_c_f32")
    # products of E2M1 values are exact and these sums stay far below 2^24 ulps of their scale: fp32 accumulation in any
    # order differs from the float64 reference by rounding only (tolerance of the GEMM parity bar: 1e-2 relative Frobenius)
    assert O.rel_frobenius(c.cpu(), ref) < 1e-5


@pytest.mark.gpu
def test_hip_attention_and_dynamic_clip_vectors(m):
    o, lse, _ = m.triton_attention_mxfp4(bf16("attn_q_bf16bits").cuda(), bf16("attn_k_bf16bits").cuda(), bf16("attn_v_bf16bits").cuda(), causal=True)
    ref = bf16("attn_out_bf16bits").float()
    # floating point through v_exp_f32: tolerance of the attention parity bar (2e-3 relative L2; equal bytes in practice)
    assert float((o.cpu().float() - ref).norm() / ref.norm()) <= 2e-3
    assert float((lse.cpu() - t("attn_lse_f32")).abs().max()) <= 1e-4
    q, s = m.convert_to_mxfp4(bf16("rne_x_bf16bits").cuda(), clip_mode="dynamic")
    assert_bytes_equal(q, t("dyn_codes"), "dynamic-clip codes")
    assert_bytes_equal(s, t("dyn_scales"), "dynamic-clip scales")


# ---------------------------------------------------------------------------------------------- vectors made by the reference
def _ref_vectors():
    return np.load(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.npz"))


@pytest.mark.parametrize("name,kw", [("row", dict(axis=-1)), ("col", dict(axis=-2)), ("2d", dict(axis=-1, is_2d_block=True))])
def test_dynamic_clip_equals_the_reference_twin(name, kw):
    """clip_mode="dynamic" on fp32 data: the oracle reproduces, byte for byte, the codes, scales and dequantised values
    that the reference's PyTorch twin computed (tests/golden/make_reference_vectors.py) -- the function its own test holds
    bit-equal to the Triton kernel for fp32 tensors (tests/unittest/mxfp4/test_mxfp_quantization.py:62-75)."""
    d = _ref_vectors()
    x = torch.from_numpy(d["dyn_x"])
    q, s = O.quantize(x, clip_mode="dynamic", **kw)
    assert torch.equal(s.contiguous(), torch.from_numpy(d[f"dyn_{name}_scales"]))
    assert torch.equal(q.contiguous(), torch.from_numpy(d[f"dyn_{name}_codes"]))
    dq = O.dequantize(q, s, torch.float32, clip_mode="dynamic", **kw)
    assert torch.equal(dq.contiguous(), torch.from_numpy(d[f"dyn_{name}_dq"]))


@pytest.mark.parametrize("name,kw", [("row", dict(axis=-1)), ("col", dict(axis=-2)), ("2d", dict(axis=-1, is_2d_block=True))])
def test_dynamic_clip_with_uos_equals_the_reference_twin(name, kw):
    """clip_mode="dynamic" together with use_uos (mxfp_quantization.py:54-78 allows the pair): the twin's fp32 bytes."""
    d = _ref_vectors()
    x = torch.from_numpy(d["dyn_x"])
    q, s = O.quantize(x, clip_mode="dynamic", use_uos=True, **kw)
    assert torch.equal(s.contiguous(), torch.from_numpy(d[f"dynuos_{name}_scales"]))
    assert torch.equal(q.contiguous(), torch.from_numpy(d[f"dynuos_{name}_codes"]))


@pytest.mark.gpu
@pytest.mark.parametrize("name,kw", [("row", dict(axis=-1)), ("col", dict(axis=-2)), ("2d", dict(axis=-1, is_2d_block=True))])
def test_hip_dynamic_clip_with_uos_equals_the_reference_twin(name, kw):
    import alto_amd.mxfp4 as m
    d = _ref_vectors()
    x = torch.from_numpy(d["dyn_x"]).cuda()
    q, s = m.convert_to_mxfp4(x, clip_mode="dynamic", use_uos=True, **kw)
    assert_bytes_equal(s.contiguous(), torch.from_numpy(d[f"dynuos_{name}_scales"]), f"dynamic+uos {name} scales")
    assert_bytes_equal(q.contiguous(), torch.from_numpy(d[f"dynuos_{name}_codes"]), f"dynamic+uos {name} codes")


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_attention_model_equals_the_reference_cpu_model(name):
    """The oracle's MXFP4 attention recurrence gives the reference CPU model's outputs (test_mxfp_pnq.py:87-149) bit for
    bit with natural exponentials, and within one bf16 rounding with the kernel's exp2 formulation."""
    from oracle.attention_oracle import attention_fwd_ref
    d = _ref_vectors()
    q, k, v = (torch.from_numpy(d[f"attn_{name}_{t}"]).view(torch.bfloat16) for t in "qkv")
    exp = torch.from_numpy(d[f"attn_{name}_out"]).view(torch.bfloat16)
    out, _ = attention_fwd_ref(q, k, v, causal=bool(d[f"attn_{name}_causal"]), use_exp2=False)
    assert torch.equal(out.view(torch.int16), exp.view(torch.int16))
    out2, _ = attention_fwd_ref(q, k, v, causal=bool(d[f"attn_{name}_causal"]), use_exp2=True)
    assert float((out2.float() - exp.float()).norm() / exp.float().norm()) < 4e-3


@pytest.mark.gpu
@pytest.mark.parametrize("name,kw", [("row", dict(axis=-1)), ("col", dict(axis=-2)), ("2d", dict(axis=-1, is_2d_block=True))])
def test_hip_dynamic_clip_equals_the_reference_twin(name, kw):
    """The HIP quantizer with clip_mode="dynamic" reproduces the reference twin's fp32 vectors byte for byte."""
    import alto_amd.mxfp4 as m
    d = _ref_vectors()
    x = torch.from_numpy(d["dyn_x"]).cuda()
    q, s = m.convert_to_mxfp4(x, clip_mode="dynamic", **kw)
    assert_bytes_equal(s.contiguous(), torch.from_numpy(d[f"dyn_{name}_scales"]), f"dynamic {name} scales")
    assert_bytes_equal(q.contiguous(), torch.from_numpy(d[f"dyn_{name}_codes"]), f"dynamic {name} codes")
    dq = m.convert_from_mxfp4(q, s, torch.float32, clip_mode="dynamic", **kw)
    assert torch.equal(dq.contiguous().cpu(), torch.from_numpy(d[f"dyn_{name}_dq"]))


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_hip_attention_close_to_the_reference_cpu_model(name):
    """The HIP attention kernel on the fixture's Q, K, V against the reference CPU model's output: relative L2 <= 4e-3
    (exp2 formulation and v_exp_f32 against libm's exp: a probability can cross an E2M1 rounding boundary)."""
    import alto_amd.mxfp4 as m
    d = _ref_vectors()
    q, k, v = (torch.from_numpy(d[f"attn_{name}_{t}"]).view(torch.bfloat16).cuda() for t in "qkv")
    exp = torch.from_numpy(d[f"attn_{name}_out"]).view(torch.bfloat16)
    out = m.triton_attention_mxfp4(q, k, v, causal=bool(d[f"attn_{name}_causal"]))
    out = out[0] if isinstance(out, (tuple, list)) else out
    assert float((out.float().cpu() - exp.float()).norm() / exp.float().norm()) < 4e-3


# --------------------------------------------------------------------------- the reference twin's other modes
_TWIN_MODES = {"none": dict(clip_mode="none"), "static": dict(clip_mode="static"), "uos": dict(clip_mode="none", use_uos=True)}
_TWIN_AXES = {"row": dict(axis=-1), "col": dict(axis=-2), "2d": dict(axis=-1, is_2d_block=True)}


def _twin_case(d, dt_name, mode, name):
    dt = torch.float32 if dt_name == "f32" else torch.bfloat16
    x = torch.from_numpy(d[f"twin_{dt_name}_x"])
    x = x if dt == torch.float32 else x.view(torch.bfloat16)
    key = f"twin_{dt_name}_{mode}_{name}"
    dq = torch.from_numpy(d[key + "_dq"])
    return dt, x, torch.from_numpy(d[key + "_codes"]), torch.from_numpy(d[key + "_scales"]), dq if dt == torch.float32 else dq.view(torch.bfloat16)


def _twin_uos_bf16_differs(dt_name, mode):
    # The twin takes log2 of the bf16 absmax IN bf16 (utils.py, torch ops on a bf16 tensor); the Triton kernel, and with it
    # the oracle and the HIP kernel, promote the division and the log2 to fp32 (tl's rule for `/`).  Where the two land on
    # different sides of an integer the scale bytes differ by one; the reference's own test skips this pairing.
    return dt_name == "bf16" and mode == "uos"


@pytest.mark.parametrize("dt_name", ["f32", "bf16"])
@pytest.mark.parametrize("mode", list(_TWIN_MODES))
@pytest.mark.parametrize("name", list(_TWIN_AXES))
def test_oracle_equals_the_reference_twin(dt_name, mode, name):
    """Scales, codes and dequantised values of the reference's PyTorch twin (tests/unittest/mxfp4/utils.py:285-400), frozen by
    tests/golden/make_reference_vectors.py, for clip none / static and the UOS rule, bf16 and fp32, byte for byte."""
    d = _ref_vectors()
    dt, x, codes, scales, dq = _twin_case(d, dt_name, mode, name)
    q, s = O.quantize(x, **_TWIN_MODES[mode], **_TWIN_AXES[name])
    if _twin_uos_bf16_differs(dt_name, mode):
        diff = (s.contiguous().to(torch.int16) - scales.to(torch.int16)).abs()
        assert int(diff.max()) <= 1, "UOS on bf16: the twin's bf16 log2 and the kernel's fp32 log2 differ by at most one step"
        return
    assert torch.equal(s.contiguous(), scales)
    assert torch.equal(q.contiguous(), codes)
    got = O.dequantize(q, s, dt, clip_mode=_TWIN_MODES[mode]["clip_mode"], **_TWIN_AXES[name]).contiguous()
    assert torch.equal(got.view(torch.int16 if dt == torch.bfloat16 else torch.int32), dq.view(torch.int16 if dt == torch.bfloat16 else torch.int32))


@pytest.mark.gpu
@pytest.mark.parametrize("dt_name", ["f32", "bf16"])
@pytest.mark.parametrize("mode", list(_TWIN_MODES))
@pytest.mark.parametrize("name", list(_TWIN_AXES))
def test_hip_equals_the_reference_twin(dt_name, mode, name):
    import alto_amd.mxfp4 as m
    d = _ref_vectors()
    dt, x, codes, scales, dq = _twin_case(d, dt_name, mode, name)
    q, s = m.convert_to_mxfp4(x.cuda(), **_TWIN_MODES[mode], **_TWIN_AXES[name])
    if _twin_uos_bf16_differs(dt_name, mode):
        eq, es = O.quantize(x, **_TWIN_MODES[mode], **_TWIN_AXES[name])          # the HIP kernel follows the Triton kernel's fp32 log2
        assert_bytes_equal(s.contiguous(), es.contiguous(), "uos bf16 scales (fp32 log2)")
        assert_bytes_equal(q.contiguous(), eq.contiguous(), "uos bf16 codes")
        return
    assert_bytes_equal(s.contiguous(), scales, f"{dt_name} {mode} {name} scales")
    assert_bytes_equal(q.contiguous(), codes, f"{dt_name} {mode} {name} codes")
    got = m.convert_from_mxfp4(q, s, dt, clip_mode=_TWIN_MODES[mode]["clip_mode"], **_TWIN_AXES[name]).contiguous().cpu()
    assert torch.equal(got.view(torch.int16 if dt == torch.bfloat16 else torch.int32), dq.view(torch.int16 if dt == torch.bfloat16 else torch.int32))
