"""Writes tests/golden/reference_vectors.npz from the reference's own CPU-runnable code.  BUILD CONTAINER ONLY: it imports
two files of the reference checkout (never copied, never shipped); the fixture it writes is data (inputs and outputs).

Two functions of the oracle have no closed form, brute force or invariant that pins them completely, so their expected
outputs are taken from the reference itself:

* ``clip_mode="dynamic"`` of the quantizer (std-based block scale).  The reference's PyTorch twin
  ``convert_to_mxfp4_pytorch`` (tests/unittest/mxfp4/utils.py:285-364) is what its own test asserts bit-equal to the Triton
  kernel for fp32 tensors (tests/unittest/mxfp4/test_mxfp_quantization.py:29,62-75); fp32 inputs only, as there.
* the MXFP4 flash-attention recurrence: ``mxfp4_pnq_reference_bhsd`` (tests/unittest/mxfp4/test_mxfp_pnq.py:87-149), the
  reference's CPU model of its kernel.

Both are plain torch on the CPU.  The import goes through the stub modules test_mxfp_pnq.py installs itself (it fakes
``alto.kernels.fp4.mxfp4.mxfp_quantization`` with BLOCK_SIZE_DEFAULT = 32, so neither Triton nor torchtitan is touched).

Run from the repository root:  python tests/golden/make_reference_vectors.py [/root/reference]
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from tests.helpers import randn_outliers  # noqa: E402


def bits16(t):
    return t.contiguous().view(torch.int16).numpy().copy()


def main():
    ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    sys.path.insert(0, os.path.join(ref_root, "tests", "unittest", "mxfp4"))
    import test_mxfp_pnq as pnq          # installs its stubs, then imports utils.py beside it
    import utils as ref_utils

    out = {}
    # ---- dynamic clip, fp32: random data with outliers plus blocks with a closed form (constant, +-a, zero, one spike)
    x = randn_outliers((64, 128), torch.float32, seed=501)
    x[0, :32] = 3.0
    x[1, :32] = torch.tensor([1.5, -1.5] * 16)
    x[2, :32] = 0.0
    x[3, :32] = 0.0
    x[3, 5] = 1000.0
    x[32:64, 96:128] = 0.25          # a constant 32 x 32 block
    out["dyn_x"] = x.numpy().copy()
    for name, kw in (("row", dict(axis=-1)), ("col", dict(axis=-2)), ("2d", dict(axis=-1, is_2d_block=True))):
        q, s = ref_utils.convert_to_mxfp4_pytorch(x, clip_mode="dynamic", **kw)
        out[f"dyn_{name}_codes"] = q.contiguous().numpy().copy()
        out[f"dyn_{name}_scales"] = s.contiguous().numpy().copy()
        dq = ref_utils.convert_from_mxfp4_pytorch(q, s, output_dtype=torch.float32, clip_mode="dynamic", **kw)
        out[f"dyn_{name}_dq"] = dq.contiguous().numpy().copy()

    # dynamic clip together with the UOS scale rule (the reference's kernel allows the pair, its own test skips it): fp32 only
    for name, kw in (("row", dict(axis=-1)), ("col", dict(axis=-2)), ("2d", dict(axis=-1, is_2d_block=True))):
        q, s = ref_utils.convert_to_mxfp4_pytorch(x, clip_mode="dynamic", use_uos=True, **kw)
        out[f"dynuos_{name}_codes"] = q.contiguous().numpy().copy()
        out[f"dynuos_{name}_scales"] = s.contiguous().numpy().copy()

    # ---- the twin's other modes (clip none / static, the UOS scale rule), bf16 and fp32: they pin the scale rule, the
    # round-to-nearest encode and the packing by bytes the reference wrote, beside the closed-form pins of the oracle.
    # The twin rounds to nearest only (no stochastic rounding), so these are RNE vectors.
    xt = randn_outliers((64, 128), torch.float32, seed=503)
    xt[5, 32:64] = 0.0
    xt[6, :32] = torch.tensor([6.0, -6.0, 5.0, 7.0] * 8)         # at and around the top of the grid
    xt[7, :32] = 2.0 ** -130                                     # below the smallest scale
    for dt_name, dt in (("f32", torch.float32), ("bf16", torch.bfloat16)):
        xx = xt.to(dt)
        out[f"twin_{dt_name}_x"] = xx.numpy().copy() if dt == torch.float32 else bits16(xx)
        for mode, mkw in (("none", dict(clip_mode="none")), ("static", dict(clip_mode="static")), ("uos", dict(clip_mode="none", use_uos=True))):
            for name, kw in (("row", dict(axis=-1)), ("col", dict(axis=-2)), ("2d", dict(axis=-1, is_2d_block=True))):
                q, s = ref_utils.convert_to_mxfp4_pytorch(xx, **mkw, **kw)
                out[f"twin_{dt_name}_{mode}_{name}_codes"] = q.contiguous().numpy().copy()
                out[f"twin_{dt_name}_{mode}_{name}_scales"] = s.contiguous().numpy().copy()
                dq = ref_utils.convert_from_mxfp4_pytorch(q, s, output_dtype=dt, clip_mode=mkw["clip_mode"], **kw)
                out[f"twin_{dt_name}_{mode}_{name}_dq"] = dq.contiguous().numpy().copy() if dt == torch.float32 else bits16(dq.contiguous())

    # ---- attention: grouped-query heads, a partial last key block, head dims 64 and 128, non-causal with Sq != Sk.
    # (Causal cases keep Sq = Sk: the CPU model ends its key loop at the unshifted query end, test_mxfp_pnq.py:125, which
    # departs from the kernel's bottom-right aligned mask, triton_flash_attention_mxfp4.py:286-294, when Sq != Sk.)
    g = torch.Generator().manual_seed(502)
    cases = {"a": (2, 1, 96, 96, 64, True), "b": (1, 1, 128, 128, 128, True), "c": (2, 1, 64, 96, 64, False)}
    for name, (hq, hk, sq, sk, d, causal) in cases.items():
        q = torch.randn(1, hq, sq, d, generator=g).bfloat16()
        k = torch.randn(1, hk, sk, d, generator=g).bfloat16()
        v = torch.randn(1, hk, sk, d, generator=g).bfloat16()
        o = pnq.mxfp4_pnq_reference_bhsd(q, k, v, causal=causal, pnq=True)
        out[f"attn_{name}_q"], out[f"attn_{name}_k"], out[f"attn_{name}_v"] = bits16(q), bits16(k), bits16(v)
        out[f"attn_{name}_out"] = bits16(o)
        out[f"attn_{name}_causal"] = np.array(int(causal))
    path = os.path.join(ROOT, "tests", "golden", "reference_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
