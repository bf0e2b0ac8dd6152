"""Writes tests/golden/mxfp4_vectors.npz: small input/output vectors of the MXFP4 path.

The reference repository holds no stored vectors for this path (its tests compare two implementations on a GPU), so
the expected outputs here come from the CPU oracle after it has been pinned by tests/test_oracle_pins.py.  The file
freezes them: a later change to the oracle or to the kernels that alters any byte fails against the fixture.

Run from the repository root:  python tests/golden/make_vectors.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import mxfp4_oracle as O  # noqa: E402
from tests.helpers import hadamard_from_seed, laplace, rand_bits, randn_outliers  # noqa: E402


def bf16_bits(t):
    return t.contiguous().view(torch.int16).numpy().copy()


def main():
    out = {}
    # 1. RNE, 1D-32 along the last dim, bf16 with outliers (the round-trip configuration, reduced to 64 x 128)
    x = randn_outliers((64, 128), torch.bfloat16, seed=11)
    q, s = O.quantize(x)
    out["rne_x_bf16bits"], out["rne_codes"], out["rne_scales"] = bf16_bits(x), q.numpy(), s.numpy()
    out["rne_dequant_bf16bits"] = bf16_bits(O.dequantize(q, s, torch.bfloat16))
    # 2. RNE, 2D 32x32 blocks, fp32 input
    w = (randn_outliers((64, 96), torch.float32, seed=12) * 0.02)
    q, s = O.quantize(w, is_2d_block=True)
    out["w2d_x_f32"], out["w2d_codes"], out["w2d_scales"] = w.numpy(), q.numpy(), s.numpy()
    # 3. fused gradient quantiser: Laplace(0, 1e-3) bf16, SR with supplied bits; row copy plain, column copy on H.dY
    g = laplace((64, 96), 1e-3, torch.bfloat16, seed=13)
    r = rand_bits((64, 96), seed=14)
    signs, perm = hadamard_from_seed(1234)
    q, s = O.quantize(g, use_sr=True, rand_bits=r)
    gh = O.rht_left(g, signs, perm)
    qc, sc = O.quantize(gh, axis=0, use_sr=True, rand_bits=r)
    out["sr_x_bf16bits"], out["sr_rand"] = bf16_bits(g), r.numpy()
    out["had_signs"], out["had_perm"] = signs.numpy(), perm.numpy()
    out["sr_row_codes"], out["sr_row_scales"] = q.numpy(), s.numpy()
    out["sr_rht_bf16bits"] = bf16_bits(gh)
    out["sr_col_codes"], out["sr_col_scales"] = qc.contiguous().numpy(), sc.contiguous().numpy()   # logical [M/2, C], [M/32, C]
    # 4. GEMM on codes: A 1D scales [64, 128], B 2D scales [96, 128] -> fp32 [64, 96]
    a = randn_outliers((64, 128), torch.bfloat16, seed=15)
    b = randn_outliers((96, 128), torch.bfloat16, seed=16) * 0.02
    aq, as_ = O.quantize(a)
    bq, bs = O.quantize(b, is_2d_block=True)
    out["gemm_a_codes"], out["gemm_a_scales"] = aq.numpy(), as_.numpy()
    out["gemm_b_codes"], out["gemm_b_scales"] = bq.numpy(), bs.numpy()
    out["gemm_c_f32"] = O.gemm_ref(aq, as_, bq, bs, use_2dblock_b=True, trans_b=True).float().numpy()
    # 5. flash-attention forward: 2 query heads on 1 KV head, 64 queries x 96 keys (the second key block is half there),
    #    head dim 64, causal (bottom-right aligned); and the dynamic-clip scales of vector 1's input
    from oracle.attention_oracle import attention_fwd_ref
    gq = torch.Generator().manual_seed(21)
    aq_ = torch.randn(1, 2, 64, 64, generator=gq).to(torch.bfloat16)
    ak_ = torch.randn(1, 1, 96, 64, generator=gq).to(torch.bfloat16)
    av_ = torch.randn(1, 1, 96, 64, generator=gq).to(torch.bfloat16)
    ao, alse = attention_fwd_ref(aq_, ak_, av_, causal=True)
    out["attn_q_bf16bits"], out["attn_k_bf16bits"], out["attn_v_bf16bits"] = bf16_bits(aq_), bf16_bits(ak_), bf16_bits(av_)
    out["attn_out_bf16bits"], out["attn_lse_f32"] = bf16_bits(ao), alse.numpy()
    qd, sd = O.quantize(x, clip_mode="dynamic")
    out["dyn_codes"], out["dyn_scales"] = qd.numpy(), sd.numpy()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "mxfp4_vectors.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes;", ", ".join(f"{k}{list(v.shape)}" for k, v in out.items()))


if __name__ == "__main__":
    main()
