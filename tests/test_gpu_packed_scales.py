"""Packed (GEMM-ready) scale layout: the converter against its definition, and the kernels that read it against the ones
that read plain scales, bit for bit."""
import numpy as np
import pytest
import torch

import oracle as O
from tests.helpers import assert_bytes_equal, randn_outliers

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def m():
    import alto_amd.mxfp4 as mod
    return mod


def pack_reference(scales: np.ndarray, rows: int, K: int, is_2d: bool) -> np.ndarray:
    """The definition: packed[kb, row, 4 (2 h + ms) + j] = scale of group 16 kb + 8 ms + 2 j + h, 127 beyond K."""
    G = K // 32
    KB = -(-G // 16)
    full = np.full((rows, KB * 16), 127, dtype=np.uint8)
    src = np.repeat(scales, 32, axis=0)[:rows] if is_2d else scales
    full[:, :G] = src
    out = np.empty((KB, rows, 16), dtype=np.uint8)
    for h in range(2):
        for ms in range(2):
            for j in range(4):
                out[:, :, 4 * (2 * h + ms) + j] = full.reshape(rows, KB, 16)[:, :, 8 * ms + 2 * j + h].T
    return out


@pytest.mark.parametrize("rows,K,is_2d", [(64, 512, False), (300, 544, False), (256, 2880, True), (96, 32, False), (1024, 4096, True)])
def test_pack_scales_against_the_definition(m, rows, K, is_2d):
    from alto_amd.mxfp4.linear import pack_scales
    g = torch.Generator().manual_seed(rows + K)
    s = torch.randint(100, 140, ((rows // 32) if is_2d else rows, K // 32), generator=g, dtype=torch.uint8)
    got = pack_scales(s.to(DEV), rows, K, is_2d)
    assert_bytes_equal(got.cpu(), torch.from_numpy(pack_reference(s.numpy(), rows, K, is_2d)), "packed scales")
    # a strided (transposed) source gives the same bytes
    st = s.t().contiguous().to(DEV).t()
    assert_bytes_equal(pack_scales(st, rows, K, is_2d).cpu(), got.cpu(), "packed scales from a strided source")


@pytest.mark.parametrize("shape", [(256, 256, 512), (300, 264, 544), (512, 384, 2880), (640, 520, 992), (384, 256, 1376), (200, 136, 704), (128, 128, 4096)])
@pytest.mark.parametrize("b_2d", [False, True])
def test_gemm_with_packed_scales_equals_the_plain_call(m, shape, b_2d):
    from alto_amd.mxfp4.linear import gemm_packed, pack_scales, packed_gemm_supported
    M, N, K = shape
    if b_2d and N % 32:
        pytest.skip("2D weight blocks need N % 32 == 0")
    a = randn_outliers((M, K), torch.bfloat16, seed=21).to(DEV)
    b = randn_outliers((N, K), torch.bfloat16, seed=22).to(DEV)
    aq, as_ = m.convert_to_mxfp4(a)
    bq, bs = m.convert_to_mxfp4(b, is_2d_block=b_2d)
    want = m.blockwise_mxfp4_gemm(aq, as_, bq, bs, trans_b=True, use_2dblock_b=b_2d, output_dtype=torch.bfloat16, out_scale=16.0 / 9.0)
    assert packed_gemm_supported(M, N, K)
    got = gemm_packed(aq, pack_scales(as_, M, K), bq, pack_scales(bs, N, K, b_2d), out_scale=16.0 / 9.0)
    assert torch.equal(got, want)
    ref = O.gemm_ref(aq.cpu(), as_.cpu(), bq.cpu(), bs.cpu(), use_2dblock_b=b_2d, trans_b=True) * (16.0 / 9.0)
    assert O.rel_frobenius(got.float().cpu(), ref) < 4e-3


def test_packed_gemm_rejects_what_the_tile_kernel_does_not_serve(m):
    from alto_amd.mxfp4.linear import gemm_packed, pack_scales, packed_gemm_supported
    M, N, K = 64, 64, 256
    assert not packed_gemm_supported(M, N, K)
    a = torch.zeros(M, K, dtype=torch.bfloat16, device=DEV)
    aq, as_ = m.convert_to_mxfp4(a)
    with pytest.raises(RuntimeError, match="not served by the tile kernel"):
        gemm_packed(aq, pack_scales(as_, M, K), aq, pack_scales(as_, N, K))


@pytest.mark.parametrize("N,K", [(768, 1280), (800, 608), (512, 2880), (264, 512)])
@pytest.mark.parametrize("sorted_form", [True, False])
def test_grouped_gemm_with_packed_scales_equals_the_plain_call(m, N, K, sorted_form):
    from alto_amd.mxfp4 import grouped_gemm as G
    from alto_amd.mxfp4.linear import pack_scales
    if N % 32:
        pytest.skip("2D weight blocks need N % 32 == 0")
    E, M = 5, 1536
    if sorted_form:
        ends = torch.tensor([200, 200, 777, 1300, 1500]).to(torch.int32)
        groups = G.groups_from_offsets(G.offsets_from_ends(ends.to(DEV)))
    else:
        idx = torch.randint(0, E, (M // 128,), generator=torch.Generator().manual_seed(3), dtype=torch.int32).repeat_interleave(128)
        groups = G.groups_from_indices(idx.to(DEV))
    a = randn_outliers((M, K), torch.bfloat16, seed=31).to(DEV)
    w = (randn_outliers((E, N, K), torch.bfloat16, seed=32) * 0.05).to(DEV)
    aq, as_ = m.convert_to_mxfp4(a)
    wq, ws = m.convert_to_mxfp4(w, is_2d_block=True)
    want = G.grouped_forward(aq, as_, wq, ws, groups, False, True, torch.bfloat16)
    a_ps, w_ps = pack_scales(as_, M, K), G.pack_expert_scales(ws, N, K, True)
    got, plan = G.grouped_forward_packed(aq, a_ps, wq, w_ps, groups, return_plan=True)
    assert torch.equal(got, want)
    again = G.grouped_forward_packed(aq, a_ps, wq, w_ps, groups, plan=plan)
    assert torch.equal(again, want)
