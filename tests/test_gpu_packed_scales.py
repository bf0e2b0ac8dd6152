"""Packed (GEMM-ready) scale layout: the converter against its definition, and the kernels that read it against the ones
that read plain scales, bit for bit."""
import numpy as np
import pytest
import torch

import oracle as O
from tests.helpers import assert_bytes_equal, hadamard_from_seed, randn_outliers

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


@pytest.mark.parametrize("M,C", [(512, 512), (96, 1056), (1024, 2880), (544, 32), (32, 4096)])
@pytest.mark.parametrize("mode", ["rne", "sr_words", "sr_philox", "sr_hw"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_quantizer_writes_the_packed_scales_itself(m, M, C, mode, dtype):
    """Codes and scales of the call with the layout flags equal those of the plain call, the scales after
    ``pack_scales``: every rounding mode, with the Hadamard transform, static clip and K tails of both outputs."""
    from alto_amd.mxfp4.linear import pack_scales
    from alto_amd.mxfp4.quantization import _prep, _quantize_call
    x = randn_outliers((M, C), dtype, seed=M + C).to(DEV)
    h = m.HadamardTransform(*hadamard_from_seed(77))
    rand = torch.randint(-2 ** 31, 2 ** 31 - 1, (1, M, C), dtype=torch.int32, generator=torch.Generator().manual_seed(3)).to(DEV)
    kw = dict(use_sr=mode != "rne", rand3=rand if mode == "sr_words" else None, hadamard=h, clip=1, use_uos=False,
              philox=(1234, 5678) if mode in ("sr_philox", "sr_hw") else None, hw_sr=mode == "sr_hw")
    x3 = _prep(x)
    rc, rs, cc, cs = _quantize_call(x3, True, True, False, **kw)
    for pr, pc in [(True, True), (True, False), (False, True)]:
        rc2, rs2, cc2, cs2 = _quantize_call(x3, True, True, False, pack_row_scales=pr, pack_col_scales=pc, **kw)
        assert_bytes_equal(rc2.cpu(), rc.cpu(), "row codes")
        assert_bytes_equal(cc2.cpu(), cc.cpu(), "column codes")
        assert_bytes_equal(rs2[0].cpu(), (pack_scales(rs[0], M, C) if pr else rs[0]).cpu(), "row scales")
        assert_bytes_equal(cs2[0].cpu(), (pack_scales(cs[0], C, M) if pc else cs[0]).cpu(), "column scales")
    # one output only
    rc3, rs3, _, _ = _quantize_call(x3, True, False, False, pack_row_scales=True, **{**kw, "hadamard": None, "clip": 0})
    rc4, rs4, _, _ = _quantize_call(x3, True, False, False, **{**kw, "hadamard": None, "clip": 0})
    assert_bytes_equal(rc3.cpu(), rc4.cpu(), "row codes alone")
    assert_bytes_equal(rs3[0].cpu(), pack_scales(rs4[0], M, C).cpu(), "row scales alone")


def test_quantize_rowcol_packed_feeds_the_packed_gemm(m):
    from alto_amd.mxfp4.linear import gemm_packed
    M, N, K = 384, 256, 1056
    a = randn_outliers((M, K), torch.bfloat16, seed=1).to(DEV)
    b = randn_outliers((N, K), torch.bfloat16, seed=2).to(DEV)
    aq, as_, _, _ = m.quantize_rowcol(a)
    bq, bs, _, _ = m.quantize_rowcol(b)
    aq2, aps, _, _ = m.quantize_rowcol(a, pack_row_scales=True)
    bq2, bps, _, _ = m.quantize_rowcol(b, pack_row_scales=True)
    want = m.blockwise_mxfp4_gemm(aq, as_, bq, bs, trans_b=True, output_dtype=torch.bfloat16)
    assert torch.equal(gemm_packed(aq2, aps, bq2, bps), want)


def test_packed_flags_are_rejected_where_they_do_not_apply(m):
    x = torch.randn(64, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="packed scales"):
        m.quantize_rowcol(x, is_2d_block=True, pack_row_scales=True)
    with pytest.raises(RuntimeError, match="packed scales"):
        m.quantize_rowcol(x, clip_mode="dynamic", pack_col_scales=True)
