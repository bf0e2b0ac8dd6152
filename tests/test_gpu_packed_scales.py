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


@pytest.mark.parametrize("M,C", [(512, 512), (96, 1056), (1056, 2880), (544, 32)])
@pytest.mark.parametrize("mode", ["rne", "sr_hw"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_quantizer_writes_packed_scales_of_2d_blocks(m, M, C, mode, dtype):
    """2D blocks (the weight): both packings' scales, packed, repeat a block's scale for its 32 rows."""
    from alto_amd.mxfp4.linear import pack_scales
    from alto_amd.mxfp4.quantization import _prep, _quantize_call
    x3 = _prep(randn_outliers((M, C), dtype, seed=M * 3 + C).to(DEV))
    kw = dict(use_sr=mode != "rne", rand3=None, hadamard=None, clip=0, use_uos=False, philox=(9, 8) if mode == "sr_hw" else None, hw_sr=mode == "sr_hw")
    rc, rs, cc, cs = _quantize_call(x3, True, True, True, **kw)
    for pr, pc in [(True, True), (True, False), (False, True)]:
        rc2, rs2, cc2, cs2 = _quantize_call(x3, True, True, True, pack_row_scales=pr, pack_col_scales=pc, **kw)
        assert_bytes_equal(rc2.cpu(), rc.cpu(), "row codes")
        assert_bytes_equal(cc2.cpu(), cc.cpu(), "column codes")
        assert_bytes_equal(rs2[0].cpu(), (pack_scales(rs[0], M, C, True) if pr else rs[0]).cpu(), "row scales")
        assert_bytes_equal(cs2[0].cpu(), (pack_scales(cs[0], C, M, True) if pc else cs[0]).cpu(), "column scales")
    rc3, rs3, _, _ = _quantize_call(x3, True, False, True, pack_row_scales=True, **kw)
    assert_bytes_equal(rc3.cpu(), rc.cpu(), "row codes alone")
    assert_bytes_equal(rs3[0].cpu(), pack_scales(rs[0], M, C, True).cpu(), "row scales alone")
    _, _, cc4, cs4 = _quantize_call(x3, False, True, True, pack_col_scales=True, **kw)
    assert_bytes_equal(cc4.cpu(), cc.cpu(), "column codes alone")
    assert_bytes_equal(cs4[0].cpu(), pack_scales(cs[0], C, M, True).cpu(), "column scales alone")


def test_packed_flags_are_rejected_where_they_do_not_apply(m):
    x = torch.randn(64, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="packed scales"):
        m.quantize_rowcol(x, clip_mode="dynamic", pack_col_scales=True)


def _count_calls(monkeypatch, module, name):
    calls = []
    real = getattr(module, name)

    def spy(*a, **k):
        calls.append(1)
        return real(*a, **k)
    monkeypatch.setattr(module, name, spy)
    return calls


@pytest.mark.parametrize("M,N,K,expect", [(512, 768, 1024, 3), (1056, 512, 2880, 3), (256, 160, 544, 1), (96, 256, 512, 0), (256, 64, 512, 0),
                                          (128, 512, 160, 1), (512, 544, 512, 3)])
@pytest.mark.parametrize("w2d", [True, False])
@pytest.mark.parametrize("mode", ["rne", "sr", "sr_hw", "static_clip"])
def test_linear_autograd_is_the_same_on_packed_scales(m, monkeypatch, M, N, K, expect, w2d, mode):
    """y, dx and dw of the linear function with packed scales switched on equal those with the switch off, bit for bit, and
    the packed GEMM serves exactly the GEMMs whose shape the tile kernel takes."""
    from alto_amd.mxfp4 import linear as L
    assert expect == sum(L.packed_gemm_supported(*s) for s in ((M, N, K), (M, K, N), (N, K, M)))
    x = randn_outliers((M, K), torch.bfloat16, seed=5).to(DEV)
    w = randn_outliers((N, K), torch.bfloat16, seed=6).to(DEV)
    go = (randn_outliers((M, N), torch.bfloat16, seed=7) / (M * N)).to(DEV)
    h = m.HadamardTransform(*hadamard_from_seed(11))
    calls = _count_calls(monkeypatch, L, "gemm_packed")
    res = []
    m.use_hardware_stochastic_rounding(mode == "sr_hw")
    try:
        for on in (True, False):
            L.use_packed_scales(on)
            torch.manual_seed(99)   # the Philox key of the backward quantizer
            xg, wg = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
            y = m.MXFP4LinearFunction.apply(xg, wg, False, w2d, mode.startswith("sr"), False, "static" if mode == "static_clip" else "none", False, h, False)
            y.backward(go)
            res.append((y.detach(), xg.grad, wg.grad))
            if on:
                assert len(calls) == expect
    finally:
        L.use_packed_scales(True)
        m.use_hardware_stochastic_rounding(True)
    assert len(calls) == expect
    for got, want, what in zip(res[0], res[1], ("y", "dx", "dw")):
        assert torch.equal(got, want), what


@pytest.mark.parametrize("N,K", [(768, 1280), (512, 2880), (288, 512), (128, 96)])
@pytest.mark.parametrize("x2d,w2d", [(False, True), (False, False), (True, True)])
@pytest.mark.parametrize("trans_weights", [True, False])
def test_grouped_autograd_is_the_same_on_packed_scales(m, monkeypatch, N, K, x2d, w2d, trans_weights):
    from alto_amd.mxfp4 import grouped_gemm as G
    from alto_amd.mxfp4 import linear as L
    E, Mt = 4, 1024
    a = randn_outliers((Mt, K), torch.bfloat16, seed=31).to(DEV)
    wts = randn_outliers((E, N, K) if trans_weights else (E, K, N), torch.bfloat16, seed=32).to(DEV)
    idx = torch.randint(0, E, (Mt // 128,), generator=torch.Generator().manual_seed(33), dtype=torch.int32).repeat_interleave(128).to(DEV)
    go = (randn_outliers((Mt, N), torch.bfloat16, seed=34) / (Mt * N)).to(DEV)
    calls = _count_calls(monkeypatch, G, "grouped_forward_packed")
    dw_calls = _count_calls(monkeypatch, G, "grouped_dw_packed")
    expect = int(G.grouped_packed_supported(Mt, N, K, E)) + int(G.grouped_packed_supported(Mt, K, N, E))
    expect_dw = int(G.grouped_dw_packed_supported(Mt, N, K, G.groups_from_indices(idx).n, E))
    res = []
    try:
        for on in (True, False):
            L.use_packed_scales(on)
            torch.manual_seed(99)
            m.HadamardFactory.configure(seed=1234)
            ag, wg = a.clone().requires_grad_(True), wts.clone().requires_grad_(True)
            out = m.mxfp4_grouped_gemm(ag, wg, idx, trans_weights=trans_weights, use_2dblock_x=x2d, use_2dblock_w=w2d, use_sr_grad=True, use_hadamard=not x2d)
            out.backward(go)
            res.append((out.detach(), ag.grad, wg.grad))
            if on:
                assert len(calls) == expect and len(dw_calls) == expect_dw
    finally:
        L.use_packed_scales(True)
    assert len(calls) == expect and len(dw_calls) == expect_dw
    for got, want, what in zip(res[0], res[1], ("out", "dx", "dw")):
        assert torch.equal(got, want), what


@pytest.mark.parametrize("N,K", [(256, 384), (512, 2880), (288, 160)])
@pytest.mark.parametrize("layout", ["sorted", "per_group", "ragged32"])
@pytest.mark.parametrize("trans_weights,is_2d", [(True, False), (False, False), (True, True)])
def test_grouped_dw_with_packed_scales_equals_the_plain_call(m, N, K, layout, trans_weights, is_2d):
    """Token-packed scales ([M/512][rows][16]): runs that start in the first and in the second half of a packed block, at
    128- and 32-token boundaries, empty experts, runs of one expert in several places; NaN poisoning of a split MX block
    included (same bits as the plain call everywhere)."""
    from alto_amd.mxfp4 import grouped_gemm as G
    from alto_amd.mxfp4.linear import pack_scales
    E = 6
    if layout == "sorted":      # 128-token boundaries, some in the second half of a 512 block, one empty expert
        offs = torch.tensor([0, 384, 384, 1280, 1408, 2304, 2560], dtype=torch.int32)
        groups = G.groups_from_offsets(offs.to(DEV))
    elif layout == "per_group":  # the reference's contract: one expert id per 128 rows, unsorted
        idx = torch.randint(0, E, (2560 // 128,), generator=torch.Generator().manual_seed(5), dtype=torch.int32).repeat_interleave(128)
        groups = G.groups_from_indices(idx.to(DEV))
    else:                        # boundaries at multiples of 32 only, one of them splitting a block (poisoned)
        offs = torch.tensor([0, 96, 800, 832, 1999, 2528, 2560], dtype=torch.int32)
        groups = G.groups_from_offsets(offs.to(DEV))
    Mt = 2560
    go = (randn_outliers((Mt, N), torch.bfloat16, seed=3) / 64).to(DEV)
    x = randn_outliers((Mt, K), torch.bfloat16, seed=4).to(DEV)
    h = None if is_2d else m.HadamardTransform(*hadamard_from_seed(8))
    _, _, gqm, gsm = m.quantize_rowcol(go, is_2d, hadamard=h, pad_codes=True)
    _, _, xqm, xsm = m.quantize_rowcol(x, is_2d, hadamard=h, pad_codes=True)
    _, _, gqm2, gps = m.quantize_rowcol(go, is_2d, hadamard=h, pad_codes=True, pack_col_scales=True)
    _, _, xqm2, xps = m.quantize_rowcol(x, is_2d, hadamard=h, pad_codes=True, pack_col_scales=True)
    assert_bytes_equal(gps.cpu(), pack_scales(gsm.transpose(0, 1), N, Mt, is_2d).cpu(), "dY scales packed along the tokens")
    assert G.grouped_dw_packed_supported(Mt, N, K, groups.n, E)
    want = G.grouped_dw(gqm.transpose(0, 1), gsm.transpose(0, 1), xqm.transpose(0, 1), xsm.transpose(0, 1), groups, E, torch.bfloat16, trans_weights, 16.0 / 9.0,
                        is_2d=is_2d)
    got = G.grouped_dw_packed(gqm2.transpose(0, 1), gps, xqm2.transpose(0, 1), xps, groups, E, trans_weights, 16.0 / 9.0)
    assert got.shape == want.shape
    assert torch.equal(torch.isnan(got), torch.isnan(want))
    if layout == "ragged32":
        assert bool(torch.isnan(want[3]).all()) and bool(torch.isnan(want[4]).all())
    assert torch.equal(torch.nan_to_num(got), torch.nan_to_num(want))


def test_packed_dw_rejects_what_the_tile_kernel_does_not_serve(m):
    from alto_amd.mxfp4 import grouped_gemm as G
    Mt, N, K, E = 256, 64, 64, 2
    assert not G.grouped_dw_packed_supported(Mt, N, K, E, E)
    z = torch.zeros(Mt, N, dtype=torch.bfloat16, device=DEV)
    _, _, q, ps = m.quantize_rowcol(z, False, pad_codes=True, pack_col_scales=True)
    groups = G.groups_from_offsets(torch.tensor([0, 128, 256], dtype=torch.int32, device=DEV))
    with pytest.raises(NotImplementedError, match="not served by the tile kernel"):
        G.grouped_dw_packed(q.transpose(0, 1), ps, q.transpose(0, 1), ps, groups, E)


def test_expert_weights_take_the_band_loop_and_keep_their_bytes(m):
    """A batch of 2D-block matrices large enough for workgroups of eight bands (whole-line column-code stores): same four
    outputs as matrix-by-matrix calls, which are below the size where that path is taken; M with a partial last group."""
    from alto_amd.mxfp4.quantization import _prep, _quantize_call
    E, R, C = 40, 1056, 5760          # 33 bands: groups of 8 + 1; 23 column tiles x 5 rows of bands x 40 >= 4096 workgroups
    w = (randn_outliers((E, R, C), torch.bfloat16, seed=12) * 0.02).to(DEV)
    kw = dict(use_sr=False, rand3=None, hadamard=None, clip=0, use_uos=False, pad_codes=True)
    big = _quantize_call(_prep(w), True, True, True, **kw)
    for e in (0, 17, E - 1):
        one = _quantize_call(_prep(w[e:e + 1]), True, True, True, **kw)
        for a, b_, what in zip(big, one, ("row codes", "row scales", "column codes", "column scales")):
            assert_bytes_equal(a[e:e + 1].cpu(), b_.cpu(), f"expert {e}: {what}")
