"""The weight-wrapper tensor routes linear-like ops and torch._grouped_mm to the MXFP4 path
(alto/kernels/dispatch/tensor.py:214-303): results and gradients equal the direct calls."""
import pytest
import torch

import oracle as O
from tests.helpers import rand_bits, randn_outliers

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def m():
    import alto_amd.mxfp4 as mod
    return mod


def _fixed_randomness(m, shape_seed):
    m.HadamardFactory.configure(seed=1234)
    m.set_rand_bits_source(lambda shp, d: rand_bits(tuple(shp), seed=shape_seed).to(d))


def test_linear_module_through_wrapper(m):
    cfg = m.TrainingOpConfig()   # production recipe: 1D x, 2D w, Hadamard, stochastic gradient rounding
    lin = torch.nn.Linear(256, 384, bias=True, dtype=torch.bfloat16, device=DEV)
    with torch.no_grad():
        lin.weight.copy_(randn_outliers((384, 256), torch.bfloat16, seed=1).to(DEV) * 0.02)
    w_plain = lin.weight.detach().clone().requires_grad_(True)
    x = randn_outliers((4, 64, 256), torch.bfloat16, seed=2).to(DEV)
    go = randn_outliers((4, 64, 384), torch.bfloat16, seed=3).to(DEV) / 1000
    try:
        _fixed_randomness(m, 7)
        x1 = x.clone().requires_grad_(True)
        y_ref = m._to_mxfp4_then_scaled_mm(x1, w_plain, cfg.use_2dblock_x, cfg.use_2dblock_w, cfg.use_sr_grad, cfg.use_dge,
                                           cfg.clip_mode, cfg.use_hadamard) + lin.bias
        y_ref.backward(go)
        m.swap_params(lin, config=cfg)
        assert isinstance(lin.weight.data, m.MXFP4TrainingWeightWrapperTensor)
        _fixed_randomness(m, 7)
        x2 = x.clone().requires_grad_(True)
        y = lin(x2)
        y.backward(go)
    finally:
        m.set_rand_bits_source(None)
    assert type(y) is torch.Tensor
    assert torch.equal(y, y_ref)
    assert torch.equal(x2.grad, x1.grad)
    assert lin.weight.grad is not None and torch.equal(lin.weight.grad, w_plain.grad)
    assert lin.bias.grad is not None


def test_mm_with_wrapped_second_operand(m):
    cfg = m.TrainingOpConfig(use_hadamard=False, use_sr_grad=False)
    w = (randn_outliers((256, 128), torch.bfloat16, seed=4) * 0.02).to(DEV)      # [K, N]: mm(x, w)
    x = randn_outliers((96, 256), torch.bfloat16, seed=5).to(DEV)
    ww = m.MXFP4TrainingWeightWrapperTensor(w, cfg)
    y = torch.mm(x, ww)
    y_ref = m._to_mxfp4_then_scaled_mm(x, w.T, False, True, False, False, "none", False)
    assert torch.equal(y, y_ref)
    y2 = torch.addmm(torch.ones(128, dtype=torch.bfloat16, device=DEV), x, ww)
    assert torch.equal(y2, y_ref + 1)


def test_grouped_mm_through_wrapper(m):
    cfg = m.TrainingOpConfig(use_hadamard=False, use_sr_grad=False)
    E, K, N = 4, 256, 384
    w = (randn_outliers((E, K, N), torch.bfloat16, seed=6) * 0.02).to(DEV)       # torch._grouped_mm layout [E, K, N]
    a = randn_outliers((512, K), torch.bfloat16, seed=7).to(DEV)
    offs = torch.tensor([128, 128, 384, 512], dtype=torch.int32, device=DEV)
    wp = torch.nn.Parameter(m.MXFP4TrainingWeightWrapperTensor(w.clone(), cfg))
    a1 = a.clone().requires_grad_(True)
    y = torch._grouped_mm(a1, wp, offs=offs)
    y.float().square().mean().backward()
    w2 = w.clone().requires_grad_(True)
    a2 = a.clone().requires_grad_(True)
    y_ref = m._quantize_then_mxfp_scaled_grouped_mm(a2, w2, offs, False, True, False, False, False, "none", False)
    y_ref.float().square().mean().backward()
    assert torch.equal(y, y_ref)
    assert torch.equal(a1.grad, a2.grad)
    assert torch.equal(wp.grad, w2.grad)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("is_2d", [True, False])
@pytest.mark.parametrize("use_uos", [False, True])
def test_fused_qdq_equals_quantize_then_dequantize(m, dtype, is_2d, use_uos):
    """One launch == the oracle's dequantize(quantize(w)) bit for bit (the de-oscillation hook, optimizer.py:123-168), and
    therefore also the two separate HIP launches."""
    w_cpu = randn_outliers((3, 96, 320), dtype, seed=11) * 0.02
    w = w_cpu.to(DEV)
    bits = torch.int16 if dtype == torch.bfloat16 else torch.int32
    for axis in (-1, -2):
        exp = O.dequantize(*O.quantize(w_cpu, axis=axis, is_2d_block=is_2d, use_uos=use_uos), dtype, axis=axis, is_2d_block=is_2d)
        got = m.quantize_dequantize(w, axis=axis, is_2d_block=is_2d, use_uos=use_uos)
        assert got.dtype == dtype and got.shape == w.shape
        assert torch.equal(got.cpu().view(bits), exp.contiguous().view(bits)), (axis, is_2d)
        q, s = m.convert_to_mxfp4(w, axis=axis, is_2d_block=is_2d, use_uos=use_uos)
        ref = m.convert_from_mxfp4(q, s, output_dtype=dtype, axis=axis, is_2d_block=is_2d)
        assert torch.equal(got.view(bits), ref.contiguous().view(bits)), (axis, is_2d)
    # the recipe-level closure, with a row count that is not a multiple of 32 (padded as the reference does)
    cfg = m.TrainingOpConfig(use_2dblock_w=is_2d, use_uos=use_uos)
    w2_cpu = randn_outliers((100, 256), dtype, seed=12) * 0.02
    got = m._make_qdq_fn_for(cfg)(w2_cpu.to(DEV), -1)
    wp = torch.nn.functional.pad(w2_cpu, (0, 0, 0, 28))
    exp = O.dequantize(*O.quantize(wp, axis=-1, is_2d_block=is_2d, use_uos=use_uos), dtype, axis=-1, is_2d_block=is_2d)[:100]
    assert got.shape == (100, 256) and torch.equal(got.cpu(), exp)


@pytest.mark.parametrize("as_parameter", [False, True])
def test_weight_cache_reuses_until_weight_changes(m, as_parameter):
    x = randn_outliers((64, 256), torch.bfloat16, seed=13).to(DEV)
    w = (randn_outliers((128, 256), torch.bfloat16, seed=14) * 0.02).to(DEV).requires_grad_(True)
    if as_parameter:   # what a module holds: the kernels see a fresh plain-tensor alias of it in every forward
        w = torch.nn.Parameter(w.detach())
    args = (False, True, False, False, "none", False)
    y0 = m._to_mxfp4_then_scaled_mm(x, w, *args)
    m.enable_weight_cache(True)
    try:
        y1 = m._to_mxfp4_then_scaled_mm(x, w, *args)
        y2 = m._to_mxfp4_then_scaled_mm(x, w, *args)
        assert m.weight_cache_stats() == {"hits": 1, "misses": 1, "entries": 1}
        assert torch.equal(y1, y0) and torch.equal(y2, y0)
        y2.float().sum().backward()          # backward of a cached forward still works
        assert w.grad is not None
        with torch.no_grad():
            w.mul_(2.0)                       # an optimizer-style in-place update invalidates the entry
        y3 = m._to_mxfp4_then_scaled_mm(x, w, *args)
        assert m.weight_cache_stats()["misses"] == 2
        m.enable_weight_cache(False)
        assert torch.equal(y3, m._to_mxfp4_then_scaled_mm(x, w, *args))
    finally:
        m.enable_weight_cache(False)


@pytest.mark.parametrize("clip_mode", ["none", "static"])
def test_dge_scales_the_weight_gradient(m, clip_mode):
    """use_dge multiplies dW by dge_bwd at the quantised weight's grid values (mxfp_linear.py:549-568), which is the
    constant fp32(1/5) on the E2M1 grid; dX and the forward result are untouched.  fp32 tensors: the reference's
    searchsorted needs the fp32 dtype of its break points."""
    x = randn_outliers((128, 256), torch.float32, seed=11).to(DEV)
    w = (randn_outliers((192, 256), torch.float32, seed=12) * 0.02).to(DEV)
    go = randn_outliers((128, 192), torch.float32, seed=13).to(DEV) / 1000
    grads = {}
    for dge in (False, True):
        xi, wi = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
        y = m._to_mxfp4_then_scaled_mm(xi, wi, False, True, False, dge, clip_mode, False)
        y.backward(go)
        grads[dge] = (y.detach(), xi.grad, wi.grad)
    assert torch.equal(grads[True][0], grads[False][0])
    assert torch.equal(grads[True][1], grads[False][1])
    f = torch.tensor(0.2, dtype=torch.float32)
    # one rounding in the GEMM epilogue (acc * (16/9 * 0.2)) versus the reference's two: within a few fp32 ulps
    torch.testing.assert_close(grads[True][2], grads[False][2] * f, rtol=4e-7, atol=0)
    assert grads[False][2].abs().max() > 0
    # against the oracle: its dW times dge_bwd evaluated element by element at the quantised weight's grid values
    xc, wc, gc = x.cpu(), w.cpu(), go.cpu()
    _, saved = O.linear_forward_ref(xc, wc, False, True, clip_mode=clip_mode)
    _, dw_ref = O.linear_backward_ref(gc, saved, False, True, clip_mode=clip_mode)
    wq, _ = O.quantize(wc, is_2d_block=True)
    factor = O.dge_bwd_ref(O.weight_grid_values(wq))
    assert factor.shape == wc.shape and float((factor - 0.2).abs().max()) < 1e-6
    assert O.rel_frobenius(grads[True][2].cpu(), dw_ref * factor.double()) < 1e-5


def test_dge_grouped_weight_gradient(m):
    E, N, K, M = 2, 128, 256, 256
    x = randn_outliers((M, K), torch.float32, seed=21).to(DEV)
    w = (randn_outliers((E, N, K), torch.float32, seed=22) * 0.02).to(DEV)
    go = randn_outliers((M, N), torch.float32, seed=23).to(DEV) / 1000
    idx = torch.arange(M, device=DEV, dtype=torch.int32) // 128
    grads = {}
    for dge in (False, True):
        xi, wi = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
        y = m.mxfp4_grouped_gemm(xi, wi, idx, use_dge=dge)
        y.backward(go)
        grads[dge] = (xi.grad, wi.grad)
    assert torch.equal(grads[True][0], grads[False][0])
    torch.testing.assert_close(grads[True][1], grads[False][1] * 0.2, rtol=4e-7, atol=0)
    assert grads[False][1].abs().max() > 0
    # against the oracle's flow times dge_bwd at the grid values of the quantised expert weights
    xc, wc, gc, ic = x.cpu(), w.cpu(), go.cpu(), idx.cpu()
    gqm, gsm = O.quantize(gc, axis=0)
    aqm, asm = O.quantize(xc, axis=0)
    dw_ref = O.grouped_gemm_dw_ref(gqm, gsm, aqm, asm, ic, E)
    wq, _ = O.quantize(wc, is_2d_block=True)
    assert O.rel_frobenius(grads[True][1].cpu(), dw_ref * O.dge_bwd_ref(O.weight_grid_values(wq)).double()) < 1e-5


def test_registered_torch_ops_run_the_hip_kernels(m):
    """torch.ops.<ns>.* (the reference registers these names as torchtitan::*) give the direct functions' results."""
    ns = m.register_torch_ops("alto_amd_test")
    x = randn_outliers((128, 256), torch.bfloat16, seed=51).to(DEV)
    w = (randn_outliers((192, 256), torch.bfloat16, seed=52) * 0.02).to(DEV)
    xq, xs = ns.convert_to_mxfp4(x)
    xq2, xs2 = m.convert_to_mxfp4(x)
    assert torch.equal(xq, xq2) and torch.equal(xs, xs2)
    cq, cs = ns.convert_to_mxfp4(x, 32, 0, False)
    cq2, cs2 = m.convert_to_mxfp4(x, axis=0)
    assert cq.shape == cq2.shape and cq.stride() == cq2.stride() and torch.equal(cq, cq2) and torch.equal(cs, cs2)
    wq, ws = ns.convert_to_mxfp4(w, 32, -1, True)
    assert torch.equal(ns.convert_from_mxfp4(wq, ws, torch.bfloat16, 32, -1, True), m.convert_from_mxfp4(wq, ws, torch.bfloat16, is_2d_block=True))
    y = ns.blockwise_mxfp4_gemm(xq, xs, wq, ws, False, True, True, True, False, True, 32, torch.bfloat16)
    assert torch.equal(y, m.blockwise_mxfp4_gemm(xq, xs, wq, ws, use_2dblock_b=True, trans_b=True, output_dtype=torch.bfloat16))
    # grouped: 2 experts x 128 rows
    idx = (torch.arange(256, device=DEV, dtype=torch.int32) // 128)
    a = randn_outliers((256, 256), torch.bfloat16, seed=53).to(DEV)
    ew = (randn_outliers((2, 192, 256), torch.bfloat16, seed=54) * 0.02).to(DEV)
    aq, as_ = m.convert_to_mxfp4(a)
    ewq, ews = m.convert_to_mxfp4(ew, is_2d_block=True)
    out = ns.mxfp4_grouped_gemm_forward(aq, ewq, idx, as_, ews)
    assert torch.equal(out, m.mxfp4_grouped_gemm_forward(aq, ewq, idx, as_, ews))
    go = randn_outliers((256, 192), torch.bfloat16, seed=55).to(DEV) / 1000
    gq, gs = m.convert_to_mxfp4(go)
    wnq, wns = m.convert_to_mxfp4(ew, axis=-2, is_2d_block=True)               # packed along N: [E, N/2, K]
    dx = ns.mxfp4_grouped_gemm_backward_inputs(gq, wnq, idx, gs, wns)
    assert torch.equal(dx, m.mxfp4_grouped_gemm_backward_inputs(gq, wnq, idx, gs, wns)) and dx.shape == (256, 256)
    gqm, gsm = m.convert_to_mxfp4(go, axis=0)
    aqm, asm_ = m.convert_to_mxfp4(a, axis=0)
    dw = ns.mxfp4_grouped_gemm_backward_weights(gqm, aqm, idx, 2, gsm, asm_, True, False, False)
    assert torch.equal(dw, m.mxfp4_grouped_gemm_backward_weights(gqm, aqm, idx, 2, gsm, asm_, use_2dblock_x=False)) and dw.shape == (2, 192, 256)


def test_forward_replays_from_a_hip_graph(m):
    """Quantizer and GEMM launches allocate nothing and sync nothing, so a linear forward can be captured once and
    replayed; every replay (with eager work and synchronisations between them) equals the eager result."""
    x = randn_outliers((256, 512), torch.bfloat16, seed=61).to(DEV)
    w = (randn_outliers((384, 512), torch.bfloat16, seed=62) * 0.02).to(DEV)
    eager = m._to_mxfp4_then_scaled_mm(x, w, False, True, False, False, "none", False)
    torch.cuda.synchronize()
    static_x = x.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):            # warm-up on the capture stream (one-time per-kernel set-up happens here)
        m._to_mxfp4_then_scaled_mm(static_x, w, False, True, False, False, "none", False)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        static_y = m._to_mxfp4_then_scaled_mm(static_x, w, False, True, False, False, "none", False)
    for i in range(3):
        static_x.copy_(x if i != 1 else x * 2)
        g.replay()
        torch.cuda.synchronize()
        ref = eager if i != 1 else m._to_mxfp4_then_scaled_mm(x * 2, w, False, True, False, False, "none", False)
        assert torch.equal(static_y, ref), f"replay {i}"
        (x.float() @ w.float().T).sum().item()   # unrelated eager work and a host sync between replays


def test_captured_stochastic_rounding_draws_fresh_words_on_every_replay(m, software_sr):
    """With the device-resident Philox state nothing about the random words is a kernel argument: a captured SR
    quantizer (fused row + column copies with the Hadamard transform) draws new words on every replay, and every replay
    equals the eager call keyed with the (key, counter) the state held before it."""
    import alto_amd.mxfp4._runtime as rt
    x = randn_outliers((128, 512), torch.bfloat16, seed=63).to(DEV)
    from tests.helpers import hadamard_from_seed
    had = m.HadamardTransform(*hadamard_from_seed(5))
    rt.enable_device_philox_state(True, seed=1234)
    try:
        state = rt.philox_device_state(x.device)
        assert state.tolist() == [1234, 0]
        static_x = x.clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):   # warm-up on the capture stream; it also moves the counter on
            m.quantize_rowcol(static_x, False, True, hadamard=had)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        words = x.numel()
        assert state.tolist() == [1234, (words + 3) // 4]
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            outs = m.quantize_rowcol(static_x, False, True, hadamard=had)
        seen = []
        for i in range(3):
            key, counter = state.tolist()
            assert counter == (i + 1) * ((words + 3) // 4)
            g.replay()
            torch.cuda.synchronize()
            got = [o.clone() for o in outs]
            bits = rt.draw_rand_bits(x.shape, x.device, key, counter)   # eager twin: the same words as a tensor
            want = m.quantize_rowcol(x, False, True, hadamard=had, rand_bits=bits)
            for a, b in zip(got, want):
                assert torch.equal(a, b), f"replay {i}"
            seen.append(got[0])
            (x.float() @ x.float().T).sum().item()
        assert not torch.equal(seen[0], seen[1]) and not torch.equal(seen[1], seen[2])
    finally:
        rt.enable_device_philox_state(False)
