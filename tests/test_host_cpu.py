"""CPU-side checks: the C-ABI library builds, loads and exports what the header declares; host logic without a GPU."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "alto_mxfp4.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(alto_mxfp4_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from alto_amd import _lib
    lib = _lib.load()
    names = header_symbols()
    assert "alto_mxfp4_quantize" in names and "alto_mxfp4_gemm" in names and len(names) >= 9
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/alto_mxfp4.h but not exported"
    assert set(names) == set(_lib.SIGNATURES), "ctypes signature table and header disagree"
    assert lib.alto_mxfp4_version() >= 1


def test_argument_validation_needs_no_gpu():
    from alto_amd import _lib
    lib = _lib.load()
    # NULL input is rejected before any HIP call
    rc = lib.alto_mxfp4_quantize(None, 0, 1, 32, 32, 32, 1024, None, None, None, None, 0, 0, None, 0, 0, 0, None, None, 0, 0, None)
    assert rc == -1 and b"NULL" in lib.alto_mxfp4_last_error()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    p += (-p) % 16
    rc = lib.alto_mxfp4_quantize(p, 0, 1, 32, 40, 40, 1280, p, p, None, None, 0, 0, None, 0, 0, 0, None, None, 0, 0, None)
    assert rc == -1 and b"C (40)" in lib.alto_mxfp4_last_error()
    rc = lib.alto_mxfp4_quantize(p, 0, 1, 32, 32, 32, 1024, p, p, p, p, 0, 0, None, 0, 0, 0, None, None, 2, 0, None)
    assert rc == -1 and b"row output only" in lib.alto_mxfp4_last_error()   # dynamic clip quantises along the contiguous dim
    rc = lib.alto_mxfp4_gemm(p, 16, p, 1, 1, 0, p, 16, p, 1, 1, 0, 32, 32, 48, p, 0, 32, 1.0, None)
    assert rc == -1 and b"K (48)" in lib.alto_mxfp4_last_error()
    bad_perm = (ctypes.c_uint8 * 32)(*([0] * 32))
    signs = (ctypes.c_int8 * 32)(*([1] * 32))
    rc = lib.alto_mxfp4_hadamard(p, 0, 32, 8, 8, p, 8, ctypes.addressof(signs), ctypes.addressof(bad_perm), None)
    assert rc == -1 and b"permutation" in lib.alto_mxfp4_last_error()


def test_argument_validation_of_the_philox_and_grouped_entry_points():
    """Rejected before any HIP call: dynamic clip with in-kernel random words, a grouped GEMM without (or with too small a)
    workspace; and the size the workspace query promises."""
    from alto_amd import _lib
    lib = _lib.load()
    buf = ctypes.create_string_buffer(1 << 16)
    p = ctypes.addressof(buf)
    p += (-p) % 16
    rc = lib.alto_mxfp4_quantize_sr_philox(p, 0, 1, 32, 32, 32, 1024, p, p, None, None, 16, 0, 0, 1, 0, None, 0, None, None, 2, 0, None)
    assert rc == -3 and b"dynamic" in lib.alto_mxfp4_last_error()
    rc = lib.alto_mxfp4_quantize_sr_philox(None, 0, 1, 32, 32, 32, 1024, p, p, None, None, 16, 0, 0, 1, 0, None, 0, None, None, 0, 0, None)
    assert rc == -1 and b"NULL" in lib.alto_mxfp4_last_error()
    M, N, K, E = 512, 256, 512, 2
    need = lib.alto_mxfp4_grouped_gemm_workspace_bytes(M, E)
    assert need == 16 + 16 * (M // 256 + E + 2)
    args = [p, K // 2, p, K // 32, 1, 0, p, N * K // 2, K // 2, p, (N // 32) * (K // 32), K // 32, 1, 1, p, None, E, E, M, N, K, p, 0, N]
    rc = lib.alto_mxfp4_grouped_gemm(*args, None, 0, None)
    assert rc == -1 and b"workspace" in lib.alto_mxfp4_last_error()
    rc = lib.alto_mxfp4_grouped_gemm(*args, p, need - 16, None)
    assert rc == -1 and b"too small" in lib.alto_mxfp4_last_error()
    rc = lib.alto_mxfp4_grouped_gemm_dw(None, 0, p, 1, 1, 0, p, 0, p, 1, 1, 0, p, None, E, E, M, N, K, p, 0, N * K, K, 1, 1.0, None)
    assert rc == -1 and b"NULL" in lib.alto_mxfp4_last_error()


def test_ops_refuse_cpu_tensors():
    import alto_amd.mxfp4 as m
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        m.convert_to_mxfp4(torch.randn(32, 32))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        m.convert_from_mxfp4(torch.zeros(32, 16, dtype=torch.uint8), torch.zeros(32, 1, dtype=torch.uint8))
    with pytest.raises(ValueError, match="Invalid clip mode"):
        m.convert_to_mxfp4(torch.randn(32, 32), clip_mode="bogus")
    with pytest.raises(RuntimeError):
        m.convert_to_mxfp4(torch.randn(32, 48))  # torch._check on the block divisibility


def test_hadamard_factory_matches_reference_draw_order():
    import oracle as O
    from alto_amd.mxfp4 import HadamardFactory
    from tests.helpers import hadamard_from_seed
    HadamardFactory.configure(seed=1234)
    t = HadamardFactory.create_transform()
    signs, perm = hadamard_from_seed(1234)
    assert torch.equal(t.signs, signs) and torch.equal(t.perm.long(), perm)
    assert torch.equal(t.weight, O.hadamard_matrix(signs, perm))
    t2 = HadamardFactory.create_transform()          # the class-level generator advances between calls
    assert not (torch.equal(t2.signs, t.signs) and torch.equal(t2.perm, t.perm))
    with pytest.raises(RuntimeError, match="MI355X only"):   # no CPU path behind the transform
        t(torch.zeros(32, 32), left_mul=False)


def test_training_op_config():
    from alto_amd.mxfp4 import TrainingOpConfig
    c = TrainingOpConfig()
    assert (c.use_2dblock_x, c.use_2dblock_w, c.use_hadamard, c.use_sr_grad, c.use_dge, c.clip_mode) == (False, True, True, True, False, "none")
    with pytest.raises(ValueError):
        TrainingOpConfig(precision="nvfp4")
    with pytest.raises(ValueError):
        TrainingOpConfig(clip_mode="x")


def test_group_helpers():
    import oracle as O
    from alto_amd.mxfp4 import grouped_gemm as G
    ends = torch.tensor([128, 128, 384, 512], dtype=torch.int32)
    idx = G.create_indices_from_offsets_nosync(ends)
    assert torch.equal(idx, O.indices_from_offsets(ends))
    g = G.groups_from_indices(idx)
    assert g.n == 4 and g.offs.tolist() == [0, 128, 256, 384, 512] and g.expert.tolist() == [0, 2, 2, 3]
    off = G.offsets_from_ends(ends)
    assert off.tolist() == [0, 128, 128, 384, 512] and G.groups_from_offsets(off).n == 4


# ----------------------------------------------------------------------------------------------- weight wrapper (CPU)
def test_weight_wrapper_passes_other_ops_through():
    """Non-GEMM ops see the plain payload; view-like ops keep the wrapper (alto/kernels/dispatch/tensor.py:33-47,101-137)."""
    import alto_amd.mxfp4 as m
    cfg = m.TrainingOpConfig()
    w = torch.randn(64, 32)
    ww = m.MXFP4TrainingWeightWrapperTensor(w, cfg)
    assert ww.shape == w.shape and ww.dtype == w.dtype and ww._data is w
    assert isinstance(ww.detach(), m.MXFP4TrainingWeightWrapperTensor)
    t = ww.t()
    assert isinstance(t, m.MXFP4TrainingWeightWrapperTensor) and t.shape == (32, 64) and t.config == cfg
    assert isinstance(ww.clone(), m.MXFP4TrainingWeightWrapperTensor)
    s = ww + 1.0
    assert type(s) is torch.Tensor and torch.equal(s, w + 1.0)
    assert torch.equal(m.linear.unwrap_weight_wrapper(ww), w)


def test_swap_params_wraps_weights_not_biases():
    import alto_amd.mxfp4 as m
    cfg = m.TrainingOpConfig()
    model = torch.nn.Sequential(torch.nn.Linear(32, 64), torch.nn.ReLU(), torch.nn.Linear(64, 32))
    m.swap_params(model, config=cfg, module_filter_fn=lambda mod, fqn: isinstance(mod, torch.nn.Linear) and fqn == "2")
    assert type(model[0].weight.data) is torch.Tensor
    assert isinstance(model[2].weight.data, m.MXFP4TrainingWeightWrapperTensor) and model[2].weight.requires_grad
    assert type(model[2].bias.data) is torch.Tensor
    with pytest.raises(ValueError):
        m.swap_params(model, config=None)


def test_dge_factor_is_one_fifth_on_the_e2m1_grid():
    """dge_bwd (alto/kernels/dge/dge.py:80-93) at a break point: |x - mid| = half_delta, so the factor is 1/k."""
    import numpy as np
    from alto_amd.mxfp4.dge import DGE_FACTOR, DGE_K, dge_bwd_e2m1_grid
    t = dge_bwd_e2m1_grid()
    assert t.shape == (16,) and t.dtype == np.float32
    assert np.float32(DGE_FACTOR) == np.float32(1.0 / DGE_K)
    assert np.all(np.abs(t - np.float32(0.2)) <= 2 * np.spacing(np.float32(0.2)))
    # an off-grid point does not give 1/k: the constant is a property of the grid, not of the formula
    bp = np.array([1.0, 1.5], dtype=np.float32)
    half, mid, x = np.float32(0.25), np.float32(1.25), np.float32(1.3)
    off = half ** np.float32(0.8) * np.abs(x - mid) ** np.float32(-0.8) / np.float32(5)
    assert abs(off - 0.2) > 0.1


def test_torch_ops_registration_and_fake_shapes():
    """The six operators exist under torch.ops with the reference's argument lists (mxfp_quantization.py:410,487,
    mxfp_linear.py:142, cg_forward.py:200, cg_backward.py:398,500) and trace with fake tensors: shapes, dtypes and the
    transposed-view strides of the quantiser outputs (mxfp_quantization.py:484)."""
    import torch
    from torch._subclasses.fake_tensor import FakeTensorMode
    import alto_amd.mxfp4 as m
    ns = m.register_torch_ops("alto_amd_test")
    assert m.register_torch_ops("alto_amd_test") is ns
    for name in ("convert_to_mxfp4", "convert_from_mxfp4", "blockwise_mxfp4_gemm", "mxfp4_grouped_gemm_forward",
                 "mxfp4_grouped_gemm_backward_inputs", "mxfp4_grouped_gemm_backward_weights"):
        assert hasattr(ns, name)
    with FakeTensorMode():
        x = torch.empty(4, 128, 64, dtype=torch.bfloat16)
        c, s = ns.convert_to_mxfp4(x)
        assert c.shape == (4, 128, 32) and s.shape == (4, 128, 2) and c.dtype == torch.uint8
        c0, s0 = ns.convert_to_mxfp4(x, 32, -2, False)
        assert c0.shape == (4, 64, 64) and s0.shape == (4, 4, 64) and c0.stride(-2) == 1      # memory [.., C][M/2]
        c2, s2 = ns.convert_to_mxfp4(x, 32, -1, True)
        assert c2.shape == (4, 128, 32) and s2.shape == (4, 4, 2)
        y = ns.convert_from_mxfp4(c, s, torch.bfloat16)
        assert y.shape == x.shape and y.dtype == torch.bfloat16
        a, a_s = torch.empty(96, 64, dtype=torch.uint8), torch.empty(96, 4, dtype=torch.uint8)
        b, b_s = torch.empty(160, 64, dtype=torch.uint8), torch.empty(5, 4, dtype=torch.uint8)
        out = ns.blockwise_mxfp4_gemm(a, a_s, b, b_s, False, True, True, True, False, True, 32, torch.bfloat16)
        assert out.shape == (96, 160) and out.dtype == torch.bfloat16
        # wgrad form: token-packed operands [M/2, N] and [M/2, K], trans_a
        gq, gs = torch.empty(64, 160, dtype=torch.uint8), torch.empty(4, 160, dtype=torch.uint8)
        xq, xs = torch.empty(64, 96, dtype=torch.uint8), torch.empty(4, 96, dtype=torch.uint8)
        dw = ns.blockwise_mxfp4_gemm(gq, gs, xq, xs, False, False, True, True, True, False)
        assert dw.shape == (160, 96) and dw.dtype == torch.float32
        idx = torch.empty(256, dtype=torch.int32)
        inp, inp_s = torch.empty(256, 64, dtype=torch.uint8), torch.empty(256, 4, dtype=torch.uint8)
        w, w_s = torch.empty(4, 160, 64, dtype=torch.uint8), torch.empty(4, 5, 4, dtype=torch.uint8)
        assert ns.mxfp4_grouped_gemm_forward(inp, w, idx, inp_s, w_s).shape == (256, 160)
        go, go_s = torch.empty(256, 80, dtype=torch.uint8), torch.empty(256, 5, dtype=torch.uint8)
        wn, wn_s = torch.empty(4, 80, 128, dtype=torch.uint8), torch.empty(4, 5, 4, dtype=torch.uint8)
        assert ns.mxfp4_grouped_gemm_backward_inputs(go, wn, idx, go_s, wn_s).shape == (256, 128)
        gom, gom_s = torch.empty(128, 160, dtype=torch.uint8), torch.empty(8, 160, dtype=torch.uint8)
        xm, xm_s = torch.empty(128, 128, dtype=torch.uint8), torch.empty(8, 128, dtype=torch.uint8)
        assert ns.mxfp4_grouped_gemm_backward_weights(gom, xm, idx, 4, gom_s, xm_s, True, False, False).shape == (4, 160, 128)


def test_weight_cache_is_keyed_by_object_identity():
    """A cache entry belongs to one tensor object: a new tensor of the same shape at the same address (what the caching
    allocator hands out after a weight is freed) must miss, an in-place update must miss, and entries die with the weight."""
    import gc
    from alto_amd.mxfp4 import linear as L
    calls = []

    def make():
        calls.append(1)
        return ("q", len(calls))

    L.enable_weight_cache(True)
    try:
        storage = torch.zeros(64, 32)
        w1 = storage.view(64, 32)
        a = L.cached_weight_quantisation(w1, "t", make)
        assert L.cached_weight_quantisation(w1, "t", make) is a and len(calls) == 1
        w2 = storage.view(64, 32)                      # another object, same address, shape, strides, version
        assert w2.data_ptr() == w1.data_ptr() and w2._version == w1._version
        b = L.cached_weight_quantisation(w2, "t", make)
        assert b is not a and len(calls) == 2
        w1.add_(1.0)                                   # in-place update bumps the version counter
        assert L.cached_weight_quantisation(w1, "t", make) is not a and len(calls) == 3
        assert L.weight_cache_stats()["entries"] == 2
        del w1, w2
        gc.collect()
        assert L.weight_cache_stats()["entries"] == 0, "entries must die with their weight"
    finally:
        L.enable_weight_cache(False)


def test_weight_cache_hits_for_a_parameter():
    """The training case: the weight is an nn.Parameter, and the plain-tensor alias the kernels work on is a new object
    in every forward.  The entry must belong to the Parameter (hit on the second forward, miss after an optimizer-style
    update, gone with the Parameter)."""
    import gc
    from alto_amd.mxfp4 import linear as L
    calls = []

    def fake_rowcol(w, *a, **k):
        calls.append(w)
        return ("q", len(calls))

    real = L.quantize_rowcol
    L.quantize_rowcol = fake_rowcol
    L.enable_weight_cache(True)
    try:
        p = torch.nn.Parameter(torch.zeros(64, 32))
        outs = []
        for _ in range(3):
            alias = L.unwrap_weight_wrapper(p)
            assert alias is not p and type(alias) is torch.Tensor
            outs.append(L._quantize_weight_2d(alias, False, owner=p))
        assert len(calls) == 1 and outs[0] is outs[1] is outs[2]
        assert L.weight_cache_stats() == {"hits": 2, "misses": 1, "entries": 1}
        with torch.no_grad():
            p.add_(1.0)
        assert L._quantize_weight_2d(L.unwrap_weight_wrapper(p), False, owner=p) is not outs[0] and len(calls) == 2
        del p, alias
        calls.clear()
        gc.collect()
        assert L.weight_cache_stats()["entries"] == 0
    finally:
        L.quantize_rowcol = real
        L.enable_weight_cache(False)


def test_product_never_imports_the_oracle_and_bench_refuses_more_than_one_gpu():
    """The oracle is the checker: nothing under the package may import it, and bench.py only inside its cpu_sample legs.
    bench.py measures one GPU and says so when asked for more."""
    import subprocess
    import sys
    pkg = os.path.join(ROOT, "alto_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(base, f), errors="replace").read()
                assert not re.search(r"^\s*(import|from)\s+oracle\b", text, flags=re.M), f"{f} imports the oracle"
    bench = open(os.path.join(ROOT, "bench.py")).read()
    for m in re.finditer(r"^(\s*)(import|from)\s+oracle\b", bench, flags=re.M):
        head = bench[:m.start()]
        last_def = head.rfind("\n    def ")
        assert last_def >= 0 and head[last_def:].lstrip().startswith("def cpu_sample"), "bench.py imports the oracle outside a cpu_sample leg"
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "one GPU" in r.stderr


def test_wrapped_weights_and_config_survive_a_weights_only_round_trip(tmp_path):
    """dispatch/tensor.py:499-503 and config.py:57 register the wrapper and the recipe as safe globals so that a state
    dict holding wrapped weights loads with torch.load(weights_only=True)."""
    import alto_amd.mxfp4 as m
    cfg = m.TrainingOpConfig(use_hadamard=False, clip_mode="static")
    w = torch.arange(64 * 32, dtype=torch.float32).reshape(64, 32)
    wrapped = m.MXFP4TrainingWeightWrapperTensor(w.clone(), cfg)
    path = tmp_path / "ckpt.pt"
    torch.save({"weight": wrapped, "config": cfg}, path)
    back = torch.load(path, weights_only=True)
    assert isinstance(back["weight"], m.MXFP4TrainingWeightWrapperTensor)
    assert back["config"] == cfg and back["weight"].config == cfg
    assert torch.equal(back["weight"]._data, w)
