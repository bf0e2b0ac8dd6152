"""The grouped GEMM entry point that allocates nothing (its pass list lives in an array inside the library's device code)
gives the bytes of the workspace entry point: two calls in a row through the C ABI, the second on a smaller problem (the
array keeps the first call's contents), ragged offsets, an empty expert, an unrouted tail."""
import pytest
import torch

import oracle as O
from tests.helpers import randn_outliers

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _call(lib, rt, name, aq, as_, wq, ws, offs, E, out, workspace=None):
    args = [aq.data_ptr(), aq.stride(0), as_.data_ptr(), as_.stride(0), as_.stride(1), 0,
            wq.data_ptr(), wq.stride(0), wq.stride(1), ws.data_ptr(), ws.stride(0), ws.stride(1), ws.stride(2), 1,
            offs.data_ptr(), None, E, E, aq.shape[0], wq.shape[1], aq.shape[1] * 2, out.data_ptr(), rt.dtype_code(out.dtype), out.stride(0)]
    if workspace is not None:
        args += [workspace.data_ptr(), workspace.numel()]
    rc = getattr(lib, name)(*args, rt.stream_ptr(out.device))
    assert rc == 0, lib.alto_mxfp4_last_error()


def test_grouped_gemm_noalloc_equals_workspace_entry_point():
    import alto_amd.mxfp4 as m
    from alto_amd.mxfp4 import _runtime as rt
    lib = rt.lib()
    E, N, K = 6, 384, 640
    w = (randn_outliers((E, N, K), torch.bfloat16, seed=2) * 0.02).to(DEV)
    wq, ws = m.convert_to_mxfp4(w, is_2d_block=True)
    for rows, sizes in ((1536, [300, 0, 517, 131, 260, 200]), (640, [100, 77, 0, 200, 3, 132])):   # second call: smaller input
        offs = torch.tensor([0] + sizes, dtype=torch.int64).cumsum(0).to(torch.int32).to(DEV)     # the rows past offs[-1] belong to nobody
        a = randn_outliers((rows, K), torch.bfloat16, seed=rows).to(DEV)
        aq, as_ = m.convert_to_mxfp4(a)
        print(f"grouped_gemm_noalloc rows={rows} sizes={sizes}", flush=True)
        for dtype in (torch.bfloat16, torch.float32):
            ref = torch.full((rows, N), float("nan"), dtype=dtype, device=DEV)
            got = torch.full((rows, N), float("nan"), dtype=dtype, device=DEV)
            wsp = torch.empty(lib.alto_mxfp4_grouped_gemm_workspace_bytes(rows, E), dtype=torch.uint8, device=DEV)
            _call(lib, rt, "alto_mxfp4_grouped_gemm", aq, as_, wq, ws, offs, E, ref, wsp)
            _call(lib, rt, "alto_mxfp4_grouped_gemm_noalloc", aq, as_, wq, ws, offs, E, got)
            torch.cuda.synchronize()
            assert not bool(torch.isnan(got).any())
            assert torch.equal(got.view(torch.int16 if dtype == torch.bfloat16 else torch.int32), ref.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))
        # and both are the oracle's result
        idx = O.indices_from_offsets(offs[1:].cpu())
        exp = O.grouped_gemm_ref(aq.cpu(), as_.cpu(), wq.cpu(), ws.cpu(), idx)
        assert O.rel_frobenius(got[:exp.shape[0]].cpu(), exp) < 1e-5
        assert bool((got[int(offs[-1]):] == 0).all())


def test_grouped_gemm_noalloc_replays_from_a_hip_graph():
    """After alto_mxfp4_init() the call makes no runtime query, so it can be captured: three replays, with the program's
    own eager work between them (new activations written into the captured input buffers), each against the eager call."""
    import alto_amd.mxfp4 as m
    from alto_amd.mxfp4 import _runtime as rt
    lib = rt.lib()
    assert lib.alto_mxfp4_init() == 0, lib.alto_mxfp4_last_error()
    E, N, K, rows = 4, 256, 512, 1024
    w = (randn_outliers((E, N, K), torch.bfloat16, seed=5) * 0.02).to(DEV)
    wq, ws = m.convert_to_mxfp4(w, is_2d_block=True)
    offs = torch.tensor([0, 300, 300, 811, 1000], dtype=torch.int32, device=DEV)
    aq, as_ = m.convert_to_mxfp4(randn_outliers((rows, K), torch.bfloat16, seed=6).to(DEV))
    out = torch.zeros((rows, N), dtype=torch.bfloat16, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _call(lib, rt, "alto_mxfp4_grouped_gemm_noalloc", aq, as_, wq, ws, offs, E, out)   # warm-up on the capture stream
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            _call(lib, rt, "alto_mxfp4_grouped_gemm_noalloc", aq, as_, wq, ws, offs, E, out)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        nq, ns = m.convert_to_mxfp4(randn_outliers((rows, K), torch.bfloat16, seed=10 + rep).to(DEV))
        aq.copy_(nq); as_.copy_(ns)
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        ref = torch.full((rows, N), float("nan"), dtype=torch.bfloat16, device=DEV)
        wsp = torch.empty(lib.alto_mxfp4_grouped_gemm_workspace_bytes(rows, E), dtype=torch.uint8, device=DEV)
        _call(lib, rt, "alto_mxfp4_grouped_gemm", aq, as_, wq, ws, offs, E, ref, wsp)
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), f"replay {rep}"


def test_grouped_gemm_noalloc_rejects_what_does_not_fit():
    from alto_amd.mxfp4 import _runtime as rt
    lib = rt.lib()
    t = torch.zeros(64, dtype=torch.uint8, device=DEV)
    # 70000 groups need more than the built-in MiB; rejected before any launch (the pointers are never used)
    rc = lib.alto_mxfp4_grouped_gemm_noalloc(t.data_ptr(), 16, t.data_ptr(), 1, 1, 0, t.data_ptr(), 16, 16, t.data_ptr(), 1, 1, 1, 0,
                                             t.data_ptr(), t.data_ptr(), 65536, 8, 256 * 65536, 128, 32, t.data_ptr(), 0, 128, None)
    assert rc == -1 and b"built-in" in lib.alto_mxfp4_last_error()
