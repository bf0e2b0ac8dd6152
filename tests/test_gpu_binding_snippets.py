"""The ctypes bindings a maintainer of the reference would add (they are printed in the integration notes), run as they
stand: raw library handle, explicit argtypes, device pointers -- checked against the oracle."""
import ctypes

import pytest
import torch

import oracle as O
from tests.helpers import randn_outliers

pytestmark = pytest.mark.gpu
DEV = "cuda"

vp, i64, i32, f32, u64 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_uint64


@pytest.fixture(scope="module")
def lib():
    from alto_amd import build
    _lib = ctypes.CDLL(build.lib_path())
    _lib.alto_mxfp4_last_error.restype = ctypes.c_char_p
    _lib.alto_mxfp4_quantize.argtypes = [vp, i32, i64, i64, i64, i64, i64, vp, vp, vp, vp, i32, i32, vp, i64, i64, i32, vp, vp, i32, i32, vp]
    _lib.alto_mxfp4_gemm.argtypes = [vp, i64, vp, i64, i64, i32, vp, i64, vp, i64, i64, i32, i64, i64, i64, vp, i32, i64, f32, vp]
    _lib.alto_mxfp4_quantize_sr_philox.argtypes = [vp, i32, i64, i64, i64, i64, i64, vp, vp, vp, vp, i64, i64, i32, u64, u64, vp, i32, vp, vp, i32, i32, vp]
    _lib.alto_mxfp4_random_bits.argtypes = [vp, i64, u64, u64, vp]
    _lib.alto_mxfp4_grouped_gemm_workspace_bytes.restype = i64
    _lib.alto_mxfp4_grouped_gemm_workspace_bytes.argtypes = [i64, i32]
    _lib.alto_mxfp4_grouped_gemm.argtypes = [vp, i64, vp, i64, i64, i32, vp, i64, i64, vp, i64, i64, i64, i32,
                                             vp, vp, i32, i32, i64, i64, i64, vp, i32, i64, vp, i64, vp]
    _lib.alto_mxfp4_quantize_ex.argtypes = [vp, i32, i64, i64, i64, i64, i64, vp, vp, vp, vp, i64, i64, i32, i32,
                                            vp, i64, i64, u64, u64, vp, i32, vp, vp, i32, i32, i32, vp]
    _lib.alto_mxfp4_gemm_ps.argtypes = [vp, i64, vp, vp, i64, vp, i64, i64, i64, vp, i64, f32, vp]
    return _lib


PACK_ROW_SCALES = 1


def _check(lib, rc):
    if rc:
        raise RuntimeError(lib.alto_mxfp4_last_error().decode())


def _stream():
    return torch.cuda.current_stream().cuda_stream


def convert_to_mxfp4_rows(lib, x):
    M, C = x.shape
    codes = torch.empty(M, C // 2, dtype=torch.uint8, device=x.device)
    scales = torch.empty(M, C // 32, dtype=torch.uint8, device=x.device)
    _check(lib, lib.alto_mxfp4_quantize(x.data_ptr(), 0 if x.dtype == torch.bfloat16 else 1, 1, M, C, x.stride(0), M * x.stride(0),
                                        codes.data_ptr(), scales.data_ptr(), None, None, 0, 0, None, 0, 0, 0, None, None, 0, 0, _stream()))
    return codes, scales


def gemm_nt(lib, a, a_s, b, b_s, b_is_2d, out_dtype):
    M, N, K = a.shape[0], b.shape[0], a.shape[1] * 2
    c = torch.empty(M, N, dtype=out_dtype, device=a.device)
    _check(lib, lib.alto_mxfp4_gemm(a.data_ptr(), a.stride(0), a_s.data_ptr(), a_s.stride(0), a_s.stride(1), 0,
                                    b.data_ptr(), b.stride(0), b_s.data_ptr(), b_s.stride(0), b_s.stride(1), int(b_is_2d),
                                    M, N, K, c.data_ptr(), 0 if out_dtype == torch.bfloat16 else 1, c.stride(0), 1.0, _stream()))
    return c


def convert_to_mxfp4_rows_sr(lib, x, seed, offset):
    M, C = x.shape
    codes = torch.empty(M, C // 2, dtype=torch.uint8, device=x.device)
    scales = torch.empty(M, C // 32, dtype=torch.uint8, device=x.device)
    _check(lib, lib.alto_mxfp4_quantize_sr_philox(x.data_ptr(), 0 if x.dtype == torch.bfloat16 else 1, 1, M, C, x.stride(0), M * x.stride(0),
                                                  codes.data_ptr(), scales.data_ptr(), None, None, C // 2, 0, 0, seed, offset, None,
                                                  0, None, None, 0, 0, _stream()))
    return codes, scales


def grouped_forward(lib, a, a_s, w, w_s, offs, N):
    M_total, K, E = a.shape[0], a.shape[1] * 2, w.shape[0]
    out = torch.empty(M_total, N, dtype=torch.bfloat16, device=a.device)
    nbytes = lib.alto_mxfp4_grouped_gemm_workspace_bytes(M_total, E)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=a.device)
    _check(lib, lib.alto_mxfp4_grouped_gemm(a.data_ptr(), a.stride(0), a_s.data_ptr(), a_s.stride(0), a_s.stride(1), 0,
                                            w.data_ptr(), w.stride(0), w.stride(1), w_s.data_ptr(), w_s.stride(0), w_s.stride(1), w_s.stride(2), 1,
                                            offs.data_ptr(), None, E, E, M_total, N, K, out.data_ptr(), 0, out.stride(0),
                                            ws.data_ptr(), nbytes, _stream()))
    return out


def convert_to_mxfp4_rows_packed(lib, x, is_2d):
    M, C = x.shape
    codes = torch.empty(M, C // 2, dtype=torch.uint8, device=x.device)
    packed = torch.empty(-(-C // 512), M, 16, dtype=torch.uint8, device=x.device)
    _check(lib, lib.alto_mxfp4_quantize_ex(x.data_ptr(), 0 if x.dtype == torch.bfloat16 else 1, 1, M, C, x.stride(0), M * x.stride(0),
                                           codes.data_ptr(), packed.data_ptr(), None, None, C // 2, 0, int(is_2d), 0,
                                           None, 0, 0, 0, 0, None, 0, None, None, 0, 0, PACK_ROW_SCALES, _stream()))
    return codes, packed


def gemm_nt_packed(lib, a, a_ps, b, b_ps):
    M, N, K = a.shape[0], b.shape[0], a.shape[1] * 2
    c = torch.empty(M, N, dtype=torch.bfloat16, device=a.device)
    _check(lib, lib.alto_mxfp4_gemm_ps(a.data_ptr(), a.stride(0), a_ps.data_ptr(), b.data_ptr(), b.stride(0), b_ps.data_ptr(),
                                       M, N, K, c.data_ptr(), c.stride(0), 1.0, _stream()))
    return c


def test_packed_scale_bindings(lib):
    """Quantizer with the layout flag + the GEMM on packed scales: same bits as the plain pair of calls, 2D weight blocks."""
    x = randn_outliers((256, 1056), torch.bfloat16, seed=76).to(DEV)
    w = (randn_outliers((384, 1056), torch.bfloat16, seed=77) * 0.02).to(DEV)
    xq, xs = convert_to_mxfp4_rows(lib, x)
    xq2, xps = convert_to_mxfp4_rows_packed(lib, x, False)
    assert torch.equal(xq, xq2)
    import alto_amd.mxfp4 as m
    wq, ws = m.convert_to_mxfp4(w, axis=-1, is_2d_block=True)
    wq2, wps = convert_to_mxfp4_rows_packed(lib, w, True)
    assert torch.equal(wq, wq2)
    want = gemm_nt(lib, xq, xs, wq, ws, True, torch.bfloat16)
    assert torch.equal(gemm_nt_packed(lib, xq2, xps, wq2, wps), want)


def test_row_quantizer_and_gemm_bindings(lib):
    x = randn_outliers((256, 512), torch.bfloat16, seed=71).to(DEV)
    w = (randn_outliers((384, 512), torch.bfloat16, seed=72) * 0.02).to(DEV)
    xq, xs = convert_to_mxfp4_rows(lib, x)
    oq, os_ = O.quantize(x.cpu(), axis=-1)
    assert torch.equal(xq.cpu(), oq) and torch.equal(xs.cpu(), os_)
    wq, ws = convert_to_mxfp4_rows(lib, w)
    y = gemm_nt(lib, xq, xs, wq, ws, False, torch.float32)
    ref = O.dequantize(oq, os_).double() @ O.dequantize(*O.quantize(w.cpu(), axis=-1)).double().T
    assert float((y.cpu().double() - ref).norm() / ref.norm()) < 1e-5


def test_philox_quantizer_binding(lib):
    x = randn_outliers((128, 256), torch.bfloat16, seed=73).to(DEV)
    codes, scales = convert_to_mxfp4_rows_sr(lib, x, 99, 7)
    bits = torch.empty(x.shape, dtype=torch.int32, device=DEV)
    _check(lib, lib.alto_mxfp4_random_bits(bits.data_ptr(), bits.numel(), 99, 7, _stream()))
    oq, os_ = O.quantize(x.cpu(), axis=-1, use_sr=True, rand_bits=bits.cpu())
    assert torch.equal(codes.cpu(), oq) and torch.equal(scales.cpu(), os_)


def test_grouped_forward_binding(lib):
    import alto_amd.mxfp4 as m
    E, N, K, M = 3, 256, 512, 640
    a = randn_outliers((M, K), torch.bfloat16, seed=74).to(DEV)
    w = (randn_outliers((E, N, K), torch.bfloat16, seed=75) * 0.02).to(DEV)
    aq, as_ = convert_to_mxfp4_rows(lib, a)
    wq, ws = m.convert_to_mxfp4(w, axis=-1, is_2d_block=True)
    offs = torch.tensor([0, 200, 200, 640], dtype=torch.int32, device=DEV)   # expert 1 is empty, boundaries off the tile grid
    out = grouped_forward(lib, aq, as_, wq, ws, offs, N)
    a_dq = O.dequantize(*O.quantize(a.cpu(), axis=-1)).double()
    ref = torch.zeros(M, N, dtype=torch.float64)
    for e, (lo, hi) in enumerate([(0, 200), (200, 200), (200, 640)]):
        if hi > lo:
            w_dq = O.dequantize(*O.quantize(w[e].cpu(), axis=-1, is_2d_block=True), is_2d_block=True).double()
            ref[lo:hi] = a_dq[lo:hi] @ w_dq.T
    assert float((out.cpu().double() - ref).norm() / ref.norm()) < 1e-2
