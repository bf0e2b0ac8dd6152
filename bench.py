#!/usr/bin/env python3
"""Benchmark of the MXFP4 hot path on one MI355X.

``python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]`` prints ONE JSON line.

The default workload is the MXFP4 fprop GEMM at the Llama-3-8B MLP up-projection shape (M=8192, N=14336, K=4096):
a "step" is one GEMM launch on operands already quantized and resident in HBM; ``value`` is TFLOP/s.  The same line
carries the fused RHT+SR gradient quantizer (config 2, GB/s) and the other GEMM shapes under ``"others"``, a
``roofline`` object for the dominant kernel of the selected workload (duration measured live with HIP events on the
launch stream) and a ``cpu_baseline`` (the CPU oracle timed on a bounded sample of the same workload on this box's
host cores).  All data is synthetic (seeded torch generators) and random-init; nothing is read from disk.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_MXFP4_TFLOPS = 10100.0   # MI355X dense FP4 MFMA peak (published), TFLOP/s
PEAK_HBM_GBS = 8000.0         # MI355X HBM3E peak (published), GB/s
METRIC = "MXFP4 GEMM TFLOPS (% MFMA peak) + quantizer GB/s, Llama-3-8B shapes, 1 MI355X"


def _laplace(shape, scale, device, gen):
    import torch
    u = (torch.rand(shape, device=device, generator=gen) - 0.5).clamp(-0.4999999, 0.4999999)
    return (-scale * torch.sign(u) * torch.log1p(-2 * u.abs())).bfloat16()


def _settle(fn, settle_ms):
    """Runs fn back to back, untimed, for settle_ms of wall time.  From idle the part's power management needs some 60 ms
    of sustained load to reach the clock it then holds (the first launches of a burst run 20 to 60 % slower); a training
    step sees the settled clock, so that is the state the timed steps are taken in.  Returns the number of calls made."""
    import torch
    n = 0
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < settle_ms:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()
        n += 8
    return n


def _bracket(fn, steps, warmup):
    """`warmup` untimed calls, then HIP events on the launch stream (torch's current stream, which every entry point is
    given) around exactly `steps` back-to-back calls.  Returns (mean ms per step, host wall ms per step)."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps, (time.perf_counter() - t0) * 1e3 / steps


def _time_steps(fn, steps, warmup, settle_ms):
    """Settling calls, then the bracket of `_bracket`: that is the reported time.  A second pass of `steps` calls with an
    event between consecutive calls gives the spread (the markers cost a couple of microseconds each, so they stay out of
    the first pass).  Returns (mean ms per step of the bracket, host wall ms per step, sorted per-step ms of the second pass)."""
    import torch
    _settle(fn, settle_ms)
    ms, wall_ms = _bracket(fn, steps, warmup)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    ev[0].record()
    for i in range(steps):
        fn()
        ev[i + 1].record()
    torch.cuda.synchronize()
    per = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(steps))
    return ms, wall_ms, per


# ------------------------------------------------------------------------------------------------ workloads
class Workload:
    name = ""
    bound = "mfma"
    kernel = ""

    def setup(self, dev, gen):
        raise NotImplementedError

    def step(self):
        raise NotImplementedError

    work = 0.0  # algorithmic FLOPs (mfma) or bytes (hbm) per step

    def cpu_sample(self):
        """-> (callable, work_of_sample, description)"""
        raise NotImplementedError


class FusedGradQuant(Workload):
    """Config 2: dY bf16 [8192, 4096] ~ Laplace(0, 1e-3) -> row copy (SR) + Hadamard column copy (SR), supplied random bits."""
    name = "cfg2_fused_rht_sr_quantizer[8192x4096]"
    bound = "hbm"
    kernel = "quant_kernel<bf16, row+col, SR, RHT>"
    M, C = 8192, 4096

    def setup(self, dev, gen):
        import torch
        import alto_amd.mxfp4 as m
        self.m = m
        self.x = _laplace((self.M, self.C), 1e-3, dev, gen)
        self.r = torch.randint(-2 ** 31, 2 ** 31, (self.M, self.C), dtype=torch.int32, device=dev, generator=gen)
        m.HadamardFactory.configure(seed=1234)
        self.h = m.HadamardFactory.create_transform()
        # algorithmic bytes: dY + random bits in, two code tensors + two scale tensors out
        self.work = self.M * self.C * 2 + self.M * self.C * 4 + 2 * (self.M * self.C // 2 + self.M * self.C // 32)

        # outputs allocated once: a step is one launch through the C ABI, as a caller that owns its buffers makes it
        from alto_amd.mxfp4 import _runtime as rt
        M, C = self.M, self.C
        u8 = dict(dtype=torch.uint8, device=dev)
        self.out = (torch.empty((M, C // 2), **u8), torch.empty((M, C // 32), **u8), torch.empty((C, M // 2), **u8), torch.empty((C, M // 32), **u8))
        self.rt, self.stream = rt, rt.stream_ptr(dev)

    def step(self):
        rt, (rc, rs, cc, cs) = self.rt, self.out
        code = rt.lib().alto_mxfp4_quantize(self.x.data_ptr(), rt.dtype_code(self.x.dtype), 1, self.M, self.C, self.C, self.M * self.C,
                                            rc.data_ptr(), rs.data_ptr(), cc.data_ptr(), cs.data_ptr(), 0, rt.ROUND_SR,
                                            self.r.data_ptr(), self.C, self.M * self.C, 1, self.h.signs.data_ptr(), self.h.perm.data_ptr(),
                                            0, 0, self.stream)
        assert code == 0, code

    def cpu_sample(self):
        import oracle as O
        rows = 2048
        x = self.x[:rows].cpu()
        r = self.r[:rows].cpu()
        signs, perm = self.h.signs, self.h.perm.long()

        def run():
            O.quantize(x, axis=-1, use_sr=True, rand_bits=r)
            O.quantize(O.rht_left(x, signs, perm), axis=0, use_sr=True, rand_bits=r)
        return run, self.work * rows / self.M, f"first {rows} of {self.M} rows, both copies"


class FusedGradQuantPhilox(FusedGradQuant):
    """The same pass as config 2 with the random words made inside the kernel (Philox4x32-10), as the autograd functions
    run it: no random tensor is read (and none has to be filled first), so the algorithmic bytes are dY in and the four
    outputs out."""
    name = "cfg2_fused_rht_sr_quantizer[8192x4096], random words made in the kernel"
    kernel = "quant_kernel<bf16, row+col, SR Philox, RHT>"

    def setup(self, dev, gen):
        super().setup(dev, gen)
        self.r = None
        self.work = self.M * self.C * 2 + 2 * (self.M * self.C // 2 + self.M * self.C // 32)

    def step(self):
        rt, (rc, rs, cc, cs) = self.rt, self.out
        code = rt.lib().alto_mxfp4_quantize_sr_philox(self.x.data_ptr(), rt.dtype_code(self.x.dtype), 1, self.M, self.C, self.C, self.M * self.C,
                                                      rc.data_ptr(), rs.data_ptr(), cc.data_ptr(), cs.data_ptr(), 0, 0, 0, 1234, 0, None,
                                                      1, self.h.signs.data_ptr(), self.h.perm.data_ptr(), 0, 0, self.stream)
        assert code == 0, code

    def cpu_sample(self):
        raise NotImplementedError("the CPU leg is the supplied-words workload's")


class FusedGradQuantHw(FusedGradQuantPhilox):
    """The same pass with the hardware's stochastic-rounding converts (what the reference runs on gfx950 with use_asm left
    at its default): one v_cvt_scalef32_sr_pk_fp4_bf16 per pair, dwords cut from Philox words made in the kernel."""
    name = "cfg2_fused_rht_sr_quantizer[8192x4096], hardware SR converts, random words made in the kernel"
    kernel = "quant_kernel<bf16, row+col, SR hardware, RHT>"

    def step(self):
        rt, (rc, rs, cc, cs) = self.rt, self.out
        code = rt.lib().alto_mxfp4_quantize_sr_hw(self.x.data_ptr(), rt.dtype_code(self.x.dtype), 1, self.M, self.C, self.C, self.M * self.C,
                                                  rc.data_ptr(), rs.data_ptr(), cc.data_ptr(), cs.data_ptr(), 0, 0, 0, 1234, 0, None,
                                                  1, self.h.signs.data_ptr(), self.h.perm.data_ptr(), 0, 0, self.stream)
        assert code == 0, code


class RneQuant(Workload):
    """Config 1: bf16 [4096, 4096] ~ N(0,1) with 1% x50 outliers, 1D-32 blocks, RNE, no Hadamard."""
    name = "cfg1_rne_quantizer[4096x4096]"
    bound = "hbm"
    kernel = "quant_kernel<bf16, row, RNE>"
    M, C = 4096, 4096

    def setup(self, dev, gen):
        import torch
        import alto_amd.mxfp4 as m
        self.m = m
        x = torch.randn(self.M, self.C, device=dev, generator=gen)
        self.x = torch.where(torch.rand(self.M, self.C, device=dev, generator=gen) < 0.01, x * 50, x).bfloat16()
        self.work = self.M * self.C * 2 + self.M * self.C // 2 + self.M * self.C // 32

        from alto_amd.mxfp4 import _runtime as rt
        u8 = dict(dtype=torch.uint8, device=dev)
        self.out = (torch.empty((self.M, self.C // 2), **u8), torch.empty((self.M, self.C // 32), **u8))
        self.rt, self.stream = rt, rt.stream_ptr(dev)

    def step(self):
        rt, (rc, rs) = self.rt, self.out
        code = rt.lib().alto_mxfp4_quantize(self.x.data_ptr(), rt.dtype_code(self.x.dtype), 1, self.M, self.C, self.C, self.M * self.C,
                                            rc.data_ptr(), rs.data_ptr(), None, None, 0, rt.ROUND_RNE, None, 0, 0, 0, None, None, 0, 0, self.stream)
        assert code == 0, code

    def cpu_sample(self):
        import oracle as O
        rows = 1024
        x = self.x[:rows].cpu()
        return (lambda: O.quantize(x)), self.work * rows / self.M, f"first {rows} of {self.M} rows"


class Gemm(Workload):
    """Dense NT GEMM on pre-quantized operands: C[M,N] = A[M,K] . B[N,K]^T."""
    bound = "mfma"
    kernel = "gemm"

    def __init__(self, name, M, N, K, a_2d, b_2d, a_kind, b_kind):
        self.name, self.M, self.N, self.K = name, M, N, K
        self.a_2d, self.b_2d, self.a_kind, self.b_kind = a_2d, b_2d, a_kind, b_kind
        self.work = 2.0 * M * N * K

    def _operand(self, rows, kind, is_2d, dev, gen):
        import torch
        if kind == "act":
            t = torch.randn(rows, self.K, device=dev, generator=gen).bfloat16()
        elif kind == "weight":
            t = (torch.randn(rows, self.K, device=dev, generator=gen) * 0.02).bfloat16()
        else:
            t = _laplace((rows, self.K), 1e-3, dev, gen)
        return self.m.convert_to_mxfp4(t, is_2d_block=is_2d)

    def setup(self, dev, gen):
        import torch
        import alto_amd.mxfp4 as m
        self.m = m
        self.aq, self.as_ = self._operand(self.M, self.a_kind, self.a_2d, dev, gen)
        self.bq, self.bs = self._operand(self.N, self.b_kind, self.b_2d, dev, gen)

    def step(self):
        import torch
        return self.m.blockwise_mxfp4_gemm(self.aq, self.as_, self.bq, self.bs, use_2dblock_a=self.a_2d, use_2dblock_b=self.b_2d,
                                           trans_b=True, output_dtype=torch.bfloat16)

    def cpu_sample(self):
        import torch
        import oracle as O
        rows = min(4096, self.M)   # about 10 s of host work per repetition at the Llama shapes
        aq, as_ = self.aq[:rows].cpu(), (self.as_[:rows // 32] if self.a_2d else self.as_[:rows]).cpu()
        bq, bs = self.bq.cpu(), self.bs.cpu()

        def run():  # the reference's dequantize-then-matmul branch (mxfp_linear.py:337-356)
            O.gemm_ref(aq, as_, bq, bs, self.a_2d, self.b_2d, trans_b=True, dtype=torch.float32)
        return run, self.work * rows / self.M, f"{rows} of {self.M} rows of A against all of B, dequantize + fp32 matmul"


class VendorGemm(Gemm):
    """The same config-3 operands through ``torch._scaled_mm`` (PyTorch's MXFP4 path into hipBLASLt): a comparator, not part of
    the product; reported beside the kernel's own number."""
    kernel = "hipBLASLt via torch._scaled_mm"

    def step(self):
        import torch
        a = self.aq.view(torch.float4_e2m1fn_x2)
        b = self.bq.view(torch.float4_e2m1fn_x2)
        return torch._scaled_mm(a, b.t(), self.as_.view(torch.float8_e8m0fnu), self.bs.view(torch.float8_e8m0fnu), out_dtype=torch.bfloat16)


class GemmPacked(Gemm):
    """The same GEMM on operands whose scales are in the packed, GEMM-ready layout (``pack_scales``; done in ``setup``)."""

    def setup(self, dev, gen):
        super().setup(dev, gen)
        from alto_amd.mxfp4 import linear as L
        self.L = L
        self.aps = L.pack_scales(self.as_, self.M, self.K, self.a_2d)
        self.bps = L.pack_scales(self.bs, self.N, self.K, self.b_2d)

    def step(self):
        return self.L.gemm_packed(self.aq, self.aps, self.bq, self.bps)

    def cpu_sample(self):
        raise NotImplementedError("reported beside the plain-scale workload, which carries the CPU leg")


class GroupedGemm(Workload):
    """Config 5: 32 experts, hidden 2880 -> 5760, 65536 routed rows with Zipf(1.1) expert skew, ragged int32 offsets [33]."""
    name = "cfg5_grouped_gemm[65536x5760x2880,E=32]"
    bound = "mfma"
    kernel = "grouped_gemm"
    E, N, K, T, TOPK = 32, 5760, 2880, 16384, 4

    def setup(self, dev, gen):
        import torch
        import alto_amd.mxfp4 as m
        from alto_amd.mxfp4 import grouped_gemm as G
        self.m, self.G = m, G
        rows = self.T * self.TOPK
        logits = torch.randn(self.T, self.E, device=dev, generator=gen)
        skew = torch.log(1.0 / torch.arange(1, self.E + 1, device=dev).float() ** 1.1)
        top = torch.topk(torch.softmax(logits + skew, dim=-1), self.TOPK, dim=-1).indices.reshape(-1)
        counts = torch.bincount(top, minlength=self.E)
        offs = torch.cat([torch.zeros(1, dtype=torch.int64, device=dev), counts.cumsum(0)]).to(torch.int32)
        self.groups = G.groups_from_offsets(offs)
        # operands as the autograd function holds them: code rows padded to whole 128-byte cache lines (K/2 = 1440 bytes
        # is not a multiple of 128), scales dense
        from alto_amd.mxfp4.quantization import _prep, _quantize_call
        a = torch.randn(rows, self.K, device=dev, generator=gen).bfloat16()
        aq, as_, _, _ = _quantize_call(_prep(a), True, False, False, False, None, None, 0, False, True)
        self.aq, self.as_ = aq[0], as_[0]
        del a
        w = (torch.randn(self.E, self.N, self.K, device=dev, generator=gen) * 0.02).bfloat16()
        self.wq, self.ws, _, _ = _quantize_call(_prep(w), True, False, True, False, None, None, 0, False, True)
        del w
        self.rows = rows
        self.work = 2.0 * rows * self.N * self.K

    def step(self):
        import torch
        return self.G.grouped_forward(self.aq, self.as_, self.wq, self.ws, self.groups, False, True, torch.bfloat16)

    def cpu_sample(self):
        import torch
        import oracle as O
        offs = self.groups.offs.cpu()
        e = int(torch.argmax(offs[1:] - offs[:-1]))
        lo = int(offs[e])
        rows = min(256, int(offs[e + 1]) - lo)
        aq, as_ = self.aq[lo:lo + rows].cpu(), self.as_[lo:lo + rows].cpu()
        wq, ws = self.wq[e].cpu(), self.ws[e].cpu()

        def run():
            O.gemm_ref(aq, as_, wq, ws, False, True, trans_b=True, dtype=torch.float32)
        return run, 2.0 * rows * self.N * self.K, f"{rows} rows of the largest expert, dequantize + fp32 matmul"


class GroupedGemmPacked(GroupedGemm):
    """Config 5 forward on operands whose scales are in the packed, GEMM-ready layout (packed in ``setup``)."""
    name = "cfg5_grouped_gemm_packed_scales[65536x5760x2880,E=32]"

    def setup(self, dev, gen):
        super().setup(dev, gen)
        from alto_amd.mxfp4.linear import pack_scales
        self.aps = pack_scales(self.as_, self.rows, self.K, False)
        self.wps = self.G.pack_expert_scales(self.ws, self.wq.shape[1], self.K, True)

    def step(self):
        return self.G.grouped_forward_packed(self.aq, self.aps, self.wq, self.wps, self.groups)

    def cpu_sample(self):
        raise NotImplementedError("reported beside the plain-scale workload, which carries the CPU leg")


class GroupedGemmDx(GroupedGemm):
    """Config 5 backward, input gradient: dX [65536, 2880] = dY [65536, 5760] . W[e] (reduction over N = 5760; the weights
    are the N-packed copy of their 2D-block quantisation), same ragged offsets."""
    name = "cfg5_grouped_dx[65536x2880x5760,E=32]"

    def setup(self, dev, gen):
        import torch
        super().setup(dev, gen)
        from alto_amd.mxfp4.quantization import _prep, _quantize_call
        go = _laplace((self.rows, self.N), 1e-3, dev, gen)
        gq, gs, _, _ = _quantize_call(_prep(go), True, False, False, False, None, None, 0, False, True)
        del go
        self.aq, self.as_ = gq[0], gs[0]
        w = (torch.randn(self.E, self.N, self.K, device=dev, generator=gen) * 0.02).bfloat16()
        _, _, self.wq, self.ws = _quantize_call(_prep(w), True, True, True, False, None, None, 0, False, True)   # [E, K, N/2], [E, K/32, N/32]
        del w
        # as in the autograd function, the input gradient reuses the pass list that the forward of the same groups wrote
        self.plan = self.G.grouped_plan(self.groups, self.E, self.rows)

    def step(self):
        import torch
        return self.G.grouped_forward(self.aq, self.as_, self.wq, self.ws, self.groups, False, True, torch.bfloat16, plan=self.plan)

    def cpu_sample(self):
        raise NotImplementedError("reported beside the forward workload, which carries the CPU leg")


class GroupedGemmDxPacked(GroupedGemmDx):
    """Config 5 input gradient on packed scales, pass list reused."""
    name = "cfg5_grouped_dx_packed_scales[65536x2880x5760,E=32]"

    def setup(self, dev, gen):
        super().setup(dev, gen)
        from alto_amd.mxfp4.linear import pack_scales
        self.aps = pack_scales(self.as_, self.rows, self.aq.shape[1] * 2, False)
        self.wps = self.G.pack_expert_scales(self.ws, self.wq.shape[1], self.aq.shape[1] * 2, True)

    def step(self):
        return self.G.grouped_forward_packed(self.aq, self.aps, self.wq, self.wps, self.groups, plan=self.plan)


class GroupedGemmDw(GroupedGemm):
    """Config 5 backward, weight gradient: dW[e] [5760, 2880] = sum over the tokens of expert e of dY^T X, token-packed
    operands, offsets rounded down to 32 rows (one MX block along the tokens belongs to one expert)."""
    name = "cfg5_grouped_dw[32x5760x2880 over 65536 tokens]"

    def setup(self, dev, gen):
        import torch
        super().setup(dev, gen)
        from alto_amd.mxfp4.quantization import _prep, _quantize_call
        offs = (self.groups.offs // 32 * 32).to(torch.int32)
        offs[-1] = self.rows
        self.groups = self.G.groups_from_offsets(offs)
        go = _laplace((self.rows, self.N), 1e-3, dev, gen)
        _, _, gq, gs = _quantize_call(_prep(go), False, True, False, False, None, None, 0, False, True)
        del go
        a = torch.randn(self.rows, self.K, device=dev, generator=gen).bfloat16()
        _, _, xq, xs = _quantize_call(_prep(a), False, True, False, False, None, None, 0, False, True)
        del a
        self.gq, self.gs, self.xq, self.xs = gq[0], gs[0], xq[0], xs[0]     # [N, M/2], [N, M/32], [K, M/2], [K, M/32]
        self.aq = self.as_ = self.wq = self.ws = None

    def step(self):
        import torch
        return self.G.grouped_dw(self.gq, self.gs, self.xq, self.xs, self.groups, self.E, torch.bfloat16)

    def cpu_sample(self):
        raise NotImplementedError("reported beside the forward workload, which carries the CPU leg")


class GroupedGemmDwPacked(GroupedGemmDw):
    """Config 5 weight gradient on operands whose scales are packed along the tokens (written that way by the quantizer)."""
    name = "cfg5_grouped_dw_packed_scales[32x5760x2880 over 65536 tokens]"

    def setup(self, dev, gen):
        super().setup(dev, gen)
        from alto_amd.mxfp4.linear import pack_scales
        self.gps = pack_scales(self.gs, self.N, self.rows)
        self.xps = pack_scales(self.xs, self.K, self.rows)

    def step(self):
        return self.G.grouped_dw_packed(self.gq, self.gps, self.xq, self.xps, self.groups, self.E)


class AttentionFwd(Workload):
    """MXFP4 flash-attention forward on pre-quantised Q, K, V: the largest case of the reference's own test list
    (tests/unittest/mxfp4/test_mxfp_attention.py:64: batch 4, 2048 tokens, 64 query / 8 KV heads, head dim 128, causal)."""
    name = "attn_fwd[b4,s2048,hq64,hk8,d128,causal]"
    bound = "mfma"
    kernel = "attention"
    B, S, HQ, HK, D = 4, 2048, 64, 8, 128

    def setup(self, dev, gen):
        import torch
        import alto_amd.mxfp4 as m
        self.m = m
        q = torch.randn(self.B, self.HQ, self.S, self.D, device=dev, generator=gen).bfloat16()
        k = torch.randn(self.B, self.HK, self.S, self.D, device=dev, generator=gen).bfloat16()
        v = torch.randn(self.B, self.HK, self.S, self.D, device=dev, generator=gen).bfloat16()
        self.q, self.k, self.v = q, k, v
        self.ops = m.quantize_qkv(q, k, v)
        # algorithmic FLOPs: the unmasked (query, key) pairs, each 2 D (QK^T) + 2 Dv (PV)
        self.work = 4.0 * self.D * self.B * self.HQ * (self.S * (self.S + 1) / 2)

    def step(self):
        qq, qs, kq, ks, vq, vs = self.ops
        return self.m.attention_mxfp4_forward(qq, kq, vq, qs, ks, vs, self.D ** -0.5, True)

    def cpu_sample(self):
        from oracle.attention_oracle import attention_fwd_ref
        q, k, v = self.q[:1, :4].cpu(), self.k[:1, :1].cpu(), self.v[:1, :1].cpu()   # 4 query heads that share one KV head

        def run():
            attention_fwd_ref(q, k, v, causal=True)
        return run, self.work * 4 / (self.B * self.HQ), "4 of 256 (batch, head) pairs at full sequence length"


class LinearStep(Workload):
    """Config 3 + 4 end to end: MXFP4LinearFunction forward and backward at the Llama-3-8B FFN shape (production flags:
    1D activations, 2D weights, Hadamard on the wgrad operands, stochastic rounding of dY): per step three quantizer
    passes over activations / gradients (plus the weight's unless cached), one fill of random words for dY and three GEMMs."""
    bound = "mfma"
    kernel = "gemm"
    M, K, N = 8192, 4096, 14336

    def __init__(self, cached, hw_sr=False):
        self.cached = cached
        self.hw_sr = hw_sr
        self.name = f"cfg3+4_linear_fwd_bwd[8192x4096->14336,{'cached' if cached else 'requantized'} weight, {'hardware SR converts (the library default)' if hw_sr else 'software SR rule'}]"
        self.work = 3 * 2.0 * self.M * self.K * self.N

    def setup(self, dev, gen):
        import torch
        import alto_amd.mxfp4 as m
        from alto_amd.mxfp4 import _runtime
        self.m, self.rt = m, _runtime
        self.x = torch.randn(self.M, self.K, device=dev, generator=gen).bfloat16().requires_grad_(True)
        self.w = (torch.randn(self.N, self.K, device=dev, generator=gen) * 0.02).bfloat16().requires_grad_(True)
        self.go = _laplace((self.M, self.N), 1e-3, dev, gen)
        g = torch.Generator().manual_seed(1234)
        signs = (torch.randint(0, 2, (32,), generator=g) * 2 - 1).to(torch.int8)
        self.h = m.HadamardTransform(signs, torch.randperm(32, generator=g))

    def step(self):
        m = self.m
        m.enable_weight_cache(self.cached)
        before = self.rt.hardware_stochastic_rounding()
        m.use_hardware_stochastic_rounding(self.hw_sr)
        try:   # the random words of the stochastic rounding are drawn inside the step (Philox fill kernel), as in training
            self.x.grad = self.w.grad = None
            y = m.MXFP4LinearFunction.apply(self.x, self.w, False, True, True, False, "none", False, self.h, False)
            y.backward(self.go)
        finally:
            m.use_hardware_stochastic_rounding(before)
            if not self.cached:
                m.enable_weight_cache(False)
        return y

    def cpu_sample(self):
        raise NotImplementedError("the end-to-end step is reported beside the per-kernel workloads, without its own CPU leg")


class GroupedStep(Workload):
    """Config 5 end to end: the grouped autograd function forward and backward at the GPT-OSS expert shape (1D activation
    blocks, 2D weight blocks, Hadamard on the dW operands, stochastic rounding of dY, ragged offsets): per step the
    quantizer passes over x, the 32 expert weights (unless cached) and dY, and the three grouped GEMMs."""
    bound = "mfma"
    kernel = "grouped_gemm"
    E, N, K, T, TOPK = 32, 5760, 2880, 16384, 4

    def __init__(self, cached, hw_sr=False):
        self.cached = cached
        self.hw_sr = hw_sr
        self.name = f"cfg5_grouped_fwd_bwd[65536x2880->5760,E=32,{'cached' if cached else 'requantized'} weights, {'hardware SR converts (the library default)' if hw_sr else 'software SR rule'}]"
        self.work = 3 * 2.0 * self.T * self.TOPK * self.K * self.N

    def setup(self, dev, gen):
        import torch
        import alto_amd.mxfp4 as m
        from alto_amd.mxfp4 import _runtime
        self.m, self.rt = m, _runtime
        rows = self.T * self.TOPK
        logits = torch.randn(self.T, self.E, device=dev, generator=gen)
        skew = torch.log(1.0 / torch.arange(1, self.E + 1, device=dev).float() ** 1.1)
        top = torch.topk(torch.softmax(logits + skew, dim=-1), self.TOPK, dim=-1).indices.reshape(-1)
        counts = torch.bincount(top, minlength=self.E)
        self.offs = torch.cat([torch.zeros(1, dtype=torch.int64, device=dev), counts.cumsum(0)]).to(torch.int32)
        self.x = torch.randn(rows, self.K, device=dev, generator=gen).bfloat16().requires_grad_(True)
        self.w = (torch.randn(self.E, self.N, self.K, device=dev, generator=gen) * 0.02).bfloat16().requires_grad_(True)
        self.go = _laplace((rows, self.N), 1e-3, dev, gen)
        m.HadamardFactory.configure(seed=1234)

    def step(self):
        m = self.m
        m.enable_weight_cache(self.cached)
        before = self.rt.hardware_stochastic_rounding()
        m.use_hardware_stochastic_rounding(self.hw_sr)
        try:
            self.x.grad = self.w.grad = None
            y = m.mxfp4_grouped_gemm(self.x, self.w, None, use_2dblock_x=False, use_2dblock_w=True, use_sr_grad=True, use_hadamard=True,
                                     offsets=self.offs)
            y.backward(self.go)
        finally:
            m.use_hardware_stochastic_rounding(before)
            if not self.cached:
                m.enable_weight_cache(False)
        return y

    def cpu_sample(self):
        raise NotImplementedError("the end-to-end step is reported beside the per-kernel workloads, without its own CPU leg")


class CopyCalibration(Workload):
    """Plain device copy of 256 MiB (torch's elementwise copy kernel): the known-size launch against which the
    FETCH_SIZE / WRITE_SIZE counters of the other kernels are scaled.  Not part of the product path."""
    name = "copy_calibration[256MiB]"
    bound = "hbm"
    kernel = "torch elementwise copy"
    BYTES = 256 << 20

    def setup(self, dev, gen):
        import torch
        self.src = torch.randint(0, 255, (self.BYTES,), dtype=torch.uint8, device=dev, generator=gen).view(torch.int32)
        self.dst = torch.empty_like(self.src)
        self.work = 2 * self.BYTES

    def step(self):
        self.dst.copy_(self.src)

    def cpu_sample(self):
        src = self.src.cpu()
        dst = src.clone()
        return (lambda: dst.copy_(src)), self.work, "the same 256 MiB copy on the host"


class MfmaProbe(Workload):
    """Register-only loop of FP4 scaled-MFMA instructions (no memory traffic): the rate the matrix pipe itself sustains
    on this part, with constant or pseudo-random FP4 operands.  A diagnostic next to the published peak, not a product path."""
    bound = "mfma"
    kernel = "mfma_probe_kernel"

    def __init__(self, random_operands):
        self.random = int(random_operands)
        self.name = f"mfma_pipe_probe[{'random' if self.random else 'constant'} operands]"

    def setup(self, dev, gen):
        import torch
        from alto_amd.mxfp4 import _runtime as rt
        self.rt, self.stream = rt, rt.stream_ptr(dev)
        self.sink = torch.zeros(512, dtype=torch.float32, device=dev)
        self.ticks = torch.zeros(2, dtype=torch.int64, device=dev)
        self.iters, self.wgs = 4000, torch.cuda.get_device_properties(dev).multi_processor_count
        self.work = 2.0 * 32 * 32 * 64 * 8 * self.iters * 8 * self.wgs

    def step(self):
        code = self.rt.lib().alto_mxfp4_probe_mfma(self.random, self.iters, self.wgs, self.sink.data_ptr(), self.ticks.data_ptr(), self.stream)
        assert code == 0, code

    def extra(self):
        """The clock the chip held during the last launch: shader-clock cycles per tick of the constant 100 MHz counter."""
        cycles, ticks = (int(v) for v in self.ticks.cpu())
        return {"clock_mhz": round(100.0 * cycles / ticks, 1) if ticks > 0 else None}

    def cpu_sample(self):
        raise NotImplementedError("the probe has no CPU counterpart")


def load_traffic(key):
    """HBM bytes per launch of the workload's dominant kernel, from the committed rocprofv3 counter summaries (or None)."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            return json.load(f).get(key, {}).get("hbm_bytes_per_launch")
    except (OSError, ValueError):
        return None


def make_workloads():
    return {
        "cfg3_fprop": Gemm("cfg3_fprop_gemm[8192x14336x4096]", 8192, 14336, 4096, False, True, "act", "weight"),
        "cfg3_fprop_packed": GemmPacked("cfg3_fprop_gemm_packed_scales[8192x14336x4096]", 8192, 14336, 4096, False, True, "act", "weight"),
        "cfg4_wgrad_packed": GemmPacked("cfg4_wgrad_gemm_packed_scales[4096x14336x8192]", 4096, 14336, 8192, False, False, "grad", "act"),
        "cfg3_fprop_vendor": VendorGemm("cfg3_fprop_gemm[8192x14336x4096] via torch._scaled_mm (1D scales on both operands)", 8192, 14336, 4096, False, False,
                                        "act", "weight"),
        "cfg2_quant": FusedGradQuant(),
        "cfg2_quant_philox": FusedGradQuantPhilox(),
        "cfg2_quant_hw_sr": FusedGradQuantHw(),
        "cfg1_quant": RneQuant(),
        # config 4: dgrad dX[8192,14336] = dY[8192,4096] . W^T-packed[14336,4096]; wgrad dW[4096,14336] over 8192 tokens
        "cfg4_dgrad": Gemm("cfg4_dgrad_gemm[8192x14336x4096]", 8192, 14336, 4096, False, True, "grad", "weight"),
        "cfg4_wgrad": Gemm("cfg4_wgrad_gemm[4096x14336x8192]", 4096, 14336, 8192, False, False, "grad", "act"),
        "cfg5_grouped": GroupedGemm(),
        "cfg5_grouped_dx": GroupedGemmDx(),
        "cfg5_grouped_packed": GroupedGemmPacked(),
        "cfg5_grouped_dx_packed": GroupedGemmDxPacked(),
        "cfg5_grouped_dw": GroupedGemmDw(),
        "cfg5_grouped_dw_packed": GroupedGemmDwPacked(),
        "attn_fwd": AttentionFwd(),
        "linear_step": LinearStep(False),
        "linear_step_cached": LinearStep(True),
        "linear_step_hw_sr": LinearStep(False, hw_sr=True),
        "linear_step_cached_hw_sr": LinearStep(True, hw_sr=True),
        "grouped_step": GroupedStep(False),
        "grouped_step_hw_sr": GroupedStep(False, hw_sr=True),
        "grouped_step_cached_hw_sr": GroupedStep(True, hw_sr=True),
        "copy_calib": CopyCalibration(),
        "mfma_probe_const": MfmaProbe(False),
        "mfma_probe_random": MfmaProbe(True),
    }


def measure(w, dev, gen, steps, warmup, settle_ms, from_idle=False):
    """from_idle: also time `steps` calls after `warmup` calls BEFORE the settling phase, after half a second without
    work, i.e. what a short burst on an idle device sees (reported beside the settled figure, never as the value)."""
    import torch
    w.setup(dev, gen)
    torch.cuda.synchronize()
    idle_ms = None
    if from_idle:
        time.sleep(0.5)
        idle_ms, _ = _bracket(w.step, steps, warmup)
    ms, wall_ms, per = _time_steps(w.step, steps, warmup, settle_ms)
    if w.bound == "mfma":
        achieved, peak, unit = w.work / (ms * 1e-3) / 1e12, PEAK_MXFP4_TFLOPS, "TFLOP/s"
    else:
        achieved, peak, unit = w.work / (ms * 1e-3) / 1e9, PEAK_HBM_GBS, "GB/s"
    res = {"workload": w.name, "kernel": w.kernel, "ms": ms, "wall_ms": wall_ms, "achieved": achieved, "peak": peak, "unit": unit,
           "bound": w.bound, "frac": achieved / peak, "ms_median": per[len(per) // 2], "ms_min": per[0], "ms_max": per[-1]}
    if idle_ms is not None:
        res["from_idle_ms"] = idle_ms
    if hasattr(w, "extra"):
        res.update(w.extra())
    return res


def _brief(r):
    """The fields of a measurement that go into "others"."""
    out = {"workload": r["workload"], "ms": round(r["ms"], 4), "ms_median": round(r["ms_median"], 4), "ms_min": round(r["ms_min"], 4),
           "ms_max": round(r["ms_max"], 4), "achieved": round(r["achieved"], 2), "unit": r["unit"], "bound": r["bound"], "frac": round(r["frac"], 4)}
    if "clock_mhz" in r:
        out["clock_mhz"] = r["clock_mhz"]
    return out


def cpu_baseline(w):
    import torch
    torch.set_num_threads(min(os.cpu_count() or 1, 16))
    fn, work, desc = w.cpu_sample()
    fn()  # warm-up
    times = []
    t_all = time.perf_counter()
    while (len(times) < 3 or time.perf_counter() - t_all < 10) and time.perf_counter() - t_all < 30:   # 10 to 30 s of CPU work
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    t = sorted(times)[len(times) // 2]
    if w.bound == "mfma":
        value, unit = work / t / 1e12, "TFLOP/s"
    else:
        value, unit = work / t / 1e9, "GB/s"
    return {"value": value, "unit": unit, "cores": torch.get_num_threads(), "kind": "port", "sample": desc, "seconds": t, "runs": len(times),
            "cpu_seconds_total": time.perf_counter() - t_all}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--settle-ms", type=float, default=150.0,
                    help="untimed back-to-back calls of each workload for this long before its warm-up and timed steps (clock settling)")
    ap.add_argument("--workload", default="cfg3_fprop", help="primary workload; one of " + ", ".join(make_workloads()))
    ap.add_argument("--only", action="store_true", help="measure the primary workload only (for profiling runs)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (every kernel works on one GPU's shard). "
              "Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py needs an MI355X: torch.cuda.is_available() is False", file=sys.stderr)
        sys.exit(1)
    from alto_amd import _lib
    _lib.load()  # fail loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)
    props = torch.cuda.get_device_properties(0)

    wl = make_workloads()
    if args.workload not in wl:
        print(f"unknown workload {args.workload}", file=sys.stderr)
        sys.exit(2)
    primary = wl[args.workload]
    res = measure(primary, dev, gen, args.steps, args.warmup, args.settle_ms, from_idle=not args.only)
    try:
        cpu = None if args.no_cpu else cpu_baseline(primary)
    except NotImplementedError as e:   # a composite workload without a CPU leg of its own
        print(f"bench.py: no cpu_baseline for {args.workload}: {e}", file=sys.stderr)
        cpu = None
    others = {}
    clock_observed = None
    if not args.only:
        for key, w in wl.items():
            if key == args.workload or key == "copy_calib":
                continue
            if key.startswith("mfma_probe"):   # the pipe's own rate and clock, reported beside the published peak
                r = measure(w, dev, gen, 3, 1, args.settle_ms)
                others[key] = _brief(r)
                if key == "mfma_probe_random":
                    clock_observed = r.get("clock_mhz")
                continue
            try:
                try:
                    r = measure(w, dev, gen, max(5, args.steps // 2), max(2, args.warmup // 2), args.settle_ms)
                except (RuntimeError, AttributeError, NotImplementedError) as e:
                    # a secondary workload that fails is reported in its place; the headline line still goes out
                    others[key] = {"workload": w.name, "error": str(e)[:200]}
                    if key != "cfg3_fprop_vendor":
                        print(f"bench: workload {key} failed: {e}", file=sys.stderr)
                    continue
                others[key] = _brief(r)
                if key == "cfg2_quant":   # the metric names the quantizer too: its own traffic figure and CPU leg
                    others[key]["traffic"] = load_traffic(key)
                    others[key]["cpu_baseline"] = None if args.no_cpu else cpu_baseline(w)
            finally:
                for attr in list(vars(w)):
                    if attr not in ("name", "work"):
                        setattr(w, attr, None)
                torch.cuda.empty_cache()

    if "from_idle_ms" in res:   # the same K steps on a device that was idle: the clock is still on its way up
        t = res["from_idle_ms"]
        rate = primary.work / (t * 1e-3) / (1e12 if res["bound"] == "mfma" else 1e9)
        from_idle = {"workload": res["workload"] + ", after 0.5 s without work, no settling calls", "ms": round(t, 4),
                     "achieved": round(rate, 2), "unit": res["unit"], "bound": res["bound"], "frac": round(rate / res["peak"], 4)}
        others[args.workload + "_from_idle"] = from_idle
    else:
        from_idle = None
    line = {
        "metric": METRIC,
        "value": round(res["achieved"], 3),
        "unit": res["unit"],
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(res["ms"], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "mxfp4 (e2m1 codes, e8m0 scales), fp32 accumulate" if res["bound"] == "mfma" else "bf16 -> e2m1/e8m0 (u8 bit ops, fp32 transform)",
        "data": "synthetic",
        # clock_mhz: what the chip held under a register-only loop of FP4 MFMAs on random operands in this run (shader
        # cycles per tick of the constant 100 MHz counter); null with --only, which skips that probe
        # settle_ms: every workload is first run untimed for this long, so that the timed steps see the clock of sustained load
        "config": {"workload": res["workload"], "device": props.name, "cus": props.multi_processor_count, "clock_mhz": clock_observed,
                   "settle_ms": args.settle_ms},
        "ms_median": round(res["ms_median"], 5), "ms_min": round(res["ms_min"], 5), "ms_max": round(res["ms_max"], 5),
        "roofline": {"bound": res["bound"], "achieved": round(res["achieved"], 3), "peak": res["peak"], "unit": res["unit"],
                     "frac": round(res["frac"], 4), "traffic": load_traffic(args.workload), "kernel": res["kernel"], "kernel_ms": round(res["ms"], 5),
                     # achieved / frac come from the event bracket around all K launches (ms_per_step), not from the per-step median
                     "timing": "HIP events around the K timed launches on the launch stream"},
        "cpu_baseline": cpu,
        # the same steps on a device that had been idle (its clock still rising): beside `value`, never instead of it
        "from_idle": from_idle,
        "others": others,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
