"""Records raw results of the gfx950 stochastic-rounding FP4 converts (run on an MI355X; writes hw_sr_vectors.npz).

    python tests/golden/make_hw_sr_vectors.py [out.npz]

The reference issues ``v_cvt_scalef32_sr_pk_fp4_bf16`` / ``_f32`` as inline assembly on gfx950
(alto/kernels/fp4/mxfp4/mxfp_quantization.py:133-182).  What the instruction computes is a property of the hardware, so the
vectors are taken from the instruction itself: a four-line probe kernel (compiled here with hipcc into a temporary
directory) applies it to chosen (value pair, random dword, scale) triples and the bytes it returns are stored beside
the inputs.  ``oracle/hw_sr.py`` must reproduce every byte (tests/test_oracle_pins.py); nothing of the product is involved.
"""
import ctypes
import os
import subprocess
import sys
import tempfile

import numpy as np
import torch

PROBE = r"""
#include <hip/hip_runtime.h>
#include <stdint.h>
typedef float f2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
__global__ void k_f32(const float* a, const float* b, const uint32_t* r, const float* s, uint32_t* out, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = __builtin_amdgcn_cvt_scalef32_sr_pk_fp4_f32(0u, f2_t{a[i], b[i]}, r[i], s[i], 0) & 0xFFu;
}
__global__ void k_bf16(const uint32_t* ab, const uint32_t* r, const float* s, uint32_t* out, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = __builtin_amdgcn_cvt_scalef32_sr_pk_fp4_bf16(0u, __builtin_bit_cast(bf2_t, ab[i]), r[i], s[i], 0) & 0xFFu;
}
extern "C" void run_f32(const float* a, const float* b, const uint32_t* r, const float* s, uint32_t* out, int n) {
  hipLaunchKernelGGL(k_f32, dim3((n + 255) / 256), dim3(256), 0, 0, a, b, r, s, out, n);
}
extern "C" void run_bf16(const uint32_t* ab, const uint32_t* r, const float* s, uint32_t* out, int n) {
  hipLaunchKernelGGL(k_bf16, dim3((n + 255) / 256), dim3(256), 0, 0, ab, r, s, out, n);
}
"""


def build_probe(tmp):
    src = os.path.join(tmp, "probe.hip")
    with open(src, "w") as f:
        f.write(PROBE)
    so = os.path.join(tmp, "libprobe.so")
    subprocess.check_call(["hipcc", "--offload-arch=gfx950", "-O2", "-shared", "-fPIC", "-o", so, src])
    return ctypes.CDLL(so)


def main(out_path):
    dev = "cuda:0"
    rng = np.random.default_rng(20250)
    with tempfile.TemporaryDirectory() as tmp:
        lib = build_probe(tmp)

        def P(t):
            return ctypes.c_void_p(t.data_ptr())

        def dev_u32(a):
            return torch.from_numpy(np.ascontiguousarray(a, dtype=np.uint32).view(np.int32)).to(dev)

        def run(fn, *arrs):
            n = len(arrs[0])
            ts = [dev_u32(a.view(np.uint32)) for a in arrs]
            out = torch.zeros(n, dtype=torch.int32, device=dev)
            fn(*[P(t) for t in ts], P(out), ctypes.c_int(n))
            torch.cuda.synchronize()
            return out.cpu().numpy().astype(np.uint8)

        # random dwords: extremes, every single bit, every single cleared bit, low masks, random ones
        one = np.uint64(1)
        bit = np.arange(32, dtype=np.uint64)
        R = np.concatenate([np.array([0, 0xFFFFFFFF], dtype=np.uint64), one << bit, ~(one << bit) & np.uint64(0xFFFFFFFF),
                            (one << (bit + one)) - one, rng.integers(0, 2 ** 32, size=90, dtype=np.uint64)]).astype(np.uint32)
        # fp32 values: every bf16-representable magnitude from 2^-6 to 8, random fp32 in that range, special cases
        grid16 = (np.arange(0x3C80, 0x4100, dtype=np.uint32) << 16).view(np.float32)
        rnd32 = rng.integers(0x3C800000, 0x41000000, size=1200, dtype=np.uint32).view(np.float32)
        spec = np.array([0.0, -0.0, 1e-30, 6.0, 5.999999, 6.0000005, 7.0, 100.0, 0.25, 0.5, 0.75, 1.0, 1.5, 2.0, 3.0, 4.0,
                         0.24999999, 0.49999997, 0.99999994, 1.9999999, 3.9999998], dtype=np.float32)
        V = np.concatenate([grid16[::3], rnd32, spec, -grid16[::11], -rnd32[::7], -spec]).astype(np.float32)
        partner = np.roll(V, 77)
        sexp = rng.integers(-20, 21, size=len(V)).astype(np.int32)          # block scale 2^sexp, value pre-multiplied by it
        scale = np.ldexp(np.float32(1.0), sexp).astype(np.float32)
        A = np.repeat((V * scale).astype(np.float32), len(R))
        Bp = np.repeat((partner * scale).astype(np.float32), len(R))
        S = np.repeat(scale, len(R))
        RR = np.tile(R, len(V))
        out32 = run(lib.run_f32, A, Bp, RR, S).reshape(len(V), len(R))
        # bf16 pairs: every pattern from 2^-7 to 8, both signs, zero
        vb = np.concatenate([np.arange(0x3C00, 0x4100, dtype=np.uint32), np.arange(0x3C00, 0x4100, 5, dtype=np.uint32) | 0x8000,
                             np.array([0, 0x8000], dtype=np.uint32)])
        pb = np.roll(vb, 333)
        sexp16 = rng.integers(-20, 21, size=len(vb)).astype(np.int32)
        shift = lambda bits, e: np.where((bits & 0x7FFF) == 0, bits, (bits.astype(np.int64) + (e.astype(np.int64) << 7)).astype(np.uint32))
        lo16, hi16 = shift(vb, sexp16), shift(pb, sexp16)
        AB = np.repeat((lo16 | (hi16 << 16)).astype(np.uint32), len(R))
        S16 = np.repeat(np.ldexp(np.float32(1.0), sexp16).astype(np.float32), len(R))
        RB = np.tile(R, len(vb))
        out16 = run(lib.run_bf16, AB, RB, S16).reshape(len(vb), len(R))
    np.savez_compressed(out_path, rand=R,
                        f32_lo=(V * scale).astype(np.float32).view(np.uint32), f32_hi=(partner * scale).astype(np.float32).view(np.uint32),
                        f32_scale_byte=(sexp + 127).astype(np.uint8), f32_out=out32,
                        bf16_lo=lo16.astype(np.uint16), bf16_hi=hi16.astype(np.uint16), bf16_scale_byte=(sexp16 + 127).astype(np.uint8), bf16_out=out16)
    print("wrote", out_path, out32.shape, out16.shape, flush=True)


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else os.path.join(os.path.dirname(os.path.abspath(__file__)), "hw_sr_vectors.npz"))
