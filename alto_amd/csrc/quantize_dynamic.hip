// MXFP4 quantisation with the std-based ("dynamic") clipping scale of
// alto/kernels/fp4/mxfp4/mxfp_quantization.py:54-59,65-70: instead of the block absmax the scale is taken from
//   max_abs = (2.92247856 / 6) * sqrt(mean(x^2) - mean(x)^2) + 1e-8     (cast to the input dtype)
// with the exponent rule of :80-85 and target_max_pow2 = 0; values beyond 6 * 2^(s-127) saturate in the encoder.
// An optional knob outside the production recipe: a plain kernel (one thread per 32-element block, a half-wave per
// 32x32 block), quantisation along the contiguous dim only.
//
// Order of the fp32 sums (the reference leaves it to Triton's reduction): the 32 elements of a block row are added in
// index order; a 32x32 block adds its 32 row sums in row order.  Squares are rounded to the input dtype before they
// are summed (a bf16 x bf16 product is a bf16 tensor in Triton; the sum itself is promoted to fp32).  The multiply
// and the add of the max_abs formula are two roundings (the reference's PyTorch twin, tests/unittest/mxfp4/utils.py:320-325).
#include "common.h"

namespace alto {
namespace {

struct DynParams {
  const void* x; int64_t ld_x, bs_x;
  const uint32_t* rand; int64_t ld_r, bs_r;
  uint8_t* codes; uint8_t* scales; int64_t ld_c;
  int M, C;
  int uos;   // scale from ceil(log2(max_abs / 7.25)) + 127 instead of the exponent rule (mxfp_quantization.py:75-78)
};

template <typename T>
__device__ __forceinline__ float round_to(float v) {
  if constexpr (sizeof(T) == 2) return (float)(__bf16)v;
  else return v;
}

template <typename T, bool B2D, bool SR>
__global__ __launch_bounds__(64) void quant_dynamic_kernel(DynParams p) {
  constexpr bool BF = sizeof(T) == 2;
  const int lane = threadIdx.x, r = lane & 31, cbl = lane >> 5;
  const int cb = blockIdx.x * 2 + cbl;
  const int row = blockIdx.y * 32 + r;
  const int64_t b = blockIdx.z;
  const bool valid = cb < p.C / 32 && row < p.M;
  float v[32];
#pragma unroll
  for (int i = 0; i < 32; ++i) v[i] = 0.0f;
  if (valid) {
    const T* src = reinterpret_cast<const T*>(p.x) + b * p.bs_x + (int64_t)row * p.ld_x + 32 * cb;
#pragma unroll
    for (int i = 0; i < 32; ++i) v[i] = (float)src[i];
  }
  float sum = 0.0f, sq = 0.0f;
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    sum = __fadd_rn(sum, v[i]);
    sq = __fadd_rn(sq, round_to<T>(__fmul_rn(v[i], v[i])));
  }
  float n = 32.0f;
  if (B2D) {   // rows of the block live in the 32 lanes of this half-wave
    float ts = 0.0f, tq = 0.0f;
    for (int j = 0; j < 32; ++j) {
      ts = __fadd_rn(ts, __shfl(sum, (lane & 32) + j, 64));
      tq = __fadd_rn(tq, __shfl(sq, (lane & 32) + j, 64));
    }
    sum = ts; sq = tq; n = 1024.0f;
  }
  const float mean_sq = __fdiv_rn(sq, n), mean = __fdiv_rn(sum, n);
  const float sd = __fsqrt_rn(__fsub_rn(mean_sq, __fmul_rn(mean, mean)));
  const float amax = round_to<T>(__fadd_rn(__fmul_rn((float)(2.92247856 / 6.0), sd), 1e-8f));
  // exponent after rounding to one mantissa bit, target_max_pow2 = 0, clamped below at 1, kept as a byte
  uint32_t e;
  if constexpr (BF) e = (((f2u(amax) >> 16) + 0x20u) >> 7) & 0x1FFu;
  else e = ((f2u(amax) + 0x200000u) >> 23) & 0x1FFu;
  uint32_t s = (e < 1u ? 1u : e) & 0xFFu;
  if (p.uos) s = e8m0_uos(amax);
  if (!valid) return;
  if (!B2D) p.scales[(b * p.M + row) * (p.C / 32) + cb] = (uint8_t)s;
  else if (r == 0) p.scales[(b * (p.M / 32) + blockIdx.y) * (p.C / 32) + cb] = (uint8_t)s;
  const float scale_f = u2f(s << 23);   // s = 255 gives +inf: every quotient is 0, as in the reference's division
  uint32_t out[4] = {0, 0, 0, 0};
  const uint32_t* rnd = SR ? p.rand + b * p.bs_r + (int64_t)row * p.ld_r + 32 * cb : nullptr;
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    const float q = __fdiv_rn(v[i], scale_f);
    const float m = __builtin_fabsf(q);
    uint32_t code = SR ? e2m1_sr_mag(m, rnd[i]) : e2m1_rne_mag(m);
    code |= (f2u(q) >> 28) & 8u;
    out[i >> 3] |= code << (4 * (i & 7));
  }
  *reinterpret_cast<uint4*>(p.codes + (b * p.M + row) * p.ld_c + 16 * cb) = make_uint4(out[0], out[1], out[2], out[3]);
}

template <typename T>
void launch(const DynParams& p, dim3 grid, hipStream_t st, bool is_2d, bool sr) {
  if (is_2d) {
    if (sr) hipLaunchKernelGGL((quant_dynamic_kernel<T, true, true>), grid, dim3(64), 0, st, p);
    else hipLaunchKernelGGL((quant_dynamic_kernel<T, true, false>), grid, dim3(64), 0, st, p);
  } else {
    if (sr) hipLaunchKernelGGL((quant_dynamic_kernel<T, false, true>), grid, dim3(64), 0, st, p);
    else hipLaunchKernelGGL((quant_dynamic_kernel<T, false, false>), grid, dim3(64), 0, st, p);
  }
}

}  // namespace

// Row output only; arguments already validated by alto_mxfp4_quantize_pitched.
int quantize_dynamic_launch(const void* x, int dtype, int64_t batch, int64_t M, int64_t C, int64_t ld_x, int64_t bs_x, uint8_t* codes,
                            uint8_t* scales, int64_t ld_codes, int is_2d, int sr, const uint32_t* rand_bits, int64_t ld_rand,
                            int64_t bs_rand, int use_uos, hipStream_t st) {
  DynParams p{x, ld_x, bs_x, rand_bits, ld_rand, bs_rand, codes, scales, ld_codes, (int)M, (int)C, use_uos ? 1 : 0};
  dim3 grid((unsigned)((C / 32 + 1) / 2), (unsigned)((M + 31) / 32), (unsigned)batch);
  if (dtype == ALTO_DT_BF16) launch<__bf16>(p, grid, st, is_2d != 0, sr != 0);
  else launch<float>(p, grid, st, is_2d != 0, sr != 0);
  return check_launch("quantize (dynamic clip)");
}

}  // namespace alto
