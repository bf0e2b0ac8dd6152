// Shared device/host helpers for the MXFP4 kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/alto_mxfp4.h"

namespace alto {

// ----------------------------------------------------------------------------- host: error reporting
void set_error(const char* fmt, ...);
int check_launch(const char* what);
int quantize_dynamic_launch(const void* x, int dtype, int64_t batch, int64_t M, int64_t C, int64_t ld_x, int64_t bs_x, uint8_t* codes,
                            uint8_t* scales, int64_t ld_codes, int is_2d, int sr, const uint32_t* rand_bits, int64_t ld_rand,
                            int64_t bs_rand, int use_uos, hipStream_t st);

// a * b * c < limit for non-negative factors; false when a factor is negative or the product leaves 64 bits on the way
inline bool product_below(int64_t limit, int64_t a, int64_t b, int64_t c = 1) {
  int64_t p;
  return a >= 0 && b >= 0 && c >= 0 && !__builtin_mul_overflow(a, b, &p) && !__builtin_mul_overflow(p, c, &p) && p < limit;
}

#define ALTO_REQUIRE(cond, ...)            \
  do {                                     \
    if (!(cond)) {                         \
      alto::set_error(__VA_ARGS__);        \
      return ALTO_MXFP4_EINVAL;            \
    }                                      \
  } while (0)

// ----------------------------------------------------------------------------- device: bit casts
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef int v8i_t __attribute__((ext_vector_type(8)));
typedef int v4i_t __attribute__((ext_vector_type(4)));
typedef float v4f_t __attribute__((ext_vector_type(4)));
typedef float v16f_t __attribute__((ext_vector_type(16)));

__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ float bf16_lo(uint32_t w) { return u2f(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return u2f(w & 0xFFFF0000u); }

// fp32 -> bf16 bits, round to nearest even (finite inputs; NaN payloads are not preserved specially)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = f2u(f);
  return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

// two floats -> packed bf16 (round to nearest even), one v_cvt_pk_bf16_f32
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef float f2_t __attribute__((ext_vector_type(2)));
  bf16x2_t p = __builtin_convertvector(f2_t{lo, hi}, bf16x2_t);
  return __builtin_bit_cast(uint32_t, p);
}

// ----------------------------------------------------------------------------- device: E8M0 scale rule
// Biased exponent of the block absmax after rounding it to one mantissa bit, minus 2, clamped below at 1.
__device__ __forceinline__ uint32_t e8m0_from_bf16_bits(uint32_t absbits16) {
  uint32_t e = ((absbits16 + 0x20u) >> 7) & 0x1FFu;
  return e > 3u ? e - 2u : 1u;
}
__device__ __forceinline__ uint32_t e8m0_from_f32_bits(uint32_t absbits32) {
  uint32_t e = ((absbits32 + 0x200000u) >> 23) & 0x1FFu;
  return e > 3u ? e - 2u : 1u;
}
// "UOS" rule: ceil(log2(absmax / 7.25)) + 127, all-zero block -> 128, clamped below at 1.
__device__ __forceinline__ uint32_t e8m0_uos(float absmax) {
  float s = ceilf(log2f(absmax / 7.25f));
  if (absmax == 0.0f) s = 1.0f;
  s += 127.0f;
  if (s < 1.0f) s = 1.0f;
  return (uint32_t)s & 0xFFu;
}

// ----------------------------------------------------------------------------- device: E2M1 encode
// Stochastic rounding of q (already divided by the scale, any sign) with 32 random bits; returns the 3-bit magnitude
// code (0..7).  The rule of the reference (triton_fp4_ops.py:49-61,79-80):
//   |q| >= 1: add the low 22 random bits under the kept mantissa bit and truncate, saturating at code 7 (the clamp of |q|
//             to 6 does the saturation: 6.0 has no bits under the kept one);
//   |q| <  1: g = 2|q| in [0, 2): code = floor(g) + (r <= trunc(frac(g) * 2^32)), an unsigned 32-bit compare.
__device__ __forceinline__ uint32_t e2m1_sr_mag(float q, uint32_t r) {
  const float m6 = __builtin_fminf(__builtin_fabsf(q), 6.0f);
  const uint32_t n = (f2u(m6) - 0x3F000000u + (r & 0x3FFFFFu)) >> 22;
  const float g = m6 + m6;
  const uint32_t thr = (uint32_t)__builtin_ldexpf(__builtin_amdgcn_fractf(g), 32);
  const uint32_t den = (uint32_t)g + (r <= thr ? 1u : 0u);
  return m6 < 1.0f ? den : n;
}

// ----------------------------------------------------------------------------- device: Philox4x32-10
// Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3" (SC'11): counter-based, so any word of the
// stream can be regenerated from (key, counter).
__device__ __forceinline__ void philox_round(uint32_t (&c)[4], uint32_t k0, uint32_t k1) {
  const uint64_t p0 = (uint64_t)0xD2511F53u * c[0], p1 = (uint64_t)0xCD9E8D57u * c[2];   // 32 x 32 -> 64 bits each
  const uint32_t lo0 = (uint32_t)p0, hi0 = (uint32_t)(p0 >> 32), lo1 = (uint32_t)p1, hi1 = (uint32_t)(p1 >> 32);
  const uint32_t n0 = hi1 ^ c[1] ^ k0, n2 = hi0 ^ c[3] ^ k1;
  c[0] = n0; c[1] = lo1; c[2] = n2; c[3] = lo0;
}

__device__ __forceinline__ uint4 philox4x32_10(uint64_t ctr_lo, uint64_t ctr_hi, uint64_t key) {
  uint32_t c[4] = {(uint32_t)ctr_lo, (uint32_t)(ctr_lo >> 32), (uint32_t)ctr_hi, (uint32_t)(ctr_hi >> 32)};
  uint32_t k0 = (uint32_t)key, k1 = (uint32_t)(key >> 32);
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    philox_round(c, k0, k1);
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return make_uint4(c[0], c[1], c[2], c[3]);
}

// Round-to-nearest-even of a non-negative magnitude; software form (used where the packed HW convert does not fit).
__device__ __forceinline__ uint32_t e2m1_rne_mag(float m) {
  uint32_t mb = f2u(m);
  uint32_t n = mb - 0x3F000000u + 0x1FFFFFu + ((mb >> 22) & 1u);
  n = (n < 0x01FFFFFFu ? n : 0x01FFFFFFu) >> 22;
  uint32_t den = f2u(m + 4194304.0f) - 0x4A800000u;
  return m < 1.0f ? den : n;
}

// E2M1 code (sign in bit 3) -> value: 0, 0.5, then (1 + m/2) * 2^(e-1)
__device__ __forceinline__ float e2m1_decode(uint32_t code) {
  uint32_t c = code & 7u;
  uint32_t bits = (((c >> 1) + 126u) << 23) | ((c & 1u) << 22);
  bits = c == 0u ? 0u : (c == 1u ? 0x3F000000u : bits);
  return u2f(bits | ((code & 8u) << 28));
}

// ----------------------------------------------------------------------------- device: cross-lane
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
// quad_perm controls: lane ^ 1 and lane ^ 2 inside each group of 4 lanes
#define ALTO_DPP_QUAD_XOR1 0xB1
#define ALTO_DPP_QUAD_XOR2 0x4E

}  // namespace alto
