// Reference-grade scaled-MFMA GEMM tile routine: one wave computes a 32x32 tile of C = A . B^T straight from
// global memory (no LDS).  It accepts every shape the API allows and serves as the fallback of the tuned kernels.
#pragma once
#include "common.h"

namespace alto {

struct OperandView {
  const uint8_t* codes;   // [rows][K/2], row stride ld (bytes)
  int64_t ld;
  const uint8_t* scales;  // element (row, g) at scales[(is_2d ? row / 32 : row) * ss_r + g * ss_k]
  int64_t ss_r, ss_k;
  int is_2d;
};

// Accumulates groups [g0, g1) (units of 32 along K) for the 32x32 tile whose A rows start at m0 and B rows at n0.
// Rows are clamped to [0, m_hi) / [0, n_hi): out-of-range rows compute garbage that the caller never stores.
__device__ __forceinline__ void mma_tile_32x32_acc(v16f_t& acc, const OperandView& A, const OperandView& B, int64_t m0, int64_t n0,
                                                   int64_t m_lo, int64_t m_hi, int64_t n_hi, int g0, int g1) {
  const int lane = threadIdx.x & 63;
  const int r = lane & 31, h = lane >> 5;
  int64_t am = m0 + r;
  am = am < m_hi ? am : m_hi - 1;
  am = am < m_lo ? m_lo : am;
  int64_t bn = n0 + r;
  bn = bn < n_hi ? bn : n_hi - 1;
  const uint8_t* ap = A.codes + am * A.ld;
  const uint8_t* bp = B.codes + bn * B.ld;
  const uint8_t* asp = A.scales + (A.is_2d ? am / 32 : am) * A.ss_r;
  const uint8_t* bsp = B.scales + (B.is_2d ? bn / 32 : bn) * B.ss_r;
  for (int g = g0 + h; g < g1 + h; g += 2) {
    const bool in = g < g1;  // the second half-wave idles on an odd tail
    v8i_t av = {0, 0, 0, 0, 0, 0, 0, 0}, bv = {0, 0, 0, 0, 0, 0, 0, 0};
    int sa = 127, sb = 127;
    if (in) {
      uint4 a4 = *reinterpret_cast<const uint4*>(ap + (int64_t)g * 16);
      uint4 b4 = *reinterpret_cast<const uint4*>(bp + (int64_t)g * 16);
      av[0] = a4.x; av[1] = a4.y; av[2] = a4.z; av[3] = a4.w;
      bv[0] = b4.x; bv[1] = b4.y; bv[2] = b4.z; bv[3] = b4.w;
      sa = asp[(int64_t)g * A.ss_k];
      sb = bsp[(int64_t)g * B.ss_k];
    }
    acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, acc, 4, 4, 0, sa, 0, sb);
  }
}

__device__ __forceinline__ v16f_t mma_tile_32x32(const OperandView& A, const OperandView& B, int64_t m0, int64_t n0,
                                                 int64_t m_lo, int64_t m_hi, int64_t n_hi, int g0, int g1) {
  v16f_t acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
  mma_tile_32x32_acc(acc, A, B, m0, n0, m_lo, m_hi, n_hi, g0, g1);
  return acc;
}

// Stores a 32x32 accumulator tile; rows in [m_lo, m_hi), columns < n_hi are written.
template <typename OutT>
__device__ __forceinline__ void store_tile_32x32(const v16f_t& acc, OutT* c, int64_t ldc, int64_t m0, int64_t n0,
                                                 int64_t m_lo, int64_t m_hi, int64_t n_hi, float out_scale) {
  const int lane = threadIdx.x & 63;
  const int64_t j = n0 + (lane & 31);
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int64_t i = m0 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
    if (i >= m_lo && i < m_hi && j < n_hi) {
      float val = acc[v] * out_scale;
      if constexpr (sizeof(OutT) == 2) {
        unsigned short hb = (unsigned short)f32_to_bf16_bits(val);
        c[i * ldc + j] = __builtin_bit_cast(OutT, hb);
      } else {
        c[i * ldc + j] = val;
      }
    }
  }
}

}  // namespace alto
