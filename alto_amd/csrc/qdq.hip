// Fused quantize -> dequantize (gfx950): y = convert_from_mxfp4(convert_to_mxfp4(x)) in one pass over x, round to
// nearest even, blocks of 32 along the contiguous dim or 32x32.  Used where only the quantisation error is wanted
// (weight de-oscillation), so no codes or scales are written.
#include "common.h"

namespace alto {
namespace {

typedef unsigned short us2q_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pk_max_u16q(uint32_t a, uint32_t b) {
  us2q_t r = __builtin_elementwise_max(__builtin_bit_cast(us2q_t, a), __builtin_bit_cast(us2q_t, b));
  return __builtin_bit_cast(uint32_t, r);
}

// One workgroup (256 threads): 32 rows x 256 columns; a lane holds 8 consecutive elements of a row for 4 rows.
template <typename T, bool B2D>
__global__ __launch_bounds__(256) void qdq_kernel(const T* __restrict__ x, int64_t ld_x, int64_t bs_x, T* __restrict__ y, int64_t ld_y,
                                                  int64_t bs_y, int M, int C, int uos) {
  constexpr bool BF = sizeof(T) == 2;
  __shared__ uint32_t blkmax[8];
  const int tid = threadIdx.x;
  const int col0 = blockIdx.x * 256, row0 = blockIdx.y * 32;
  const int64_t b = blockIdx.z;
  if (B2D) {
    if (tid < 8) blkmax[tid] = 0;
    __syncthreads();
  }
  const int chunk = tid & 31;
  const int c = col0 + chunk * 8;
  uint32_t w[4][BF ? 4 : 8];
  uint32_t amax[4];
  bool valid[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = (tid >> 5) + 8 * i;
    valid[i] = (row0 + r < M) && (c < C);
#pragma unroll
    for (int e = 0; e < (BF ? 4 : 8); ++e) w[i][e] = 0;
    if (valid[i]) {
      const uint4* src = reinterpret_cast<const uint4*>(x + b * bs_x + (int64_t)(row0 + r) * ld_x + c);
      uint4 v0 = src[0];
      w[i][0] = v0.x; w[i][1] = v0.y; w[i][2] = v0.z; w[i][3] = v0.w;
      if constexpr (!BF) {
        uint4 v1 = src[1];
        w[i][4] = v1.x; w[i][5] = v1.y; w[i][6] = v1.z; w[i][7] = v1.w;
      }
    }
    uint32_t a;
    if constexpr (BF) {
      a = pk_max_u16q(pk_max_u16q(w[i][0] & 0x7FFF7FFFu, w[i][1] & 0x7FFF7FFFu), pk_max_u16q(w[i][2] & 0x7FFF7FFFu, w[i][3] & 0x7FFF7FFFu));
      a = max(a & 0xFFFFu, a >> 16);
    } else {
      a = 0;
#pragma unroll
      for (int e = 0; e < 8; ++e) a = max(a, w[i][e] & 0x7FFFFFFFu);
    }
    a = max(a, dpp_u32<ALTO_DPP_QUAD_XOR1>(a));
    a = max(a, dpp_u32<ALTO_DPP_QUAD_XOR2>(a));
    amax[i] = a;
    if (B2D && (tid & 3) == 0) atomicMax(&blkmax[chunk >> 2], a);
  }
  if (B2D) __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (!valid[i]) continue;
    const int r = (tid >> 5) + 8 * i;
    const uint32_t a = B2D ? blkmax[chunk >> 2] : amax[i];
    uint32_t s;
    if (uos) s = e8m0_uos(BF ? u2f(a << 16) : u2f(a));
    else s = BF ? e8m0_from_bf16_bits(a) : e8m0_from_f32_bits(a);
    const float scale_f = u2f(s << 23);
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if constexpr (BF) v[e] = (e & 1) ? bf16_hi(w[i][e >> 1]) : bf16_lo(w[i][e >> 1]);
      else v[e] = u2f(w[i][e]);
    }
    uint32_t codes = 0;
    codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, v[0], v[1], scale_f, 0);
    codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, v[2], v[3], scale_f, 1);
    codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, v[4], v[5], scale_f, 2);
    codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(codes, v[6], v[7], scale_f, 3);
    float o[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = e2m1_decode((codes >> (4 * e)) & 0xFu) * scale_f;
    T* dst = y + b * bs_y + (int64_t)(row0 + r) * ld_y + c;
    if constexpr (BF) {
      uint4 pk;
      pk.x = f32_to_bf16_bits(o[0]) | (f32_to_bf16_bits(o[1]) << 16);
      pk.y = f32_to_bf16_bits(o[2]) | (f32_to_bf16_bits(o[3]) << 16);
      pk.z = f32_to_bf16_bits(o[4]) | (f32_to_bf16_bits(o[5]) << 16);
      pk.w = f32_to_bf16_bits(o[6]) | (f32_to_bf16_bits(o[7]) << 16);
      *reinterpret_cast<uint4*>(dst) = pk;
    } else {
      *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
      *reinterpret_cast<float4*>(dst + 4) = make_float4(o[4], o[5], o[6], o[7]);
    }
  }
}

}  // namespace
}  // namespace alto

extern "C" int alto_mxfp4_qdq(const void* x, int dtype, int64_t batch, int64_t M, int64_t C, int64_t ld_x, int64_t bs_x,
                              void* y, int64_t ld_y, int64_t bs_y, int is_2d, int use_uos, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(x && y, "qdq: NULL pointer");
  ALTO_REQUIRE(dtype == ALTO_DT_BF16 || dtype == ALTO_DT_F32, "qdq: dtype %d is neither bf16 (0) nor f32 (1)", dtype);
  ALTO_REQUIRE(batch >= 0 && M >= 0 && C >= 0 && C % 32 == 0, "qdq: C (%lld) must be a multiple of 32", (long long)C);
  ALTO_REQUIRE(!is_2d || M % 32 == 0, "qdq: 2D blocks need M (%lld) %% 32 == 0", (long long)M);
  ALTO_REQUIRE(M < (1ll << 31) && C < (1ll << 31) && batch < 65536 && (M + 31) / 32 <= 65535, "qdq: size out of range");
  const int64_t vec = dtype == ALTO_DT_BF16 ? 8 : 4;
  ALTO_REQUIRE(ld_x >= C && ld_y >= C && ld_x % vec == 0 && ld_y % vec == 0 && bs_x % vec == 0 && bs_y % vec == 0,
               "qdq: row/batch strides must be >= C and multiples of %lld elements", (long long)vec);
  ALTO_REQUIRE(((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0, "qdq: x and y must be 16-byte aligned");
  if (batch == 0 || M == 0 || C == 0) return ALTO_MXFP4_OK;
  dim3 grid((unsigned)((C + 255) / 256), (unsigned)((M + 31) / 32), (unsigned)batch);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int uos = use_uos ? 1 : 0;
  if (dtype == ALTO_DT_BF16) {
    if (is_2d) hipLaunchKernelGGL((qdq_kernel<__bf16, true>), grid, dim3(256), 0, st, (const __bf16*)x, ld_x, bs_x, (__bf16*)y, ld_y, bs_y, (int)M, (int)C, uos);
    else hipLaunchKernelGGL((qdq_kernel<__bf16, false>), grid, dim3(256), 0, st, (const __bf16*)x, ld_x, bs_x, (__bf16*)y, ld_y, bs_y, (int)M, (int)C, uos);
  } else {
    if (is_2d) hipLaunchKernelGGL((qdq_kernel<float, true>), grid, dim3(256), 0, st, (const float*)x, ld_x, bs_x, (float*)y, ld_y, bs_y, (int)M, (int)C, uos);
    else hipLaunchKernelGGL((qdq_kernel<float, false>), grid, dim3(256), 0, st, (const float*)x, ld_x, bs_x, (float*)y, ld_y, bs_y, (int)M, (int)C, uos);
  }
  return check_launch("qdq");
}
