// MXFP4 dequantizer and nibble transpose (gfx950).
#include "common.h"

namespace alto {
namespace {

// one thread: 8 codes (one dword of packed data) of one row
template <typename OutT>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t* __restrict__ codes, const uint8_t* __restrict__ scales,
                                                      int64_t R, int64_t C, int is_2d, OutT* __restrict__ out,
                                                      int64_t osr, int64_t osc, int static_clip) {
  const int64_t chunks_per_row = C / 8;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= R * chunks_per_row) return;
  const int64_t r = idx / chunks_per_row;
  const int64_t c0 = (idx % chunks_per_row) * 8;
  const uint32_t w = *reinterpret_cast<const uint32_t*>(codes + r * (C / 2) + c0 / 2);
  const uint32_t s = scales[(is_2d ? r / 32 : r) * (C / 32) + c0 / 32];
  const float sf = u2f(s << 23);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float v = e2m1_decode((w >> (4 * e)) & 0xFu) * sf;
    if (static_clip) v = v * (4.0f / 3.0f);
    OutT o;
    if constexpr (sizeof(OutT) == 2) {
      unsigned short hb = (unsigned short)f32_to_bf16_bits(v);
      o = __builtin_bit_cast(OutT, hb);
    } else {
      o = v;
    }
    out[r * osr + (c0 + e) * osc] = o;
  }
}

// 64x64 code tile through LDS: in [R][C/2] (packed along C) -> out [C][R/2] (packed along R)
__global__ __launch_bounds__(256) void transpose_codes_kernel(const uint8_t* __restrict__ in, int64_t R, int64_t C, uint8_t* __restrict__ out) {
  __shared__ uint8_t t[64][65];  // unpacked codes
  const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
  const int tid = threadIdx.x;
  // 64 rows x 32 bytes: thread reads one byte at a time (8 passes)
#pragma unroll
  for (int pass = 0; pass < 8; ++pass) {
    int lr = pass * 8 + tid / 32, lb = tid % 32;
    int64_t r = r0 + lr, cb = c0 / 2 + lb;
    uint8_t v = (r < R && cb < C / 2) ? in[r * (C / 2) + cb] : 0;
    t[lr][2 * lb] = v & 0xF;
    t[lr][2 * lb + 1] = v >> 4;
  }
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 8; ++pass) {
    int lc = pass * 8 + tid / 32, lb = tid % 32;  // output row = column lc, output byte lb covers rows 2lb, 2lb+1
    int64_t c = c0 + lc, rb = r0 / 2 + lb;
    if (c < C && rb < R / 2) out[c * (R / 2) + rb] = t[2 * lb][lc] | (t[2 * lb + 1][lc] << 4);
  }
}

}  // namespace
}  // namespace alto

extern "C" int alto_mxfp4_dequantize(const uint8_t* codes, const uint8_t* scales, int64_t R, int64_t C, int is_2d,
                                     void* out, int out_dtype, int64_t out_stride_r, int64_t out_stride_c,
                                     int clip_mode, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(codes && scales && out, "dequantize: NULL pointer");
  ALTO_REQUIRE(R >= 0 && C >= 0 && C % 32 == 0, "dequantize: C (%lld) must be a multiple of 32", (long long)C);
  ALTO_REQUIRE(!is_2d || R % 32 == 0, "dequantize: 2D blocks need R (%lld) %% 32 == 0", (long long)R);
  ALTO_REQUIRE(out_dtype == ALTO_DT_BF16 || out_dtype == ALTO_DT_F32, "dequantize: bad out_dtype %d", out_dtype);
  ALTO_REQUIRE((reinterpret_cast<uintptr_t>(codes) & 3) == 0, "dequantize: codes must be 4-byte aligned");
  ALTO_REQUIRE((reinterpret_cast<uintptr_t>(out) & (out_dtype == ALTO_DT_F32 ? 3 : 1)) == 0, "dequantize: out must be aligned to its element size");
  ALTO_REQUIRE(R < (1ll << 31) && C < (1ll << 31) && product_below(1ll << 39, R, C / 8), "dequantize: %lld x %lld exceeds the grid", (long long)R, (long long)C);
  if (R == 0 || C == 0) return ALTO_MXFP4_OK;
  const int64_t n = R * (C / 8);
  dim3 grid((unsigned)((n + 255) / 256));
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int sc = clip_mode == ALTO_CLIP_STATIC;
  if (out_dtype == ALTO_DT_BF16)
    hipLaunchKernelGGL(dequant_kernel<__bf16>, grid, dim3(256), 0, st, codes, scales, R, C, is_2d, (__bf16*)out, out_stride_r, out_stride_c, sc);
  else
    hipLaunchKernelGGL(dequant_kernel<float>, grid, dim3(256), 0, st, codes, scales, R, C, is_2d, (float*)out, out_stride_r, out_stride_c, sc);
  return check_launch("dequantize");
}

extern "C" int alto_mxfp4_transpose_codes(const uint8_t* in, int64_t R, int64_t C, uint8_t* out, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(in && out, "transpose_codes: NULL pointer");
  ALTO_REQUIRE(R >= 0 && C >= 0 && R % 2 == 0 && C % 2 == 0, "transpose_codes: R and C must be even");
  ALTO_REQUIRE(R < (1ll << 31) && C < (1ll << 31), "transpose_codes: size out of range");
  if (R == 0 || C == 0) return ALTO_MXFP4_OK;
  dim3 grid((unsigned)((C + 63) / 64), (unsigned)((R + 63) / 64));
  ALTO_REQUIRE(grid.y <= 65535u, "transpose_codes: R too large");
  hipLaunchKernelGGL(transpose_codes_kernel, grid, dim3(256), 0, reinterpret_cast<hipStream_t>(stream), in, R, C, out);
  return check_launch("transpose_codes");
}
