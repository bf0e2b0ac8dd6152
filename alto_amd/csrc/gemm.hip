// Block-scaled MXFP4 GEMM entry point (dense): C[M][N] = A[M][K] . B[N][K]^T on gfx950 scaled MFMA.
#include "common.h"
#include "gemm_simple.h"
#include "gemm_tiled.h"

namespace alto {
namespace {

template <typename OutT>
__global__ __launch_bounds__(256) void gemm_simple_kernel(OperandView A, OperandView B, int64_t M, int64_t N, int G,
                                                          OutT* c, int64_t ldc, float out_scale) {
  const int wave = threadIdx.x >> 6;
  const int64_t m0 = (int64_t)blockIdx.y * 64 + (wave >> 1) * 32;
  const int64_t n0 = (int64_t)blockIdx.x * 64 + (wave & 1) * 32;
  if (m0 >= M || n0 >= N) return;
  v16f_t acc = mma_tile_32x32(A, B, m0, n0, 0, M, N, 0, G);
  store_tile_32x32<OutT>(acc, c, ldc, m0, n0, 0, M, N, out_scale);
}

}  // namespace
}  // namespace alto

extern "C" int alto_mxfp4_gemm(const uint8_t* a, int64_t lda, const uint8_t* a_scales, int64_t a_ss_r, int64_t a_ss_k, int a_is_2d,
                               const uint8_t* b, int64_t ldb, const uint8_t* b_scales, int64_t b_ss_r, int64_t b_ss_k, int b_is_2d,
                               int64_t M, int64_t N, int64_t K, void* c, int c_dtype, int64_t ldc, float out_scale, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(a && b && a_scales && b_scales && c, "gemm: NULL pointer");
  ALTO_REQUIRE(M >= 0 && N >= 0 && K >= 0, "gemm: negative size");
  ALTO_REQUIRE(K % 32 == 0, "gemm: K (%lld) must be a multiple of 32", (long long)K);
  ALTO_REQUIRE(!a_is_2d || M % 32 == 0, "gemm: 2D scales for A need M (%lld) %% 32 == 0", (long long)M);
  ALTO_REQUIRE(!b_is_2d || N % 32 == 0, "gemm: 2D scales for B need N (%lld) %% 32 == 0", (long long)N);
  ALTO_REQUIRE(lda >= K / 2 && ldb >= K / 2 && lda % 16 == 0 && ldb % 16 == 0, "gemm: lda/ldb must be >= K/2 and multiples of 16 bytes");
  ALTO_REQUIRE(((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15) == 0, "gemm: a and b must be 16-byte aligned");
  ALTO_REQUIRE(ldc >= N, "gemm: ldc < N");
  ALTO_REQUIRE(a_ss_r >= 0 && a_ss_k >= 0 && b_ss_r >= 0 && b_ss_k >= 0, "gemm: negative scale stride");
  ALTO_REQUIRE(c_dtype == ALTO_DT_BF16 || c_dtype == ALTO_DT_F32, "gemm: bad c_dtype %d", c_dtype);
  ALTO_REQUIRE((reinterpret_cast<uintptr_t>(c) & (c_dtype == ALTO_DT_F32 ? 3 : 1)) == 0, "gemm: c must be aligned to its element size");
  ALTO_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), "gemm: size out of range");
  if (M == 0 || N == 0) return ALTO_MXFP4_OK;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  OperandView A{a, lda, a_scales, a_ss_r, a_ss_k, a_is_2d};
  OperandView B{b, ldb, b_scales, b_ss_r, b_ss_k, b_is_2d};

  if (gemm_tiled_supported(A, B, M, N, K, c, c_dtype, ldc)) {
    gemm_tiled_launch(A, B, M, N, K, c, c_dtype, ldc, out_scale, st);
    return check_launch("gemm(tiled)");
  }
  dim3 grid((unsigned)((N + 63) / 64), (unsigned)((M + 63) / 64));
  ALTO_REQUIRE(grid.y <= 65535u, "gemm: M too large for the fallback kernel");
  if (c_dtype == ALTO_DT_BF16)
    hipLaunchKernelGGL(gemm_simple_kernel<__bf16>, grid, dim3(256), 0, st, A, B, M, N, (int)(K / 32), (__bf16*)c, ldc, out_scale);
  else
    hipLaunchKernelGGL(gemm_simple_kernel<float>, grid, dim3(256), 0, st, A, B, M, N, (int)(K / 32), (float*)c, ldc, out_scale);
  return check_launch("gemm");
}

extern "C" int64_t alto_mxfp4_packed_scales_bytes(int64_t rows, int64_t K) {
  if (rows < 0 || K < 0 || K % 32 != 0) return 0;
  const int64_t blocks = (K / 32 + 15) / 16;
  return alto::product_below(INT64_MAX, blocks, rows, 16) ? blocks * rows * 16 : 0;
}

extern "C" int alto_mxfp4_pack_scales(const uint8_t* scales, int64_t ss_r, int64_t ss_k, int is_2d, int64_t rows, int64_t K, uint8_t* packed, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(scales && packed, "pack_scales: NULL pointer");
  ALTO_REQUIRE(rows >= 0 && K >= 0 && K % 32 == 0, "pack_scales: K (%lld) must be a multiple of 32", (long long)K);
  ALTO_REQUIRE(!is_2d || rows % 32 == 0, "pack_scales: 2D scales need rows (%lld) %% 32 == 0", (long long)rows);
  ALTO_REQUIRE((reinterpret_cast<uintptr_t>(packed) & 15) == 0, "pack_scales: packed must be 16-byte aligned");
  ALTO_REQUIRE((K / 32 + 15) / 16 <= 65535 && rows < (1ll << 31), "pack_scales: size out of range");
  if (rows == 0 || K == 0) return ALTO_MXFP4_OK;
  pack_scales_launch(scales, ss_r, ss_k, is_2d, rows, K / 32, packed, reinterpret_cast<hipStream_t>(stream));
  return check_launch("pack_scales");
}

extern "C" int alto_mxfp4_gemm_ps(const uint8_t* a, int64_t lda, const uint8_t* a_packed, const uint8_t* b, int64_t ldb, const uint8_t* b_packed,
                                  int64_t M, int64_t N, int64_t K, void* c, int64_t ldc, float out_scale, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(a && b && a_packed && b_packed && c, "gemm_ps: NULL pointer");
  ALTO_REQUIRE(M >= 0 && N >= 0 && K >= 0 && K % 32 == 0, "gemm_ps: K (%lld) must be a multiple of 32", (long long)K);
  ALTO_REQUIRE(lda >= K / 2 && ldb >= K / 2 && lda % 16 == 0 && ldb % 16 == 0, "gemm_ps: lda/ldb must be >= K/2 and multiples of 16 bytes");
  ALTO_REQUIRE(((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(a_packed) | reinterpret_cast<uintptr_t>(b_packed)) & 15) == 0,
               "gemm_ps: a, b and their packed scales must be 16-byte aligned");
  ALTO_REQUIRE(ldc >= N, "gemm_ps: ldc < N");
  ALTO_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), "gemm_ps: size out of range");
  if (M == 0 || N == 0) return ALTO_MXFP4_OK;
  const int64_t KB = (K / 32 + 15) / 16;
  OperandView A{a, lda, a_packed, 16, M * 16, 0};
  OperandView B{b, ldb, b_packed, 16, N * 16, 0};
  // the packed form exists for the 256x256 tile kernel only: same shape conditions as alto_mxfp4_gemm's choice of it
  OperandView Ap{a, lda, a_packed, 1, 1, 0}, Bp{b, ldb, b_packed, 1, 1, 0};
  if (!(gemm_tiled_supported(Ap, Bp, M, N, K, c, ALTO_DT_BF16, ldc) && product_below(1ll << 31, KB, M, 16) && product_below(1ll << 31, KB, N, 16))) {
    set_error("gemm_ps: shape (%lld, %lld, %lld) is not served by the tile kernel; use alto_mxfp4_gemm with plain scales", (long long)M, (long long)N, (long long)K);
    return ALTO_MXFP4_ENOTIMPL;
  }
  gemm_tiled_launch_ps(A, B, M, N, K, c, ldc, out_scale, reinterpret_cast<hipStream_t>(stream));
  return check_launch("gemm_ps");
}
