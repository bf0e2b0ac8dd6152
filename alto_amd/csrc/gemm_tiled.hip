// Tuned LDS-tiled MXFP4 GEMM for gfx950: dense entry (one 256x256 tile per 512-thread workgroup, XCD-aware tile order).
#include <mutex>

#include "gemm_tiled.h"
#include "gemm_tile.h"

namespace alto {
namespace {

// Workgroups are dealt round-robin to the 8 XCDs (each with its own L2).  Every XCD gets a contiguous range of the
// tile sequence, and the sequence walks 8 N-tiles per M-tile before moving on, so the ~32 tiles an XCD has in flight
// share A rows and B rows through its L2.
__device__ __forceinline__ bool tile_coords(int wg, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int T = tiles_m * tiles_n;
  const int per_xcd = (T + 7) / 8;
  const int u = (wg & 7) * per_xcd + (wg >> 3);
  if ((wg >> 3) >= per_xcd || u >= T) return false;
  const int GN = 8;
  const int in_group = GN * tiles_m;
  const int group = u / in_group;
  const int first_n = group * GN;
  const int gsize = (tiles_n - first_n) < GN ? (tiles_n - first_n) : GN;
  const int w = u % in_group;
  tn = first_n + w % gsize;
  tm = w / gsize;
  return true;
}

template <typename OutT, bool KTAIL, int LMS, int NST, bool PS>
__global__ __launch_bounds__(GT_THREADS) void gemm_tiled_kernel(OperandView A, OperandView B, int64_t M, int64_t N, int G,
                                                         OutT* c, int64_t ldc, float out_scale, int tiles_m, int tiles_n) {
  extern __shared__ __align__(16) uint8_t smem[];
  int tm, tn;
  if (!tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn)) return;
  const int KB = (G + 15) / 16;
  TileArgs ta{A, B, (int64_t)tm * GT_TM, (int64_t)tn * GT_TN, 0, M, N, G, out_scale,
              (M - 1) * A.ld + G * 16, (N - 1) * B.ld + G * 16,
              PS ? KB * A.ss_k : ((A.is_2d ? M / 32 : M) - 1) * A.ss_r + G, PS ? KB * B.ss_k : ((B.is_2d ? N / 32 : N) - 1) * B.ss_r + G, 0, G};
  gemm_tile_256x256<OutT, KTAIL, LMS, NST, PS>(ta, c, ldc, smem);
}

// Plain scales of one operand -> the packed form the PS kernels read: dst[(kb * rows + row) * 16 + 4 (2 h + ms) + j] =
// scale of group 16 kb + 8 ms + 2 j + h of that row, 127 beyond G.  One thread per (row, block).
__global__ __launch_bounds__(256) void pack_scales_kernel(const uint8_t* __restrict__ src, int64_t ss_r, int64_t ss_k, int is_2d, int64_t rows, int G,
                                                          uint8_t* __restrict__ dst) {
  const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int kb = blockIdx.y;
  if (row >= rows) return;
  const uint8_t* sr = src + (is_2d ? (row >> 5) : row) * ss_r;
  uint32_t w[4];
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const int h = d >> 1, ms = d & 1;
    uint32_t v = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int g = 16 * kb + 8 * ms + 2 * j + h;
      v |= (uint32_t)(g < G ? sr[g * ss_k] : (uint8_t)127) << (8 * j);
    }
    w[d] = v;
  }
  *reinterpret_cast<uint4*>(dst + ((int64_t)kb * rows + row) * 16) = make_uint4(w[0], w[1], w[2], w[3]);
}

template <typename OutT, bool KTAIL, int LMS = -1, int NST = 4, bool PS = false>
int launch_tiled(const OperandView& A, const OperandView& B, int64_t M, int64_t N, int64_t K, void* c, int64_t ldc, float out_scale, hipStream_t st) {
  // the opt-in for > 64 KB of dynamic LDS is per function, set once per process (two host threads may make their first
  // call together: forward on the caller's thread, backward on the autograd thread)
  auto kern = gemm_tiled_kernel<OutT, KTAIL, LMS, NST, PS>;
  static std::once_flag once;
  static hipError_t attr_rc = hipSuccess;
  std::call_once(once, [&] { attr_rc = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, GT_LDS_BYTES); });
  if (attr_rc != hipSuccess) return -1;
  const int tiles_m = (int)((M + GT_TM - 1) / GT_TM), tiles_n = (int)((N + GT_TN - 1) / GT_TN);
  const int T = tiles_m * tiles_n;
  const int per_xcd = (T + 7) / 8;
  hipLaunchKernelGGL(kern, dim3((unsigned)(per_xcd * 8)), dim3(GT_THREADS), GT_LDS_BYTES, st, A, B, M, N, (int)(K / 32), (OutT*)c, ldc, out_scale, tiles_m, tiles_n);
  return 0;
}

}  // namespace

bool gemm_tiled_supported(const OperandView& A, const OperandView& B, int64_t M, int64_t N, int64_t K, const void* c, int c_dtype, int64_t ldc) {
  (void)c_dtype;
  // small problems do not fill 256x256 tiles; the direct kernel handles them
  if (M < 128 || N < 128 || K < 512) return false;   // (scale rows are read 16 bytes = 512 K at a time)
  // the tile kernel reads scale rows with unit stride along K and stores C in aligned 16-byte groups
  if (A.ss_k != 1 || B.ss_k != 1) return false;
  if (!product_below(1ll << 31, M, A.ld) || !product_below(1ll << 31, N, B.ld)) return false;   // 32-bit buffer offsets
  if (!product_below(1ll << 31, M, A.ss_r) || !product_below(1ll << 31, N, B.ss_r)) return false;
  if (N % 8 != 0 || ldc % 8 != 0 || (reinterpret_cast<uintptr_t>(c) & 15) != 0) return false;
  const int64_t tiles = ((M + GT_TM - 1) / GT_TM) * ((N + GT_TN - 1) / GT_TN);
  return tiles < (1ll << 28);
}

void gemm_tiled_launch(const OperandView& A, const OperandView& B, int64_t M, int64_t N, int64_t K, void* c, int c_dtype, int64_t ldc,
                       float out_scale, hipStream_t st) {
  const bool tail = (K / 32) % 16 != 0;   // K not a multiple of 512: the last scale block of a row is partial
#define ALTO_TILED_LAUNCH(T, ...) launch_tiled<T, __VA_ARGS__>(A, B, M, N, K, c, ldc, out_scale, st)
  if (!tail) {
    if (c_dtype == ALTO_DT_BF16) ALTO_TILED_LAUNCH(__bf16, false);
    else ALTO_TILED_LAUNCH(float, false);
  } else if (c_dtype != ALTO_DT_BF16) {
    ALTO_TILED_LAUNCH(float, true);   // (fp32 output: the general ending)
  } else {
    // K is known here: the kernel that ends the reduction exactly where K ends
    int lms, nst;
    gemm_tile_last_stage(K / 32, lms, nst);
    switch (lms * 4 + nst - 1) {
      case 0: ALTO_TILED_LAUNCH(__bf16, true, 0, 1); break;
      case 1: ALTO_TILED_LAUNCH(__bf16, true, 0, 2); break;
      case 2: ALTO_TILED_LAUNCH(__bf16, true, 0, 3); break;
      case 3: ALTO_TILED_LAUNCH(__bf16, true, 0, 4); break;
      case 4: ALTO_TILED_LAUNCH(__bf16, true, 1, 1); break;
      case 5: ALTO_TILED_LAUNCH(__bf16, true, 1, 2); break;
      case 6: ALTO_TILED_LAUNCH(__bf16, true, 1, 3); break;
      default: ALTO_TILED_LAUNCH(__bf16, true, 1, 4); break;
    }
  }
#undef ALTO_TILED_LAUNCH
}

// Both operands with packed scales (A.scales / B.scales = packed base, ss_k = bytes per block), bf16 output.
void gemm_tiled_launch_ps(const OperandView& A, const OperandView& B, int64_t M, int64_t N, int64_t K, void* c, int64_t ldc, float out_scale,
                          hipStream_t st) {
  const bool tail = (K / 32) % 16 != 0;
#define ALTO_TILED_LAUNCH(...) launch_tiled<__bf16, __VA_ARGS__, true>(A, B, M, N, K, c, ldc, out_scale, st)
  if (!tail) {
    ALTO_TILED_LAUNCH(false, -1, 4);
  } else {
    int lms, nst;
    gemm_tile_last_stage(K / 32, lms, nst);
    switch (lms * 4 + nst - 1) {
      case 0: ALTO_TILED_LAUNCH(true, 0, 1); break;
      case 1: ALTO_TILED_LAUNCH(true, 0, 2); break;
      case 2: ALTO_TILED_LAUNCH(true, 0, 3); break;
      case 3: ALTO_TILED_LAUNCH(true, 0, 4); break;
      case 4: ALTO_TILED_LAUNCH(true, 1, 1); break;
      case 5: ALTO_TILED_LAUNCH(true, 1, 2); break;
      case 6: ALTO_TILED_LAUNCH(true, 1, 3); break;
      default: ALTO_TILED_LAUNCH(true, 1, 4); break;
    }
  }
#undef ALTO_TILED_LAUNCH
}

void pack_scales_launch(const uint8_t* src, int64_t ss_r, int64_t ss_k, int is_2d, int64_t rows, int64_t G, uint8_t* dst, hipStream_t st) {
  const int KB = (int)((G + 15) / 16);
  hipLaunchKernelGGL(pack_scales_kernel, dim3((unsigned)((rows + 255) / 256), (unsigned)KB), dim3(256), 0, st, src, ss_r, ss_k, is_2d, rows, (int)G, dst);
}

}  // namespace alto
