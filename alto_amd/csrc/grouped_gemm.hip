// Ragged grouped MXFP4 GEMMs for MoE experts (gfx950): forward / dX (rows grouped by expert) and dW (reduction grouped by expert).
#include "common.h"
#include "gemm_simple.h"

namespace alto {
namespace {

// Maps a linear tile index onto (group, first row) by walking the offsets: group g owns ceil(len_g / tile_m) row
// tiles.  Index num_groups stands for the unrouted tail [offs[G], M_total), which is zero-filled.
struct TileRef {
  int group;  // -1: no such tile
  int64_t m0, m_lo, m_hi;
};

__device__ __forceinline__ TileRef locate_tile(const int32_t* offs, int num_groups, int64_t M_total, int64_t t, int tile_m) {
  TileRef ref{-1, 0, 0, 0};
  int64_t lo = offs[0];
  for (int g = 0; g <= num_groups; ++g) {
    int64_t hi = g < num_groups ? (int64_t)offs[g + 1] : M_total;
    hi = hi < lo ? lo : (hi > M_total ? M_total : hi);  // malformed offsets never index out of the buffers
    int64_t nt = (hi - lo + tile_m - 1) / tile_m;
    if (t < nt) {
      ref.group = g;
      ref.m_lo = lo;
      ref.m_hi = hi;
      ref.m0 = lo + t * tile_m;
      return ref;
    }
    t -= nt;
    lo = hi;
  }
  return ref;
}

template <typename OutT>
__global__ __launch_bounds__(256) void grouped_simple_kernel(OperandView A, const uint8_t* w, int64_t w_stride_e, int64_t ldw,
                                                             const uint8_t* w_scales, int64_t ws_stride_e, int64_t ws_r, int64_t ws_k, int w_is_2d,
                                                             const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts,
                                                             int64_t M_total, int64_t N, int G, OutT* out, int64_t ldo) {
  TileRef t = locate_tile(offs, num_groups, M_total, blockIdx.y, 64);
  if (t.group < 0) return;
  int expert = num_experts;  // "no expert": zero fill
  if (t.group < num_groups) {
    expert = group_expert ? group_expert[t.group] : t.group;
    if (expert < 0 || expert >= num_experts) expert = num_experts;
  }
  const int wave = threadIdx.x >> 6;
  const int64_t m0 = t.m0 + (wave >> 1) * 32;
  const int64_t n0 = (int64_t)blockIdx.x * 64 + (wave & 1) * 32;
  if (m0 >= t.m_hi || n0 >= N) return;
  v16f_t acc;
  if (expert == num_experts) {
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
  } else {
    OperandView B{w + expert * w_stride_e, ldw, w_scales + expert * ws_stride_e, ws_r, ws_k, w_is_2d};
    acc = mma_tile_32x32(A, B, m0, n0, t.m_lo, t.m_hi, N, 0, G);
  }
  store_tile_32x32<OutT>(acc, out, ldo, m0, n0, t.m_lo, t.m_hi, N, 1.0f);
}

// dW[e] tile (n0, k0): reduction over the token groups of expert e
template <typename OutT>
__global__ __launch_bounds__(256) void grouped_dw_simple_kernel(OperandView GO, OperandView X, const int32_t* offs, const int32_t* group_expert,
                                                                int num_groups, int64_t M_total, int64_t N, int64_t K,
                                                                OutT* dw, int64_t s_e, int64_t s_n, int64_t s_k, float out_scale) {
  const int e = blockIdx.z;
  const int wave = threadIdx.x >> 6;
  const int64_t n0 = (int64_t)blockIdx.y * 64 + (wave >> 1) * 32;
  const int64_t k0 = (int64_t)blockIdx.x * 64 + (wave & 1) * 32;
  if (n0 >= N || k0 >= K) return;
  v16f_t acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
  const int gmax = (int)(M_total / 32);
  if (group_expert == nullptr) {
    int g0 = offs[e] / 32, g1 = offs[e + 1] / 32;
    g0 = g0 < 0 ? 0 : g0;
    g1 = g1 > gmax ? gmax : g1;
    mma_tile_32x32_acc(acc, GO, X, n0, k0, 0, N, K, g0, g1);
  } else {
    for (int g = 0; g < num_groups; ++g) {
      if (group_expert[g] != e) continue;
      int g0 = offs[g] / 32, g1 = offs[g + 1] / 32;
      g0 = g0 < 0 ? 0 : g0;
      g1 = g1 > gmax ? gmax : g1;
      mma_tile_32x32_acc(acc, GO, X, n0, k0, 0, N, K, g0, g1);
    }
  }
  const int lane = threadIdx.x & 63;
  const int64_t j = k0 + (lane & 31);
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int64_t i = n0 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
    if (i < N && j < K) {
      float val = acc[v] * out_scale;
      OutT* dst = dw + e * s_e + i * s_n + j * s_k;
      if constexpr (sizeof(OutT) == 2) {
        unsigned short hb = (unsigned short)f32_to_bf16_bits(val);
        *dst = __builtin_bit_cast(OutT, hb);
      } else {
        *dst = val;
      }
    }
  }
}

}  // namespace
}  // namespace alto

extern "C" int alto_mxfp4_grouped_gemm(const uint8_t* a, int64_t lda, const uint8_t* a_scales, int64_t a_ss_r, int64_t a_ss_k, int a_is_2d,
                                       const uint8_t* w, int64_t w_stride_e, int64_t ldw,
                                       const uint8_t* w_scales, int64_t ws_stride_e, int64_t ws_r, int64_t ws_k, int w_is_2d,
                                       const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts,
                                       int64_t M_total, int64_t N, int64_t K, void* out, int out_dtype, int64_t ldo, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(a && a_scales && w && w_scales && offs && out, "grouped_gemm: NULL pointer");
  ALTO_REQUIRE(num_groups > 0 && num_groups <= 65536, "grouped_gemm: num_groups (%d) out of range", num_groups);
  ALTO_REQUIRE(group_expert != nullptr || num_groups == num_experts, "grouped_gemm: without group_expert, num_groups must equal num_experts");
  ALTO_REQUIRE(num_experts > 0 && num_experts <= 4096, "grouped_gemm: num_experts (%d) out of range", num_experts);
  ALTO_REQUIRE(M_total >= 0 && N >= 0 && K >= 0 && K % 32 == 0, "grouped_gemm: K (%lld) must be a multiple of 32", (long long)K);
  ALTO_REQUIRE(!w_is_2d || N % 32 == 0, "grouped_gemm: 2D weight scales need N (%lld) %% 32 == 0", (long long)N);
  ALTO_REQUIRE(!a_is_2d || M_total % 32 == 0, "grouped_gemm: 2D activation scales need M_total %% 32 == 0");
  ALTO_REQUIRE(lda >= K / 2 && ldw >= K / 2 && lda % 16 == 0 && ldw % 16 == 0 && w_stride_e % 16 == 0,
               "grouped_gemm: lda/ldw/w_stride_e must be >= K/2 and multiples of 16 bytes");
  ALTO_REQUIRE(((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(w)) & 15) == 0, "grouped_gemm: a and w must be 16-byte aligned");
  ALTO_REQUIRE(ldo >= N, "grouped_gemm: ldo < N");
  ALTO_REQUIRE(out_dtype == ALTO_DT_BF16 || out_dtype == ALTO_DT_F32, "grouped_gemm: bad out_dtype %d", out_dtype);
  if (M_total == 0 || N == 0) return ALTO_MXFP4_OK;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  OperandView A{a, lda, a_scales, a_ss_r, a_ss_k, a_is_2d};
  // upper bound on row tiles: every expert (and the zero tail) may end with one partial tile
  const int64_t tiles = M_total / 64 + num_groups + 2;
  ALTO_REQUIRE(tiles <= 65535, "grouped_gemm: M_total too large for the fallback kernel");
  dim3 grid((unsigned)((N + 63) / 64), (unsigned)tiles);
  if (out_dtype == ALTO_DT_BF16)
    hipLaunchKernelGGL(grouped_simple_kernel<__bf16>, grid, dim3(256), 0, st, A, w, w_stride_e, ldw, w_scales, ws_stride_e, ws_r, ws_k, w_is_2d,
                       offs, group_expert, num_groups, num_experts, M_total, N, (int)(K / 32), (__bf16*)out, ldo);
  else
    hipLaunchKernelGGL(grouped_simple_kernel<float>, grid, dim3(256), 0, st, A, w, w_stride_e, ldw, w_scales, ws_stride_e, ws_r, ws_k, w_is_2d,
                       offs, group_expert, num_groups, num_experts, M_total, N, (int)(K / 32), (float*)out, ldo);
  return check_launch("grouped_gemm");
}

extern "C" int alto_mxfp4_grouped_gemm_dw(const uint8_t* go, int64_t ld_go, const uint8_t* go_scales, int64_t gs_r, int64_t gs_k,
                                          const uint8_t* x, int64_t ld_xq, const uint8_t* x_scales, int64_t xs_r, int64_t xs_k,
                                          const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts,
                                          int64_t M_total, int64_t N, int64_t K, void* dw, int dw_dtype, int64_t dw_stride_e, int64_t dw_stride_n, int64_t dw_stride_k,
                                          float out_scale, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(go && go_scales && x && x_scales && offs && dw, "grouped_gemm_dw: NULL pointer");
  ALTO_REQUIRE(num_experts > 0 && num_experts <= 65535, "grouped_gemm_dw: num_experts (%d) out of range", num_experts);
  ALTO_REQUIRE(num_groups > 0 && num_groups <= 65536, "grouped_gemm_dw: num_groups (%d) out of range", num_groups);
  ALTO_REQUIRE(group_expert != nullptr || num_groups == num_experts, "grouped_gemm_dw: without group_expert, num_groups must equal num_experts");
  ALTO_REQUIRE(M_total >= 0 && M_total % 32 == 0, "grouped_gemm_dw: M_total (%lld) must be a multiple of 32", (long long)M_total);
  ALTO_REQUIRE(ld_go >= M_total / 2 && ld_xq >= M_total / 2 && ld_go % 16 == 0 && ld_xq % 16 == 0,
               "grouped_gemm_dw: ld_go/ld_xq must be >= M_total/2 and multiples of 16 bytes");
  ALTO_REQUIRE(((reinterpret_cast<uintptr_t>(go) | reinterpret_cast<uintptr_t>(x)) & 15) == 0, "grouped_gemm_dw: go and x must be 16-byte aligned");
  ALTO_REQUIRE(dw_dtype == ALTO_DT_BF16 || dw_dtype == ALTO_DT_F32, "grouped_gemm_dw: bad dw_dtype %d", dw_dtype);
  if (N == 0 || K == 0) return ALTO_MXFP4_OK;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  OperandView GO{go, ld_go, go_scales, gs_r, gs_k, 0};
  OperandView X{x, ld_xq, x_scales, xs_r, xs_k, 0};
  dim3 grid((unsigned)((K + 63) / 64), (unsigned)((N + 63) / 64), (unsigned)num_experts);
  ALTO_REQUIRE(grid.y <= 65535u, "grouped_gemm_dw: N too large");
  if (dw_dtype == ALTO_DT_BF16)
    hipLaunchKernelGGL(grouped_dw_simple_kernel<__bf16>, grid, dim3(256), 0, st, GO, X, offs, group_expert, num_groups, M_total, N, K, (__bf16*)dw, dw_stride_e, dw_stride_n, dw_stride_k, out_scale);
  else
    hipLaunchKernelGGL(grouped_dw_simple_kernel<float>, grid, dim3(256), 0, st, GO, X, offs, group_expert, num_groups, M_total, N, K, (float*)dw, dw_stride_e, dw_stride_n, dw_stride_k, out_scale);
  return check_launch("grouped_gemm_dw");
}
