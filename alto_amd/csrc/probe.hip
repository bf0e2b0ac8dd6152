// Diagnostic: how fast does the FP4 matrix pipe run on this part when nothing else is in the way?
// A register-only loop of independent v_mfma_scale_f32_32x32x64_f8f6f4 instructions (8 accumulators per wave, two waves
// per SIMD, no memory traffic).  With constant operands the chip holds a higher clock than with random FP4 codes, so
// both are offered: the second is the ceiling a GEMM on real data can approach.
#include "common.h"

namespace alto {
namespace {

// `ticks` (may be NULL): workgroup 0 records how many shader-clock cycles (s_memtime) and how many ticks of the constant
// 100 MHz counter (s_memrealtime) its loop took: their ratio is the clock the chip held under this load.
__global__ __launch_bounds__(512) void mfma_probe_kernel(float* sink, int iters, int random_operands, uint64_t* ticks) {
  v8i_t a[4], b[2];
  uint32_t x = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 99u;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = v8i_t{0x22222222, 0x22222222, 0x22222222, 0x22222222, 0, 0, 0, 0};
    if (random_operands)
      for (int j = 0; j < 4; ++j) { x = x * 1664525u + 1013904223u; a[i][j] = (int)(x ^ (x >> 13)); }
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    b[i] = v8i_t{0x22222222, 0x22222222, 0x22222222, 0x22222222, 0, 0, 0, 0};
    if (random_operands)
      for (int j = 0; j < 4; ++j) { x = x * 1664525u + 1013904223u; b[i][j] = (int)(x ^ (x >> 11)); }
  }
  int sa = 0x7F7F7F7F, sb = 0x7F7F7F7F;
  v16f_t acc[4][2];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[t][u][v] = 0.0f;
  const uint64_t c0 = __builtin_readcyclecounter(), w0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
    asm volatile("" : "+v"(sa), "+v"(sb));
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int u = 0; u < 2; ++u) acc[t][u] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b[u], a[t], acc[t][u], 4, 4, 0, sb, 0, sa);
  }
  const uint64_t c1 = __builtin_readcyclecounter(), w1 = __builtin_amdgcn_s_memrealtime();
  if (ticks != nullptr && blockIdx.x == 0 && threadIdx.x == 0) {
    ticks[0] = c1 - c0;
    ticks[1] = w1 - w0;
  }
  float s = 0.0f;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int v = 0; v < 16; ++v) s += acc[t][u][v];
  if (s == 12345.678f) sink[threadIdx.x] = s;   // keeps the loop alive; practically never taken
}

}  // namespace
}  // namespace alto

extern "C" int alto_mxfp4_probe_mfma(int random_operands, int iters, int workgroups, float* sink, uint64_t* ticks, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(sink != nullptr, "probe_mfma: sink is NULL (needs 512 floats of device memory)");
  ALTO_REQUIRE((reinterpret_cast<uintptr_t>(sink) & 3) == 0 && (reinterpret_cast<uintptr_t>(ticks) & 7) == 0, "probe_mfma: sink must be 4-byte and ticks 8-byte aligned");
  ALTO_REQUIRE(iters > 0 && iters <= (1 << 24) && workgroups > 0 && workgroups <= 65535, "probe_mfma: iters/workgroups out of range");
  hipLaunchKernelGGL(mfma_probe_kernel, dim3((unsigned)workgroups), dim3(512), 0, reinterpret_cast<hipStream_t>(stream), sink, iters,
                     random_operands ? 1 : 0, ticks);
  return check_launch("probe_mfma");
}
