// Random bits for stochastic rounding: Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as
// 1, 2, 3", SC'11), counter-based, so any element can be regenerated from (seed, offset, index).  The reference draws its
// bits inside the Triton kernel with tl.randint4x (alto/kernels/fp4/fp4_common/triton_fp4_ops.py:15-18), the same
// generator family; here the bits are a tensor the quantizer (and the CPU oracle) reads, and this kernel fills it at
// memory speed: word 4 c + j of the output is word j of philox4x32_10(counter = (c + offset) as 128 bits, key = seed).
#include "common.h"

namespace alto {
namespace {

__global__ __launch_bounds__(256) void random_bits_kernel(uint32_t* __restrict__ out, int64_t n, uint64_t seed, uint64_t offset) {
  const int64_t quads = (n + 3) / 4;
  for (int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x; q < quads; q += (int64_t)gridDim.x * 256) {
    const uint64_t lo = (uint64_t)q + offset;
    const uint4 w = philox4x32_10(lo, lo < offset ? 1ull : 0ull, seed);   // 128-bit counter: the carry goes into the high half
    if (4 * q + 4 <= n) {
      *reinterpret_cast<uint4*>(out + 4 * q) = w;
    } else {
      const uint32_t v[4] = {w.x, w.y, w.z, w.w};
      for (int j = 0; 4 * q + j < n; ++j) out[4 * q + j] = v[j];
    }
  }
}

}  // namespace
}  // namespace alto

extern "C" int alto_mxfp4_random_bits(uint32_t* out, int64_t n, uint64_t seed, uint64_t offset, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(n >= 0 && n < (1ll << 48), "random_bits: count out of range");
  if (n == 0) return ALTO_MXFP4_OK;
  ALTO_REQUIRE(out != nullptr, "random_bits: NULL output");
  ALTO_REQUIRE((reinterpret_cast<uintptr_t>(out) & 15) == 0, "random_bits: out must be 16-byte aligned");
  const int64_t quads = (n + 3) / 4;
  int64_t blocks = (quads + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;   // grid-stride beyond 32 workgroups per CU
  hipLaunchKernelGGL(random_bits_kernel, dim3((unsigned)blocks), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), out, n, seed, offset);
  return check_launch("random_bits");
}
