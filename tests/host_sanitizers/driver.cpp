// Host-side robustness driver for the C ABI, meant to be linked against a build of the library whose HOST code carries
// AddressSanitizer and UndefinedBehaviorSanitizer (the device code is built as always).  It needs no GPU: every call
// either fails its argument checks or fails at the launch, and both must come back as an error code with a message.
// What is under test is the host code in front of the kernels: argument validation, size arithmetic at extreme values
// (no signed overflow, no out-of-range shift), the choice of grids and kernel variants, the per-device tables and the
// error string.  A sanitizer report aborts the process.
//
// Every entry point has one valid argument set.  A call takes that set and replaces zero to three of its arguments by
// values from a small pool of plausible and extreme ones (a fixed generator picks: a failure names its call index), so
// most calls get past most checks and many reach the code that chooses the kernel and the grid.
#include <cinttypes>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "alto_mxfp4.h"

namespace {

uint64_t g_state = 0x243F6A8885A308D3ull;
uint64_t next_u64() {   // splitmix64
  uint64_t z = (g_state += 0x9E3779B97F4A7C15ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

const int64_t kSizes[] = {-1, 0, 1, 2, 8, 16, 31, 32, 33, 64, 96, 128, 160, 256, 288, 512, 1024, 2880, 4096, 5760, 8192, 14336, 65536,
                          (1ll << 20), (1ll << 24), (1ll << 26), (1ll << 31) - 32, (1ll << 31) - 1, (1ll << 31), (1ll << 31) + 32, (1ll << 32),
                          (1ll << 33), (1ll << 40), (1ll << 62), INT64_MAX, INT64_MIN};
const int kInts[] = {-1, 0, 1, 2, 3, 4, 5, 7, 8, 32, 64, 255, 4096, 65535, 65536, 1 << 20, INT32_MAX, INT32_MIN};
const float kFloats[] = {1.0f, 0.0f, -1.0f, 0.088388f, 1e30f, __builtin_nanf(""), __builtin_inff()};

alignas(256) unsigned char g_mem[4096];   // stands in for device memory: the host code must never read or write through it
int8_t g_signs[32];
uint8_t g_perm[32];
uint8_t g_zeros[32];

void* pool_ptr() {
  switch (next_u64() & 3) {
    case 0: return nullptr;
    case 1: return g_mem + 1;   // misaligned
    case 2: return g_mem + 4;
    default: return g_mem + 512;
  }
}

// s: sizes and strides, i: flags / modes / counts, p: device pointers, signs / perm: host arrays the Hadamard entries read
struct Args {
  int64_t s[16];
  int i[8];
  void* p[10];
  float f;
  uint64_t u[2];
  const int8_t* signs;
  const uint8_t* perm;
};

struct Entry {
  const char* name;
  int ns, ni, np;   // how many of s, i, p the entry reads
  Args valid;
  int (*call)(const Args&);
  long calls, ok, launches;
};

void* const D = g_mem + 256;   // a well-aligned "device" pointer
#define P(T, k) static_cast<T*>(a.p[k])

Entry g_entries[] = {
    // x, dtype, batch, M, C, ld_x, bs_x, row_codes, row_scales, col_codes, col_scales, is_2d, rounding, rand, ld_rand, bs_rand, hadamard, ...
    {"quantize", 7, 6, 6, {{1, 64, 256, 256, 64 * 256, 256, 64 * 256}, {0, 0, 0, 0, 0, 0}, {D, D, D, D, D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_quantize(a.p[0], a.i[0], a.s[0], a.s[1], a.s[2], a.s[3], a.s[4], P(uint8_t, 1), P(uint8_t, 2), P(uint8_t, 3), P(uint8_t, 4),
                                  a.i[1], a.i[2], P(const uint32_t, 5), a.s[5], a.s[6], a.i[3], a.signs, a.perm, a.i[4], a.i[5], nullptr);
     }},
    {"quantize_pitched", 9, 6, 6, {{1, 64, 256, 256, 64 * 256, 256, 64 * 256, 128, 32}, {0, 0, 1, 1, 0, 0}, {D, D, D, D, D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_quantize_pitched(a.p[0], a.i[0], a.s[0], a.s[1], a.s[2], a.s[3], a.s[4], P(uint8_t, 1), P(uint8_t, 2), P(uint8_t, 3),
                                          P(uint8_t, 4), a.s[7], a.s[8], a.i[1], a.i[2], P(const uint32_t, 5), a.s[5], a.s[6], a.i[3], a.signs, a.perm,
                                          a.i[4], a.i[5], nullptr);
     }},
    {"quantize_sr_philox", 7, 5, 6, {{1, 64, 256, 256, 64 * 256, 128, 32}, {0, 0, 1, 0, 0}, {D, D, D, D, D, D}, 1.0f, {1234, 5}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_quantize_sr_philox(a.p[0], a.i[0], a.s[0], a.s[1], a.s[2], a.s[3], a.s[4], P(uint8_t, 1), P(uint8_t, 2), P(uint8_t, 3),
                                            P(uint8_t, 4), a.s[5], a.s[6], a.i[1], a.u[0], a.u[1], P(const uint64_t, 5), a.i[2], a.signs, a.perm,
                                            a.i[3], a.i[4], nullptr);
     }},
    {"quantize_sr_hw", 7, 5, 6, {{1, 64, 256, 256, 64 * 256, 128, 32}, {0, 0, 1, 0, 0}, {D, D, D, D, D, D}, 1.0f, {1234, 5}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_quantize_sr_hw(a.p[0], a.i[0], a.s[0], a.s[1], a.s[2], a.s[3], a.s[4], P(uint8_t, 1), P(uint8_t, 2), P(uint8_t, 3),
                                        P(uint8_t, 4), a.s[5], a.s[6], a.i[1], a.u[0], a.u[1], P(const uint64_t, 5), a.i[2], a.signs, a.perm, a.i[3],
                                        a.i[4], nullptr);
     }},
    {"quantize_ex", 9, 7, 7, {{4, 512, 512, 512, 512 * 512, 256, 256, 512, 512 * 512}, {0, 1, 0, 0, 0, 0, 3}, {D, D, D, D, D, D, D}, 1.0f, {1234, 5}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_quantize_ex(a.p[0], a.i[0], a.s[0], a.s[1], a.s[2], a.s[3], a.s[4], P(uint8_t, 1), P(uint8_t, 2), P(uint8_t, 3), P(uint8_t, 4),
                                     a.s[5], a.s[6], a.i[1], a.i[2], P(const uint32_t, 5), a.s[7], a.s[8], a.u[0], a.u[1], P(const uint64_t, 6),
                                     a.i[3], a.signs, a.perm, a.i[4], a.i[5], a.i[6], nullptr);
     }},
    {"quantize_sr_hw_words", 3, 1, 0, {{1, 64, 256}, {0}, {}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) { return alto_mxfp4_quantize_sr_hw_words(a.i[0], a.s[0], a.s[1], a.s[2]) < 0 ? -100 : 0; }},
    {"philox_advance", 0, 0, 1, {{}, {}, {D}, 1.0f, {1000, 0}, g_signs, g_perm},
     [](const Args& a) { return alto_mxfp4_philox_advance(P(uint64_t, 0), a.u[0], nullptr); }},
    {"hadamard", 4, 1, 2, {{64, 256, 256, 256}, {0}, {D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) { return alto_mxfp4_hadamard(a.p[0], a.i[0], a.s[0], a.s[1], a.s[2], a.p[1], a.s[3], a.signs, a.perm, nullptr); }},
    {"hadamard_apply", 4, 3, 2, {{64, 256, 256, 256}, {1, 1, 1}, {D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_hadamard_apply(a.p[0], a.i[0], a.s[0], a.s[1], a.s[2], a.p[1], a.s[3], a.signs, a.perm, a.i[1], a.i[2], nullptr);
     }},
    {"dequantize", 4, 3, 3, {{64, 256, 256, 1}, {0, 0, 0}, {D, D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_dequantize(P(const uint8_t, 0), P(const uint8_t, 1), a.s[0], a.s[1], a.i[0], a.p[2], a.i[1], a.s[2], a.s[3], a.i[2], nullptr);
     }},
    {"transpose_codes", 2, 0, 2, {{64, 256}, {}, {D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) { return alto_mxfp4_transpose_codes(P(const uint8_t, 0), a.s[0], a.s[1], P(uint8_t, 1), nullptr); }},
    // a, lda, a_scales, a_ss_r, a_ss_k, a_is_2d, b, ldb, b_scales, b_ss_r, b_ss_k, b_is_2d, M, N, K, c, c_dtype, ldc, out_scale
    {"gemm", 10, 3, 5, {{512, 32, 1, 512, 32, 1, 256, 256, 1024, 256}, {0, 0, 0}, {D, D, D, D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_gemm(P(const uint8_t, 0), a.s[0], P(const uint8_t, 1), a.s[1], a.s[2], a.i[0], P(const uint8_t, 2), a.s[3], P(const uint8_t, 3),
                              a.s[4], a.s[5], a.i[1], a.s[6], a.s[7], a.s[8], a.p[4], a.i[2], a.s[9], a.f, nullptr);
     }},
    {"gemm_small", 10, 3, 5, {{32, 2, 1, 32, 2, 1, 32, 48, 64, 48}, {0, 0, 1}, {D, D, D, D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_gemm(P(const uint8_t, 0), a.s[0], P(const uint8_t, 1), a.s[1], a.s[2], a.i[0], P(const uint8_t, 2), a.s[3], P(const uint8_t, 3),
                              a.s[4], a.s[5], a.i[1], a.s[6], a.s[7], a.s[8], a.p[4], a.i[2], a.s[9], a.f, nullptr);
     }},
    {"packed_scales_bytes", 2, 0, 0, {{256, 1024}, {}, {}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) { return alto_mxfp4_packed_scales_bytes(a.s[0], a.s[1]) < 0 ? -100 : 0; }},
    {"pack_scales", 4, 1, 2, {{32, 1, 256, 1024}, {0}, {D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) { return alto_mxfp4_pack_scales(P(const uint8_t, 0), a.s[0], a.s[1], a.i[0], a.s[2], a.s[3], P(uint8_t, 1), nullptr); }},
    {"gemm_ps", 6, 0, 5, {{512, 512, 256, 256, 1024, 256}, {}, {D, D, D, D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_gemm_ps(P(const uint8_t, 0), a.s[0], P(const uint8_t, 1), P(const uint8_t, 2), a.s[1], P(const uint8_t, 3), a.s[2], a.s[3],
                                 a.s[4], a.p[4], a.s[5], a.f, nullptr);
     }},
    // a, lda, a_scales, a_ss_r, a_ss_k, a_is_2d, w, w_stride_e, ldw, w_scales, ws_stride_e, ws_r, ws_k, w_is_2d, offs, group_expert, G, E, M_total, N, K,
    // out, out_dtype, ldo, workspace, workspace_bytes
    {"grouped_gemm", 14, 5, 8, {{512, 32, 1, 256 * 512, 512, 256 * 32, 32, 1, 1024, 256, 1024, 256, 65536}, {0, 0, 4, 4, 0}, {D, D, D, D, D, D, D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_grouped_gemm(P(const uint8_t, 0), a.s[0], P(const uint8_t, 1), a.s[1], a.s[2], a.i[0], P(const uint8_t, 2), a.s[3], a.s[4],
                                      P(const uint8_t, 3), a.s[5], a.s[6], a.s[7], a.i[1], P(const int32_t, 4), P(const int32_t, 5), a.i[2], a.i[3],
                                      a.s[8], a.s[9], a.s[10], a.p[6], a.i[4], a.s[11], a.p[7], a.s[12], nullptr);
     }},
    {"grouped_gemm_plan", 2, 2, 3, {{1024, 65536}, {4, 4}, {D, D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) { return alto_mxfp4_grouped_gemm_plan(P(const int32_t, 0), P(const int32_t, 1), a.i[0], a.i[1], a.s[0], a.p[2], a.s[1], nullptr); }},
    {"grouped_gemm_planned", 14, 5, 8, {{512, 32, 1, 256 * 512, 512, 256 * 32, 32, 1, 1024, 256, 1024, 256, 65536}, {0, 0, 4, 4, 0}, {D, D, D, D, D, D, D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_grouped_gemm_planned(P(const uint8_t, 0), a.s[0], P(const uint8_t, 1), a.s[1], a.s[2], a.i[0], P(const uint8_t, 2), a.s[3], a.s[4],
                                              P(const uint8_t, 3), a.s[5], a.s[6], a.s[7], a.i[1], P(const int32_t, 4), P(const int32_t, 5), a.i[2],
                                              a.i[3], a.s[8], a.s[9], a.s[10], a.p[6], a.i[4], a.s[11], a.p[7], a.s[12], nullptr);
     }},
    // a, lda, a_packed, w, w_stride_e, ldw, w_packed, wp_stride_e, offs, group_expert, G, E, M_total, N, K, out, ldo, workspace, bytes, plan_built
    {"grouped_gemm_ps", 9, 3, 8, {{512, 256 * 512, 512, 2 * 256 * 16, 1024, 256, 1024, 256, 65536}, {4, 4, 0}, {D, D, D, D, D, D, D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_grouped_gemm_ps(P(const uint8_t, 0), a.s[0], P(const uint8_t, 1), P(const uint8_t, 2), a.s[1], a.s[2], P(const uint8_t, 3),
                                         a.s[3], P(const int32_t, 4), P(const int32_t, 5), a.i[0], a.i[1], a.s[4], a.s[5], a.s[6], a.p[6], a.s[7], a.p[7],
                                         a.s[8], a.i[2], nullptr);
     }},
    {"grouped_gemm_noalloc", 12, 5, 7, {{512, 32, 1, 256 * 512, 512, 256 * 32, 32, 1, 1024, 256, 1024, 256}, {0, 0, 4, 4, 0}, {D, D, D, D, D, D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_grouped_gemm_noalloc(P(const uint8_t, 0), a.s[0], P(const uint8_t, 1), a.s[1], a.s[2], a.i[0], P(const uint8_t, 2), a.s[3], a.s[4],
                                              P(const uint8_t, 3), a.s[5], a.s[6], a.s[7], a.i[1], P(const int32_t, 4), P(const int32_t, 5), a.i[2],
                                              a.i[3], a.s[8], a.s[9], a.s[10], a.p[6], a.i[4], a.s[11], nullptr);
     }},
    {"grouped_workspace_bytes", 1, 1, 0, {{1024}, {4}, {}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) { return alto_mxfp4_grouped_gemm_workspace_bytes(a.s[0], a.i[0]) < 0 ? -100 : 0; }},
    // go, ld_go, go_scales, gs_r, gs_k, go_is_2d, x, ld_xq, x_scales, xs_r, xs_k, x_is_2d, offs, group_expert, G, E, M_total, N, K, dw, dw_dtype,
    // dw_stride_e, dw_stride_n, dw_stride_k, out_scale
    {"grouped_gemm_dw", 12, 5, 7, {{512, 32, 1, 512, 32, 1, 1024, 256, 512, 256 * 512, 512, 1}, {0, 0, 4, 4, 0}, {D, D, D, D, D, D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_grouped_gemm_dw(P(const uint8_t, 0), a.s[0], P(const uint8_t, 1), a.s[1], a.s[2], a.i[0], P(const uint8_t, 2), a.s[3],
                                         P(const uint8_t, 3), a.s[4], a.s[5], a.i[1], P(const int32_t, 4), P(const int32_t, 5), a.i[2], a.i[3], a.s[6],
                                         a.s[7], a.s[8], a.p[6], a.i[4], a.s[9], a.s[10], a.s[11], a.f, nullptr);
     }},
    {"grouped_gemm_dw_small", 12, 5, 7, {{64, 4, 1, 64, 4, 1, 128, 48, 64, 48 * 64, 64, 1}, {0, 0, 2, 2, 1}, {D, D, D, D, D, D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_grouped_gemm_dw(P(const uint8_t, 0), a.s[0], P(const uint8_t, 1), a.s[1], a.s[2], a.i[0], P(const uint8_t, 2), a.s[3],
                                         P(const uint8_t, 3), a.s[4], a.s[5], a.i[1], P(const int32_t, 4), P(const int32_t, 5), a.i[2], a.i[3], a.s[6],
                                         a.s[7], a.s[8], a.p[6], a.i[4], a.s[9], a.s[10], a.s[11], a.f, nullptr);
     }},
    {"grouped_gemm_dw_ps", 8, 2, 7, {{512, 512, 1024, 256, 512, 256 * 512, 512, 1}, {4, 4}, {D, D, D, D, D, D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_grouped_gemm_dw_ps(P(const uint8_t, 0), a.s[0], P(const uint8_t, 1), P(const uint8_t, 2), a.s[1], P(const uint8_t, 3),
                                            P(const int32_t, 4), P(const int32_t, 5), a.i[0], a.i[1], a.s[2], a.s[3], a.s[4], a.p[6], a.s[5], a.s[6],
                                            a.s[7], a.f, nullptr);
     }},
    {"qdq", 7, 3, 2, {{1, 64, 256, 256, 64 * 256, 256, 64 * 256}, {0, 0, 0}, {D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_qdq(a.p[0], a.i[0], a.s[0], a.s[1], a.s[2], a.s[3], a.s[4], a.p[1], a.s[5], a.s[6], a.i[1], a.i[2], nullptr);
     }},
    // B, Hq, Hk, Sq, Sk, Sk_used, D, Dv
    {"attention_fwd", 8, 1, 8, {{2, 8, 2, 256, 256, 256, 128, 128}, {1}, {D, D, D, D, D, D, D, D}, 0.088388f, {0, 0}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_attention_fwd(a.p[0], a.p[1], a.p[2], a.p[3], a.p[4], a.p[5], a.p[6], P(float, 7), a.s[0], a.s[1], a.s[2], a.s[3], a.s[4], a.s[5],
                                       a.s[6], a.s[7], a.f, a.i[0], nullptr);
     }},
    {"attention_fwd_ex", 13, 1, 10, {{2, 8, 2, 256, 320, 288, 64, 64, 8 * 256 * 288, 256 * 288, 288, 8, 1}, {0}, {D, D, D, D, D, D, D, D, D, D}, 0.088388f, {0, 0}, g_signs, g_perm},
     [](const Args& a) {
       return alto_mxfp4_attention_fwd_ex(a.p[0], a.p[1], a.p[2], a.p[3], a.p[4], a.p[5], a.p[6], P(float, 7), a.s[0], a.s[1], a.s[2], a.s[3], a.s[4],
                                          a.s[5], a.s[6], a.s[7], a.f, a.i[0], P(const float, 8), a.s[8], a.s[9], a.s[10], P(const float, 9), a.s[11],
                                          a.s[12], nullptr);
     }},
    {"random_bits", 1, 0, 1, {{4096}, {}, {D}, 1.0f, {7, 9}, g_signs, g_perm},
     [](const Args& a) { return alto_mxfp4_random_bits(P(uint32_t, 0), a.s[0], a.u[0], a.u[1], nullptr); }},
    {"probe_mfma", 0, 3, 2, {{}, {1, 16, 256}, {D, D}, 1.0f, {0, 0}, g_signs, g_perm},
     [](const Args& a) { return alto_mxfp4_probe_mfma(a.i[0], a.i[1], a.i[2], P(float, 0), P(uint64_t, 1), nullptr); }},
};
constexpr int kEntries = sizeof(g_entries) / sizeof(g_entries[0]);

void mutate(Args& a, const Entry& e) {
  const int fields = e.ns + e.ni + e.np + 4;   // + float, one of the two u64, signs, perm
  int k = (int)(next_u64() % (uint64_t)fields);
  const uint64_t r = next_u64();
  if (k < e.ns) { a.s[k] = kSizes[r % (sizeof(kSizes) / sizeof(kSizes[0]))]; return; }
  k -= e.ns;
  if (k < e.ni) { a.i[k] = kInts[r % (sizeof(kInts) / sizeof(kInts[0]))]; return; }
  k -= e.ni;
  if (k < e.np) { a.p[k] = pool_ptr(); return; }
  k -= e.np;
  switch (k) {
    case 0: a.f = kFloats[r % 7]; break;
    case 1: a.u[r & 1] = (r & 2) ? ~0ull - (r >> 60) : next_u64(); break;
    case 2: a.signs = (r & 1) ? nullptr : reinterpret_cast<const int8_t*>(g_zeros); break;
    default: a.perm = (r & 1) ? nullptr : g_zeros; break;
  }
}

}  // namespace

int main(int argc, char** argv) {
  const long rounds = argc > 1 ? std::atol(argv[1]) : 2000;
  if (argc > 2) g_state ^= std::strtoull(argv[2], nullptr, 0);   // another sequence of calls
  for (int k = 0; k < 32; ++k) {
    g_signs[k] = (k * 7 % 3 == 0) ? -1 : 1;
    g_perm[k] = (uint8_t)((k * 5 + 3) % 32);
  }
  std::printf("version %d\n", alto_mxfp4_version());
  (void)alto_mxfp4_init();   // no device here: must fail cleanly or do nothing
  long calls = 0;
  for (long it = 0; it < rounds; ++it) {
    for (int n = 0; n < kEntries; ++n) {
      Entry& e = g_entries[n];
      Args a = e.valid;
      const int changes = (int)(next_u64() % 4);
      for (int c = 0; c < changes; ++c) mutate(a, e);
      const int rc = e.call(a);
      ++calls;
      ++e.calls;
      if (rc == -100) {
        std::fprintf(stderr, "call %ld (%s): a size query returned a negative number\n", calls, e.name);
        return 2;
      }
      if (rc == 0) { ++e.ok; continue; }   // size queries, empty problems
      const char* msg = alto_mxfp4_last_error();
      if (msg == nullptr || std::strlen(msg) == 0) {
        std::fprintf(stderr, "call %ld (%s): error code %d without a message\n", calls, e.name, rc);
        return 2;
      }
      // a launch that fails for want of a device has passed every argument check and chosen its kernel and grid
      if (std::strstr(msg, "launch failed") != nullptr || std::strstr(msg, "could not reserve") != nullptr || std::strstr(msg, "no current HIP device") != nullptr)
        ++e.launches;
    }
  }
  for (unsigned k = 0; k < sizeof(g_mem); ++k)
    if (g_mem[k] != 0) {
      std::fprintf(stderr, "host code wrote through a pointer that stands for device memory (byte %u)\n", k);
      return 3;
    }
  int never = 0;
  for (int n = 0; n < kEntries; ++n) {
    const Entry& e = g_entries[n];
    std::printf("%-24s calls %6ld  returned 0 %6ld  reached the launch %6ld\n", e.name, e.calls, e.ok, e.launches);
    if (e.launches == 0 && e.ok == 0) ++never;
  }
  if (never != 0 && rounds >= 100) {
    std::fprintf(stderr, "%d entry points never got past their argument checks: their valid argument set is not valid\n", never);
    return 4;
  }
  std::printf("calls %ld\n", calls);
  return 0;
}
