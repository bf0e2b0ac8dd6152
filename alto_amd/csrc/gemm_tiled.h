// Tuned LDS-tiled MXFP4 GEMM (declarations).  See gemm_tiled.hip.
#pragma once
#include "gemm_simple.h"

namespace alto {
bool gemm_tiled_supported(const OperandView& A, const OperandView& B, int64_t M, int64_t N, int64_t K, const void* c, int c_dtype, int64_t ldc);
void gemm_tiled_launch(const OperandView& A, const OperandView& B, int64_t M, int64_t N, int64_t K, void* c, int c_dtype, int64_t ldc,
                       float out_scale, hipStream_t st);
// Packed scales (see pack_scales_kernel): the converter, and the tiled GEMM on operands that bring them (bf16 output).
void pack_scales_launch(const uint8_t* src, int64_t ss_r, int64_t ss_k, int is_2d, int64_t rows, int64_t G, uint8_t* dst, hipStream_t st);
void gemm_tiled_launch_ps(const OperandView& A, const OperandView& B, int64_t M, int64_t N, int64_t K, void* c, int64_t ldc, float out_scale,
                          hipStream_t st);
}  // namespace alto
