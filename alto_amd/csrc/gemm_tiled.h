// Tuned LDS-tiled MXFP4 GEMM (declarations).  See gemm_tiled.hip.
#pragma once
#include "gemm_simple.h"

namespace alto {
bool gemm_tiled_supported(const OperandView& A, const OperandView& B, int64_t M, int64_t N, int64_t K, const void* c, int c_dtype, int64_t ldc);
void gemm_tiled_launch(const OperandView& A, const OperandView& B, int64_t M, int64_t N, int64_t K, void* c, int c_dtype, int64_t ldc,
                       float out_scale, hipStream_t st);
}  // namespace alto
