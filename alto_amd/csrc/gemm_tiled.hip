// Tuned LDS-tiled MXFP4 GEMM for gfx950 (placeholder until the tiled kernel lands: reports "unsupported").
#include "gemm_tiled.h"

namespace alto {
bool gemm_tiled_supported(const OperandView&, const OperandView&, int64_t, int64_t, int64_t, const void*, int, int64_t) { return false; }
void gemm_tiled_launch(const OperandView&, const OperandView&, int64_t, int64_t, int64_t, void*, int, int64_t, float, hipStream_t) {}
}  // namespace alto
