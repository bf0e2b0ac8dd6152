// LDS-tiled MXFP4 GEMM tile for gfx950: one workgroup of 256 threads (4 waves, 2x2) computes a 256x256 tile of
// C = A . B^T with v_mfma_scale_f32_32x32x64_f8f6f4; each wave owns 128x128 (4x4 MFMA tiles, 256 accumulator registers).
//
// Data path per K stage of 128 elements (64 B per operand row):
//   global --128-bit loads--> registers (two stages in flight) --ds_write_b128--> LDS ring of 3 stages (32 KB each)
//   LDS --ds_read_b128--> MFMA operands.  A 16-byte piece holds one MX block (32 codes); lane (r, h) of the MFMA takes
//   piece 2h + j of row r at K step j, so a row's four pieces are XOR-swizzled by (row / 2) % 4 inside its 64 bytes,
//   which makes every 8 consecutive rows of a fragment read cover all 32 banks.
// Scales: one byte per row per 32 K (1D) or per 32 rows (2D).  They are staged through LDS per block of 512 K
//   (16 bytes per row, rows at a 20-byte pitch) so that 1D and 2D scales look alike to the MFMA loop, which reads the two
//   bytes a lane needs for a stage with one 16-bit LDS load and selects between them with op_sel.
// The MFMA takes B rows as its first operand: accumulator registers then run along N (4 consecutive columns per lane),
// so a lane converts and stores 8 contiguous bytes of a C row at a time.
#pragma once
#include "gemm_simple.h"

namespace alto {

constexpr int GT_TM = 256, GT_TN = 256, GT_TK = 128;
constexpr int GT_STAGE_BYTES = (GT_TM + GT_TN) * (GT_TK / 2);   // 32768
constexpr int GT_NSTAGE = 4;
constexpr int GT_SCALE_PITCH = 5;                                // dwords per row (16 B + 4 B pad)
constexpr int GT_SCALE_BUF_DW = (GT_TM + GT_TN) * GT_SCALE_PITCH;  // one buffer, in dwords
constexpr int GT_LDS_BYTES = GT_NSTAGE * GT_STAGE_BYTES + 2 * GT_SCALE_BUF_DW * 4;  // 131072 + 20480 = 151552

struct TileArgs {
  OperandView A, B;
  int64_t m0, n0;          // first row of the tile in A / B
  int64_t m_lo, m_hi;      // valid A rows [m_lo, m_hi): loads clamp, stores mask
  int64_t n_hi;            // valid B rows [0, n_hi)
  int G;                   // number of 32-wide K groups
  float out_scale;
  int64_t a_bytes, b_bytes;    // extent of the code buffers in bytes (< 2^31), for the buffer descriptors
  int64_t as_bytes, bs_bytes;  // extent of the scale buffers in bytes (< 2^31)
};

// One 256x256 tile.  KTAIL = false requires G % 4 == 0 (K a multiple of 128): then every scale dword of a row is
// either fully inside K or fully beyond it and the main loop is branch-free.  KTAIL = true additionally handles a last
// partial dword of a scale row with byte loads.
template <typename OutT, bool KTAIL>
__device__ __forceinline__ void gemm_tile_256x256(const TileArgs& ta, OutT* __restrict__ c, int64_t ldc, uint8_t* smem) {
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int wm = wave >> 1, wn = wave & 1;
  const int r = lane & 31, h = lane >> 5;
  uint32_t* sscale = reinterpret_cast<uint32_t*>(smem + GT_NSTAGE * GT_STAGE_BYTES);
  const int KB = (ta.G + 15) / 16;       // loop iterations: blocks of 512 K = 4 stages of 128 K
  const int kbytes = ta.G * 16;

  // ---- global -> register staging: instruction i (0..7) of this thread moves one 16-byte piece.
  // Piece (i, wave, lane): operand = i / 4 (0: A, 1: B); chunk q = 4 * (i % 4) + wave covers tile rows 16q .. 16q+15;
  // lane l holds row 16q + l / 4, slot l % 4, which stores global piece (l % 4) ^ ((l / 8) % 4) of that row.
  // Raw buffer loads: 32-bit per-lane byte offsets, the K offset of the stage rides in the scalar offset, and a piece
  // beyond the end of K gets an out-of-range offset, for which the hardware returns zeros.
  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(ta.A.codes), 0, (int)ta.a_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(ta.B.codes), 0, (int)ta.b_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_as = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(ta.A.scales), 0, (int)ta.as_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_bs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(ta.B.scales), 0, (int)ta.bs_bytes, 0x00020000);
  uint32_t goff[8];
  uint32_t ldst[8];
  int gpiece;
  {
    const int rr = lane >> 2;
    gpiece = (lane & 3) ^ ((rr >> 1) & 3);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int q = 4 * (i & 3) + wave;
      const int trow = 16 * q + rr;
      if (i < 4) {
        int64_t row = ta.m0 + trow;
        row = row < ta.m_hi ? row : ta.m_hi - 1;
        row = row < ta.m_lo ? ta.m_lo : row;
        goff[i] = (uint32_t)(row * ta.A.ld + gpiece * 16);
      } else {
        int64_t row = ta.n0 + trow;
        row = row < ta.n_hi ? row : ta.n_hi - 1;
        goff[i] = (uint32_t)(row * ta.B.ld + gpiece * 16);
      }
      ldst[i] = (i < 4 ? 0 : GT_TM * 64) + q * 1024 + lane * 16;
    }
  }
  // ---- fragment read offsets (bytes inside a stage): rows of this wave's sub-tiles, pieces 2h + j swizzled
  uint32_t a_off, b_off;   // for j = 0; j = 1 is the same address ^ 16
  {
    const int sw = (r >> 1) & 3;
    const int slot = (r & 15) * 4 + ((2 * h) ^ sw);
    a_off = (uint32_t)((128 * wm + r) >> 4) * 1024 + slot * 16;
    b_off = GT_TM * 64 + (uint32_t)((128 * wn + r) >> 4) * 1024 + slot * 16;
  }
  // scale read offsets (bytes): row * 20 + 2h within a block buffer
  const uint32_t sa_off = (uint32_t)(128 * wm + r) * (GT_SCALE_PITCH * 4) + 2 * h;
  const uint32_t sb_off = (uint32_t)(GT_TM + 128 * wn + r) * (GT_SCALE_PITCH * 4) + 2 * h;

  // scale staging: thread t owns A row t and B row t of the tile (unit stride along K, any byte alignment)
  uint32_t soff_a, soff_b;
  {
    int64_t ra = ta.m0 + tid;
    ra = ra < ta.m_hi ? ra : ta.m_hi - 1;
    ra = ra < ta.m_lo ? ta.m_lo : ra;
    int64_t rb = ta.n0 + tid;
    rb = rb < ta.n_hi ? rb : ta.n_hi - 1;
    soff_a = (uint32_t)((ta.A.is_2d ? (ra >> 5) : ra) * ta.A.ss_r);
    soff_b = (uint32_t)((ta.B.is_2d ? (rb >> 5) : rb) * ta.B.ss_r);
  }
  uint32_t sreg[8];

  v16f_t acc[4][4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[t][u][v] = 0.0f;

  uint4 pre[2][8];
  auto gload = [&](int s, uint4 (&dst)[8]) {
    const int koff = s * 64;
    const bool in = koff + gpiece * 16 < kbytes;   // whole piece inside K (K is a multiple of 32 codes = 16 bytes)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t off = in ? goff[i] : 0x80000000u;
      v4i_t v = __builtin_amdgcn_raw_buffer_load_b128(i < 4 ? rsrc_a : rsrc_b, (int)off, koff, 0);
      dst[i] = make_uint4((uint32_t)v[0], (uint32_t)v[1], (uint32_t)v[2], (uint32_t)v[3]);
    }
  };
  auto lwrite = [&](int slot, const uint4 (&src)[8]) {
    uint8_t* base = smem + slot * GT_STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < 8; ++i) *reinterpret_cast<uint4*>(base + ldst[i]) = src[i];
  };
  // 16 scale bytes of K block kb for this thread's A row and B row; groups at or beyond G read as 127 (scale 1.0) so
  // that the zero codes of a K tail never meet a NaN scale byte.
  auto sload = [&](int kb) {
    const int rem = ta.G - kb * 16;   // wave-uniform
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int n = rem - 4 * d;
      uint32_t wa = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsrc_as, (int)soff_a, kb * 16 + 4 * d, 0);
      uint32_t wb = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsrc_bs, (int)soff_b, kb * 16 + 4 * d, 0);
      const uint32_t keep = n >= 4 ? 0xFFFFFFFFu : 0u;
      wa = (wa & keep) | (0x7F7F7F7Fu & ~keep);
      wb = (wb & keep) | (0x7F7F7F7Fu & ~keep);
      if (KTAIL && n > 0 && n < 4) {   // last, partial dword of the row: bytes one by one, never past the row
        uint32_t a0 = __builtin_amdgcn_raw_buffer_load_b8(rsrc_as, (int)soff_a, kb * 16 + 4 * d, 0);
        uint32_t b0 = __builtin_amdgcn_raw_buffer_load_b8(rsrc_bs, (int)soff_b, kb * 16 + 4 * d, 0);
        uint32_t a1 = 127, b1 = 127, a2 = 127, b2 = 127;
        if (n > 1) {
          a1 = __builtin_amdgcn_raw_buffer_load_b8(rsrc_as, (int)soff_a, kb * 16 + 4 * d + 1, 0);
          b1 = __builtin_amdgcn_raw_buffer_load_b8(rsrc_bs, (int)soff_b, kb * 16 + 4 * d + 1, 0);
        }
        if (n > 2) {
          a2 = __builtin_amdgcn_raw_buffer_load_b8(rsrc_as, (int)soff_a, kb * 16 + 4 * d + 2, 0);
          b2 = __builtin_amdgcn_raw_buffer_load_b8(rsrc_bs, (int)soff_b, kb * 16 + 4 * d + 2, 0);
        }
        wa = (a0 & 0xFF) | ((a1 & 0xFF) << 8) | ((a2 & 0xFF) << 16) | (127u << 24);
        wb = (b0 & 0xFF) | ((b1 & 0xFF) << 8) | ((b2 & 0xFF) << 16) | (127u << 24);
      }
      sreg[d] = wa;
      sreg[4 + d] = wb;
    }
  };
  auto swrite = [&](int kb) {
    uint32_t* buf = sscale + (kb & 1) * GT_SCALE_BUF_DW;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      buf[tid * GT_SCALE_PITCH + d] = sreg[d];
      buf[(GT_TM + tid) * GT_SCALE_PITCH + d] = sreg[4 + d];
    }
  };
  // MFMAs of one stage held in LDS slot `slot`; `i` = stage index inside the 512-K block (selects the scale dword)
  auto compute = [&](int slot, int i, const uint8_t* sblock) {
    const uint8_t* base = smem + slot * GT_STAGE_BYTES;
    const uint8_t* sbase = sblock + i * 4;
    int sa[4], sb[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      sa[t] = *reinterpret_cast<const unsigned short*>(sbase + sa_off + t * 32 * GT_SCALE_PITCH * 4);
      sb[t] = *reinterpret_cast<const unsigned short*>(sbase + sb_off + t * 32 * GT_SCALE_PITCH * 4);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      v8i_t af[4], bf[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        uint4 a4 = *reinterpret_cast<const uint4*>(base + ((a_off + t * 2048) ^ (j * 16)));
        uint4 b4 = *reinterpret_cast<const uint4*>(base + ((b_off + t * 2048) ^ (j * 16)));
        af[t] = v8i_t{(int)a4.x, (int)a4.y, (int)a4.z, (int)a4.w, 0, 0, 0, 0};
        bf[t] = v8i_t{(int)b4.x, (int)b4.y, (int)b4.z, (int)b4.w, 0, 0, 0, 0};
      }
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          if (j == 0)
            acc[t][u] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bf[u], af[t], acc[t][u], 4, 4, 0, sb[u], 0, sa[t]);
          else
            acc[t][u] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bf[u], af[t], acc[t][u], 4, 4, 1, sb[u], 1, sa[t]);
        }
    }
  };

  // ---- prologue: stages 0 and 1 into LDS, stage 2 in flight; scale block 0 in LDS, block 1 in flight.
  // Stages beyond K load zeros and blocks beyond K load unit scales, so nothing below is conditional.
  sload(0);
  gload(0, pre[0]);
  gload(1, pre[1]);
  swrite(0);
  lwrite(0, pre[0]);
  lwrite(1, pre[1]);
  gload(2, pre[0]);
  sload(1);

  // ---- main loop: one iteration = one 512-K block = 4 stages; LDS slot = stage % 4, register buffer = stage % 2.
  // Per stage: barrier; issue the global loads of stage s+3; MFMAs of stage s; park stage s+2 (loaded one stage ago)
  // in the slot that stage s-2 used.
  for (int kb = 0; kb < KB; ++kb) {
    const int s = kb * 4;
    const uint8_t* sblock = reinterpret_cast<const uint8_t*>(sscale + (kb & 1) * GT_SCALE_BUF_DW);
    __syncthreads();
    gload(s + 3, pre[1]);
    compute(0, 0, sblock);
    lwrite(2, pre[0]);

    __syncthreads();
    gload(s + 4, pre[0]);
    compute(1, 1, sblock);
    lwrite(3, pre[1]);
    swrite(kb + 1);          // block kb+1 -> the other scale buffer (last read in iteration kb-1)

    __syncthreads();
    gload(s + 5, pre[1]);
    compute(2, 2, sblock);
    lwrite(0, pre[0]);
    sload(kb + 2);

    __syncthreads();
    gload(s + 6, pre[0]);
    compute(3, 3, sblock);
    lwrite(1, pre[1]);
  }

  // ---- epilogue: accumulator register v of tile (t, u) is C[m][n] with
  //   m = m0 + 128 wm + 32 t + r,  n = n0 + 128 wn + 32 u + 8 (v / 4) + 4 h + v % 4
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int64_t m = ta.m0 + 128 * wm + 32 * t + r;
    const bool mok = m >= ta.m_lo && m < ta.m_hi;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) {
        const int64_t n = ta.n0 + 128 * wn + 32 * u + 8 * vq + 4 * h;
        float f0 = acc[t][u][4 * vq + 0] * ta.out_scale, f1 = acc[t][u][4 * vq + 1] * ta.out_scale;
        float f2 = acc[t][u][4 * vq + 2] * ta.out_scale, f3 = acc[t][u][4 * vq + 3] * ta.out_scale;
        OutT* dst = c + m * ldc + n;
        if (mok && n + 4 <= ta.n_hi) {   // N, ldc multiples of 4 and c 16-byte aligned (host-checked): aligned vector store
          if constexpr (sizeof(OutT) == 2) {
            uint2 o;
            o.x = f32_to_bf16_bits(f0) | (f32_to_bf16_bits(f1) << 16);
            o.y = f32_to_bf16_bits(f2) | (f32_to_bf16_bits(f3) << 16);
            *reinterpret_cast<uint2*>(dst) = o;
          } else {
            *reinterpret_cast<float4*>(dst) = make_float4(f0, f1, f2, f3);
          }
        }
      }
    }
  }
}

}  // namespace alto
