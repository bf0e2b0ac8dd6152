// LDS-tiled MXFP4 GEMM tile for gfx950: one workgroup of 512 threads (8 waves, 2 x 4) computes a 256x256 tile of
// C = A . B^T with v_mfma_scale_f32_32x32x64_f8f6f4; each wave owns 128 (M) x 64 (N) = 4 x 2 MFMA tiles (128 accumulator
// registers), so two waves share every SIMD and cover each other's waits.
//
// Data path per K stage of 128 elements (64 B per operand row):
//   global --buffer_load_dwordx4 ... lds (no register staging, two stages in flight)--> LDS ring of 4 stages (32 KB each)
//   LDS --ds_read_b128--> MFMA operands.  (LDS instructions cost issue time on the SIMD that also issues the MFMAs -- about
//   12 clocks per ds_read_b128 and 40 per ds_write_b128 -- so the operand tiles never pass through ds_write.)  A 16-byte piece holds one MX block (32 codes); lane (r, h) of the MFMA takes
//   piece 2h + j of row r at K step j, so a row's four pieces are XOR-swizzled by (row / 4) % 4 inside its 64 bytes:
//   16 consecutive rows of a fragment read then cover the 64 LDS banks exactly once (ds_read_b128 serves 16 lanes per clock).
// Scales: one byte per row per 32 K (1D) or per 32 rows (2D).  They are staged through LDS per block of 512 K (16 bytes
//   per row, rows at a 20-byte pitch) so that 1D and 2D scales look alike to the MFMA loop; inside a row the bytes are
//   regrouped so that the 8 bytes a lane needs for the 4 stages of a block are contiguous, and op_sel picks the byte.
// The MFMA takes B rows as its first operand: accumulator registers then run along N (4 consecutive columns per lane).
// bf16 results go through LDS (swizzled 16-byte chunks) so that the global stores are whole 512-byte row segments.
#pragma once
#include <type_traits>

#include "gemm_simple.h"

namespace alto {

constexpr int GT_TM = 256, GT_TN = 256, GT_TK = 128;
constexpr int GT_THREADS = 512;
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

typedef v16f_t TileAcc[4][2];   // per wave: 4 (M) x 2 (N) MFMA tiles of 32x32

__device__ __forceinline__ void gemm_tile_zero(TileAcc& acc) {
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[t][u][v] = 0.0f;
}

// K loop of one 256x256 tile: acc += A[m0.., :] . B[n0.., :]^T over G groups of 32.  KTAIL = false requires G % 4 == 0
// (K a multiple of 128): then every scale dword of a row is either fully inside K or fully beyond it and the main loop
// is branch-free.  KTAIL = true additionally handles a last partial dword of a scale row with byte loads.  Requirements
// checked by the host: unit-stride scale rows, operand extents below 2^31 bytes.  Every thread of the workgroup must
// call it; it may be called again (same or other operands) to keep accumulating.
template <bool KTAIL>
__device__ __forceinline__ void gemm_tile_mainloop(const TileArgs& ta, TileAcc& acc, uint8_t* smem) {
  __syncthreads();   // the LDS ring may still be read by a previous call
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;   // the wave index lives in a scalar register
  const int wm = wave >> 2, wn = wave & 3;
  const int r = lane & 31, h = lane >> 5;
  uint32_t* sscale = reinterpret_cast<uint32_t*>(smem + GT_NSTAGE * GT_STAGE_BYTES);
  const int KB = (ta.G + 15) / 16;       // loop iterations: blocks of 512 K = 4 stages of 128 K
  const int kbytes = ta.G * 16;

  // ---- global -> register staging: instruction i (0..3) of this thread moves one 16-byte piece.
  // Piece (i, wave, lane): operand = i / 2 (0: A, 1: B); chunk q = 8 * (i % 2) + wave covers tile rows 16q .. 16q+15;
  // lane l holds row 16q + l / 4, slot l % 4, which stores global piece (l % 4) ^ ((l / 16) % 4) of that row.
  // Raw buffer loads: 32-bit per-lane byte offsets, the K offset of the stage rides in the scalar offset, and a piece
  // beyond the end of K gets an out-of-range offset, for which the hardware returns zeros.
  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(ta.A.codes), 0, (int)ta.a_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(ta.B.codes), 0, (int)ta.b_bytes, 0x00020000);
  uint32_t goff[4];
  uint32_t ldst[4];
  int gpiece;
  {
    const int rr = lane >> 2;
    gpiece = (lane & 3) ^ ((rr >> 2) & 3);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = 8 * (i & 1) + wave;
      const int trow = 16 * q + rr;
      if (i < 2) {
        int64_t row = ta.m0 + trow;
        row = row < ta.m_hi ? row : ta.m_hi - 1;
        row = row < ta.m_lo ? ta.m_lo : row;
        goff[i] = (uint32_t)(row * ta.A.ld + gpiece * 16);
      } else {
        int64_t row = ta.n0 + trow;
        row = row < ta.n_hi ? row : ta.n_hi - 1;
        goff[i] = (uint32_t)(row * ta.B.ld + gpiece * 16);
      }
      ldst[i] = (i < 2 ? 0 : GT_TM * 64) + q * 1024;   // wave-uniform chunk base; the hardware adds 16 * lane
    }
  }
  // ---- fragment read offsets (bytes inside a stage): rows of this wave's sub-tiles, pieces 2h + j swizzled
  uint32_t a_off, b_off;   // for j = 0; j = 1 is the same address ^ 16
  {
    const int sw = (r >> 2) & 3;
    const int slot = (r & 15) * 4 + ((2 * h) ^ sw);
    a_off = (uint32_t)((128 * wm + r) >> 4) * 1024 + slot * 16;
    b_off = GT_TM * 64 + (uint32_t)((64 * wn + r) >> 4) * 1024 + slot * 16;
  }
  // scale read offsets (bytes): row * 20 + 8h within a block buffer
  const uint32_t sa_off = (uint32_t)(128 * wm + r) * (GT_SCALE_PITCH * 4) + 8 * h;
  const uint32_t sb_off = (uint32_t)(GT_TM + 64 * wn + r) * (GT_SCALE_PITCH * 4) + 8 * h;

  // scale staging: thread t owns tile row t of A (t < 256) or tile row t - 256 of B (unit stride along K, any alignment)
  const bool s_is_a = tid < GT_TM;   // wave-uniform
  const __amdgpu_buffer_rsrc_t rsrc_s = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t*>(s_is_a ? ta.A.scales : ta.B.scales), 0, (int)(s_is_a ? ta.as_bytes : ta.bs_bytes), 0x00020000);
  uint32_t soff;
  {
    int64_t row;
    if (s_is_a) {
      row = ta.m0 + tid;
      row = row < ta.m_hi ? row : ta.m_hi - 1;
      row = row < ta.m_lo ? ta.m_lo : row;
      soff = (uint32_t)((ta.A.is_2d ? (row >> 5) : row) * ta.A.ss_r);
    } else {
      row = ta.n0 + (tid - GT_TM);
      row = row < ta.n_hi ? row : ta.n_hi - 1;
      soff = (uint32_t)((ta.B.is_2d ? (row >> 5) : row) * ta.B.ss_r);
    }
  }
  uint32_t sreg[4];

  // Direct-to-LDS load of stage s into ring slot `slot`: lane l of instruction i lands at chunk base + 16 l.
  typedef __attribute__((address_space(3))) uint8_t lds_u8;
  lds_u8* const lds = (lds_u8*)smem;
  auto gload = [&](int s, int slot) {
    const int koff = s * 64;
    // a piece beyond K gets bit 31 set in its offset: out of range for the descriptor, so zeros land in LDS
    const uint32_t oob = (koff + gpiece * 16 < kbytes) ? 0u : 0x80000000u;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t off = goff[i] | oob;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(i < 2 ? rsrc_a : rsrc_b, (__attribute__((address_space(3))) void*)(lds + slot * GT_STAGE_BYTES + ldst[i]),
                                               16, (int)off, koff, 0, 0);
    }
  };
  // 16 scale bytes of K block kb for this thread's row; groups at or beyond G read as 127 (scale 1.0) so that the zero
  // codes of a K tail never meet a NaN scale byte.
  auto sload = [&](int kb) {
    const int rem = ta.G - kb * 16;   // wave-uniform
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int n = rem - 4 * d;
      uint32_t w = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsrc_s, (int)soff, kb * 16 + 4 * d, 0);
      const uint32_t keep = n >= 4 ? 0xFFFFFFFFu : 0u;
      w = (w & keep) | (0x7F7F7F7Fu & ~keep);
      if (KTAIL && n > 0 && n < 4) {   // last, partial dword of the row: bytes one by one, never past the row
        uint32_t b0 = __builtin_amdgcn_raw_buffer_load_b8(rsrc_s, (int)soff, kb * 16 + 4 * d, 0);
        uint32_t b1 = 127, b2 = 127;
        if (n > 1) b1 = __builtin_amdgcn_raw_buffer_load_b8(rsrc_s, (int)soff, kb * 16 + 4 * d + 1, 0);
        if (n > 2) b2 = __builtin_amdgcn_raw_buffer_load_b8(rsrc_s, (int)soff, kb * 16 + 4 * d + 2, 0);
        w = (b0 & 0xFF) | ((b1 & 0xFF) << 8) | ((b2 & 0xFF) << 16) | (127u << 24);
      }
      sreg[d] = w;
    }
  };
  // LDS row layout (4 dwords): [h=0: stages 0,1 | h=0: stages 2,3 | h=1: stages 0,1 | h=1: stages 2,3], where the
  // half-wave h of the MFMA uses groups 4i + 2h + {0, 1} at stage i; byte (2 (i % 2) + j) of dword (2h + i / 2).
  auto swrite = [&](int kb) {
    uint32_t* row = sscale + (kb & 1) * GT_SCALE_BUF_DW + tid * GT_SCALE_PITCH;
    row[0] = __builtin_amdgcn_perm(sreg[1], sreg[0], 0x05040100u);
    row[1] = __builtin_amdgcn_perm(sreg[3], sreg[2], 0x05040100u);
    row[2] = __builtin_amdgcn_perm(sreg[1], sreg[0], 0x07060302u);
    row[3] = __builtin_amdgcn_perm(sreg[3], sreg[2], 0x07060302u);
  };

  // Fragment / scale registers: F0 = pieces of K step j = 0 of the current stage (read during the previous stage),
  // F1 = pieces of step j = 1, S = this block's scale bytes (8 per lane and sub-tile, selected by op_sel).
  v8i_t fa0[4], fb0[2], fa1[4], fb1[2];
  int sa[4][2], sb[2][2];
  auto read_frags = [&](int slot, int j, v8i_t (&fa)[4], v8i_t (&fb)[2]) {
    const uint8_t* base = smem + slot * GT_STAGE_BYTES;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      uint4 a4 = *reinterpret_cast<const uint4*>(base + ((a_off + t * 2048) ^ (j * 16)));
      fa[t] = v8i_t{(int)a4.x, (int)a4.y, (int)a4.z, (int)a4.w, 0, 0, 0, 0};
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      uint4 b4 = *reinterpret_cast<const uint4*>(base + ((b_off + u * 2048) ^ (j * 16)));
      fb[u] = v8i_t{(int)b4.x, (int)b4.y, (int)b4.z, (int)b4.w, 0, 0, 0, 0};
    }
  };
  auto read_scales = [&](const uint8_t* sblock, int (&xa)[4][2], int (&xb)[2][2]) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const uint32_t* p = reinterpret_cast<const uint32_t*>(sblock + sa_off + t * 32 * GT_SCALE_PITCH * 4);
      xa[t][0] = (int)p[0];
      xa[t][1] = (int)p[1];
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const uint32_t* p = reinterpret_cast<const uint32_t*>(sblock + sb_off + u * 32 * GT_SCALE_PITCH * 4);
      xb[u][0] = (int)p[0];
      xb[u][1] = (int)p[1];
    }
  };
  // 8 MFMAs of K step J of stage I (inside its block)
  auto mfma8 = [&](auto ic, auto jc, const v8i_t (&fa)[4], const v8i_t (&fb)[2]) {
    constexpr int I = decltype(ic)::value, J = decltype(jc)::value;
    constexpr int SEL = 2 * (I & 1) + J, D = I >> 1;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int u = 0; u < 2; ++u)
        acc[t][u] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[u], fa[t], acc[t][u], 4, 4, SEL, sb[u][D], SEL, sa[t][D]);
  };
  // Barrier between stages.  At most the 4 loads of the youngest stage may still be in flight, so the stage read next is
  // complete for this wave (vmcnt is in issue order), its LDS writes (scales) are done, and after the barrier that holds
  // for every wave.  The asm keeps the compiler from moving LDS accesses across it.
  auto stage_barrier = [&]() { asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

  // One stage s = 4 kb + I: LDS slot I; the next stage lives in slot (I + 1) % 4.
  //   barrier (stage s+1 has landed for every wave); issue the loads of stage s+3 into the slot stage s-1 used;
  //   6 x {MFMA, LDS read}   j=0 MFMAs 0-5 + the j=1 pieces of this stage;  2 more j=0 MFMAs
  //   6 x {MFMA, LDS read}   j=1 MFMAs 0-5 + the next stage's j=0 pieces;   2 more j=1 MFMAs
  auto stage = [&](auto ic, int s) {
    constexpr int I = decltype(ic)::value;
    stage_barrier();
    gload(s + 3, (I + 3) & 3);
    read_frags(I, 1, fa1, fb1);
    mfma8(ic, std::integral_constant<int, 0>{}, fa0, fb0);
    read_frags((I + 1) & 3, 0, fa0, fb0);
    mfma8(ic, std::integral_constant<int, 1>{}, fa1, fb1);
    __builtin_amdgcn_sched_group_barrier(0x020, 4, 0);
#pragma unroll
    for (int q = 0; q < 6; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
#pragma unroll
    for (int q = 0; q < 6; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- prologue: stages 0, 1, 2 in flight into their slots; scale block 0 in LDS, block 1 in flight; then the first
  // stage's j=0 pieces and the first block's scales in registers.  Stages beyond K load zeros and blocks beyond K load
  // unit scales, so nothing below is conditional.
  sload(0);
  gload(0, 0);
  swrite(0);
  sload(1);
  gload(1, 1);
  gload(2, 2);
  asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");   // stage 0 and scale block 0 visible to all
  read_frags(0, 0, fa0, fb0);
  read_scales(reinterpret_cast<const uint8_t*>(sscale), sa, sb);

  // ---- main loop: one iteration = one 512-K block = 4 stages; LDS slot = stage % 4.
  for (int kb = 0; kb < KB; ++kb) {
    const int s = kb * 4;
    const uint8_t* sblock_next = reinterpret_cast<const uint8_t*>(sscale + ((kb + 1) & 1) * GT_SCALE_BUF_DW);
    stage(std::integral_constant<int, 0>{}, s + 0);
    stage(std::integral_constant<int, 1>{}, s + 1);
    swrite(kb + 1);          // block kb+1 -> the other scale buffer (last read in iteration kb-1); visible after the next barrier
    sload(kb + 2);
    stage(std::integral_constant<int, 2>{}, s + 2);
    stage(std::integral_constant<int, 3>{}, s + 3);
    read_scales(sblock_next, sa, sb);   // next block's scales (written two stages ago)
  }
  // loads of the (zero-filled) stages past the end may still be landing in the ring the epilogue reuses
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// Stores the tile: accumulator register v of MFMA tile (t, u) is C[m][n] with
//   m = m0 + 128 wm + 32 t + r,  n = n0 + 64 wn + 32 u + 8 (v / 4) + 4 h + v % 4.
// Rows outside [m_lo, m_hi) and columns at or beyond n_hi are not written.  Host-checked: N % 8 == 0, ldc % 8 == 0,
// 16-byte aligned c.
template <typename OutT>
__device__ __forceinline__ void gemm_tile_store(const TileArgs& ta, TileAcc& acc, OutT* __restrict__ c, int64_t ldc, uint8_t* smem) {
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int wm = wave >> 2, wn = wave & 3;
  const int r = lane & 31, h = lane >> 5;
  if constexpr (sizeof(OutT) == 2) {
    // bf16: the 256x256 tile (128 KB) is assembled in LDS as rows of 32 16-byte chunks, chunk index XORed with row % 32
    // (conflict-free for the 8-byte writes of 32 different rows and for the row-wise 16-byte reads), then stored as
    // whole rows: 32 lanes x 16 bytes = one 512-byte row segment per half-wave.
    __syncthreads();   // every wave is done reading operand pieces
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int ml = 128 * wm + 32 * t + r;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) {
          const int chunk = 8 * wn + 4 * u + vq;
          float f0 = acc[t][u][4 * vq + 0] * ta.out_scale, f1 = acc[t][u][4 * vq + 1] * ta.out_scale;
          float f2 = acc[t][u][4 * vq + 2] * ta.out_scale, f3 = acc[t][u][4 * vq + 3] * ta.out_scale;
          uint2 o;
          o.x = f32_to_bf16_bits(f0) | (f32_to_bf16_bits(f1) << 16);
          o.y = f32_to_bf16_bits(f2) | (f32_to_bf16_bits(f3) << 16);
          *reinterpret_cast<uint2*>(smem + ml * 512 + ((chunk ^ (ml & 31)) << 4) + 8 * h) = o;
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 16; ++it) {
      const int id = it * GT_THREADS + tid;
      const int row = id >> 5, ch = id & 31;
      const uint4 v = *reinterpret_cast<const uint4*>(smem + row * 512 + ((ch ^ (row & 31)) << 4));
      const int64_t m = ta.m0 + row, n = ta.n0 + 8 * ch;
      if (m >= ta.m_lo && m < ta.m_hi && n + 8 <= ta.n_hi) *reinterpret_cast<uint4*>(c + m * ldc + n) = v;
    }
  } else {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int64_t m = ta.m0 + 128 * wm + 32 * t + r;
      const bool mok = m >= ta.m_lo && m < ta.m_hi;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) {
          const int64_t n = ta.n0 + 64 * wn + 32 * u + 8 * vq + 4 * h;
          if (mok && n + 4 <= ta.n_hi)
            *reinterpret_cast<float4*>(c + m * ldc + n) = make_float4(acc[t][u][4 * vq + 0] * ta.out_scale, acc[t][u][4 * vq + 1] * ta.out_scale,
                                                                        acc[t][u][4 * vq + 2] * ta.out_scale, acc[t][u][4 * vq + 3] * ta.out_scale);
        }
      }
    }
  }
}

template <typename OutT, bool KTAIL>
__device__ __forceinline__ void gemm_tile_256x256(const TileArgs& ta, OutT* __restrict__ c, int64_t ldc, uint8_t* smem) {
  TileAcc acc;
  gemm_tile_zero(acc);
  gemm_tile_mainloop<KTAIL>(ta, acc, smem);
  gemm_tile_store<OutT>(ta, acc, c, ldc, smem);
}

}  // namespace alto
