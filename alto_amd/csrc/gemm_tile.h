// LDS-tiled MXFP4 GEMM tile for gfx950: one workgroup of 512 threads (8 waves, 2 x 4) computes a 256x256 tile of
// C = A . B^T with v_mfma_scale_f32_32x32x64_f8f6f4; each wave owns 128 (M) x 64 (N) = 4 x 2 MFMA tiles (128 accumulator
// registers), so two waves share every SIMD and cover each other's waits.
//
// Data path per macro stage of 256 K elements (128 B = one cache line per operand row):
//   global --buffer_load_dwordx4 ... lds (no register staging)--> LDS ring of 2 stages (64 KB each)
//   LDS --ds_read_b128--> MFMA operands, four K steps of 64 per stage.
//   The loads ask for whole 128-byte lines (8 lanes per row): the path from L2 into the compute unit moves whole lines,
//   so half-line requests (a 128-K stage) cost twice the fill bandwidth, which is what bounds this kernel before the
//   MFMA pipe does.  LDS instructions cost issue time on the SIMD that also issues the MFMAs -- about 12 clocks per
//   ds_read_b128 and 40 per ds_write_b128 -- so the operand tiles never pass through ds_write.
//   A 16-byte piece holds one MX block (32 codes); lane (r, h) of the MFMA takes piece 2j + h of row r at K step j, so a
//   row's eight pieces are XOR-swizzled by (row / 2) % 8 inside its 128 bytes: 16 consecutive rows of a fragment read
//   then cover the 64 LDS banks exactly once (ds_read_b128 serves 16 lanes per clock).
// Scales: one byte per row per 32 K (1D) or per 32 rows (2D).  They are staged through LDS per block of 512 K (16 bytes
//   per row, rows at a 20-byte pitch) so that 1D and 2D scales look alike to the MFMA loop; inside a row the bytes are
//   regrouped so that the 8 bytes a lane needs for the 8 K steps of a block are contiguous, and op_sel picks the byte.
// The MFMA takes B rows as its first operand: accumulator registers then run along N (4 consecutive columns per lane).
// bf16 results go through LDS (swizzled 16-byte chunks) so that the global stores are whole 512-byte row segments; the
// stores are non-temporal: nobody re-reads the tile soon, and as ordinary stores its 128 KB push operand lines that the
// neighbouring workgroups still share out of the XCD's L2 (the grouped kernels, whose output is large, gain 5 to 10 %).
#pragma once
#include <type_traits>

#include "gemm_simple.h"

namespace alto {

constexpr int GT_TM = 256, GT_TN = 256, GT_TK = 256;
constexpr int GT_THREADS = 512;
constexpr int GT_STAGE_BYTES = (GT_TM + GT_TN) * (GT_TK / 2);   // 65536
constexpr int GT_NSTAGE = 2;
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
  int s_k0;                    // first scale byte of this reduction inside the operands' scale rows (0 unless a sub-range of K)
  int s_row;                   // length of a whole scale row in bytes (>= 16): loads never reach past it
  int k_lead = 0;              // the first k_lead (< 8) K groups of the reduction read as zero codes: a reduction over a
                               // sub-range of K starts at the 128-byte line that holds its first group, so that every
                               // operand load is one whole line, and the groups before the range drop out this way
  int ps_q0 = 0;               // packed scales, reduction over a sub-range of K: the 512-K block of the packed layout that
  int ps_sh = 0;               // holds the range's first stage, and 1 when that stage is the block's second half
};

// Every field of TileArgs is the same for all lanes.  When the struct arrives through memory (a real function call) the
// compiler no longer knows that and would wrap each buffer load in a per-lane loop; this copies the fields into
// scalar registers.
__device__ __forceinline__ int64_t uniform_i64(int64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ OperandView uniform_view(const OperandView& v) {
  OperandView o;
  o.codes = reinterpret_cast<const uint8_t*>(uniform_i64(reinterpret_cast<int64_t>(v.codes)));
  o.ld = uniform_i64(v.ld);
  o.scales = reinterpret_cast<const uint8_t*>(uniform_i64(reinterpret_cast<int64_t>(v.scales)));
  o.ss_r = uniform_i64(v.ss_r);
  o.ss_k = uniform_i64(v.ss_k);
  o.is_2d = __builtin_amdgcn_readfirstlane(v.is_2d);
  return o;
}
__device__ __forceinline__ TileArgs uniform_args(const TileArgs& t) {
  TileArgs o;
  o.A = uniform_view(t.A);
  o.B = uniform_view(t.B);
  o.m0 = uniform_i64(t.m0); o.n0 = uniform_i64(t.n0);
  o.m_lo = uniform_i64(t.m_lo); o.m_hi = uniform_i64(t.m_hi); o.n_hi = uniform_i64(t.n_hi);
  o.G = __builtin_amdgcn_readfirstlane(t.G);
  o.out_scale = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, t.out_scale)));
  o.a_bytes = uniform_i64(t.a_bytes); o.b_bytes = uniform_i64(t.b_bytes);
  o.as_bytes = uniform_i64(t.as_bytes); o.bs_bytes = uniform_i64(t.bs_bytes);
  o.s_k0 = __builtin_amdgcn_readfirstlane(t.s_k0); o.s_row = __builtin_amdgcn_readfirstlane(t.s_row);
  o.k_lead = __builtin_amdgcn_readfirstlane(t.k_lead);
  o.ps_q0 = __builtin_amdgcn_readfirstlane(t.ps_q0); o.ps_sh = __builtin_amdgcn_readfirstlane(t.ps_sh);
  return o;
}

typedef v16f_t TileAcc[4][2];   // per wave: 4 (M) x 2 (N) MFMA tiles of 32x32

__device__ __forceinline__ void gemm_tile_zero(TileAcc& acc) {
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[t][u][v] = 0.0f;
}

// Per-thread state of the global -> LDS operand loads and the scale loads of one tile.
//   Operands: instruction i (0..7) of a wave moves chunk q = 8 i + wave = 8 tile rows x 128 bytes (whole cache lines).
//   Chunks 0..31 are A rows, 32..63 B rows.  Lane l holds row 8 q + l / 8, slot l % 8, which stores global piece
//   (l % 8) ^ ((row / 2) % 8) of that row.  Raw buffer loads: 32-bit per-lane byte offsets, the K offset of the stage
//   rides in the scalar offset, and a piece beyond the end of K gets an out-of-range offset, for which the hardware
//   returns zeros.  (Per-load offsets are recomputed at every stage rather than kept in 8 registers.)
//   Scales: thread t owns tile row t of A (t < 256) or tile row t - 256 of B (unit stride along K, any alignment).
struct TileLoader {
  __amdgpu_buffer_rsrc_t rsrc_a, rsrc_b, rsrc_s;
  int wave, gpiece, arow0, brow0, a_last, a_first, b_last, kbytes, G, s_k0, s_row, k_lead;
  uint32_t ld_a, ld_b, soff;

  __device__ __forceinline__ void init(const TileArgs& ta) {
    const int tid = threadIdx.x;
    wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // the wave index lives in a scalar register
    const int lane = tid & 63;
    rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(ta.A.codes), 0, (int)ta.a_bytes, 0x00020000);
    rsrc_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(ta.B.codes), 0, (int)ta.b_bytes, 0x00020000);
    gpiece = (lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7);
    arow0 = (int)ta.m0 + 8 * wave + (lane >> 3);
    brow0 = (int)ta.n0 + 8 * wave + (lane >> 3);
    a_last = (int)ta.m_hi - 1;
    a_first = (int)ta.m_lo;
    b_last = (int)ta.n_hi - 1;
    ld_a = (uint32_t)ta.A.ld;
    ld_b = (uint32_t)ta.B.ld;
    kbytes = ta.G * 16;
    G = ta.G;
    s_k0 = ta.s_k0;
    s_row = ta.s_row;
    k_lead = ta.k_lead;
    const bool s_is_a = wave < GT_TM / 64;   // scalar: the descriptor choice below must be provably wave-uniform
    rsrc_s = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(s_is_a ? ta.A.scales : ta.B.scales), 0,
                                               (int)(s_is_a ? ta.as_bytes : ta.bs_bytes), 0x00020000);
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

  // Direct-to-LDS load of stage s into ring slot `slot`, instructions i0 .. i1-1 of the stage's eight (0-3: A rows,
  // 4-7: B rows): lane l of instruction i lands at chunk base + 16 l.
  __device__ __forceinline__ void gload(uint8_t* smem, int s, int slot, int i0, int i1) const {
    typedef __attribute__((address_space(3))) uint8_t lds_u8;
    lds_u8* const lds = (lds_u8*)smem;
    const int koff = __builtin_amdgcn_readfirstlane(s * 128);   // scalar offset operand: must live in an SGPR
    // a piece beyond K gets bit 31 set in its offset: out of range for the descriptor, so zeros land in LDS
    const uint32_t oob = (koff + gpiece * 16 < kbytes && s * 8 + gpiece >= k_lead) ? 0u : 0x80000000u;
#pragma unroll
    for (int i = i0; i < i1; ++i) {
      int row;
      uint32_t off;
      if (i < 4) {
        row = arow0 + 64 * i;
        row = row < a_last ? row : a_last;
        row = row > a_first ? row : a_first;
        off = (uint32_t)row * ld_a;
      } else {
        row = brow0 + 64 * (i - 4);
        row = row < b_last ? row : b_last;
        off = (uint32_t)row * ld_b;
      }
      off = (off + gpiece * 16) | oob;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(i < 4 ? rsrc_a : rsrc_b,
                                               (__attribute__((address_space(3))) void*)(lds + slot * GT_STAGE_BYTES + (8 * i + wave) * 1024),
                                               16, (int)off, koff, 0, 0);
    }
  }

  // 16 scale bytes of K block kb for this thread's row, in two parts so that nothing touches the loaded registers until
  // they are used (the wave would otherwise sit out the load's latency right here, two blocks before the bytes are needed):
  // sload sends the load, sfix -- called when the bytes go to LDS -- makes groups at or beyond G read as 127 (scale 1.0),
  // so that the zero codes of a K tail never meet a NaN scale byte.
  template <bool KTAIL>
  __device__ __forceinline__ void sload(int kb, v4i_t& raw) const {
    const int kb16 = __builtin_amdgcn_readfirstlane(kb * 16);
    if constexpr (!KTAIL) {   // G % 4 == 0 and the whole K range: every dword is all inside or all beyond K, one 16-byte load
      raw = __builtin_amdgcn_raw_buffer_load_b128(rsrc_s, (int)soff, kb16, 0);
      return;
    }
    // General case (any G, any sub-range of K): still one 16-byte load per row.  A block that would reach past the end
    // of the scale row is loaded from the last 16 bytes of the row instead (and shifted down by the difference in sfix),
    // so no byte from beyond the row (possibly beyond the buffer) is ever used.
    const int want = s_k0 + kb16;                     // where the block starts in the scale row
    const int last = s_row - 16;
    const int off = __builtin_amdgcn_readfirstlane(want < last ? want : last);
    raw = __builtin_amdgcn_raw_buffer_load_b128(rsrc_s, (int)soff, off, 0);
  }
  // FAST: the caller knows that the block lies inside its scale row and inside K (every block but the last of a
  // reduction): the bytes are used as loaded
  template <bool KTAIL, bool FAST = false>
  __device__ __forceinline__ void sfix(int kb, const v4i_t& L, uint32_t (&sreg)[4]) const {
    if constexpr (KTAIL && FAST) {
#pragma unroll
      for (int d = 0; d < 4; ++d) sreg[d] = (uint32_t)L[d];
      return;
    }
    const int rem = G - kb * 16;   // wave-uniform
    if constexpr (!KTAIL) {
#pragma unroll
      for (int d = 0; d < 4; ++d) sreg[d] = rem - 4 * d >= 4 ? (uint32_t)L[d] : 0x7F7F7F7Fu;
      return;
    }
    // bytes at or beyond G become 127; all shift amounts and masks are wave-uniform and applied with mask arithmetic
    const int want = s_k0 + kb * 16;
    const int last = s_row - 16;
    const int off = want < last ? want : last;
    int sh = want - off;                                 // bytes to shift down: 0 unless clamped
    sh = sh > 16 ? 16 : sh;
    const int q = sh >> 2, rb = sh & 3;
    int valid = rem < 0 ? 0 : (rem > 16 ? 16 : rem);     // bytes of this block that lie inside K
    uint32_t mq[5];
#pragma unroll
    for (int c = 0; c < 5; ++c) mq[c] = (uint32_t)(-(int)(q == c));   // all ones for the dword shift in effect
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      uint32_t lo = 0, hi = 0;
#pragma unroll
      for (int c = 0; c < 5; ++c) {
        const uint32_t xl = d + c < 4 ? (uint32_t)L[(d + c) & 3] : 0x7F7F7F7Fu;
        const uint32_t xh = d + c + 1 < 4 ? (uint32_t)L[(d + c + 1) & 3] : 0x7F7F7F7Fu;
        lo |= xl & mq[c];
        hi |= xh & mq[c];
      }
      const uint32_t w = __builtin_amdgcn_alignbyte(hi, lo, (uint32_t)rb);
      int nv = valid - 4 * d;
      nv = nv < 0 ? 0 : (nv > 4 ? 4 : nv);
      const uint32_t keep = (uint32_t)((1ull << (8 * nv)) - 1ull);
      sreg[d] = (w & keep) | (0x7F7F7F7Fu & ~keep);
    }
  }
};

// K loop of one 256x256 tile: acc += A[m0.., :] . B[n0.., :]^T over G groups of 32.  KTAIL = false requires G % 16 == 0
// (K a multiple of 512) and s_k0 == 0: then every 16-byte scale block of a row lies inside the row.  KTAIL = true
// handles any G and any start inside the scale rows (a reduction over a sub-range of K).  Requirements
// checked by the host: unit-stride scale rows, operand extents below 2^31 bytes.  Every thread of the workgroup must
// call it; it may be called again (same or other operands) to keep accumulating.
// How the reduction ends (KTAIL only; K is padded to whole 512-K blocks otherwise):
//   LMS = -1  every 512-K block that holds any K runs both of its 256-K stages in full (any G, nothing known at compile time)
//   LMS = -2  as -1, but a last block whose second stage lies wholly beyond K runs its first stage only (tested at run
//             time; for callers whose G differs from call to call)
//   LMS = 0/1 the caller knows G when it picks the kernel: the last stage that holds any K is stage LMS of its block and
//             has NST (1 .. 4) K steps of 64; it runs exactly those, without the wait and the barrier of a full stage
//             (nothing is loaded behind it), the stage before it loads nothing beyond K, and no stage beyond it runs at
//             all.  No run-time test: the tile needs nearly every register, and control flow around its MFMAs makes the
//             compiler spill.  Without a K tail the reduction always ends this way (LMS = 1, NST = 4).
// PS: both operands bring their scale bytes in the packed form of alto_mxfp4_pack_scales -- [block of 512 K][row][16 bytes
// in the order of the LDS row below, bytes beyond K = 127] -- with OperandView::scales the base of it and
// OperandView::ss_k the bytes from one block to the next (rows x 16).  A block of a tile's 256 + 256 rows is then 8 runs of
// 1 KB, which the eight waves move straight into LDS with one load each (no registers, no fix-up, no ds_write; 8 cache
// lines per load instead of the 64 of per-row scale rows).  Needs the end of K at compile time (LMS >= 0, or no K tail).
template <bool KTAIL, int LMS = -1, int NST = 4, int PS = 0>
__device__ __forceinline__ void gemm_tile_mainloop(const TileArgs& ta, TileAcc& acc, uint8_t* smem) {
  static_assert(PS != 1 || !KTAIL || LMS >= 0, "packed scales: the end of K must be known at compile time");
  static_assert(PS != 2 || (KTAIL && LMS < 0), "packed scales of a sub-range of K: the generic endings only");
  constexpr int SP = PS ? 4 : GT_SCALE_PITCH;   // dwords per row of a scale buffer in LDS
  TileLoader ld;
  v4i_t sraw;   // scale bytes of a later block, as loaded
  __syncthreads();   // the LDS ring may still be read by a previous call
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;   // the wave index lives in a scalar register
  const int wm = wave >> 2, wn = wave & 3;
  const int r = lane & 31, h = lane >> 5;
  uint32_t* sscale = reinterpret_cast<uint32_t*>(smem + GT_NSTAGE * GT_STAGE_BYTES);
  const int KB = (ta.G + 15) / 16;       // loop iterations: blocks of 512 K = 2 macro stages

  // ---- fragment read offsets (bytes inside a stage): row * 128 + ((2 j + h) ^ ((row / 2) % 8)) * 16; the j-dependent
  // part is an XOR with 32 j
  uint32_t a_off, b_off;   // for j = 0
  {
    const int c0 = (h ^ ((r >> 1) & 7)) << 4;
    a_off = (uint32_t)(128 * wm + r) * 128 + c0;
    b_off = GT_TM * 128 + (uint32_t)(64 * wn + r) * 128 + c0;
  }
  // scale read offsets (bytes): row * 20 + 8h within a block buffer
  const uint32_t sa_off = (uint32_t)(128 * wm + r) * (SP * 4) + 8 * h;
  const uint32_t sb_off = (uint32_t)(GT_TM + 64 * wn + r) * (SP * 4) + 8 * h;

  // LDS row layout (4 dwords): [h=0: K 0..255 | h=0: K 256..511 | h=1: K 0..255 | h=1: K 256..511], where the half-wave h
  // of the MFMA uses group 8 ms + 2 j + h at K step j of macro stage ms: byte j of dword 2 h + ms.
  auto swrite = [&](int kb, auto fastc) {
    uint32_t sreg[4];
    ld.template sfix<KTAIL, decltype(fastc)::value>(kb, sraw, sreg);
    uint32_t* row = sscale + (kb & 1) * GT_SCALE_BUF_DW + tid * GT_SCALE_PITCH;
    row[0] = __builtin_amdgcn_perm(sreg[1], sreg[0], 0x06040200u);   // groups 0, 2, 4, 6
    row[1] = __builtin_amdgcn_perm(sreg[3], sreg[2], 0x06040200u);   // groups 8, 10, 12, 14
    row[2] = __builtin_amdgcn_perm(sreg[1], sreg[0], 0x07050301u);   // groups 1, 3, 5, 7
    row[3] = __builtin_amdgcn_perm(sreg[3], sreg[2], 0x07050301u);   // groups 9, 11, 13, 15
  };

  // Fragment / scale registers: F0 = pieces of K step j = 0 of the current stage (read during the previous stage),
  // F1 = pieces of step j = 1, S = this block's scale bytes (8 per lane and sub-tile, selected by op_sel).
  v8i_t fa0[4], fb0[2], fa1[4], fb1[2];
  int sa[4][2], sb[2][2], sa_next[4][2], sb_next[2][2];
  auto read_frags = [&](int slot, int j, v8i_t (&fa)[4], v8i_t (&fb)[2]) {
    const uint8_t* base = smem + slot * GT_STAGE_BYTES;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      uint4 a4 = *reinterpret_cast<const uint4*>(base + ((a_off ^ (j * 32)) + t * 4096));
      fa[t] = v8i_t{(int)a4.x, (int)a4.y, (int)a4.z, (int)a4.w, 0, 0, 0, 0};
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      uint4 b4 = *reinterpret_cast<const uint4*>(base + ((b_off ^ (j * 32)) + u * 4096));
      fb[u] = v8i_t{(int)b4.x, (int)b4.y, (int)b4.z, (int)b4.w, 0, 0, 0, 0};
    }
  };
  // PS == 2: the reduction starts at stage ps_sh (0 / 1) of packed block ps_q0, so block kn of this loop takes its first
  // stage's bytes from packed block kn, dword 2 h + sh, and its second stage's from packed block kn + sh, dword 2 h + 1 - sh
  // (packed block q sits in scale buffer q & 1).
  const int sh = PS == 2 ? ta.ps_sh : 0;
  auto read_scales2 = [&](int kn, int (&xa)[4][2], int (&xb)[2][2]) {
    const uint32_t o0 = (uint32_t)((kn & 1) * (GT_TM + GT_TN) * SP * 4 + 4 * sh);
    const uint32_t o1 = (uint32_t)(((kn + sh) & 1) * (GT_TM + GT_TN) * SP * 4 + 4 - 4 * sh);
    const uint8_t* sb8 = reinterpret_cast<const uint8_t*>(sscale);
    const uint8_t *a0 = sb8 + (sa_off + o0), *a1 = sb8 + (sa_off + o1), *b0 = sb8 + (sb_off + o0), *b1 = sb8 + (sb_off + o1);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      xa[t][0] = *reinterpret_cast<const int*>(a0 + t * 32 * SP * 4);
      xa[t][1] = *reinterpret_cast<const int*>(a1 + t * 32 * SP * 4);
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      xb[u][0] = *reinterpret_cast<const int*>(b0 + u * 32 * SP * 4);
      xb[u][1] = *reinterpret_cast<const int*>(b1 + u * 32 * SP * 4);
    }
  };
  auto read_scales = [&](const uint8_t* sblock, int (&xa)[4][2], int (&xb)[2][2]) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const uint32_t* p = reinterpret_cast<const uint32_t*>(sblock + sa_off + t * 32 * SP * 4);
      xa[t][0] = (int)p[0];
      xa[t][1] = (int)p[1];
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const uint32_t* p = reinterpret_cast<const uint32_t*>(sblock + sb_off + u * 32 * SP * 4);
      xb[u][0] = (int)p[0];
      xb[u][1] = (int)p[1];
    }
  };
  // packed scales: block kb of this wave's 64 rows (waves 0-3: A rows, 4-7: B rows), 1 KB, straight into scale buffer kb & 1
  const bool ps_a = wave < GT_TM / 64;   // scalar
  const __amdgpu_buffer_rsrc_t rsrc_ps = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(ps_a ? ta.A.scales : ta.B.scales), 0,
                                                                           (int)(ps_a ? ta.as_bytes : ta.bs_bytes), 0x00020000);
  const int ps_row0 = __builtin_amdgcn_readfirstlane((int)((ps_a ? ta.m0 + 64 * wave : ta.n0 + 64 * (wave - GT_TM / 64)) * 16));
  const int ps_blk = __builtin_amdgcn_readfirstlane((int)(ps_a ? ta.A.ss_k : ta.B.ss_k));
  const int ps_q0 = PS == 2 ? ta.ps_q0 : 0;
  auto sdma = [&](int kb) {   // packed block ps_q0 + kb -> scale buffer kb & 1
    typedef __attribute__((address_space(3))) uint8_t lds_u8s;
    const int so = __builtin_amdgcn_readfirstlane((kb + ps_q0) * ps_blk + ps_row0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_ps, (__attribute__((address_space(3))) void*)((lds_u8s*)sscale + (kb & 1) * (GT_TM + GT_TN) * SP * 4 + wave * 1024), 16,
                                             lane * 16, so, 0, 0);
  };
  // 8 MFMAs of K step J (0..3) of macro stage MS (0..1 inside its 512-K block): scale byte J of dword MS
  auto mfma8 = [&](auto msc, auto jc, const v8i_t (&fa)[4], const v8i_t (&fb)[2]) {
    constexpr int MS = decltype(msc)::value, J = decltype(jc)::value;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int u = 0; u < 2; ++u)
        acc[t][u] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[u], fa[t], acc[t][u], 4, 4, J, sb[u][MS], J, sa[t][MS]);
  };
  auto interleave = [&]() {   // 6 x {MFMA, LDS read}, 2 more MFMAs
#pragma unroll
    for (int q = 0; q < 6; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
  };
  auto interleave_loads = [&]() {   // the same with one global->LDS load after every second MFMA
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (q < 2) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
  };
  // One macro stage s = 2 kb + MS (256 K, LDS slot MS), four K steps of 64.  Pieces of step j+1 are read while step j
  // multiplies.  Before the last step: wait for this wave's loads of stage s+1 and meet the other waves -- then stage
  // s+1 is in LDS for everyone and nobody reads this stage's slot any more (its step-3 pieces are in registers), so the
  // loads of stage s+2 go out into it: half of them during the last step, half during the first step of the next
  // stage, one load per two MFMAs.  (A wave issues in order, and the address unit takes a 1 KB load about every 16
  // clocks per compute unit: a burst of eight loads per wave would hold the MFMAs behind it for a thousand clocks.)
  // PEN (the stage before the last one, when the end of K is known at compile time): nothing beyond K is loaded.
  auto stage = [&](auto msc, int s, int kb, auto fastc, auto penc) {
    constexpr int MS = decltype(msc)::value;
    constexpr bool PEN = decltype(penc)::value;
    __builtin_amdgcn_s_setprio(2);
    ld.gload(smem, s + 1, MS ^ 1, 4, 8);
    mfma8(msc, std::integral_constant<int, 0>{}, fa0, fb0);
    read_frags(MS, 1, fa1, fb1);
    interleave_loads();
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_setprio(1);
    mfma8(msc, std::integral_constant<int, 1>{}, fa1, fb1);
    read_frags(MS, 2, fa0, fb0);
    interleave();
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_setprio(0);
    mfma8(msc, std::integral_constant<int, 2>{}, fa0, fb0);
    read_frags(MS, 3, fa1, fb1);
    interleave();
    __builtin_amdgcn_sched_barrier(0);
    // (the wait as a builtin: the compiler's own wait insertion then knows that nothing is outstanding behind it and does
    // not guard later uses of registers loaded before this point)
    __builtin_amdgcn_s_waitcnt(0);
    asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_s_setprio(3);
    if constexpr (MS == 0 && !PEN) {
      if constexpr (PS) {
        sdma(kb + 1 + sh);       // block kb+1 (+1 with a half-block shift) -> the buffer whose bytes are all in registers; this block's second stage waits for it
      } else {
        swrite(kb + 1, fastc);   // block kb+1 -> the other scale buffer (last read at the end of block kb-1)
        ld.template sload<KTAIL>(kb + 2, sraw);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (!PEN) ld.gload(smem, s + 2, MS, 0, 4);
    if constexpr (MS == 1) {   // the next block's scales (in LDS since this stage's barrier) ride along with the last step
      if constexpr (PS == 2) read_scales2(kb + 1, sa_next, sb_next);
      else read_scales(reinterpret_cast<const uint8_t*>(sscale + ((kb + 1) & 1) * (GT_TM + GT_TN) * SP), sa_next, sb_next);
    }
    mfma8(msc, std::integral_constant<int, 3>{}, fa1, fb1);
    read_frags(MS ^ 1, 0, fa0, fb0);
    if constexpr (PEN) interleave();
    else interleave_loads();
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- prologue: stage 0 and scale block 0 into LDS, stage 1 and scale block 1 in flight; then the first step's pieces
  // and the first block's scales in registers.  Stages beyond K load zeros and blocks beyond K load unit scales, so
  // nothing below is conditional.
  ld.init(ta);
  if constexpr (PS) {
    sdma(0);
    if constexpr (PS == 2) sdma(sh);   // with the shift, block 0 also needs packed block 1 (without: block 0 once more)
    ld.gload(smem, 0, 0, 0, 8);
    (void)sraw;
  } else {
    ld.template sload<KTAIL>(0, sraw);
    ld.gload(smem, 0, 0, 0, 8);
    swrite(0, std::false_type{});
    ld.template sload<KTAIL>(1, sraw);
  }
  ld.gload(smem, 1, 1, 0, 4);   // the other half goes out in the first step of the loop
  asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)\n\ts_barrier" ::: "memory");   // all but stage 1's four loads
  read_frags(0, 0, fa0, fb0);
  if constexpr (PS == 2) read_scales2(0, sa, sb);
  else read_scales(reinterpret_cast<const uint8_t*>(sscale), sa, sb);

  // ---- main loop: one iteration = one 512-K block = 2 macro stages
  const int NS = (ta.G + 7) / 8;         // macro stages that hold any K at all
  // ENDS: where K ends is known at compile time (always without a K tail: the second stage of the last block, in full)
  constexpr bool ENDS = KTAIL ? LMS >= 0 : LMS != -3;   // (-3: a caller without a K tail that wants the plain loop over whole blocks)
  constexpr int ELMS = KTAIL ? LMS : 1, ENST = KTAIL ? NST : 4;
  static_assert(!ENDS || (ELMS >= 0 && ELMS <= 1 && ENST >= 1 && ENST <= 4), "last stage: 0 or 1, with 1 to 4 K steps");
  const int KBF = ENDS ? (NS > 0 ? (NS - 1) / 2 : 0) : (KTAIL && LMS == -2 ? NS / 2 : KB);   // whole blocks in the loops
  using F = std::false_type;
  using T = std::true_type;
  int kb = 0;
  auto block = [&](int kb, auto fastc, auto penc) {
    stage(std::integral_constant<int, 0>{}, 2 * kb, kb, fastc, F{});
    stage(std::integral_constant<int, 1>{}, 2 * kb + 1, kb, F{}, penc);
#pragma unroll
    for (int t = 0; t < 4; ++t) { sa[t][0] = sa_next[t][0]; sa[t][1] = sa_next[t][1]; }
#pragma unroll
    for (int u = 0; u < 2; ++u) { sb[u][0] = sb_next[u][0]; sb[u][1] = sb_next[u][1]; }
  };
  if constexpr (KTAIL && !PS) {
    // Iteration kb passes scale block kb + 1 on to LDS.  Only the last block that holds any K (KB - 1, passed on by
    // iteration KB - 2) can reach past its row or past K and needs its bytes fixed; earlier ones are used as loaded,
    // later ones are never read.  Three loops in a row rather than a test inside one: the tile needs nearly every
    // register, and a branch inside the loop body makes the compiler spill.
    // With the end of K known, iteration KB - 2 is the last of the loops (KBF = KB - 1); when the last stage is the
    // first of its block, the second stage of that iteration is the one before it.
    const int kfull = KB - 2;
    for (; kb < kfull && kb < KBF; ++kb) block(kb, T{}, F{});
    for (; kb < kfull + 1 && kb < KBF; ++kb) block(kb, F{}, std::bool_constant<ENDS && ELMS == 0>{});
    if constexpr (!ENDS)
      for (; kb < KBF; ++kb) block(kb, T{}, F{});
  } else {
    for (; kb < KBF; ++kb) block(kb, F{}, F{});
  }
  if constexpr (KTAIL && LMS == -2) {
    if (NS & 1) stage(std::integral_constant<int, 0>{}, 2 * kb, kb, F{}, F{});   // the last block's second stage lies wholly beyond K
  }
  if constexpr (ENDS) {
    if constexpr (ELMS == 1) stage(std::integral_constant<int, 0>{}, 2 * kb, kb, T{}, T{});   // the stage before the last
    // The last stage, only the steps it has: its step-0 pieces are in fa0 / fb0 and its loads have landed (the stage before
    // has waited and met the other waves), its scale bytes are in sa / sb; nothing is loaded behind it, so it neither
    // waits nor meets anybody.
    using LM = std::integral_constant<int, ELMS>;
    if constexpr (ENST > 1) read_frags(ELMS, 1, fa1, fb1);
    mfma8(LM{}, std::integral_constant<int, 0>{}, fa0, fb0);
    if constexpr (ENST > 2) read_frags(ELMS, 2, fa0, fb0);
    if constexpr (ENST > 1) mfma8(LM{}, std::integral_constant<int, 1>{}, fa1, fb1);
    if constexpr (ENST > 3) read_frags(ELMS, 3, fa1, fb1);
    if constexpr (ENST > 2) mfma8(LM{}, std::integral_constant<int, 2>{}, fa0, fb0);
    if constexpr (ENST > 3) mfma8(LM{}, std::integral_constant<int, 3>{}, fa1, fb1);
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
    // LDS byte offset of this lane's 8 bytes of (u, vq): row r of the 32-row band, chunk (8 wn + 4 u + vq) ^ r
    auto stage_out = [&](auto scaled) {
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) {
          const uint32_t off = (uint32_t)(128 * wm + r) * 512 + (((8 * wn + 4 * u + vq) ^ r) << 4) + 8 * h;
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            float f0 = acc[t][u][4 * vq + 0], f1 = acc[t][u][4 * vq + 1], f2 = acc[t][u][4 * vq + 2], f3 = acc[t][u][4 * vq + 3];
            if constexpr (decltype(scaled)::value) {
              f0 *= ta.out_scale; f1 *= ta.out_scale; f2 *= ta.out_scale; f3 *= ta.out_scale;
            }
            uint2 o;
            o.x = pack_bf16x2(f0, f1);
            o.y = pack_bf16x2(f2, f3);
            *reinterpret_cast<uint2*>(smem + off + t * (32 * 512)) = o;
          }
        }
    };
    if (ta.out_scale == 1.0f) stage_out(std::false_type{});
    else stage_out(std::true_type{});
    __syncthreads();
    // thread -> chunk ch of rows row0 + 16 it: the XOR term alternates between two values
    const int row0 = tid >> 5, ch = tid & 31;
    const uint32_t rd_even = (uint32_t)row0 * 512 + ((ch ^ row0) << 4), rd_odd = (uint32_t)(row0 + 16) * 512 + ((ch ^ (row0 + 16)) << 4);
    const bool full = ta.m0 >= ta.m_lo && ta.m0 + GT_TM <= ta.m_hi && ta.n0 + GT_TN <= ta.n_hi && ldc < (1 << 22);
    if (full) {   // no bounds to check; one 64-bit tile origin plus 32-bit offsets
      OutT* origin = c + ta.m0 * ldc + ta.n0;
      const uint32_t step = (uint32_t)ldc * 16;
      uint32_t eoff = (uint32_t)row0 * (uint32_t)ldc + 8 * ch;
#pragma unroll
      for (int it = 0; it < 16; it += 2) {
        const uint4 v0 = *reinterpret_cast<const uint4*>(smem + rd_even + (it / 2) * (32 * 512));
        const uint4 v1 = *reinterpret_cast<const uint4*>(smem + rd_odd + (it / 2) * (32 * 512));
        __builtin_nontemporal_store(*reinterpret_cast<const v4i_t*>(&v0), reinterpret_cast<v4i_t*>(origin + eoff));
        __builtin_nontemporal_store(*reinterpret_cast<const v4i_t*>(&v1), reinterpret_cast<v4i_t*>(origin + (eoff + step)));
        eoff += 2 * step;
      }
    } else {
#pragma unroll
      for (int it = 0; it < 16; ++it) {
        const int row = row0 + 16 * it;
        const uint4 v = *reinterpret_cast<const uint4*>(smem + ((it & 1) ? rd_odd : rd_even) + (it / 2) * (32 * 512));
        const int64_t m = ta.m0 + row, n = ta.n0 + 8 * ch;
        if (m >= ta.m_lo && m < ta.m_hi && n + 8 <= ta.n_hi) __builtin_nontemporal_store(*reinterpret_cast<const v4i_t*>(&v), reinterpret_cast<v4i_t*>(c + m * ldc + n));
      }
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

// LMS / NST: how the reduction ends, as in gemm_tile_mainloop.
template <typename OutT, bool KTAIL, int LMS = -1, int NST = 4, int PS = 0>
__device__ __forceinline__ void gemm_tile_256x256(const TileArgs& ta, OutT* __restrict__ c, int64_t ldc, uint8_t* smem) {
  TileAcc acc;
  gemm_tile_zero(acc);
  // (with fp32 output and no K tail the specialised ending pushes the register allocation into spilling: plain loop there)
  gemm_tile_mainloop<KTAIL, (!KTAIL && sizeof(OutT) == 4) ? -3 : LMS, NST, PS>(ta, acc, smem);
  gemm_tile_store<OutT>(ta, acc, c, ldc, smem);
}

// The (LMS, NST) pair of a reduction over G groups of 32 whose length is known at launch (see gemm_tile_mainloop):
// stage of the last block that holds the end of K, and its number of 64-wide K steps.  G must not be a multiple of 16.
inline void gemm_tile_last_stage(int64_t G, int& lms, int& nst) {
  const int64_t ns = (G + 7) / 8;
  lms = (int)((ns - 1) & 1);
  nst = (int)((G - 8 * (ns - 1) + 1) / 2);
}

}  // namespace alto
