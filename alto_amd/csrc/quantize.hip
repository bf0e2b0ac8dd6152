// Fused MXFP4 quantizer for gfx950.
//
// One workgroup (256 threads) owns a tile of 32 rows x 256 columns of a row-major matrix and can emit,
// from a single read of the tile,
//   * the row output  (blocks of 32 along the contiguous dim):   codes [M][C/2], scales [M][C/32]
//   * the column output (blocks of 32 along the row dim):        codes [C][M/2], scales [C][M/32]
//     optionally preceded by the randomized 32-point Hadamard transform along the row dim
//   * or, for 2D 32x32 blocks, both packings with one shared scale per block.
//
// Row phase: a lane holds 8 consecutive elements (one 128-bit load for bf16); 4 lanes form one MX block,
// so the block absmax is two DPP quad steps.  The raw tile is parked in LDS (at a permuted row when the
// Hadamard permutation is active).  Column phase: thread t owns column t of the tile and reads its 32 rows
// from LDS, so the transform, the absmax and the packing along rows are all in-thread.
#include "common.h"

namespace alto {
namespace {

constexpr int TILE_C = 256;
constexpr int STAGE_PITCH = 9;  // dwords per thread in the private byte-permutation scratch (36 B: conflict-free)

struct QuantParams {
  const void* x;
  int64_t ld_x, bs_x;
  int M, C;
  const uint32_t* rand;
  int64_t ld_r, bs_r;
  uint64_t seed, ctr0;            // in-kernel Philox: key and first counter (used when philox_state is NULL)
  const uint64_t* philox_state;   // device memory {key, first counter}, or NULL
  uint8_t* row_codes;
  uint8_t* row_scales;
  uint8_t* col_codes;
  uint8_t* col_scales;
  int64_t ld_rc, ld_cc;  // row pitch in bytes of the row / column code outputs (>= C/2, M/2)
  uint32_t sign_mask;    // bit k set: Q[k] == -1 (k = position after the permutation)
  uint32_t sign_nib[4];  // the same signs as code bits in row order: bit 4 r + 3 set when row r of a block sits at a position with Q == -1
  uint32_t perm4[8];     // row j of a block -> position perm[j], four bytes per word
  uint32_t pinv4[8];     // position k -> row
  int clip_row;          // 1: multiply by 3/4 (in the input dtype) before encoding the row output
  int clip_col;
  int uos;
  int unit_shift;        // column-output launches: log2 of the bands per unit of the workgroup mapping (3 .. 7)
  int pack_rs, pack_cs;  // 1: the row / column scales go out in the packed form of alto_mxfp4_pack_scales, matrix after matrix
};

// byte position of K group g16 (0..15) inside the 16 bytes of a row and 512-K block of packed scales: 4 (2 h + ms) + j with
// g16 = 8 ms + 2 j + h
__device__ __forceinline__ int packed_scale_pos(int g16) { return 4 * (2 * (g16 & 1) + (g16 >> 3)) + ((g16 >> 1) & 3); }

// byte k of a packed table that lives in scalar registers (k is a compile-time constant where this is used)
__device__ __forceinline__ int packed_byte(const uint32_t (&t)[8], int k) { return (int)((t[k >> 2] >> (8 * (k & 3))) & 0xFFu); }

typedef unsigned short us2_t __attribute__((ext_vector_type(2)));
typedef float f2_t __attribute__((ext_vector_type(2)));
typedef unsigned int v4u_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
  us2_t r = __builtin_elementwise_max(__builtin_bit_cast(us2_t, a), __builtin_bit_cast(us2_t, b));
  return __builtin_bit_cast(uint32_t, r);
}

// z / float32(sqrt(32)) correctly rounded, without the full division sequence: one Newton correction with FMAs.
__device__ __forceinline__ float div_sqrt32(float z) {
  const float c = 5.656854152679443f;
  const float rc = 0.17677669529663689f;  // nearest fp32 to 1/c
  float q = z * rc;
  float r = __builtin_fmaf(-q, c, z);
  r = __builtin_fmaxf(r, -3.0e38f);  // z = +-inf gives r = NaN: drop it so that the quotient stays +-inf like a true division
  return __builtin_fmaf(r, rc, q);
}

// (z * sign) / float32(sqrt(32)) with `flip` = 0 or 0x80000000.  The sign of the quotient is taken from the dividend so
// that signed zeros come out as a true division gives them (the FMA correction alone would turn -0 into +0).
__device__ __forceinline__ float div_sqrt32_signed(float z, uint32_t flip) {
  uint32_t q = f2u(div_sqrt32(z));
  uint32_t s = f2u(z) ^ flip;
  return u2f((q & 0x7FFFFFFFu) | (s & 0x80000000u));
}

template <typename T>
__device__ __forceinline__ float round_to_T(float v) {
  if constexpr (sizeof(T) == 2) {   // float -> bf16 (round to nearest even, one v_cvt_pk_bf16_f32 per pair) -> float
    const __bf16 b = (__bf16)v;
    return u2f((uint32_t)__builtin_bit_cast(unsigned short, b) << 16);
  }
  return v;
}

// SR: 0 = round to nearest even, 1 = stochastic with supplied random words, 2 = stochastic with Philox words made here,
// 3 = stochastic with the hardware converts v_cvt_scalef32_sr_pk_fp4_{bf16,f32} (one random dword per PAIR of
// neighbouring elements along the quantisation axis, as the reference's gfx950 path has it,
// mxfp_quantization.py:133-182), dwords cut from Philox words made here.  What the instruction does with the dword
// (measured on the instruction itself): the element in the low half is rounded by adding the dword's top bits under
// the kept mantissa bit and truncating -- bits 31..10 for an fp32 source, bits 31..26 for a bf16 source -- and the
// element in the high half by the same rule with the dword shifted left by one.  A bf16 pair therefore consumes
// the top 7 bits of its dword only, and four pairs share one Philox word (pair k of the four gets word << 8 k).
// Which word belongs to which pair is a function of (batch, row, column) alone:
//   nb = ceil(M / 32) row bands; row-copy calls R = batch nb C (bf16) or 4 batch nb C (fp32);
//   row copy, element (b, i, j):  bf16  call ((b nb + i/32) (C/8) + j/8) 8 + i%8, word (i%32)/8, shift 8 ((j%8)/2)
//                                 fp32  call that * 4 + (i%32)/8,              word (j%8)/2
//   column copy, rows (2p, 2p+1) of band i/32, column j (after the Hadamard transform, in output row order):
//                                 bf16  call R + (b nb + i/32) C + j,  word (p%16)/4, shift 8 (p%4)
//                                 fp32  call R + ((b nb + i/32) C + j) 4 + (p%16)/4,  word p%4
//   where "call c" is the Philox4x32-10 block with the 128-bit counter offset + c.  A 2D-block quantisation has one
//   set of codes: its column packing holds the codes of the row copy.
// Memory is addressed through buffer descriptors that start at the tile (32-bit per-lane offsets, row steps as scalar
// offsets; an offset with bit 31 set is out of range: such a load returns zeros and such a store is dropped, which is
// how rows past M and columns past C are masked).
// BPW: 32-row bands one workgroup walks (1, or 8 for 2D blocks with a column output: the workgroup then holds the eight
// 16-byte pieces of a 128-byte line of every column's codes and stores whole lines, eight columns per wave instruction,
// instead of one piece of 64 different lines per instruction).
template <typename T, bool DO_ROW, bool DO_COL, int SR, bool RHT, bool B2D, bool GEN, int BPW = 1>
__global__ __launch_bounds__(256) void quant_kernel(const QuantParams p) {
  static_assert(BPW == 1 || (BPW == 8 && DO_COL && B2D), "bands per workgroup: 1, or 8 for the column output of 2D blocks");
  constexpr bool BF = sizeof(T) == 2;
  // Both phases consume the same random word per element.  Supplied words (SR == 1): each phase loads them in its own
  // layout, and the column phase's loads go out at the very start, beside the row phase's, so the second request for a
  // line meets the first one in the L2 and memory is read once (measured: fetch = 1.03 x the tensor); staging them in
  // LDS instead costs 32 KB per workgroup, i.e. occupancy, and is 5 % slower.  Words made here (SR == 2) are staged in
  // LDS: making them twice would cost more than the occupancy.
  constexpr bool EARLY = DO_COL && SR == 1;
  constexpr bool STASH = DO_COL && SR == 2;
  constexpr bool HW = SR == 3;
  constexpr bool DEFER_FLIP = RHT && DO_COL && !HW;   // the Hadamard signs go onto the finished column codes
  constexpr bool XCODES = HW && B2D && DO_COL;   // 2D blocks: the column packing takes the row phase's codes through LDS
  constexpr int OOB = (int)0x80000000;
  // the column phase of the hardware mode brings its transformed values back to row order through a private strip per
  // thread (17 dwords of bf16 pairs or 33 dwords of fp32: odd pitches, conflict-free), which reuses the tile's memory
  constexpr int STRIP = BF ? 17 : 33;
  // the column phase hands the hardware converts two rows at a time (stochastic mode with 1D blocks, round to nearest always)
  constexpr bool PAIRS = (HW && !B2D) || SR == 0;
  constexpr int TILE_ELEMS = !DO_COL ? 8 : ((PAIRS && RHT) ? (256 * STRIP * 4 + (int)sizeof(T) - 1) / (int)sizeof(T) : 32 * TILE_C);
  __shared__ __align__(16) T tile[TILE_ELEMS];
  __shared__ __align__(8) uint8_t xcodes[XCODES ? 32 * TILE_C : 8];
  __shared__ __align__(16) uint32_t stash[STASH ? 32 * TILE_C : 4];
  __shared__ uint32_t blkmax[8];
  __shared__ uint8_t sperm[32];
  static_assert(!(DO_COL && RHT) || sizeof(T) * 32 * TILE_C >= 256 * STAGE_PITCH * 4, "the byte scratch of the column phase reuses the tile");

  const int tid = threadIdx.x;
  const int M = p.M, C = p.C;
  // Workgroup -> (column tile bx, 32-row band by; with BPW > 1 read "row of BPW bands" for "band" below).  With a column
  // output the grid is one-dimensional per matrix: consecutive workgroups go to the 8 XCDs in turn, so 8 x 2^unit_shift consecutive ones are laid out as 8 XCDs (one unit = column tile
  // x group of 2^unit_shift bands each, neighbouring column tiles first) x the unit's consecutive bands.  The 16-byte pieces
  // that make up a 128-byte line of the column codes (8 bands), and the bytes of a line of plain column scales (128 bands),
  // are then written through one XCD's L2 within a short time of each other and leave it as whole lines (measured: 65536 x
  // 5760 in 260-300 us instead of 403).  Without a column output: (column tiles, bands).
  const int nby = (M + 31) >> 5;
  int bx, by0;   // column tile; first band of this workgroup
  if constexpr (DO_COL) {
    const unsigned wg = blockIdx.x, us = (unsigned)p.unit_shift;
    const unsigned unit = (wg >> (3 + us)) * 8 + (wg & 7), tiles_x = (unsigned)(C + TILE_C - 1) / TILE_C;
    bx = (int)(unit % tiles_x);
    by0 = (int)(((unit / tiles_x) << us) + ((wg >> 3) & ((1u << us) - 1))) * BPW;
    if (by0 >= nby) return;   // (whole workgroup: padding of the last group of bands / of the units to a multiple of 8)
  } else {
    bx = (int)blockIdx.x;
    by0 = (int)blockIdx.y;
  }
  const int col0 = bx * TILE_C;
  const int64_t b = blockIdx.z;

  if (RHT || B2D) {
    if (tid < 32) sperm[tid] = (uint8_t)((p.perm4[tid >> 2] >> (8 * (tid & 3))) & 0xFFu);
    if (BPW == 1 && tid < 8) blkmax[tid] = 0;
    __syncthreads();
  }
  // column codes of the bands walked so far, oldest first (shifted down one place per band: static register indices)
  uint32_t colacc[BPW > 1 ? BPW : 1][4];
  int bands_done = 0;
#pragma unroll 1
  for (int bi = 0; bi < BPW; ++bi) {
    const int by = by0 + bi;
    if (BPW > 1) {
      if (by >= nby) break;
      __syncthreads();   // the previous band's column phase is done with the tile (and with blkmax)
      if (B2D) {
        if (tid < 8) blkmax[tid] = 0;
        __syncthreads();
      }
    }
    const int row0 = by * 32;

    const int rows_here = M - row0 < 32 ? M - row0 : 32;
    const T* xt = reinterpret_cast<const T*>(p.x) + b * p.bs_x + (int64_t)row0 * p.ld_x;
    const __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<T*>(xt), 0, (int)(((int64_t)(rows_here - 1) * p.ld_x + C) * (int64_t)sizeof(T)), 0x00020000);
    const uint32_t* rt_ = SR == 1 ? p.rand + b * p.bs_r + (int64_t)row0 * p.ld_r : nullptr;
    const __amdgpu_buffer_rsrc_t rsrc_r = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t*>(rt_), 0, SR == 1 ? (int)(((int64_t)(rows_here - 1) * p.ld_r + C) * 4) : 0, 0x00020000);
    const int ldx_b = (int)p.ld_x * (int)sizeof(T), ldr_b = (int)p.ld_r * 4;   // row pitches in bytes

    // Philox: element (b, i, j) consumes word ((b M + i) C + j) of the stream, i.e. word j % 4 of the block with the
    // counter ctr0 + ((b M + i) C + j) / 4.  A lane owns 8 consecutive elements of a row = two blocks.
    uint64_t key = 0, ctr0 = 0, qbase = 0;
    if constexpr (SR == 2 || HW) {
      key = p.philox_state ? p.philox_state[0] : p.seed;
      ctr0 = p.philox_state ? p.philox_state[1] : p.ctr0;
      qbase = ctr0 + (((uint64_t)b * (uint64_t)M + (uint64_t)row0) * (uint64_t)C >> 2);
    }
    const uint64_t band = (uint64_t)b * nby + by;   // hardware mode: index of this 32-row band

    // ------------------------------------------------------------------ row phase
    const int chunk = tid & 31, rsub = tid >> 5;
    const int c = col0 + chunk * 8;
    const bool cok = c < C;
    uint32_t w[4][BF ? 4 : 8];
    uint32_t rr[4][((SR == 1 || SR == 2) && (DO_ROW || STASH)) ? 8 : 1];
    constexpr bool ROW_CODES = DO_ROW || XCODES;   // the row phase encodes (and stores, when DO_ROW)
    uint32_t hw_row[4][(HW && ROW_CODES) ? (BF ? 1 : 4) : 1];
    if constexpr (HW && ROW_CODES) {
      const uint64_t call = (band * (uint64_t)(C >> 3) + (uint64_t)((col0 >> 3) + (tid & 31))) * 8 + (uint64_t)(tid >> 5);
      if constexpr (BF) {
        const uint64_t q = ctr0 + call;
        const uint4 a = philox4x32_10(q, q < ctr0 ? 1ull : 0ull, key);
        hw_row[0][0] = a.x; hw_row[1][0] = a.y; hw_row[2][0] = a.z; hw_row[3][0] = a.w;
      } else {
  #pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint64_t q = ctr0 + call * 4 + (uint64_t)i;
          const uint4 a = philox4x32_10(q, q < ctr0 ? 1ull : 0ull, key);
          hw_row[i][0] = a.x; hw_row[i][1] = a.y; hw_row[i][2] = a.z; hw_row[i][3] = a.w;
        }
      }
    }
    uint32_t amax_i[4];
    bool valid[4];
  #pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = rsub + 8 * i;
      valid[i] = (row0 + r < M) && cok;
      // rows past M are out of the descriptor's range and read as zeros; columns past C get an out-of-range offset
      const int voff = valid[i] ? rsub * ldx_b + c * (int)sizeof(T) : OOB;
      const v4i_t v0 = __builtin_amdgcn_raw_buffer_load_b128(rsrc_x, voff, 8 * i * ldx_b, 0);
      w[i][0] = v0[0]; w[i][1] = v0[1]; w[i][2] = v0[2]; w[i][3] = v0[3];
      if constexpr (!BF) {
        const v4i_t v1 = __builtin_amdgcn_raw_buffer_load_b128(rsrc_x, voff, 8 * i * ldx_b + 16, 0);
        w[i][4] = v1[0]; w[i][5] = v1[1]; w[i][6] = v1[2]; w[i][7] = v1[3];
      }
      if constexpr (SR == 1 && (DO_ROW || STASH)) {
        const int roff = valid[i] ? rsub * ldr_b + c * 4 : OOB;
        const v4i_t r0 = __builtin_amdgcn_raw_buffer_load_b128(rsrc_r, roff, 8 * i * ldr_b, 0);
        const v4i_t r1 = __builtin_amdgcn_raw_buffer_load_b128(rsrc_r, roff, 8 * i * ldr_b + 16, 0);
        rr[i][0] = r0[0]; rr[i][1] = r0[1]; rr[i][2] = r0[2]; rr[i][3] = r0[3];
        rr[i][4] = r1[0]; rr[i][5] = r1[1]; rr[i][6] = r1[2]; rr[i][7] = r1[3];
      }
    }
    uint32_t rc[EARLY ? 32 : 1];
    if constexpr (EARLY) {
      const int cvoff = (col0 + tid < C) ? tid * 4 + col0 * 4 : OOB;
  #pragma unroll
      for (int k = 0; k < 32; ++k) {
        const int row = RHT ? packed_byte(p.pinv4, k) : k;
        rc[k] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsrc_r, cvoff, __builtin_amdgcn_readfirstlane(row * ldr_b), 0);
      }
    }
  #pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = rsub + 8 * i;
      if constexpr (SR == 2) {
        const uint64_t q0 = qbase + (uint64_t)(uint32_t)((r * C + c) >> 2), q1 = q0 + 1;   // 128-bit counters: the carry goes up
        const uint4 a = philox4x32_10(q0, q0 < ctr0 ? 1ull : 0ull, key);
        const uint4 d = philox4x32_10(q1, q1 < ctr0 ? 1ull : 0ull, key);
        rr[i][0] = a.x; rr[i][1] = a.y; rr[i][2] = a.z; rr[i][3] = a.w;
        rr[i][4] = d.x; rr[i][5] = d.y; rr[i][6] = d.z; rr[i][7] = d.w;
      }
      if (DO_COL) {
        const int pos = RHT ? sperm[r] : r;
        uint4* dst = reinterpret_cast<uint4*>(&tile[pos * TILE_C + chunk * 8]);
        dst[0] = make_uint4(w[i][0], w[i][1], w[i][2], w[i][3]);
        if constexpr (!BF) dst[1] = make_uint4(w[i][4], w[i][5], w[i][6], w[i][7]);
        if constexpr (STASH) {   // the word of row r waits at the position its element takes in the transform
          uint4* sd = reinterpret_cast<uint4*>(&stash[pos * TILE_C + chunk * 8]);
          sd[0] = make_uint4(rr[i][0], rr[i][1], rr[i][2], rr[i][3]);
          sd[1] = make_uint4(rr[i][4], rr[i][5], rr[i][6], rr[i][7]);
        }
      }
      if (DO_ROW || B2D) {
        uint32_t a;
        if constexpr (BF) {
          a = pk_max_u16(pk_max_u16(w[i][0] & 0x7FFF7FFFu, w[i][1] & 0x7FFF7FFFu),
                         pk_max_u16(w[i][2] & 0x7FFF7FFFu, w[i][3] & 0x7FFF7FFFu));
          a = max(a & 0xFFFFu, a >> 16);
        } else {
          a = 0;
  #pragma unroll
          for (int e = 0; e < 8; ++e) a = max(a, w[i][e] & 0x7FFFFFFFu);
        }
        a = max(a, dpp_u32<ALTO_DPP_QUAD_XOR1>(a));
        a = max(a, dpp_u32<ALTO_DPP_QUAD_XOR2>(a));
        amax_i[i] = a;
        if (B2D && (tid & 3) == 0) atomicMax(&blkmax[chunk >> 2], a);
      }
    }
    if (B2D || DO_COL) __syncthreads();

    if (ROW_CODES || B2D) {
      // descriptors of the row outputs start at the tile's first row
      const __amdgpu_buffer_rsrc_t rsrc_rc = __builtin_amdgcn_make_buffer_rsrc(
          DO_ROW ? p.row_codes + (b * M + row0) * p.ld_rc : nullptr, 0, DO_ROW ? 0x7FFFFFFF : 0, 0x00020000);
      // Row scales, plain: [M][C/32], the byte of (row, group g) at row * (C/32) + g.  Packed (per matrix): the 16 groups of
      // a row's 512-element block share 16 bytes, ((g / 16) M + row) 16 + packed_scale_pos(g % 16).  One store serves both:
      // the row pitch and the lane's column term are chosen here, outside the loop.
      // With 2D blocks the packed form repeats the block's scale for each of its 32 rows (the GEMM reads one layout).
      const bool prs = DO_ROW && p.pack_rs;
      const bool rs_rows = DO_ROW && (!B2D || prs);   // a scale byte per row goes out
      const int ldrs = prs ? 16 : C / 32;
      const int rs_col = prs ? ((c >> 9) * M) * 16 + packed_scale_pos((c >> 5) & 15) : (c >> 5);
      const __amdgpu_buffer_rsrc_t rsrc_rs = __builtin_amdgcn_make_buffer_rsrc(
          rs_rows ? p.row_scales + (prs ? (b * (int64_t)((C + 511) >> 9) * M + row0) * 16 : (b * M + row0) * (int64_t)(C / 32)) : nullptr, 0,
          rs_rows ? 0x7FFFFFFF : 0, 0x00020000);
      const int ldrc = (int)p.ld_rc;
      if (prs && ((C >> 5) & 15) != 0 && col0 + TILE_C >= C) {   // packed: the groups of the last block beyond C read as 127
        const bool last = (tid & 3) == 0 && (c >> 5) == (C >> 5) - 1;
        for (int gp = (C >> 5) & 15; gp < 16; ++gp) {
          const int off = rsub * 16 + ((c >> 9) * M) * 16 + packed_scale_pos(gp);
  #pragma unroll
          for (int i = 0; i < 4; ++i) __builtin_amdgcn_raw_buffer_store_b8((uint8_t)127, rsrc_rs, (last && valid[i]) ? off : OOB, 8 * i * 16, 0);
        }
      }
      uint32_t blk = B2D ? blkmax[chunk >> 2] : 0;
  #pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t a = B2D ? blk : amax_i[i];
        uint32_t s;
        if (GEN && p.uos) s = e8m0_uos(BF ? u2f(a << 16) : u2f(a));
        else s = BF ? e8m0_from_bf16_bits(a) : e8m0_from_f32_bits(a);
        // scales
        if (!B2D || prs)   // (descriptor without range when no per-row byte is due)
          __builtin_amdgcn_raw_buffer_store_b8((uint8_t)s, rsrc_rs, (valid[i] && (tid & 3) == 0) ? rsub * ldrs + rs_col : OOB, 8 * i * ldrs, 0);
        if (B2D && i == 0 && rsub == 0 && (tid & 3) == 0 && valid[0]) {
          if (DO_ROW && !prs) p.row_scales[(b * (M / 32) + by) * (C / 32) + (c >> 5)] = (uint8_t)s;
          if (DO_COL && !p.pack_cs) p.col_scales[(b * (C / 32) + (c >> 5)) * (M / 32) + by] = (uint8_t)s;
        }
        if constexpr (ROW_CODES) {
        const float scale_f = u2f(s << 23);
        float v[8];
  #pragma unroll
        for (int e = 0; e < 8; ++e) {
          if constexpr (BF) v[e] = (e & 1) ? bf16_hi(w[i][e >> 1]) : bf16_lo(w[i][e >> 1]);
          else v[e] = u2f(w[i][e]);
          if (GEN && p.clip_row) v[e] = round_to_T<T>(v[e] * 0.75f);
        }
        uint32_t out = 0;
        if constexpr (SR == 0) {
          out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, v[0], v[1], scale_f, 0);
          out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, v[2], v[3], scale_f, 1);
          out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, v[4], v[5], scale_f, 2);
          out = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(out, v[6], v[7], scale_f, 3);
        } else if constexpr (HW) {
          uint32_t by[4];   // byte 0 of each result holds the pair's two codes; the other bytes are not defined
  #pragma unroll
          for (int e = 0; e < 4; ++e) {
            if constexpr (BF) {
              const uint32_t src = (GEN && p.clip_row) ? pack_bf16x2(v[2 * e], v[2 * e + 1]) : w[i][e];
              by[e] = __builtin_amdgcn_cvt_scalef32_sr_pk_fp4_bf16(0u, __builtin_bit_cast(bf16x2_t, src), hw_row[i][0] << (8 * e), scale_f, 0);
            } else {
              by[e] = __builtin_amdgcn_cvt_scalef32_sr_pk_fp4_f32(0u, f2_t{v[2 * e], v[2 * e + 1]}, hw_row[i][e], scale_f, 0);
            }
          }
          out = __builtin_amdgcn_perm(by[1], by[0], 0x0C0C0400u) | __builtin_amdgcn_perm(by[3], by[2], 0x04000C0Cu);
        } else {
          const float inv = u2f((254u - s) << 23);
          // sign bits of the eight codes from four hardware converts (their magnitudes are not used): 5 instructions
          // instead of 16
          uint32_t sg = 0;
          if constexpr (BF) {
            sg = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(sg, __builtin_bit_cast(bf16x2_t, w[i][0]), scale_f, 0);
            sg = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(sg, __builtin_bit_cast(bf16x2_t, w[i][1]), scale_f, 1);
            sg = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(sg, __builtin_bit_cast(bf16x2_t, w[i][2]), scale_f, 2);
            sg = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(sg, __builtin_bit_cast(bf16x2_t, w[i][3]), scale_f, 3);
          } else {
            sg = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(sg, v[0], v[1], scale_f, 0);
            sg = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(sg, v[2], v[3], scale_f, 1);
            sg = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(sg, v[4], v[5], scale_f, 2);
            sg = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(sg, v[6], v[7], scale_f, 3);
          }
          out = sg & 0x88888888u;
  #pragma unroll
          for (int e = 0; e < 8; ++e) out |= e2m1_sr_mag(v[e] * inv, rr[i][e]) << (4 * e);
        }
        if constexpr (DO_ROW) __builtin_amdgcn_raw_buffer_store_b32(out, rsrc_rc, valid[i] ? rsub * ldrc + (c >> 1) : OOB, 8 * i * ldrc, 0);
        if constexpr (XCODES) {   // one code per byte, in column order, for the column packing
          const uint32_t ev = out & 0x0F0F0F0Fu, od = (out >> 4) & 0x0F0F0F0Fu;
          uint2 two;
          two.x = __builtin_amdgcn_perm(od, ev, 0x05010400u);
          two.y = __builtin_amdgcn_perm(od, ev, 0x07030602u);
          *reinterpret_cast<uint2*>(&xcodes[(rsub + 8 * i) * TILE_C + chunk * 8]) = two;
        }
        }
      }
    }

    // ------------------------------------------------------------------ column phase
    if (DO_COL) {
      const int cc = col0 + tid;
      const bool cvalid = cc < C;
      float z[32];
      uint32_t zp[(BF && RHT) ? 16 : 1];   // the transformed column as packed bf16 pairs
  #pragma unroll
      for (int k = 0; k < 32; ++k) {
        if (BF) z[k] = u2f((uint32_t)reinterpret_cast<const unsigned short*>(tile)[k * TILE_C + tid] << 16);
        else z[k] = reinterpret_cast<const float*>(tile)[k * TILE_C + tid];
      }
      if (RHT) {
        __syncthreads();   // every thread holds its column: the tile's memory becomes the byte scratch used further down
  #pragma unroll
        for (int h = 1; h < 32; h <<= 1) {
  #pragma unroll
          for (int k = 0; k < 32; ++k) {
            if ((k & h) == 0) {
              float a0 = z[k], a1 = z[k + h];
              z[k] = a0 + a1;
              z[k + h] = a0 - a1;
            }
          }
        }
        // z * (+-1) / float32(sqrt(32)), correctly rounded: quotient estimate, one FMA correction, special cases and the
        // sign by the division fix-up instruction.
  #pragma unroll
        for (int k = 0; k < 32; ++k) {
          // Q[k] = -1: folded into the (wave-uniform) constants in the hardware mode; the software rule, which is short of
          // scalar registers (the 64 signed constants made it spill 24 of them into vector lanes), divides by +sqrt(32) and
          // flips the sign bits of the finished codes instead (DEFER_FLIP below: rounding, absmax and both encodes are
          // symmetric in the sign)
          const uint32_t flip = DEFER_FLIP ? 0u : ((p.sign_mask >> k) & 1u) << 31;
          const float ck = u2f(f2u(5.656854152679443f) ^ flip);
          const float rck = u2f(f2u(0.17677669529663689f) ^ flip);
          const float q = z[k] * rck;
          // v_div_fixup_f32 gives the quotient its sign (sign(z) ^ sign(ck), so -0 stays -0) and returns +-inf for z = +-inf,
          // where the correction term is NaN; otherwise it passes the magnitude through (measured against a max + bit-field
          // insert pair doing the same: 0.6 % faster with the software rule, 1.4 % with the hardware converts)
          z[k] = __builtin_amdgcn_div_fixupf(__builtin_fmaf(__builtin_fmaf(-q, ck, z[k]), rck, q), ck, z[k]);
        }
        if constexpr (BF) {   // round to bf16 two at a time
  #pragma unroll
          for (int k = 0; k < 32; k += 2) {
            zp[k >> 1] = pack_bf16x2(z[k], z[k + 1]);   // the hardware convert takes the packed pairs as they are
            z[k] = u2f(zp[k >> 1] << 16);
            z[k + 1] = u2f(zp[k >> 1] & 0xFFFF0000u);
          }
        }
      }
      uint32_t s;
      if (B2D) {
        uint32_t a = blkmax[tid >> 5];
        if (GEN && p.uos) s = e8m0_uos(BF ? u2f(a << 16) : u2f(a));
        else s = BF ? e8m0_from_bf16_bits(a) : e8m0_from_f32_bits(a);
      } else {
        float am = 0.0f;
  #pragma unroll
        for (int k = 0; k < 32; k += 2) am = __builtin_fmaxf(__builtin_fmaxf(am, __builtin_fabsf(z[k])), __builtin_fabsf(z[k + 1]));
        if (GEN && p.uos) s = e8m0_uos(am);
        else s = BF ? e8m0_from_bf16_bits(f2u(am) >> 16) : e8m0_from_f32_bits(f2u(am));
      }
      // Column scales, plain 1D: [C][M/32], this band's byte of column cc at cc (M/32) + band (2D blocks: the row phase wrote
      // the block's byte).  Packed (per matrix, 1D or 2D blocks): ((band / 16) C + cc) 16 + packed_scale_pos(band % 16); the
      // last band also writes the 127s of the groups beyond M.
      {
        const bool pcs = p.pack_cs;
        const int cs_pitch = pcs ? 16 : M / 32;
        const uint8_t* cs_blk = p.col_scales + ((b * (int64_t)((M + 511) >> 9) + (by >> 4)) * C + col0) * 16;
        const __amdgpu_buffer_rsrc_t rsrc_cs = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint8_t*>(pcs ? cs_blk + packed_scale_pos(by & 15) : p.col_scales + (b * C + col0) * (int64_t)(M / 32) + by), 0, 0x7FFFFFFF, 0x00020000);
        if (!B2D || pcs) __builtin_amdgcn_raw_buffer_store_b8((uint8_t)s, rsrc_cs, cvalid ? tid * cs_pitch : OOB, 0, 0);
        if (pcs && by == (M >> 5) - 1 && ((M >> 5) & 15) != 0) {
          const __amdgpu_buffer_rsrc_t rsrc_pad = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(cs_blk), 0, 0x7FFFFFFF, 0x00020000);
          for (int gp = (M >> 5) & 15; gp < 16; ++gp)
            __builtin_amdgcn_raw_buffer_store_b8((uint8_t)127, rsrc_pad, cvalid ? tid * 16 + packed_scale_pos(gp) : OOB, 0, 0);
        }
      }
      const float scale_f = u2f(s << 23);
      const float inv = u2f((254u - s) << 23);
      uint32_t codes[32];
      uint32_t out[4];
      if constexpr (HW && B2D) {
        // 2D blocks have one set of codes: the row phase left them in LDS, one per byte
        __syncthreads();
  #pragma unroll
        for (int k = 0; k < 32; ++k) codes[k] = xcodes[k * TILE_C + tid];
      } else if constexpr (PAIRS) {
        // transformed values back to row order (a private strip in LDS undoes the permutation), then one hardware
        // convert per pair of rows
        if (GEN && p.clip_col) {
  #pragma unroll
          for (int k = 0; k < 32; ++k) z[k] = round_to_T<T>(z[k] * 0.75f);
        }
        uint32_t* strip = reinterpret_cast<uint32_t*>(tile) + tid * STRIP;
        const uint64_t nrow = (uint64_t)gridDim.z * nby * (uint64_t)C;   // calls of the row copy: batch * bands * C
        uint32_t by[16];
        if constexpr (BF) {
          uint32_t pr[16];
  #pragma unroll
          for (int j = 0; j < 16; ++j) pr[j] = (RHT && !(GEN && p.clip_col)) ? zp[RHT ? j : 0] : pack_bf16x2(z[2 * j], z[2 * j + 1]);
          if (RHT) {
            unsigned short* s16 = reinterpret_cast<unsigned short*>(strip);
  #pragma unroll
            for (int j = 0; j < 16; ++j) {
              s16[packed_byte(p.pinv4, 2 * j)] = (unsigned short)pr[j];
              s16[packed_byte(p.pinv4, 2 * j + 1)] = (unsigned short)(pr[j] >> 16);
            }
            asm volatile("" ::: "memory");   // same thread reads what it wrote: LDS ops of one wave complete in order
  #pragma unroll
            for (int j = 0; j < 16; ++j) pr[j] = strip[j];
          }
          if constexpr (HW) {
            const uint64_t q = ctr0 + nrow + band * (uint64_t)C + (uint64_t)cc;
            const uint4 a = philox4x32_10(q, q < ctr0 ? 1ull : 0ull, key);
            const uint32_t wd[4] = {a.x, a.y, a.z, a.w};
  #pragma unroll
            for (int j = 0; j < 16; ++j)
              by[j] = __builtin_amdgcn_cvt_scalef32_sr_pk_fp4_bf16(0u, __builtin_bit_cast(bf16x2_t, pr[j]), wd[j >> 2] << (8 * (j & 3)), scale_f, 0);
          } else {
  #pragma unroll
            for (int j = 0; j < 4; ++j) {
              uint32_t o = 0;
              o = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(o, __builtin_bit_cast(bf16x2_t, pr[4 * j + 0]), scale_f, 0);
              o = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(o, __builtin_bit_cast(bf16x2_t, pr[4 * j + 1]), scale_f, 1);
              o = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(o, __builtin_bit_cast(bf16x2_t, pr[4 * j + 2]), scale_f, 2);
              o = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(o, __builtin_bit_cast(bf16x2_t, pr[4 * j + 3]), scale_f, 3);
              out[j] = o;
            }
          }
        } else {
          if (RHT) {
            float* sf = reinterpret_cast<float*>(strip);
  #pragma unroll
            for (int k = 0; k < 32; ++k) sf[packed_byte(p.pinv4, k)] = z[k];
            asm volatile("" ::: "memory");
  #pragma unroll
            for (int k = 0; k < 32; ++k) z[k] = sf[k];
          }
          if constexpr (HW) {
  #pragma unroll
            for (int g = 0; g < 4; ++g) {
              const uint64_t q = ctr0 + 4 * nrow + (band * (uint64_t)C + (uint64_t)cc) * 4 + (uint64_t)g;
              const uint4 a = philox4x32_10(q, q < ctr0 ? 1ull : 0ull, key);
              const uint32_t wd[4] = {a.x, a.y, a.z, a.w};
  #pragma unroll
              for (int e = 0; e < 4; ++e)
                by[4 * g + e] = __builtin_amdgcn_cvt_scalef32_sr_pk_fp4_f32(0u, f2_t{z[8 * g + 2 * e], z[8 * g + 2 * e + 1]}, wd[e], scale_f, 0);
            }
          } else {
  #pragma unroll
            for (int j = 0; j < 4; ++j) {
              uint32_t o = 0;
              o = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(o, z[8 * j + 0], z[8 * j + 1], scale_f, 0);
              o = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(o, z[8 * j + 2], z[8 * j + 3], scale_f, 1);
              o = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(o, z[8 * j + 4], z[8 * j + 5], scale_f, 2);
              o = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(o, z[8 * j + 6], z[8 * j + 7], scale_f, 3);
              out[j] = o;
            }
          }
        }
        if constexpr (HW) {
  #pragma unroll
          for (int j = 0; j < 4; ++j)
            out[j] = __builtin_amdgcn_perm(by[4 * j + 1], by[4 * j], 0x0C0C0400u) | __builtin_amdgcn_perm(by[4 * j + 3], by[4 * j + 2], 0x04000C0Cu);
        }
      }
      if constexpr (!HW && !PAIRS) {
  #pragma unroll
      for (int k = 0; k < 32; ++k) {
        float v = z[k];
        if (GEN && p.clip_col) v = round_to_T<T>(v * 0.75f);
        if constexpr (SR == 0) {
          codes[k] = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(0u, v, 0.0f, scale_f, 0) & 0xFu;
        } else {
          uint32_t r;
          if constexpr (EARLY) r = rc[k];
          else r = stash[k * TILE_C + tid];
          const float q = v * inv;
          codes[k] = e2m1_sr_mag(q, r) | ((f2u(q) >> 28) & 8u);
        }
      }
      }
      if constexpr (PAIRS) {
        // out[] is complete
      } else if (RHT) {
        // undo the permutation: position k belongs to row perm_inv[k]; a private byte scratch in LDS does the indexing
        uint32_t* stage = reinterpret_cast<uint32_t*>(tile);
        uint8_t* sb = reinterpret_cast<uint8_t*>(stage + tid * STAGE_PITCH);
  #pragma unroll
        for (int k = 0; k < 32; ++k) sb[packed_byte(p.pinv4, k)] = (uint8_t)codes[k];
        // same thread reads what it wrote: LDS ops of one wave complete in order, no barrier needed
        uint32_t d[8];
  #pragma unroll
        for (int j = 0; j < 8; ++j) d[j] = stage[tid * STAGE_PITCH + j];
  #pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t ta = d[2 * j] | (d[2 * j] >> 4);
          uint32_t tb = d[2 * j + 1] | (d[2 * j + 1] >> 4);
          out[j] = __builtin_amdgcn_perm(tb, ta, 0x06040200u);
        }
      } else {
  #pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t o = 0;
  #pragma unroll
          for (int e = 0; e < 8; ++e) o |= codes[8 * j + e] << (4 * e);
          out[j] = o;
        }
      }
      if constexpr (DEFER_FLIP) {
  #pragma unroll
        for (int j = 0; j < 4; ++j) out[j] ^= p.sign_nib[j];
      }
      if constexpr (BPW == 1) {
        const __amdgpu_buffer_rsrc_t rsrc_cc = __builtin_amdgcn_make_buffer_rsrc(
            p.col_codes + (b * C + col0) * p.ld_cc + by * 16, 0, 0x7FFFFFFF, 0x00020000);
        __builtin_amdgcn_raw_buffer_store_b128(v4u_t{out[0], out[1], out[2], out[3]}, rsrc_cc, cvalid ? tid * (int)p.ld_cc : OOB, 0, 0);
      } else {
  #pragma unroll
        for (int q = 0; q + 1 < BPW; ++q)
  #pragma unroll
          for (int j = 0; j < 4; ++j) colacc[q][j] = colacc[q + 1][j];
  #pragma unroll
        for (int j = 0; j < 4; ++j) colacc[BPW - 1][j] = out[j];
      }
    }
    ++bands_done;
  }   // bands of this workgroup

  if constexpr (BPW > 1) {
    // Column codes out, whole lines: colacc[q] is the piece of band by0 + q - (BPW - bands_done) of this thread's column.
    // In two halves of 128 columns through the first 16 KB of the tile: the column's thread writes its BPW pieces (slot
    // XORed with the column so that neighbouring columns spread over the banks), then lane l of a wave takes piece l % 8
    // of column l / 8: one store instruction covers 8 columns x 128 bytes.
    uint4* stage = reinterpret_cast<uint4*>(tile);
    static_assert(sizeof(tile) >= 128 * BPW * 16, "the column-code staging reuses the tile");
    const __amdgpu_buffer_rsrc_t rsrc_cc = __builtin_amdgcn_make_buffer_rsrc(
        p.col_codes + (b * C + col0) * p.ld_cc + by0 * 16, 0, 0x7FFFFFFF, 0x00020000);
    const int first = BPW - bands_done;   // pieces below this index hold nothing
#pragma unroll 1
    for (int half = 0; half < 2; ++half) {
      __syncthreads();
      if ((tid >> 7) == half) {
        const int cl = tid & 127;
#pragma unroll
        for (int q = 0; q < BPW; ++q) stage[cl * BPW + (q ^ (cl & 7))] = make_uint4(colacc[q][0], colacc[q][1], colacc[q][2], colacc[q][3]);
      }
      __syncthreads();
#pragma unroll
      for (int j = 0; j < 128 * BPW / 256; ++j) {
        const int idx = j * 256 + tid, cl = idx >> 3, q = (idx & 7) ^ (cl & 7);
        const uint4 v = stage[idx];
        const int ccol = col0 + half * 128 + cl;
        __builtin_amdgcn_raw_buffer_store_b128(v4u_t{v.x, v.y, v.z, v.w}, rsrc_cc,
                                               (ccol < C && q >= first) ? (half * 128 + cl) * (int)p.ld_cc + (q - first) * 16 : OOB, 0, 0);
      }
    }
  }
}

// The 32-point butterfly both standalone kernels share: z holds the block in permuted order (z[k] = element perm^-1[k]).
// `in_flip` / `out_flip` are sign masks over k: the inverse transform (W^T) applies diag(Q) to the input, the forward
// transform to the output, and the other mask is zero.
__device__ __forceinline__ void hadamard32(float (&z)[32], uint32_t in_flip, uint32_t out_flip) {
#pragma unroll
  for (int k = 0; k < 32; ++k) z[k] = u2f(f2u(z[k]) ^ (((in_flip >> k) & 1u) << 31));
#pragma unroll
  for (int h = 1; h < 32; h <<= 1) {
#pragma unroll
    for (int k = 0; k < 32; ++k) {
      if ((k & h) == 0) {
        float a0 = z[k], a1 = z[k + h];
        z[k] = a0 + a1;
        z[k + h] = a0 - a1;
      }
    }
  }
#pragma unroll
  for (int k = 0; k < 32; ++k) z[k] = div_sqrt32_signed(z[k], ((out_flip >> k) & 1u) << 31);
}

template <typename T>
__device__ __forceinline__ float load_as_f32(const T* q) {
  if constexpr (sizeof(T) == 2) return u2f((uint32_t)__builtin_bit_cast(unsigned short, *q) << 16);
  else return *q;
}

template <typename T>
__device__ __forceinline__ void store_from_f32(T* q, float v) {
  if constexpr (sizeof(T) == 2) *q = __builtin_bit_cast(T, (unsigned short)f32_to_bf16_bits(v));
  else *q = v;
}

// Standalone transform along the rows' index (W or W^T from the left): thread t owns one column, loads the 32 rows of
// a block in permuted order, runs the same butterfly as the fused quantizer and writes each position back to the row
// it came from.
template <typename T>
__global__ __launch_bounds__(256) void hadamard_kernel(const T* __restrict__ x, int64_t ld_x, T* __restrict__ y, int64_t ld_y, int C,
                                                       const QuantParams p, uint32_t in_flip, uint32_t out_flip) {
  const int cc = blockIdx.x * 256 + threadIdx.x;
  if (cc >= C) return;
  const int64_t row0 = (int64_t)blockIdx.y * 32;
  float z[32];
#pragma unroll
  for (int k = 0; k < 32; ++k) z[k] = load_as_f32(&x[(row0 + packed_byte(p.pinv4, k)) * ld_x + cc]);
  hadamard32(z, in_flip, out_flip);
#pragma unroll
  for (int k = 0; k < 32; ++k) store_from_f32(&y[(row0 + packed_byte(p.pinv4, k)) * ld_y + cc], z[k]);
}

// Standalone transform along the columns' index (W or W^T from the right): a workgroup takes 256 chunks of 32
// neighbouring elements of a row.  Half a wave moves one chunk between memory and LDS (whole 128- or 64-byte
// segments); then thread t picks chunk t out of LDS in permuted order (pitch 33 dwords: no bank conflicts either
// way), runs the butterfly and puts the results back for the same half-wave pattern to store.
template <typename T>
__global__ __launch_bounds__(256) void hadamard_rows_kernel(const T* __restrict__ x, int64_t ld_x, T* __restrict__ y, int64_t ld_y,
                                                            int chunks_per_row, int64_t n_chunks, const QuantParams p,
                                                            uint32_t in_flip, uint32_t out_flip) {
  __shared__ float tile[256 * 33];
  const int tid = threadIdx.x, j = tid & 31, grp = tid >> 5;
  const int64_t base = (int64_t)blockIdx.x * 256;
  const int64_t g0 = base + grp * 32;   // the first of the 32 chunks this half-wave moves
  int64_t row = g0 / chunks_per_row;
  int ch = (int)(g0 - row * chunks_per_row);
  {
    int64_t r = row;
    int c = ch;
    for (int i = 0; i < 32; ++i) {
      if (g0 + i < n_chunks) tile[(grp * 32 + i) * 33 + j] = load_as_f32(&x[r * ld_x + c * 32 + j]);
      if (++c == chunks_per_row) { c = 0; ++r; }
    }
  }
  __syncthreads();
  if (base + tid < n_chunks) {
    float z[32];
#pragma unroll
    for (int k = 0; k < 32; ++k) z[k] = tile[tid * 33 + packed_byte(p.pinv4, k)];
    hadamard32(z, in_flip, out_flip);
#pragma unroll
    for (int k = 0; k < 32; ++k) tile[tid * 33 + packed_byte(p.pinv4, k)] = z[k];
  }
  __syncthreads();
  for (int i = 0; i < 32; ++i) {
    if (g0 + i < n_chunks) store_from_f32(&y[row * ld_y + ch * 32 + j], tile[(grp * 32 + i) * 33 + j]);
    if (++ch == chunks_per_row) { ch = 0; ++row; }
  }
}

// Validates signs/perm (host arrays) and fills the kernel-side description.
int fill_hadamard(QuantParams& p, const int8_t* signs, const uint8_t* perm, const char* who) {
  p.sign_mask = 0;
  uint32_t seen = 0;
  ALTO_REQUIRE(signs != nullptr, "%s: hadamard set but signs is NULL", who);
  for (int w = 0; w < 8; ++w) p.perm4[w] = p.pinv4[w] = 0;
  for (int j = 0; j < 32; ++j) {
    int k = perm ? perm[j] : j;
    ALTO_REQUIRE(k >= 0 && k < 32 && !((seen >> k) & 1u), "%s: perm is not a permutation of 0..31", who);
    seen |= 1u << k;
    p.perm4[j >> 2] |= (uint32_t)k << (8 * (j & 3));
    p.pinv4[k >> 2] |= (uint32_t)j << (8 * (k & 3));
  }
  for (int k = 0; k < 32; ++k) {
    ALTO_REQUIRE(signs[k] == 1 || signs[k] == -1, "%s: signs[%d] = %d is not +1/-1", who, k, (int)signs[k]);
    if (signs[k] < 0) p.sign_mask |= 1u << k;
  }
  for (int w = 0; w < 4; ++w) p.sign_nib[w] = 0;
  for (int r = 0; r < 32; ++r)
    if ((p.sign_mask >> (perm ? perm[r] : r)) & 1u) p.sign_nib[r >> 3] |= 8u << (4 * (r & 7));
  return ALTO_MXFP4_OK;
}

// bpw8: the caller laid the grid out for workgroups of 8 bands (column outputs of large 2D-block tensors, !GEN only)
template <typename T, bool DO_ROW, bool DO_COL, int SR, bool RHT, bool B2D, bool GEN>
void launch(const QuantParams& p, dim3 grid, hipStream_t st, bool bpw8) {
  if constexpr (DO_COL && B2D && !GEN) {
    if (bpw8) {
      hipLaunchKernelGGL((quant_kernel<T, DO_ROW, DO_COL, SR, RHT, B2D, GEN, 8>), grid, dim3(256), 0, st, p);
      return;
    }
  }
  hipLaunchKernelGGL((quant_kernel<T, DO_ROW, DO_COL, SR, RHT, B2D, GEN, 1>), grid, dim3(256), 0, st, p);
}

template <typename T, int SR, bool GEN>
void dispatch_mode(const QuantParams& p, dim3 grid, hipStream_t st, bool do_row, bool do_col, bool rht, bool b2d, bool bpw8) {
  if (b2d) {
    if (do_row && do_col) launch<T, true, true, SR, false, true, GEN>(p, grid, st, bpw8);
    else if (do_row) launch<T, true, false, SR, false, true, GEN>(p, grid, st, bpw8);
    else launch<T, false, true, SR, false, true, GEN>(p, grid, st, bpw8);
  } else if (do_row && do_col) {
    if (rht) launch<T, true, true, SR, true, false, GEN>(p, grid, st, bpw8);
    else launch<T, true, true, SR, false, false, GEN>(p, grid, st, bpw8);
  } else if (do_row) {
    launch<T, true, false, SR, false, false, GEN>(p, grid, st, bpw8);
  } else {
    if (rht) launch<T, false, true, SR, true, false, GEN>(p, grid, st, bpw8);
    else launch<T, false, true, SR, false, false, GEN>(p, grid, st, bpw8);
  }
}

template <typename T>
void dispatch(const QuantParams& p, dim3 grid, hipStream_t st, bool do_row, bool do_col, bool rht, bool b2d, int sr, bool gen, bool bpw8) {
  if (gen) {
    if (sr == 3) dispatch_mode<T, 3, true>(p, grid, st, do_row, do_col, rht, b2d, bpw8);
    else if (sr == 2) dispatch_mode<T, 2, true>(p, grid, st, do_row, do_col, rht, b2d, bpw8);
    else if (sr == 1) dispatch_mode<T, 1, true>(p, grid, st, do_row, do_col, rht, b2d, bpw8);
    else dispatch_mode<T, 0, true>(p, grid, st, do_row, do_col, rht, b2d, bpw8);
  } else {
    if (sr == 3) dispatch_mode<T, 3, false>(p, grid, st, do_row, do_col, rht, b2d, bpw8);
    else if (sr == 2) dispatch_mode<T, 2, false>(p, grid, st, do_row, do_col, rht, b2d, bpw8);
    else if (sr == 1) dispatch_mode<T, 1, false>(p, grid, st, do_row, do_col, rht, b2d, bpw8);
    else dispatch_mode<T, 0, false>(p, grid, st, do_row, do_col, rht, b2d, bpw8);
  }
}

}  // namespace
}  // namespace alto

namespace alto {
namespace {

// one-thread kernel: moves the counter of a device-resident Philox state past the blocks a quantizer call consumed
__global__ void philox_advance_kernel(uint64_t* state, uint64_t blocks) { state[1] += blocks; }

// sr_mode: 0 round to nearest even, 1 stochastic with the words in rand_bits, 2 stochastic with Philox words made in the kernel,
// 3 stochastic with the hardware converts (dwords cut from Philox words made in the kernel)
int quantize_impl(const void* x, int dtype, int64_t batch, int64_t M, int64_t C, int64_t ld_x, int64_t bs_x,
                  uint8_t* row_codes, uint8_t* row_scales, uint8_t* col_codes, uint8_t* col_scales,
                  int64_t ld_row_codes, int64_t ld_col_codes, int is_2d, int sr_mode,
                  const uint32_t* rand_bits, int64_t ld_rand, int64_t bs_rand, uint64_t seed, uint64_t offset, const uint64_t* philox_state,
                  int hadamard, const int8_t* signs, const uint8_t* perm, int clip_mode, int use_uos, void* stream, int flags = 0) {
  if (ld_row_codes == 0) ld_row_codes = C / 2;
  if (ld_col_codes == 0) ld_col_codes = M / 2;
  ALTO_REQUIRE(row_codes == nullptr || (ld_row_codes >= C / 2 && ld_row_codes % 4 == 0), "quantize: ld_row_codes must be >= C/2 and a multiple of 4 bytes");
  ALTO_REQUIRE(col_codes == nullptr || (ld_col_codes >= M / 2 && ld_col_codes % 16 == 0), "quantize: ld_col_codes must be >= M/2 and a multiple of 16 bytes");
  ALTO_REQUIRE(ld_row_codes < (1ll << 26) && ld_col_codes < (1ll << 23), "quantize: code row pitch out of range");
  const bool do_row = row_codes != nullptr, do_col = col_codes != nullptr;
  ALTO_REQUIRE(x != nullptr, "quantize: x is NULL");
  ALTO_REQUIRE(dtype == ALTO_DT_BF16 || dtype == ALTO_DT_F32, "quantize: dtype %d is neither bf16 (0) nor f32 (1)", dtype);
  ALTO_REQUIRE(do_row || do_col, "quantize: neither a row nor a column output was requested");
  ALTO_REQUIRE(!do_row || row_scales != nullptr, "quantize: row_codes given without row_scales");
  ALTO_REQUIRE(!do_col || col_scales != nullptr, "quantize: col_codes given without col_scales");
  ALTO_REQUIRE(batch >= 0 && M >= 0 && C >= 0, "quantize: negative size");
  ALTO_REQUIRE(M < (1ll << 31) && C < (1ll << 31) && batch < 65536, "quantize: size out of range");
  ALTO_REQUIRE(C % 8 == 0, "quantize: C (%lld) must be a multiple of 8", (long long)C);
  ALTO_REQUIRE(!do_row || C % 32 == 0, "quantize: row output needs C (%lld) %% 32 == 0", (long long)C);
  ALTO_REQUIRE(!(do_col || is_2d) || M % 32 == 0, "quantize: column output / 2D blocks need M (%lld) %% 32 == 0", (long long)M);
  ALTO_REQUIRE(!is_2d || C % 32 == 0, "quantize: 2D blocks need C (%lld) %% 32 == 0", (long long)C);
  const int64_t vec = dtype == ALTO_DT_BF16 ? 8 : 4;
  ALTO_REQUIRE(ld_x >= C && ld_x % vec == 0 && bs_x % vec == 0, "quantize: ld_x/bs_x must be >= C and multiples of %lld elements", (long long)vec);
  ALTO_REQUIRE((reinterpret_cast<uintptr_t>(x) & 15) == 0, "quantize: x must be 16-byte aligned");
  ALTO_REQUIRE(ld_x < (1ll << 24) && ld_rand < (1ll << 24), "quantize: row strides of 2^24 elements or more are not supported");
  if (sr_mode == 1) {
    ALTO_REQUIRE(rand_bits != nullptr, "quantize: stochastic rounding needs rand_bits");
    ALTO_REQUIRE(ld_rand >= C && ld_rand % 4 == 0 && bs_rand % 4 == 0, "quantize: ld_rand/bs_rand must be >= C and multiples of 4");
    ALTO_REQUIRE((reinterpret_cast<uintptr_t>(rand_bits) & 15) == 0, "quantize: rand_bits must be 16-byte aligned");
  }
  ALTO_REQUIRE(!hadamard || (!is_2d && do_col), "quantize: the Hadamard transform applies to a 1D column output only");
  ALTO_REQUIRE(clip_mode == ALTO_CLIP_NONE || clip_mode == ALTO_CLIP_STATIC || clip_mode == ALTO_CLIP_DYNAMIC, "quantize: bad clip_mode %d", clip_mode);
  const bool pack_rs = (flags & 1) != 0, pack_cs = (flags & 2) != 0;
  if (pack_rs || pack_cs) {
    ALTO_REQUIRE(clip_mode != ALTO_CLIP_DYNAMIC, "quantize: packed scales are not written with the dynamic clip");
    ALTO_REQUIRE((!pack_rs || row_codes) && (!pack_cs || col_codes), "quantize: packed scales asked for an output that is not produced");
    ALTO_REQUIRE(M % 32 == 0 && M * C < (1ll << 36), "quantize: packed scales need M %% 32 == 0 and M * C < 2^36");
    ALTO_REQUIRE(((reinterpret_cast<uintptr_t>(pack_rs ? row_scales : nullptr) | reinterpret_cast<uintptr_t>(pack_cs ? col_scales : nullptr)) & 15) == 0,
                 "quantize: packed scales must be 16-byte aligned");
  }
  if (batch == 0 || M == 0 || C == 0) return ALTO_MXFP4_OK;
  if (clip_mode == ALTO_CLIP_DYNAMIC) {   // std-based scale: separate plain kernel, quantisation along the contiguous dim
    ALTO_REQUIRE(do_row && !do_col && !hadamard,
                 "quantize: clip_mode=dynamic gives the row output only (no column output, no Hadamard); transpose on the host");
    if (sr_mode >= 2) {
      set_error("quantize: clip_mode=dynamic takes its random words from a tensor (fill one with alto_mxfp4_random_bits)");
      return ALTO_MXFP4_ENOTIMPL;
    }
    ALTO_REQUIRE(ld_row_codes % 16 == 0, "quantize: clip_mode=dynamic needs 16-byte aligned code rows");
    ALTO_REQUIRE((M + 31) / 32 <= 65535, "quantize: M (%lld) exceeds 65535 row blocks", (long long)M);
    return quantize_dynamic_launch(x, dtype, batch, M, C, ld_x, bs_x, row_codes, row_scales, ld_row_codes, is_2d, sr_mode == 1,
                                   rand_bits, ld_rand, bs_rand, use_uos, reinterpret_cast<hipStream_t>(stream));
  }

  QuantParams p;
  p.x = x; p.ld_x = ld_x; p.bs_x = bs_x; p.M = (int)M; p.C = (int)C;
  p.rand = rand_bits; p.ld_r = ld_rand; p.bs_r = bs_rand;
  p.seed = seed; p.ctr0 = offset; p.philox_state = philox_state;
  p.row_codes = row_codes; p.row_scales = row_scales; p.col_codes = col_codes; p.col_scales = col_scales;
  p.ld_rc = ld_row_codes; p.ld_cc = ld_col_codes;
  p.sign_mask = 0;
  for (int w = 0; w < 4; ++w) p.sign_nib[w] = 0;
  for (int w = 0; w < 8; ++w) p.perm4[w] = p.pinv4[w] = 0x03020100u + 0x04040404u * (uint32_t)w;   // identity
  if (hadamard) {
    int rc = fill_hadamard(p, signs, perm, "quantize");
    if (rc != ALTO_MXFP4_OK) return rc;
  }
  const bool both = do_row && do_col;
  p.clip_row = (clip_mode == ALTO_CLIP_STATIC && !both) ? 1 : 0;
  p.clip_col = (clip_mode == ALTO_CLIP_STATIC) ? 1 : 0;
  if (!do_col) p.clip_col = 0;
  if (!do_row) p.clip_row = 0;
  p.uos = use_uos ? 1 : 0;
  p.pack_rs = pack_rs ? 1 : 0;
  p.pack_cs = pack_cs ? 1 : 0;
  const bool gen = p.clip_row || p.clip_col || p.uos;

  const int64_t tiles_x = (C + TILE_C - 1) / TILE_C, bands = (M + 31) / 32;
  // Column outputs of large 2D-block tensors (weights): workgroups of 8 bands, which store their column codes as whole
  // lines, eight columns per wave instruction, instead of one 16-byte piece of 64 different lines per instruction
  // (measured: the 32 x 5760 x 2880 expert weights 408 -> 357 us with packed scales; a timing-only build with contiguous
  // column stores: 267).  It pays from about 16 workgroups per CU on (8 experts: 94 -> 96 us, 14336 x 4096: 32 -> 38 us), and
  // the 1D-block kernels, bound by their vector instructions, lose 5-40 % to the band loop's barriers and registers:
  // all of those keep one band per workgroup.  ALTO_MXFP4_QUANT_BANDS=1|8 overrides the choice (tests, measurements).
  static const int force_bpw = [] { const char* e = getenv("ALTO_MXFP4_QUANT_BANDS"); return e ? atoi(e) : 0; }();
  const bool bpw8 = do_col && is_2d && !gen && (force_bpw == 8 || (force_bpw != 1 && tiles_x * ((bands + 7) / 8) * batch >= 4096));
  const int64_t wrows = bpw8 ? (bands + 7) / 8 : bands;   // workgroup rows
  // With a column output: 2^unit_shift workgroup rows per unit, units padded to a multiple of 8.  The largest unit (up to the
  // 128 bands of a line of plain column scales) whose padding launches at most 5 % more workgroups than there are tiles;
  // single-band workgroups take at least the 8 bands of a line of column codes.
  const int us_min = bpw8 ? 0 : 3;
  int us = bpw8 ? 4 : 7;
  auto padded = [&](int sh) { return ((tiles_x * ((wrows + (1ll << sh) - 1) >> sh) + 7) / 8 * 8) << sh; };
  while (us > us_min && padded(us) * 20 > tiles_x * wrows * 21) --us;
  p.unit_shift = us;
  ALTO_REQUIRE(do_col ? padded(us) < (1ll << 31) : (tiles_x < (1ll << 31) && bands <= 65535), "quantize: %lld x %lld exceeds the grid", (long long)M, (long long)C);
  const dim3 grid = do_col ? dim3((unsigned)padded(us), 1, (unsigned)batch) : dim3((unsigned)tiles_x, (unsigned)bands, (unsigned)batch);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (dtype == ALTO_DT_BF16) dispatch<__bf16>(p, grid, st, do_row, do_col, hadamard != 0, is_2d != 0, sr_mode, gen, bpw8);
  else dispatch<float>(p, grid, st, do_row, do_col, hadamard != 0, is_2d != 0, sr_mode, gen, bpw8);
  return check_launch("quantize");
}

}  // namespace
}  // namespace alto

extern "C" int alto_mxfp4_quantize(const void* x, int dtype, int64_t batch, int64_t M, int64_t C, int64_t ld_x, int64_t bs_x,
                                   uint8_t* row_codes, uint8_t* row_scales, uint8_t* col_codes, uint8_t* col_scales,
                                   int is_2d, int rounding, const uint32_t* rand_bits, int64_t ld_rand, int64_t bs_rand,
                                   int hadamard, const int8_t* signs, const uint8_t* perm,
                                   int clip_mode, int use_uos, void* stream) {
  return alto_mxfp4_quantize_pitched(x, dtype, batch, M, C, ld_x, bs_x, row_codes, row_scales, col_codes, col_scales, 0, 0, is_2d, rounding,
                                     rand_bits, ld_rand, bs_rand, hadamard, signs, perm, clip_mode, use_uos, stream);
}

extern "C" int alto_mxfp4_quantize_pitched(const void* x, int dtype, int64_t batch, int64_t M, int64_t C, int64_t ld_x, int64_t bs_x,
                                           uint8_t* row_codes, uint8_t* row_scales, uint8_t* col_codes, uint8_t* col_scales,
                                           int64_t ld_row_codes, int64_t ld_col_codes,
                                           int is_2d, int rounding, const uint32_t* rand_bits, int64_t ld_rand, int64_t bs_rand,
                                           int hadamard, const int8_t* signs, const uint8_t* perm,
                                           int clip_mode, int use_uos, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(rounding == ALTO_ROUND_RNE || rounding == ALTO_ROUND_SR, "quantize: bad rounding mode %d", rounding);
  return quantize_impl(x, dtype, batch, M, C, ld_x, bs_x, row_codes, row_scales, col_codes, col_scales, ld_row_codes, ld_col_codes, is_2d,
                       rounding == ALTO_ROUND_SR ? 1 : 0, rand_bits, ld_rand, bs_rand, 0, 0, nullptr, hadamard, signs, perm, clip_mode, use_uos, stream);
}

extern "C" int alto_mxfp4_quantize_sr_philox(const void* x, int dtype, int64_t batch, int64_t M, int64_t C, int64_t ld_x, int64_t bs_x,
                                             uint8_t* row_codes, uint8_t* row_scales, uint8_t* col_codes, uint8_t* col_scales,
                                             int64_t ld_row_codes, int64_t ld_col_codes, int is_2d,
                                             uint64_t seed, uint64_t offset, const uint64_t* philox_state,
                                             int hadamard, const int8_t* signs, const uint8_t* perm,
                                             int clip_mode, int use_uos, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(C < (1ll << 26), "quantize_sr_philox: C (%lld) out of range", (long long)C);
  ALTO_REQUIRE((reinterpret_cast<uintptr_t>(philox_state) & 7) == 0, "quantize_sr_philox: philox_state must be 8-byte aligned");
  return quantize_impl(x, dtype, batch, M, C, ld_x, bs_x, row_codes, row_scales, col_codes, col_scales, ld_row_codes, ld_col_codes, is_2d,
                       2, nullptr, 0, 0, seed, offset, philox_state, hadamard, signs, perm, clip_mode, use_uos, stream);
}

extern "C" int alto_mxfp4_quantize_sr_hw(const void* x, int dtype, int64_t batch, int64_t M, int64_t C, int64_t ld_x, int64_t bs_x,
                                         uint8_t* row_codes, uint8_t* row_scales, uint8_t* col_codes, uint8_t* col_scales,
                                         int64_t ld_row_codes, int64_t ld_col_codes, int is_2d,
                                         uint64_t seed, uint64_t offset, const uint64_t* philox_state,
                                         int hadamard, const int8_t* signs, const uint8_t* perm,
                                         int clip_mode, int use_uos, void* stream) {
  using namespace alto;
  ALTO_REQUIRE((reinterpret_cast<uintptr_t>(philox_state) & 7) == 0, "quantize_sr_hw: philox_state must be 8-byte aligned");
  return quantize_impl(x, dtype, batch, M, C, ld_x, bs_x, row_codes, row_scales, col_codes, col_scales, ld_row_codes, ld_col_codes, is_2d,
                       3, nullptr, 0, 0, seed, offset, philox_state, hadamard, signs, perm, clip_mode, use_uos, stream);
}

extern "C" int64_t alto_mxfp4_quantize_sr_hw_words(int dtype, int64_t batch, int64_t M, int64_t C) {
  if (batch < 0 || M < 0 || C < 0 || M >= (1ll << 31) || C >= (1ll << 31) || batch >= 65536) return 0;   // sizes no quantizer call accepts
  const int64_t nb = (M + 31) / 32;
  const int64_t per_column = 4 * (dtype == ALTO_DT_BF16 ? 2 : 8) * batch * nb;   // < 2^5 * 2^16 * 2^26
  return alto::product_below(INT64_MAX, per_column, C) ? per_column * C : 0;
}

extern "C" int alto_mxfp4_quantize_ex(const void* x, int dtype, int64_t batch, int64_t M, int64_t C, int64_t ld_x, int64_t bs_x,
                                      uint8_t* row_codes, uint8_t* row_scales, uint8_t* col_codes, uint8_t* col_scales,
                                      int64_t ld_row_codes, int64_t ld_col_codes, int is_2d, int sr_mode,
                                      const uint32_t* rand_bits, int64_t ld_rand, int64_t bs_rand, uint64_t seed, uint64_t offset,
                                      const uint64_t* philox_state, int hadamard, const int8_t* signs, const uint8_t* perm,
                                      int clip_mode, int use_uos, int flags, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(sr_mode >= 0 && sr_mode <= 3, "quantize_ex: sr_mode %d is not 0 (nearest even), 1 (words given), 2 (Philox in the kernel) or 3 (hardware converts)", sr_mode);
  ALTO_REQUIRE((flags & ~3) == 0, "quantize_ex: unknown flags 0x%x", flags);
  ALTO_REQUIRE(sr_mode < 2 || C < (1ll << 26), "quantize_ex: C (%lld) out of range for words made in the kernel", (long long)C);
  ALTO_REQUIRE(sr_mode < 2 || philox_state == nullptr || (reinterpret_cast<uintptr_t>(philox_state) & 7) == 0, "quantize_ex: philox_state must be 8-byte aligned");
  return quantize_impl(x, dtype, batch, M, C, ld_x, bs_x, row_codes, row_scales, col_codes, col_scales, ld_row_codes, ld_col_codes, is_2d, sr_mode,
                       sr_mode == 1 ? rand_bits : nullptr, ld_rand, bs_rand, seed, offset, sr_mode >= 2 ? philox_state : nullptr, hadamard, signs, perm,
                       clip_mode, use_uos, stream, flags);
}

extern "C" int alto_mxfp4_philox_advance(uint64_t* philox_state, uint64_t words, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(philox_state != nullptr && (reinterpret_cast<uintptr_t>(philox_state) & 7) == 0, "philox_advance: philox_state must be a non-NULL 8-byte aligned device pointer");
  hipLaunchKernelGGL(philox_advance_kernel, dim3(1), dim3(1), 0, reinterpret_cast<hipStream_t>(stream), philox_state, (words + 3) / 4);
  return check_launch("philox_advance");
}

extern "C" int alto_mxfp4_hadamard_apply(const void* x, int dtype, int64_t M, int64_t C, int64_t ld_x, void* y, int64_t ld_y,
                                         const int8_t* signs, const uint8_t* perm, int inverse, int left_mul, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(x && y, "hadamard: NULL pointer");
  ALTO_REQUIRE(dtype == ALTO_DT_BF16 || dtype == ALTO_DT_F32, "hadamard: bad dtype %d", dtype);
  ALTO_REQUIRE(M >= 0 && C >= 0, "hadamard: negative size");
  ALTO_REQUIRE(!left_mul || M % 32 == 0, "hadamard: M (%lld) must be a multiple of 32", (long long)M);
  ALTO_REQUIRE(left_mul || C % 32 == 0, "hadamard: C (%lld) must be a multiple of 32 for a multiplication from the right", (long long)C);
  ALTO_REQUIRE(ld_x >= C && ld_y >= C, "hadamard: row stride smaller than C");
  ALTO_REQUIRE(M < (1ll << 31) && C < (1ll << 31), "hadamard: size out of range");
  ALTO_REQUIRE(((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & (dtype == ALTO_DT_BF16 ? 1 : 3)) == 0, "hadamard: x and y must be aligned to their element size");
  QuantParams p{};
  int rc = fill_hadamard(p, signs, perm, "hadamard");
  if (rc != ALTO_MXFP4_OK) return rc;
  if (M == 0 || C == 0) return ALTO_MXFP4_OK;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (left_mul) {
    // y = W x (or W^T x): out[i] = sum_j W[i][j] x[j]
    ALTO_REQUIRE(M / 32 <= 65535, "hadamard: size out of range");
    const uint32_t in_flip = inverse ? p.sign_mask : 0u, out_flip = inverse ? 0u : p.sign_mask;
    dim3 grid((unsigned)((C + 255) / 256), (unsigned)(M / 32));
    if (dtype == ALTO_DT_BF16)
      hipLaunchKernelGGL(hadamard_kernel<__bf16>, grid, dim3(256), 0, st, (const __bf16*)x, ld_x, (__bf16*)y, ld_y, (int)C, p, in_flip, out_flip);
    else
      hipLaunchKernelGGL(hadamard_kernel<float>, grid, dim3(256), 0, st, (const float*)x, ld_x, (float*)y, ld_y, (int)C, p, in_flip, out_flip);
  } else {
    // y = x W: out[j] = sum_i x[i] W[i][j] = (W^T x^T)[j], so the row vector sees the transpose of what a column sees
    const uint32_t in_flip = inverse ? 0u : p.sign_mask, out_flip = inverse ? p.sign_mask : 0u;
    const int64_t n_chunks = M * (C / 32);
    ALTO_REQUIRE((n_chunks + 255) / 256 < (1ll << 31), "hadamard: size out of range");
    dim3 grid((unsigned)((n_chunks + 255) / 256));
    if (dtype == ALTO_DT_BF16)
      hipLaunchKernelGGL(hadamard_rows_kernel<__bf16>, grid, dim3(256), 0, st, (const __bf16*)x, ld_x, (__bf16*)y, ld_y, (int)(C / 32), n_chunks, p, in_flip, out_flip);
    else
      hipLaunchKernelGGL(hadamard_rows_kernel<float>, grid, dim3(256), 0, st, (const float*)x, ld_x, (float*)y, ld_y, (int)(C / 32), n_chunks, p, in_flip, out_flip);
  }
  return check_launch("hadamard");
}

extern "C" int alto_mxfp4_hadamard(const void* x, int dtype, int64_t M, int64_t C, int64_t ld_x, void* y, int64_t ld_y,
                                   const int8_t* signs, const uint8_t* perm, void* stream) {
  return alto_mxfp4_hadamard_apply(x, dtype, M, C, ld_x, y, ld_y, signs, perm, 0, 1, stream);
}
