// MXFP4 flash-attention forward for gfx950: S = Q K^T and O = P V both on v_mfma_scale_f32_32x32x64_f8f6f4, with the
// probabilities re-quantised to MXFP4 in registers and the row sums taken from the SAME quantised probabilities
// (the recurrence of alto/kernels/fp4/mxfp4/triton_flash_attention_mxfp4.py:168-400,640-890, key blocks of 64).
//
// One wave owns 32 query rows of one head.  The MFMA is issued as (first = rows that land in registers, second = rows
// that land in lanes): S tiles and O tiles keep the query row in the lane (lane % 32) and spread keys / value columns
// over the 16 accumulator registers, so the per-row softmax state (running max, rescale factor) is one scalar per lane
// and the only cross-lane traffic is between the two lanes (l, l ^ 32) that share a row.
#include <type_traits>
#include <utility>

#include "common.h"

namespace alto {

struct AttnArgs {
  const uint8_t* q;  const uint8_t* qs;    // [B, Hq, Sq, D/2],  [B, Hq, Sq/32, D/32]
  const uint8_t* k;  const uint8_t* ks;    // [B, Hk, Sk, D/2],  [B, Hk, Sk/32, D/32]
  const uint8_t* vt; const uint8_t* vs;    // [B, Hk, Dv, Sk/2] packed along keys, [B, Hk, Sk/32, Dv/32]
  void* out; float* lse;                   // [B, Hq, Sq, Dv] bf16, [B, Hq, Sq] fp32
  int Hq, Hk, Sq, Sk, Sk_used;             // Sk keys are allocated (a multiple of 64), the first Sk_used exist
  float sm_scale;
  int causal;
  // optional additive terms on the scaled scores (triton_flash_attention_mxfp4.py:288-299), fp32:
  const float* bias;  int64_t bias_sb, bias_sh, bias_sm, bias_bytes;   // element (b, h, m, n) at b sb + h sh + m sm + n; NULL: none
  const float* alibi; int64_t alibi_sb, alibi_sh;                      // slope of (b, h) at b sb + h sh; NULL: none
};

#ifndef ATTN_WG_PER_CU
#define ATTN_WG_PER_CU 3
#endif
constexpr float ATTN_RCP_LN2 = 1.4426950408889634f;
constexpr float ATTN_LN2 = 0.6931471824645996f;

__device__ __forceinline__ v8i_t frag16(const uint8_t* p) {
  const uint4 w = *reinterpret_cast<const uint4*>(p);
  return v8i_t{(int)w.x, (int)w.y, (int)w.z, (int)w.w, 0, 0, 0, 0};
}
template <int N, typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) { (f(std::integral_constant<int, I>{}), ...); }
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) { static_for_impl<N>(static_cast<F&&>(f), std::make_integer_sequence<int, N>{}); }

typedef unsigned v2u_t __attribute__((ext_vector_type(2)));
// v_permlane32_swap(a, b) returns {a of lanes 0..31 | b of lanes 0..31,  a of lanes 32..63 | b of lanes 32..63}
// (first | second half of the wave): a value and its copy come back as the low half's and the high half's values.
__device__ __forceinline__ float pair_max(float v) {   // max over the two lanes l and l ^ 32
  const v2u_t p = __builtin_amdgcn_permlane32_swap(f2u(v), f2u(v), false, false);
  return fmaxf(u2f(p[0]), u2f(p[1]));
}

// NK = D / 64 (MFMA K steps of Q K^T), ND = Dv / 32 (output tiles).
// The four waves of a workgroup own 128 consecutive query rows of one head and walk the key blocks together: a block's
// K codes (64 rows x D/2 bytes) and V codes (Dv rows x 32 bytes) are fetched once per workgroup, two blocks ahead, with
// direct-to-LDS loads (16 bytes per lane, 1 KB per wave instruction, no registers in between) into a three-slot ring;
// one barrier per block.  (Fetching the pieces per wave straight from global memory made the vector-memory path the
// bound: 8 KB per wave and block in scattered 16-byte accesses.  One block ahead through registers left the waves
// waiting for the load at the end of every block: the kernel ran at 38 % VALU issue with the matrix pipes at 11 %.)
constexpr int ATTN_RING = 3;
template <int NK, int ND>
struct AttnTile {
  static constexpr int D = NK * 64, DV = ND * 32;
  static constexpr int K_BYTES = 64 * (D / 2), V_BYTES = DV * 32;       // one block of K codes, of V codes
  static constexpr int SLOT = K_BYTES + V_BYTES;
};

// The body of the kernel as a function of its own because of the `__restrict__` on the outputs: inlining then marks the
// direct-to-LDS loads as not aliasing them, and only with that mark does the compiler's wait insertion keep those loads
// in flight across the LDS reads that follow (unmarked, it puts an `s_waitcnt vmcnt(0)` before the next LDS read).
// BIASED: the scores get a.bias and / or the ALiBi term -slope |row + Sk - Sq - key| added after the scaling and the mask,
// before the running maximum (:288-308); a separate instantiation, the plain one carries none of it.
template <int NK, int ND, bool BIASED>
__device__ __forceinline__ void attn_fwd_body(const AttnArgs& a, __bf16* __restrict__ out, float* __restrict__ lse_out, uint8_t* ring) {
  constexpr int D = NK * 64, DV = ND * 32;
  constexpr int K_BYTES = AttnTile<NK, ND>::K_BYTES, V_BYTES = AttnTile<NK, ND>::V_BYTES, SLOT = AttnTile<NK, ND>::SLOT;
  constexpr int K_PIECES = K_BYTES / 16, V_PIECES = V_BYTES / 16;
  constexpr int PIECES = K_PIECES + V_PIECES;             // 16-byte pieces of one block, K first; both multiples of 64
  constexpr int DMA_MAX = (PIECES + 255) / 256;           // loads per wave and block: DMA_MAX, or one less for the last waves

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, h = lane >> 5;
  // grid (heads, batch, row blocks): with a causal mask every head's longest rows are dispatched before anybody's shorter
  // ones, so the launch ends with the cheapest workgroups
  const int qblk = a.causal ? (int)(gridDim.z - 1 - blockIdx.z) : (int)blockIdx.z;
  const int q0 = (qblk * 4 + wave) * 32;
  const bool live = q0 < a.Sq;                    // a wave past the last row still helps with loads and barriers
  const int hq = blockIdx.x, b = blockIdx.y;
  const int hk = hq / (a.Hq / a.Hk);
  const int64_t bhq = (int64_t)b * a.Hq + hq, bhk = (int64_t)b * a.Hk + hk;
  const int qrow = live ? q0 + r : 0;
  const int shift = a.Sk_used - a.Sq;                  // causal mask is aligned to the bottom-right corner

  // ---- Q pieces: row qrow, K step ks, half h -> 16 bytes; one scale byte per (32-row block, 32-column block)
  v8i_t qf[NK];
  int qsc[NK];
#pragma unroll
  for (int s = 0; s < NK; ++s) {
    qf[s] = frag16(a.q + (bhq * a.Sq + qrow) * (D / 2) + s * 32 + h * 16);
    qsc[s] = a.qs[(bhq * (a.Sq / 32) + qrow / 32) * (D / 32) + 2 * s + h];
  }

  v16f_t acc_o[ND], acc_l;
#pragma unroll
  for (int d = 0; d < ND; ++d)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc_o[d][v] = 0.0f;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc_l[v] = 0.0f;
  float m_i = -__builtin_inff();                   // running row max of S * sm_scale * log2(e)
  const float c2 = a.sm_scale * ATTN_RCP_LN2;
  const float cs = BIASED ? 1.0f : c2;   // what is left to multiply once the scores are in the base-2 domain
  // bias rows of this (batch, head): a descriptor over the rest of the tensor (no range when there is no bias: loads give 0)
  const __amdgpu_buffer_rsrc_t rsrc_bias = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>((BIASED && a.bias) ? a.bias + b * a.bias_sb + hq * a.bias_sh : nullptr), 0,
      (BIASED && a.bias) ? (int)(a.bias_bytes - (b * a.bias_sb + hq * a.bias_sh) * 4) : 0, 0x00020000);
  const float slope2 = (BIASED && a.alibi) ? a.alibi[b * a.alibi_sb + hq * a.alibi_sh] * ATTN_RCP_LN2 : 0.0f;

  const v8i_t ones = v8i_t{0x22222222, 0x22222222, 0x22222222, 0x22222222, 0, 0, 0, 0};   // E2M1 code 2 = 1.0

  // blocks this wave needs, and the most any wave of the workgroup needs (the last wave's rows reach furthest)
  const int all_blk = (a.Sk_used + 63) / 64;
  int nblk = all_blk, wg_blk = all_blk;
  if (a.causal) {
    const int lim = (q0 + 32 + shift + 63) / 64;
    nblk = lim < all_blk ? lim : all_blk;
    int q_end = qblk * 128 + 128;
    q_end = q_end < a.Sq ? q_end : a.Sq;
    const int wlim = (q_end + shift + 63) / 64;
    wg_blk = wlim < all_blk ? wlim : all_blk;
  }
  if (!live) nblk = 0;

  // ---- cooperative fetch of one block: wave instruction j moves pieces [256 j + 64 wave, + 64) of the block, K pieces
  // first (contiguous in memory), then V pieces (piece p = 16 bytes of row p / 2, half p % 2); the piece index is also the
  // position in the slot.  Blocks beyond the keys are out of the descriptors' range and arrive as zeros.
  typedef __attribute__((address_space(3))) uint8_t lds_u8;
  const __amdgpu_buffer_rsrc_t rsrc_k = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(a.k + bhk * a.Sk * (D / 2)), 0, a.Sk * (D / 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_v = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(a.vt + bhk * DV * (int64_t)(a.Sk / 2)), 0, DV * (a.Sk / 2), 0x00020000);
  // Where a piece sits inside its row of the slot: the LDS serves a 16-byte read of 16 lanes per pass from 64 banks
  // (256 bytes), and the 16 lanes of a fragment read ask for the same piece of 16 consecutive rows.  With PR pieces per
  // row, 16 / PR rows share a 256-byte line; piece c of row `row` goes to position c ^ ((row / (16 / PR)) % PR), which
  // spreads those 16 reads over all banks.  (Rows of 96 bytes, D = 192, keep the plain order.)  The loads put the pieces
  // there: lane i of a load fills position p0 + i and fetches the piece that belongs there.
  constexpr int KPR = D / 32, KSW = (KPR == 2 || KPR == 4 || KPR == 8) ? 16 / KPR : 0;   // pieces per K row; rows per swizzle step
  const int n_dma = (PIECES - 64 * wave + 255) / 256;   // this wave's loads per block (wave-uniform)
  auto dma = [&](int kb, int slot) {
    lds_u8* base = (lds_u8*)ring + slot * SLOT;
#pragma unroll
    for (int j = 0; j < DMA_MAX; ++j) {
      const int p0 = 256 * j + 64 * wave;   // wave-uniform
      if (PIECES % 256 != 0 && p0 >= PIECES) continue;
      if (p0 < K_PIECES) {
        const int p = p0 + lane, row = p / KPR;
        const int c = KSW ? (p % KPR) ^ ((row / (KSW ? KSW : 1)) % KPR) : p % KPR;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_k, (__attribute__((address_space(3))) void*)(base + p0 * 16), 16, (row * KPR + c) * 16,
                                                 __builtin_amdgcn_readfirstlane(kb * K_BYTES), 0, 0);
      } else {
        const int p = p0 - K_PIECES + lane, row = p >> 1;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_v, (__attribute__((address_space(3))) void*)(base + p0 * 16), 16,
                                                 row * (a.Sk / 2) + (((p & 1) ^ ((row >> 3) & 1)) * 16), __builtin_amdgcn_readfirstlane(kb * 32), 0, 0);
      }
    }
  };
  const int k_swz = KSW ? ((r / (KSW ? KSW : 1)) % KPR) * 16 : 0;   // XOR on the byte offset of a piece inside its K row
  const int v_swz = ((r >> 3) & 1) * 16;                            // and inside its 32-byte V row
  auto wait_dma = [&](bool one_block_in_flight) {   // this wave's loads are done, except the youngest block's if asked
    if (!one_block_in_flight) __builtin_amdgcn_s_waitcnt(0x0070 | 0x0F00 | 0);                      // vmcnt(0)
    else if (n_dma == DMA_MAX) __builtin_amdgcn_s_waitcnt(0x0070 | 0x0F00 | (DMA_MAX & 15));        // vmcnt(DMA_MAX)
    else __builtin_amdgcn_s_waitcnt(0x0070 | 0x0F00 | ((DMA_MAX - 1) & 15));
  };
  // Scale bytes of a block: 2 D/32 bytes of K (key tile t, 32-column block j at byte t D/32 + j) and 2 Dv/32 bytes of V
  // (key tile t, column block d at byte t Dv/32 + d) sit at wave-uniform, 4-byte aligned addresses: whole dwords, one
  // block ahead; the MFMA picks a byte of a dword with op_sel, the lane half h shifts its byte into place.
  constexpr int KS_DW = 2 * (D / 32) / 4, VS_DW = (2 * (DV / 32) + 3) / 4;
  uint32_t ksw[KS_DW], vsw[VS_DW], ksw_next[KS_DW], vsw_next[VS_DW];
  auto fetch_scales = [&](int kb, uint32_t (&kw)[KS_DW], uint32_t (&vw)[VS_DW]) {
    const uint32_t* kp = reinterpret_cast<const uint32_t*>(a.ks + (bhk * (a.Sk / 32) + kb * 2) * (D / 32));
    const uint32_t* vp = reinterpret_cast<const uint32_t*>(a.vs + (bhk * (a.Sk / 32) + kb * 2) * (DV / 32));
#pragma unroll
    for (int i = 0; i < KS_DW; ++i) kw[i] = kp[i];
#pragma unroll
    for (int i = 0; i < VS_DW; ++i) vw[i] = vp[i];
  };
  if (wg_blk > 0) {
    fetch_scales(0, ksw_next, vsw_next);
    dma(0, 0);
    if (wg_blk > 1) dma(1, 1);
  }
  // (the bare barrier instruction: `__syncthreads()` would first wait for every outstanding load, the prefetched block's
  // included; the ring is written by the direct-to-LDS loads only, and wait_dma has waited for this wave's part)
  wait_dma(wg_blk > 1);
  asm volatile("s_barrier" ::: "memory");

  int slot = 0;   // of block kb
  for (int kb = 0; kb < wg_blk; ++kb) {
    const int key0 = kb * 64;
    const uint8_t* tile = ring + slot * SLOT;
#pragma unroll
    for (int i = 0; i < KS_DW; ++i) ksw[i] = ksw_next[i];
#pragma unroll
    for (int i = 0; i < VS_DW; ++i) vsw[i] = vsw_next[i];
    // the next block's scale bytes, then the codes of the block after it (into the slot the previous block used: every wave
    // left it at the last barrier); both travel during this block's arithmetic
    if (kb + 1 < wg_blk) fetch_scales(kb + 1, ksw_next, vsw_next);
    if (kb + 2 < wg_blk) dma(kb + 2, slot == 0 ? ATTN_RING - 1 : slot - 1);
    if (kb < nblk) {
      v4f_t bb[BIASED ? 2 : 1][BIASED ? 4 : 1];   // bias of this lane's 32 scores: keys key0 + 32 t + 8 g + 4 h + (0..3)
      if constexpr (BIASED) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const v4i_t w = __builtin_amdgcn_raw_buffer_load_b128(rsrc_bias, (int)((qrow * a.bias_sm + key0 + 32 * t + 8 * g + 4 * h) * 4), 0, 0);
            bb[t][g] = __builtin_bit_cast(v4f_t, w);
          }
      }
      // ---- S = Q K^T for two 32-key tiles; K scale of (tile t, step s, half h) = byte t D/32 + 2 s + h
      v16f_t S[2];
      int ksh[KS_DW];
#pragma unroll
      for (int i = 0; i < KS_DW; ++i) ksh[i] = (int)(ksw[i] >> (8 * h));
      static_for<2>([&](auto tc) {
        constexpr int t = decltype(tc)::value;
#pragma unroll
        for (int v = 0; v < 16; ++v) S[t][v] = 0.0f;
        static_for<NK>([&](auto sc) {
          constexpr int s = decltype(sc)::value;
          constexpr int byte = t * (D / 32) + 2 * s;
          const v8i_t kf = frag16(tile + (32 * t + r) * (D / 2) + ((32 * s + 16 * h) ^ k_swz));
          S[t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kf, qf[s], S[t], 4, 4, byte % 4, ksh[byte / 4], 0, qsc[s]);
        });
      });
      if constexpr (BIASED) {   // scores into the base-2 domain with their additive terms
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int key = key0 + 32 * t + 8 * (v >> 2) + 4 * h + (v & 3);
            float x = __builtin_fmaf(bb[t][v >> 2][v & 3], ATTN_RCP_LN2, S[t][v] * c2);
            x = __builtin_fmaf(-slope2, __builtin_fabsf((float)(qrow + shift - key)), x);
            S[t][v] = x;
          }
      }
      // ---- mask (only blocks the diagonal crosses or that reach past the last key), running max kept in the base-2 domain: m = max(S) * sm_scale * log2(e)
      if ((a.causal && key0 + 63 > q0 + shift) || key0 + 64 > a.Sk_used) {
        asm volatile("" ::: "memory");   // keep this a branch: most blocks skip it
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int key = key0 + 32 * t + 8 * (v >> 2) + 4 * h + (v & 3);
            if ((a.causal && key > qrow + shift) || key >= a.Sk_used) S[t][v] = -__builtin_inff();
          }
      }
      float tmx[2];   // row maximum of each 32-key tile (exp2 is monotonic: its largest probability comes from this score)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        float x = -__builtin_inff();
#pragma unroll
        for (int v = 0; v < 16; ++v) x = fmaxf(x, S[t][v]);
        tmx[t] = pair_max(x);
      }
      const float mx = fmaxf(tmx[0], tmx[1]);
      float m_new = fmaxf(m_i, mx * cs);
      // a bias may hide every key a row has seen so far (-inf): such a row keeps m = -inf and takes exp2(-inf - 0) = 0
      // everywhere instead of exp2(-inf + inf)
      const float m_sub = (BIASED && m_new == -__builtin_inff()) ? 0.0f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m_i - m_sub);
      m_i = m_new;
      m_new = m_sub;

      // ---- probabilities, one E8M0 scale per (row, 32 keys), E2M1 codes (round to nearest even)
      uint32_t c[2][2];
      int psc[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int v = 0; v < 16; ++v) S[t][v] = __builtin_amdgcn_exp2f(__builtin_fmaf(S[t][v], cs, -m_new));
        const float am = __builtin_amdgcn_exp2f(__builtin_fmaf(tmx[t], cs, -m_new));   // = max of the 32 values above
        const uint32_t e = e8m0_from_f32_bits(f2u(am));
        psc[t] = (int)e;
        const float scale_f = u2f(e << 23);
#pragma unroll
        for (int w = 0; w < 2; ++w) {
          uint32_t o = 0;
          o = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(o, S[t][8 * w + 0], S[t][8 * w + 1], scale_f, 0);
          o = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(o, S[t][8 * w + 2], S[t][8 * w + 3], scale_f, 1);
          o = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(o, S[t][8 * w + 4], S[t][8 * w + 5], scale_f, 2);
          o = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(o, S[t][8 * w + 6], S[t][8 * w + 7], scale_f, 3);
          c[t][w] = o;
        }
      }
      // Lane (r, h) multiplies tile h of this block and needs that tile's 32 codes of row r in key order; it holds the
      // keys 8 g + 4 h + (0..3) of both tiles.  One half-wave swap per dword hands lane (r, 0) the tile-0 codes of lane
      // (r, 1) and lane (r, 1) the tile-1 codes of lane (r, 0); in both halves the swapped pair is then {keys 8 g + 0..3,
      // keys 8 g + 4..7} = {p[0], p[1]}, interleaved 16 bits at a time.
      const v2u_t p0 = __builtin_amdgcn_permlane32_swap(c[0][0], c[1][0], false, false);
      const v2u_t p1 = __builtin_amdgcn_permlane32_swap(c[0][1], c[1][1], false, false);
      const v8i_t pf = v8i_t{(int)__builtin_amdgcn_perm(p0[1], p0[0], 0x05040100u), (int)__builtin_amdgcn_perm(p0[1], p0[0], 0x07060302u),
                             (int)__builtin_amdgcn_perm(p1[1], p1[0], 0x05040100u), (int)__builtin_amdgcn_perm(p1[1], p1[0], 0x07060302u),
                             0, 0, 0, 0};
      const int pscale = h ? psc[1] : psc[0];

      // ---- row sums of the quantised probabilities (a column of ones) and O += P V
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {   // the row maxima settle after a few blocks
        acc_l[0] *= alpha;                                     // all 16 registers hold the row sum; only [0] is read
#pragma unroll
        for (int d = 0; d < ND; ++d)
#pragma unroll
          for (int v = 0; v < 16; ++v) acc_o[d][v] *= alpha;
      }
      acc_l = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ones, pf, acc_l, 4, 4, 0, 127, 0, pscale);
      // V scale of (key tile h, column block d) = byte h Dv/32 + d
      const int vsh = DV == 128 ? (int)(h ? vsw[VS_DW - 1] : vsw[0]) : (int)(vsw[0] >> (16 * h));
      static_for<ND>([&](auto dc) {
        constexpr int d = decltype(dc)::value;
        const v8i_t vf = frag16(tile + K_BYTES + (32 * d + r) * 32 + ((16 * h) ^ v_swz));
        acc_o[d] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vf, pf, acc_o[d], 4, 4, d, vsh, 0, pscale);
      });
    }
    wait_dma(kb + 2 < wg_blk);   // block kb + 1 has landed (this wave's part; the barrier collects the others')
    asm volatile("s_barrier" ::: "memory");
    slot = slot == ATTN_RING - 1 ? 0 : slot + 1;
  }
  if (!live) return;

  // ---- O = acc / l, bf16; log-sum-exp
  const float l = acc_l[0];
  const float rl = 1.0f / l;
  __bf16* orow = out + (bhq * a.Sq + qrow) * DV;
#pragma unroll
  for (int d = 0; d < ND; ++d)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      bf16x2_t lo, hi;
      lo[0] = (__bf16)(acc_o[d][4 * g + 0] * rl);
      lo[1] = (__bf16)(acc_o[d][4 * g + 1] * rl);
      hi[0] = (__bf16)(acc_o[d][4 * g + 2] * rl);
      hi[1] = (__bf16)(acc_o[d][4 * g + 3] * rl);
      uint2 w;
      w.x = __builtin_bit_cast(uint32_t, lo);
      w.y = __builtin_bit_cast(uint32_t, hi);
      *reinterpret_cast<uint2*>(orow + 32 * d + 8 * g + 4 * h) = w;
    }
  if (h == 0) lse_out[bhq * a.Sq + qrow] = (m_i + log2f(l)) * ATTN_LN2;
}

template <int NK, int ND, bool BIASED>
__global__ __launch_bounds__(256, BIASED ? 2 : ATTN_WG_PER_CU) void attn_fwd_kernel(AttnArgs a) {
  __shared__ __attribute__((aligned(16))) uint8_t ring[ATTN_RING * AttnTile<NK, ND>::SLOT];
  attn_fwd_body<NK, ND, BIASED>(a, reinterpret_cast<__bf16*>(a.out), a.lse, ring);
}

template <int NK, int ND>
static int launch_attn(const AttnArgs& a, int B, hipStream_t st) {
  dim3 grid((unsigned)a.Hq, (unsigned)B, (unsigned)((a.Sq + 127) / 128));
  if (a.bias || a.alibi) hipLaunchKernelGGL((attn_fwd_kernel<NK, ND, true>), grid, dim3(256), 0, st, a);
  else hipLaunchKernelGGL((attn_fwd_kernel<NK, ND, false>), grid, dim3(256), 0, st, a);
  return check_launch("attention_fwd");
}

template <int NK>
static int launch_attn_nd(const AttnArgs& a, int B, int Dv, hipStream_t st) {
  switch (Dv) {
    case 64: return launch_attn<NK, 2>(a, B, st);
    case 128: return launch_attn<NK, 4>(a, B, st);
  }
  return ALTO_MXFP4_EINVAL;
}

}  // namespace alto

extern "C" int alto_mxfp4_attention_fwd_ex(const void* q_codes, const void* q_scales, const void* k_codes, const void* k_scales,
                                           const void* vt_codes, const void* v_scales, void* out, float* lse, int64_t B, int64_t Hq,
                                           int64_t Hk, int64_t Sq, int64_t Sk, int64_t Sk_used, int64_t D, int64_t Dv, float sm_scale,
                                           int causal, const float* bias, int64_t bias_sb, int64_t bias_sh, int64_t bias_sm,
                                           const float* alibi_slopes, int64_t alibi_sb, int64_t alibi_sh, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(!alibi_slopes || (alibi_sb >= 0 && alibi_sh >= 0), "attention_fwd: negative alibi strides");
  ALTO_REQUIRE(q_codes && q_scales && k_codes && k_scales && vt_codes && v_scales && out && lse, "attention_fwd: null pointer");
  ALTO_REQUIRE(B > 0 && Hq > 0 && Hk > 0 && Hq % Hk == 0, "attention_fwd: Hq=%lld must be a positive multiple of Hk=%lld", (long long)Hq, (long long)Hk);
  ALTO_REQUIRE(Sq > 0 && Sq % 32 == 0, "attention_fwd: Sq=%lld must be a positive multiple of 32", (long long)Sq);
  ALTO_REQUIRE(Sk > 0 && Sk % 64 == 0, "attention_fwd: Sk=%lld must be a positive multiple of 64", (long long)Sk);
  ALTO_REQUIRE(D == 64 || D == 128 || D == 192 || D == 256, "attention_fwd: head dim D=%lld must be 64, 128, 192 or 256", (long long)D);
  ALTO_REQUIRE(Dv == 64 || Dv == 128, "attention_fwd: value dim Dv=%lld must be 64 or 128", (long long)Dv);
  ALTO_REQUIRE(Sk_used > 0 && Sk_used <= Sk && Sk - Sk_used < 64 && Sk_used % 32 == 0,
               "attention_fwd: Sk_used=%lld must be a multiple of 32 in (Sk - 64, Sk]", (long long)Sk_used);
  ALTO_REQUIRE(!causal || Sq <= Sk_used, "attention_fwd: causal attention needs Sq <= Sk (got %lld > %lld)", (long long)Sq, (long long)Sk_used);
  ALTO_REQUIRE(B <= 65535 && (Sq + 127) / 128 <= 65535, "attention_fwd: B and Sq / 128 must fit a grid dimension");
  ALTO_REQUIRE(Hq < (1ll << 31) && Sk < (1ll << 31) && product_below(1ll << 40, B * Sq, Hq, D > Dv ? D : Dv), "attention_fwd: tensor too large");
  int64_t bias_bytes = 0;
  if (bias) {   // (B, Hq, Sq and Sk_used are in range here)
    ALTO_REQUIRE(bias_sb >= 0 && bias_sh >= 0 && bias_sm >= Sk_used && bias_sm % 4 == 0 && (uintptr_t)bias % 16 == 0,
                 "attention_fwd: bias rows must be 16-byte aligned with unit stride along the keys (row stride %lld)", (long long)bias_sm);
    ALTO_REQUIRE(product_below(1ll << 29, Sq, bias_sm) && product_below(1ll << 30, B - 1, bias_sb) && product_below(1ll << 30, Hq - 1, bias_sh),
                 "attention_fwd: bias tensor too large");
    bias_bytes = ((B - 1) * bias_sb + (Hq - 1) * bias_sh + (Sq - 1) * bias_sm + Sk_used) * 4;
    ALTO_REQUIRE(bias_bytes < (1ll << 32), "attention_fwd: bias tensor too large");
  }
  ALTO_REQUIRE(((uintptr_t)q_codes | (uintptr_t)k_codes | (uintptr_t)vt_codes) % 16 == 0 && (uintptr_t)out % 8 == 0,
               "attention_fwd: code pointers must be 16-byte aligned, out 8-byte aligned");
  ALTO_REQUIRE(((uintptr_t)k_scales | (uintptr_t)v_scales | (uintptr_t)lse | (uintptr_t)alibi_slopes) % 4 == 0,
               "attention_fwd: K and V scale pointers, lse and the alibi slopes must be 4-byte aligned");
  AttnArgs a{(const uint8_t*)q_codes, (const uint8_t*)q_scales, (const uint8_t*)k_codes, (const uint8_t*)k_scales,
             (const uint8_t*)vt_codes, (const uint8_t*)v_scales, out, lse, (int)Hq, (int)Hk, (int)Sq, (int)Sk, (int)Sk_used, sm_scale, causal ? 1 : 0,
             bias, bias_sb, bias_sh, bias_sm, bias_bytes, alibi_slopes, alibi_sb, alibi_sh};
  hipStream_t st = (hipStream_t)stream;
  switch (D) {
    case 64: return launch_attn_nd<1>(a, (int)B, (int)Dv, st);
    case 128: return launch_attn_nd<2>(a, (int)B, (int)Dv, st);
    case 192: return launch_attn_nd<3>(a, (int)B, (int)Dv, st);
    case 256: return launch_attn_nd<4>(a, (int)B, (int)Dv, st);
  }
  return ALTO_MXFP4_EINVAL;
}

extern "C" int alto_mxfp4_attention_fwd(const void* q_codes, const void* q_scales, const void* k_codes, const void* k_scales,
                                        const void* vt_codes, const void* v_scales, void* out, float* lse, int64_t B, int64_t Hq,
                                        int64_t Hk, int64_t Sq, int64_t Sk, int64_t Sk_used, int64_t D, int64_t Dv, float sm_scale,
                                        int causal, void* stream) {
  return alto_mxfp4_attention_fwd_ex(q_codes, q_scales, k_codes, k_scales, vt_codes, v_scales, out, lse, B, Hq, Hk, Sq, Sk, Sk_used, D, Dv, sm_scale,
                                     causal, nullptr, 0, 0, 0, nullptr, 0, 0, stream);
}
