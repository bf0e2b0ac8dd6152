// Ragged grouped MXFP4 GEMMs for MoE experts (gfx950): forward / dX (rows grouped by expert) and dW (reduction grouped by expert).
#include <mutex>

#include "common.h"
#include "gemm_simple.h"
#include "gemm_tile.h"

// Pass-list memory of alto_mxfp4_grouped_gemm_noalloc: one array per GPU, part of the loaded code object (each GPU the
// library runs on holds its own copy at its own address until the process ends).  In host code the name is only a
// handle for hipGetSymbolAddress; kernels get the address that call returns.
constexpr int64_t ALTO_NOALLOC_SCRATCH_BYTES = 1 << 20;
static __device__ __align__(256) unsigned char scratch[ALTO_NOALLOC_SCRATCH_BYTES];

namespace alto {
namespace {

// Maps a linear tile index onto (group, first row) by walking the offsets: group g owns ceil(len_g / tile_m) row
// tiles.  Index num_groups stands for the unrouted tail [offs[G], M_total), which is zero-filled.
struct TileRef {
  int group;  // -1: no such tile
  int64_t m0, m_lo, m_hi;
};

__device__ __forceinline__ TileRef locate_tile(const int32_t* offs, int num_groups, int64_t M_total, int64_t t, int tile_m) {
  TileRef ref{-1, 0, 0, 0};
  int64_t lo = offs[0];
  for (int g = 0; g <= num_groups; ++g) {
    int64_t hi = g < num_groups ? (int64_t)offs[g + 1] : M_total;
    hi = hi < lo ? lo : (hi > M_total ? M_total : hi);  // malformed offsets never index out of the buffers
    int64_t nt = (hi - lo + tile_m - 1) / tile_m;
    if (t < nt) {
      ref.group = g;
      ref.m_lo = lo;
      ref.m_hi = hi;
      ref.m0 = lo + t * tile_m;
      return ref;
    }
    t -= nt;
    lo = hi;
  }
  return ref;
}

__device__ __forceinline__ int clamp_off(const int32_t* offs, int g, int64_t M_total) {
  const int64_t v = offs[g];
  return (int)(v < 0 ? 0 : (v > M_total ? M_total : v));
}

template <typename OutT>
__global__ __launch_bounds__(256) void grouped_simple_kernel(OperandView A, const uint8_t* w, int64_t w_stride_e, int64_t ldw,
                                                             const uint8_t* w_scales, int64_t ws_stride_e, int64_t ws_r, int64_t ws_k, int w_is_2d,
                                                             const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts,
                                                             int64_t M_total, int64_t N, int G, OutT* out, int64_t ldo) {
  TileRef t = locate_tile(offs, num_groups, M_total, blockIdx.y, 64);
  if (t.group < 0) return;
  int expert = num_experts;  // "no expert": zero fill
  if (t.group < num_groups) {
    expert = group_expert ? group_expert[t.group] : t.group;
    if (expert < 0 || expert >= num_experts) expert = num_experts;
  }
  const int wave = threadIdx.x >> 6;
  const int64_t m0 = t.m0 + (wave >> 1) * 32;
  const int64_t n0 = (int64_t)blockIdx.x * 64 + (wave & 1) * 32;
  if (m0 >= t.m_hi || n0 >= N) return;
  v16f_t acc;
  if (expert == num_experts) {
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
  } else {
    OperandView B{w + expert * w_stride_e, ldw, w_scales + expert * ws_stride_e, ws_r, ws_k, w_is_2d};
    acc = mma_tile_32x32(A, B, m0, n0, t.m_lo, t.m_hi, N, 0, G);
  }
  store_tile_32x32<OutT>(acc, out, ldo, m0, n0, t.m_lo, t.m_hi, N, 1.0f);
}

// dW[e] tile (n0, k0): reduction over the token groups of expert e
template <typename OutT>
__global__ __launch_bounds__(256) void grouped_dw_simple_kernel(OperandView GO, OperandView X, const int32_t* offs, const int32_t* group_expert,
                                                                int num_groups, int64_t M_total, int64_t N, int64_t K,
                                                                OutT* dw, int64_t s_e, int64_t s_n, int64_t s_k, float out_scale) {
  const int e = blockIdx.z;
  const int wave = threadIdx.x >> 6;
  const int64_t n0 = (int64_t)blockIdx.y * 64 + (wave >> 1) * 32;
  const int64_t k0 = (int64_t)blockIdx.x * 64 + (wave & 1) * 32;
  if (n0 >= N || k0 >= K) return;
  v16f_t acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
  int bad = 0;   // a boundary of this expert's token ranges that is not a multiple of 32: the MX blocks along the token dim
                 // would be shared with another expert, so the gradient is poisoned with NaN instead of being silently wrong
  if (group_expert == nullptr) {
    const int lo = clamp_off(offs, e, M_total), hi = clamp_off(offs, e + 1, M_total);
    if (hi > lo) bad = (lo | hi) & 31;
    int g0 = lo / 32, g1 = hi / 32;
    mma_tile_32x32_acc(acc, GO, X, n0, k0, 0, N, K, g0, g1);
  } else {
    for (int g = 0; g < num_groups; ++g) {
      if (group_expert[g] != e) continue;
      const int lo = clamp_off(offs, g, M_total), hi = clamp_off(offs, g + 1, M_total);
      if (hi > lo) {   // a boundary shared with a neighbouring group of the same expert splits nothing
        if (!(g > 0 && group_expert[g - 1] == e)) bad |= lo & 31;
        if (!(g + 1 < num_groups && group_expert[g + 1] == e)) bad |= hi & 31;
      }
      int g0 = lo / 32, g1 = hi / 32;
      mma_tile_32x32_acc(acc, GO, X, n0, k0, 0, N, K, g0, g1);
    }
  }
  if (bad) {
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = __builtin_nanf("");
  }
  const int lane = threadIdx.x & 63;
  const int64_t j = k0 + (lane & 31);
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int64_t i = n0 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
    if (i < N && j < K) {
      float val = acc[v] * out_scale;
      OutT* dst = dw + e * s_e + i * s_n + j * s_k;
      if constexpr (sizeof(OutT) == 2) {
        unsigned short hb = (unsigned short)f32_to_bf16_bits(val);
        *dst = __builtin_bit_cast(OutT, hb);
      } else {
        *dst = val;
      }
    }
  }
}

// ----------------------------------------------------------------------------- 256x256 tiles (large problems)

// Tile order of the grouped kernels.  As in the dense kernel an XCD (wg % 8) works on 8 neighbouring N-tiles of a few row
// bands at a time, so its L2 shares the A rows and the expert's weight rows; but the row bands are dealt to the XCDs
// round-robin (band tm belongs to XCD tm % 8) instead of in contiguous ranges: a band that an expert boundary cuts runs
// once per segment, such bands cluster where the small experts sit, and contiguous ranges left one XCD with most of them.
__device__ __forceinline__ bool grouped_tile_coords(int wg, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int k = wg & 7, j = wg >> 3;
  const int nb = (tiles_m - k + 7) / 8;          // bands of this XCD
  if (nb <= 0 || j >= nb * tiles_n) return false;
  const int GN = 8;
  const int group = j / (GN * nb);
  const int first_n = group * GN;
  const int gsize = (tiles_n - first_n) < GN ? (tiles_n - first_n) : GN;
  const int w = j - group * GN * nb;
  tn = first_n + w % gsize;
  tm = k + 8 * (w / gsize);
  return true;
}
// workgroups to launch for that order: 8 x the tile count of the XCD with the most bands
__host__ __device__ inline int64_t grouped_grid_size(int64_t tiles_m, int64_t tiles_n) { return 8 * ((tiles_m + 7) / 8) * tiles_n; }

template <typename OutT>
__device__ __forceinline__ void zero_rows(OutT* out, int64_t ldo, int64_t r0, int64_t r1, int64_t n0, int64_t n1) {
  constexpr int PER = 16 / sizeof(OutT);
  const int chunks = (int)((n1 - n0) / PER);   // N % 8 == 0 and n0 % 256 == 0: whole 16-byte chunks
  const int64_t total = (r1 - r0) * chunks;
  for (int64_t i = threadIdx.x; i < total; i += GT_THREADS) {
    const int64_t row = r0 + i / chunks;
    const int ch = (int)(i % chunks);
    *reinterpret_cast<uint4*>(out + row * ldo + n0 + (int64_t)ch * PER) = make_uint4(0, 0, 0, 0);
  }
}

// ---- pass list.  The output rows are cut into passes: a pass is the part of one 256-row band that one expert serves
// (adjacent groups of the same expert merge; rows that no group owns, or whose expert id is out of range, form passes of
// expert -1 that are zero-filled).  A small plan kernel walks the offsets once and writes the list to a workspace in
// device memory; the GEMM kernel then runs one workgroup per (pass, 256-column tile), exactly like the dense kernel:
// no loop around the tile routine (which needs nearly every vector register), and passes of one band run in parallel.
//   workspace: int32 n_pass, 3 x pad, then n_pass x {band row, first row, end row, expert}
struct PassWalk {
  const int32_t* offs;
  const int32_t* group_expert;
  int num_groups, num_experts;
  int64_t M_total;
  __device__ __forceinline__ int off_at(int g) const { return clamp_off(offs, g, M_total); }
  __device__ __forceinline__ int expert_of(int g) const { return group_expert ? group_expert[g] : g; }
  // calls emit(first row, end row, expert) for every pass of band tm, in row order
  template <typename F>
  __device__ __forceinline__ void band(int tm, F&& emit) const {
    const int Mt = (int)M_total;
    const int row0 = tm * GT_TM;
    const int row1 = row0 + GT_TM < Mt ? row0 + GT_TM : Mt;
    int lo = 0, hi = num_groups;   // first group that ends after row0
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (off_at(mid + 1) > row0) hi = mid; else lo = mid + 1;
    }
    int g = lo, cur = row0;
    while (cur < row1) {
      int e = -1, seg_end = row1;
      while (g < num_groups && off_at(g + 1) <= cur) ++g;
      if (g < num_groups) {
        const int start = off_at(g);
        if (start > cur) {   // rows before the next group
          seg_end = start < row1 ? start : row1;
        } else {
          e = expert_of(g);
          int end = off_at(g + 1);
          while (end < row1 && g + 1 < num_groups && expert_of(g + 1) == e) {
            ++g;
            const int e2 = off_at(g + 1);
            end = e2 > end ? e2 : end;
          }
          seg_end = end < row1 ? end : row1;
          ++g;
          if (e < 0 || e >= num_experts) e = -1;
        }
      }
      emit(cur, seg_end, e);
      cur = seg_end;
    }
  }
};

constexpr int PLAN_THREADS = 256;

// One workgroup.  Two ways to cut the rows into passes, same list format:
//  * groups in expert order (group_expert == NULL, the sorted form of torch._grouped_mm): every group is tiled from its
//    own first row in steps of 256, so an expert has at most one partial tile (about E / 2 partial tiles in all, where
//    cutting fixed 256-row bands at the expert boundaries gives one extra pass per boundary); the rows before the first
//    and after the last group are tiled the same way as zero-fill passes.  Item i of the walk: 0 = head, 1..G = groups,
//    G + 1 = tail; thread t owns a block of consecutive items.
//  * per-group expert ids (the reference's form, one id per aligned 128-row group, any order): thread t owns the bands
//    [t nb, (t + 1) nb) and emits, per band, one pass per run of groups of the same expert.
// Either way a thread counts its passes, an exclusive scan of the counts gives its offset, and it writes them there,
// so the list is in row order.
// Inclusive scan over the workgroup's PLAN_THREADS values (thread order): inside a wave with lane shuffles, across the four
// waves through four words of LDS -- two barriers instead of the two per doubling step of a scan through LDS.
template <typename Op>
__device__ __forceinline__ int plan_scan(int v, Op op, int* part) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int u = __shfl_up(v, d, 64);
    if (lane >= d) v = op(v, u);
  }
  if (lane == 63) part[w] = v;
  __syncthreads();
  for (int k = 0; k < w; ++k) v = op(v, part[k]);
  __syncthreads();   // `part` may be written again
  return v;
}

__global__ __launch_bounds__(PLAN_THREADS) void grouped_plan_kernel(PassWalk wk, int tiles_m, int32_t* ws, int max_pass) {
  __shared__ int part[PLAN_THREADS / 64];
  __shared__ int carry[PLAN_THREADS];
  const int t = threadIdx.x;
  const bool sorted = wk.group_expert == nullptr;
  const int items = sorted ? wk.num_groups + 2 : tiles_m;
  const int per = (items + PLAN_THREADS - 1) / PLAN_THREADS;
  const int i0 = t * per, i1 = (i0 + per) < items ? (i0 + per) : items;
  const int Mt = (int)wk.M_total;
  // Sorted form: item i ends at E(i) = offs[i] (head: offs[0]; tail: M_total) and starts at the running maximum of the
  // ends before it, so the items tile [0, M_total) without overlap whatever the offsets are: a group whose end lies
  // below an earlier end is empty, one that starts below it is cut (the fallback kernel's row search does the same).
  auto item_end_load = [&](int i) { return i == wk.num_groups + 1 ? Mt : wk.off_at(i); };
  const int first_end = (sorted && i0 < i1) ? item_end_load(i0) : 0;   // (the usual case is one item per thread: one load in all)
  auto item_end = [&](int i) { return i == i0 ? first_end : item_end_load(i); };
  int start = 0;   // running maximum of the ends before item i0
  if (sorted) {
    int lm = 0;
    for (int i = i0; i < i1; ++i) { const int v = item_end(i); lm = v > lm ? v : lm; }
    carry[t] = plan_scan(lm, [](int a, int b) { return a > b ? a : b; }, part);   // inclusive max scan
    __syncthreads();
    start = t > 0 ? carry[t - 1] : 0;
  }
  auto item = [&](int i, int& run, int& lo, int& hi, int& e) {   // `run` carries the running maximum along the thread's items
    e = (i >= 1 && i <= wk.num_groups && (i - 1) < wk.num_experts) ? i - 1 : -1;
    lo = run;
    const int end = item_end(i);
    hi = end > lo ? end : lo;
    run = hi;
  };
  auto walk = [&](auto&& emit) {
    int run = start;
    for (int i = i0; i < i1; ++i) {
      if (sorted) {
        int lo, hi, e;
        item(i, run, lo, hi, e);
        for (int r = lo; r < hi; r += GT_TM) emit(r, r, r + GT_TM < hi ? r + GT_TM : hi, e);
      } else {
        wk.band(i, [&](int lo, int hi, int e) { emit(i * GT_TM, lo, hi, e); });
      }
    }
  };
  int cnt = 0;
  walk([&](int, int, int, int) { ++cnt; });
  const int upto = plan_scan(cnt, [](int a, int b) { return a + b; }, part);   // passes of threads 0 .. t
  int at = upto - cnt;
  int4* list = reinterpret_cast<int4*>(ws + 4);
  walk([&](int row0, int lo, int hi, int e) {
    if (at < max_pass) list[at] = make_int4(row0, lo, hi, e);
    ++at;
  });
  if (t == PLAN_THREADS - 1) ws[0] = upto < max_pass ? upto : max_pass;
}

template <typename OutT, bool KTAIL, int LMS, int NST, bool PS>
__global__ __launch_bounds__(GT_THREADS) void grouped_tiled_kernel(OperandView A, const uint8_t* w, int64_t w_stride_e, int64_t ldw,
                                                                   const uint8_t* w_scales, int64_t ws_stride_e, int64_t ws_r, int w_is_2d,
                                                                   const int32_t* plan, int64_t M_total, int64_t N, int G, OutT* out, int64_t ldo, int tiles_n) {
  extern __shared__ __align__(16) uint8_t smem[];
  const int n_pass = __builtin_amdgcn_readfirstlane(plan[0]);
  int pi, tn;
  if (!grouped_tile_coords(blockIdx.x, n_pass, tiles_n, pi, tn)) return;
  const int4 d = reinterpret_cast<const int4*>(plan + 4)[pi];
  const int row0 = __builtin_amdgcn_readfirstlane(d.x), m_lo = __builtin_amdgcn_readfirstlane(d.y), m_hi = __builtin_amdgcn_readfirstlane(d.z);
  const int e = __builtin_amdgcn_readfirstlane(d.w);
  const int n0 = tn * GT_TN;
  if (e < 0) {
    const int n1 = n0 + GT_TN < (int)N ? n0 + GT_TN : (int)N;
    zero_rows<OutT>(out, ldo, m_lo, m_hi, n0, n1);
    return;
  }
  // (packed scales: A.scales / w_scales + e * ws_stride_e are the packed bases, ss_k the bytes from block to block)
  OperandView B{w + e * w_stride_e, ldw, w_scales + e * ws_stride_e, ws_r, PS ? N * 16 : 1, w_is_2d};
  const int KB = (G + 15) / 16;
  TileArgs ta{A, B, row0, n0, m_lo, m_hi, N, G, 1.0f,
              (M_total - 1) * A.ld + G * 16, (N - 1) * ldw + G * 16,
              PS ? KB * A.ss_k : ((A.is_2d ? M_total / 32 : M_total) - 1) * A.ss_r + G, PS ? KB * N * 16 : ((w_is_2d ? N / 32 : N) - 1) * ws_r + G, 0, G};
  gemm_tile_256x256<OutT, KTAIL, LMS, NST, PS>(ta, out, ldo, smem);
}

// dW[e] tile: rows [256 tm, +256) of the first operand (P) x rows [256 tn, +256) of the second (Q), reduced over the
// token ranges of expert e.  With per-group expert ids, the runs of adjacent groups of this expert are found with one
// ballot per 64 groups (bit masks kept in LDS behind the tile's own buffers); every run is one pass of the K loop into
// the same accumulators, in increasing token order.
constexpr int GT_DW_MAX_GROUPS = 32768;
constexpr int GT_DW_LDS_BYTES = GT_LDS_BYTES + 2 * (GT_DW_MAX_GROUPS / 64) * 8;   // + 8 KB of masks

// The body of the kernel as a function of its own because of the `__restrict__` on the output: inlining then marks every
// memory operation in here, the global->LDS loads of the K loop included, as not aliasing the output, and only with that
// mark does the compiler's wait insertion keep those loads in flight across the LDS reads that follow them (unmarked, it
// puts an `s_waitcnt vmcnt(0)` before the next fragment read, twice per stage, and the loop runs at the load latency).
// PS: the operands' scales are in the packed form of alto_mxfp4_pack_scales along the tokens ([M_total / 512 blocks][rows][16],
// P.ss_k / Q.ss_k = bytes per block); a run starts at a 256-token line, i.e. at the first or the second half of a block.
template <typename OutT, bool PS>
__device__ __forceinline__ void grouped_dw_tile(const OperandView& P, const OperandView& Q, int64_t NP, int64_t NQ,
                                                const int32_t* offs, const int32_t* group_expert, int num_groups,
                                                int64_t M_total, OutT* __restrict__ dw, int64_t s_e, int64_t ld, float out_scale,
                                                int tiles_p, int tiles_q, int xq_log2, uint8_t* smem) {
  const int e = blockIdx.y;
  int tm, tn;
  {
    // Each XCD (blockIdx.x % 8) owns one rectangular block of every expert's tile grid, the XCDs forming a
    // (8 >> xq_log2) x (1 << xq_log2) arrangement: its ~32 resident workgroups then share the P and Q bands of one
    // expert's token range through its L2, and each band is fetched by few XCDs.
    const int k = blockIdx.x & 7, j = blockIdx.x >> 3;
    const int xq = 1 << xq_log2, xp = 8 >> xq_log2;
    const int bp = (tiles_p + xp - 1) / xp, bq = (tiles_q + xq - 1) / xq;
    const int p0 = (k >> xq_log2) * bp, q0 = (k & (xq - 1)) * bq;
    const int np = tiles_p - p0 < bp ? tiles_p - p0 : bp, nq = tiles_q - q0 < bq ? tiles_q - q0 : bq;
    if (np <= 0 || nq <= 0 || j >= np * nq) return;
    tm = p0 + j / nq;
    tn = q0 + j % nq;
  }
  TileAcc acc;
  gemm_tile_zero(acc);
  const int64_t p_bytes = (NP - 1) * P.ld + M_total / 2, q_bytes = (NQ - 1) * Q.ld + M_total / 2;
  const int64_t ps_bytes = PS ? ((M_total + 511) / 512) * P.ss_k : ((P.is_2d ? NP / 32 : NP) - 1) * P.ss_r + M_total / 32;
  const int64_t qs_bytes = PS ? ((M_total + 511) / 512) * Q.ss_k : ((Q.is_2d ? NQ / 32 : NQ) - 1) * Q.ss_r + M_total / 32;
  // Boundaries of this expert's token runs; one that is not a multiple of 32 would share an MX block along the token dim
  // with another expert: the tile is then poisoned with NaN instead of being silently wrong.
  int bad = 0;
  auto tok = [&](int g) { return (int64_t)clamp_off(offs, g, M_total); };
  uint64_t* mstart = reinterpret_cast<uint64_t*>(smem + GT_LDS_BYTES);
  uint64_t* mend = mstart + GT_DW_MAX_GROUPS / 64;
  const int words = group_expert ? (num_groups + 63) >> 6 : 0;
  for (int base = 0; base < words * 64; base += GT_THREADS) {
    const int gi = base + (int)threadIdx.x;
    bool first = false, last = false;
    if (gi < num_groups && group_expert[gi] == e) {
      first = gi == 0 || group_expert[gi - 1] != e;
      last = gi == num_groups - 1 || group_expert[gi + 1] != e;
    }
    const uint64_t bs = __ballot(first), be = __ballot(last);
    if ((threadIdx.x & 63) == 0 && (gi >> 6) < words) {
      mstart[gi >> 6] = bs;
      mend[gi >> 6] = be;
    }
  }
  __syncthreads();
  auto word = [&](const uint64_t* p, int i) {   // same LDS word for every lane -> scalar registers
    const uint64_t v = p[i];
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return ((uint64_t)hi << 32) | lo;
  };
  int wi = -1;           // current mask word; -1: not started
  uint64_t ms = 0, me = 0;
  int64_t t0 = 0, t1 = 0;
  bool direct_done = false;
  while (true) {
    // next run [t0, t1) of this expert's tokens
    bool have = false;
    if (group_expert == nullptr) {
      if (!direct_done) {
        t0 = tok(e);
        t1 = tok(e + 1);
        direct_done = true;
        have = true;
      }
    } else {
      while (true) {
        if (ms == 0 && me == 0) {
          if (++wi >= words) break;
          ms = word(mstart, wi);
          me = word(mend, wi);
          continue;
        }
        const int bs = ms ? __builtin_ctzll(ms) : 64, be = me ? __builtin_ctzll(me) : 64;
        if (bs <= be) {   // a run starts at this group; its end is this bit or a later one
          t0 = tok(wi * 64 + bs);
          ms &= ms - 1;
        } else {
          t1 = tok(wi * 64 + be + 1);
          me &= me - 1;
          have = true;
          break;
        }
      }
    }
    if (!have) break;
    if (t1 <= t0) continue;
    bad |= (int)(t0 | t1) & 31;
    t0 &= ~(int64_t)31;
    t1 &= ~(int64_t)31;
    if (t1 <= t0) continue;
    // The codes start at the 128-byte line (256 tokens) that holds the run's first token, so that every operand load is one
    // whole line; the groups of that line that lie before the run read as zeros (k_lead).  The scale rows keep their
    // base and the offset of the line rides in s_k0.
    const int64_t ta0 = t0 & ~(int64_t)255;
    OperandView Pv = P, Qv = Q;
    Pv.codes += ta0 / 2;
    Qv.codes += ta0 / 2;
    TileArgs ta{Pv, Qv, (int64_t)tm * GT_TM, (int64_t)tn * GT_TN, 0, NP, NQ, (int)((t1 - ta0) / 32), out_scale,
                p_bytes - ta0 / 2, q_bytes - ta0 / 2, ps_bytes, qs_bytes, (int)(ta0 / 32), (int)(M_total / 32), (int)((t0 - ta0) / 32),
                (int)(ta0 >> 9), (int)(ta0 >> 8) & 1};
    gemm_tile_mainloop<true, -2, 4, PS ? 2 : 0>(ta, acc, smem);
  }
  if (bad) {
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][u][v] = __builtin_nanf("");
  }
  TileArgs ta{P, Q, (int64_t)tm * GT_TM, (int64_t)tn * GT_TN, 0, NP, NQ, 0, out_scale, 0, 0, 0, 0, 0, 0};
  gemm_tile_store<OutT>(ta, acc, dw + e * s_e, ld, smem);
}

template <typename OutT, bool PS = false>
__global__ __launch_bounds__(GT_THREADS) void grouped_dw_tiled_kernel(OperandView P, OperandView Q, int64_t NP, int64_t NQ,
                                                                      const int32_t* offs, const int32_t* group_expert, int num_groups,
                                                                      int64_t M_total, OutT* dw, int64_t s_e, int64_t ld, float out_scale,
                                                                      int tiles_p, int tiles_q, int xq_log2) {
  extern __shared__ __align__(16) uint8_t smem[];
  grouped_dw_tile<OutT, PS>(P, Q, NP, NQ, offs, group_expert, num_groups, M_total, dw, s_e, ld, out_scale, tiles_p, tiles_q, xq_log2, smem);
}

// upper bound on the number of passes: every band is one, every group start inside a band adds one, plus the unrouted head and tail
inline int64_t grouped_max_passes(int64_t M_total, int64_t num_groups) { return (M_total + GT_TM - 1) / GT_TM + num_groups + 2; }
inline int64_t grouped_workspace_bytes(int64_t M_total, int64_t num_groups) { return 16 + 16 * grouped_max_passes(M_total, num_groups); }

template <typename OutT, bool KTAIL, int LMS = -1, int NST = 4, bool PS = false>
int launch_grouped_tiled(const OperandView& A, const uint8_t* w, int64_t w_stride_e, int64_t ldw, const uint8_t* w_scales, int64_t ws_stride_e,
                         int64_t ws_r, int w_is_2d, const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts,
                         int64_t M_total, int64_t N, int64_t K, void* out, int64_t ldo, int32_t* plan, bool build_plan, hipStream_t st) {
  // the opt-in for > 64 KB of dynamic LDS is per function, set once per process (thread-safe: forward and backward may
  // make their first calls from two host threads)
  auto kern = grouped_tiled_kernel<OutT, KTAIL, LMS, NST, PS>;
  static std::once_flag once;
  static hipError_t attr_rc = hipSuccess;
  std::call_once(once, [&] { attr_rc = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, GT_LDS_BYTES); });
  if (attr_rc != hipSuccess) return -1;
  const int tiles_m = (int)((M_total + GT_TM - 1) / GT_TM), tiles_n = (int)((N + GT_TN - 1) / GT_TN);
  const int max_pass = (int)grouped_max_passes(M_total, num_groups);
  PassWalk wk{offs, group_expert, num_groups, num_experts, M_total};
  if (build_plan) hipLaunchKernelGGL(grouped_plan_kernel, dim3(1), dim3(PLAN_THREADS), 0, st, wk, tiles_m, plan, max_pass);
  hipLaunchKernelGGL(kern, dim3((unsigned)grouped_grid_size(max_pass, tiles_n)), dim3(GT_THREADS), GT_LDS_BYTES, st, A, w, w_stride_e, ldw, w_scales, ws_stride_e, ws_r,
                     w_is_2d, plan, M_total, N, (int)(K / 32), (OutT*)out, ldo, tiles_n);
  return 0;
}

template <typename OutT, bool PS = false>
int launch_dw_tiled(const OperandView& P, const OperandView& Q, int64_t NP, int64_t NQ, const int32_t* offs, const int32_t* group_expert,
                    int num_groups, int num_experts, int64_t M_total, void* dw, int64_t s_e, int64_t ld, float out_scale, hipStream_t st) {
  auto kern = grouped_dw_tiled_kernel<OutT, PS>;
  static std::once_flag once;
  static hipError_t attr_rc = hipSuccess;
  std::call_once(once, [&] { attr_rc = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, GT_DW_LDS_BYTES); });
  if (attr_rc != hipSuccess) return -1;
  const int tiles_p = (int)((NP + GT_TM - 1) / GT_TM), tiles_q = (int)((NQ + GT_TN - 1) / GT_TN);
  // split of the 8 XCDs over the tile grid: the smallest blocks (least idle workgroups), then the smallest perimeter
  int xq_log2 = 0;
  int64_t best_area = -1, best_per = 0;
  for (int l = 0; l < 4; ++l) {
    const int xq = 1 << l, xp = 8 >> l;
    const int64_t bp = (tiles_p + xp - 1) / xp, bq = (tiles_q + xq - 1) / xq;
    if (best_area < 0 || bp * bq < best_area || (bp * bq == best_area && bp + bq < best_per)) {
      best_area = bp * bq;
      best_per = bp + bq;
      xq_log2 = l;
    }
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)(8 * best_area), (unsigned)num_experts), dim3(GT_THREADS), GT_DW_LDS_BYTES, st, P, Q, NP, NQ, offs,
                     group_expert, num_groups, M_total, (OutT*)dw, s_e, ld, out_scale, tiles_p, tiles_q, xq_log2);
  return 0;
}

}  // namespace
}  // namespace alto

namespace alto {
namespace {

// `plan` = device memory for the pass list (plan_bytes of it), needed by the tiled path only
int grouped_gemm_impl(const uint8_t* a, int64_t lda, const uint8_t* a_scales, int64_t a_ss_r, int64_t a_ss_k, int a_is_2d,
                      const uint8_t* w, int64_t w_stride_e, int64_t ldw,
                      const uint8_t* w_scales, int64_t ws_stride_e, int64_t ws_r, int64_t ws_k, int w_is_2d,
                      const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts,
                      int64_t M_total, int64_t N, int64_t K, void* out, int out_dtype, int64_t ldo,
                      void* plan, int64_t plan_bytes, const char* plan_name, bool build_plan, void* stream, bool ps = false) {
  ALTO_REQUIRE(a && a_scales && w && w_scales && offs && out, "grouped_gemm: NULL pointer");
  ALTO_REQUIRE(((reinterpret_cast<uintptr_t>(offs) | reinterpret_cast<uintptr_t>(group_expert)) & 3) == 0, "grouped_gemm: offs and group_expert must be 4-byte aligned");
  ALTO_REQUIRE(num_groups > 0 && num_groups <= 65536, "grouped_gemm: num_groups (%d) out of range", num_groups);
  ALTO_REQUIRE(group_expert != nullptr || num_groups == num_experts, "grouped_gemm: without group_expert, num_groups must equal num_experts");
  ALTO_REQUIRE(num_experts > 0 && num_experts <= 4096, "grouped_gemm: num_experts (%d) out of range", num_experts);
  ALTO_REQUIRE(M_total >= 0 && N >= 0 && K >= 0 && K % 32 == 0, "grouped_gemm: K (%lld) must be a multiple of 32", (long long)K);
  ALTO_REQUIRE(M_total < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), "grouped_gemm: size out of range");
  ALTO_REQUIRE(!w_is_2d || N % 32 == 0, "grouped_gemm: 2D weight scales need N (%lld) %% 32 == 0", (long long)N);
  ALTO_REQUIRE(!a_is_2d || M_total % 32 == 0, "grouped_gemm: 2D activation scales need M_total %% 32 == 0");
  ALTO_REQUIRE(lda >= K / 2 && ldw >= K / 2 && lda % 16 == 0 && ldw % 16 == 0 && w_stride_e % 16 == 0,
               "grouped_gemm: lda/ldw/w_stride_e must be >= K/2 and multiples of 16 bytes");
  ALTO_REQUIRE(((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(w)) & 15) == 0, "grouped_gemm: a and w must be 16-byte aligned");
  ALTO_REQUIRE(ldo >= N, "grouped_gemm: ldo < N");
  ALTO_REQUIRE(a_ss_r >= 0 && a_ss_k >= 0 && ws_stride_e >= 0 && ws_r >= 0 && ws_k >= 0 && w_stride_e >= 0, "grouped_gemm: negative stride");
  ALTO_REQUIRE(out_dtype == ALTO_DT_BF16 || out_dtype == ALTO_DT_F32, "grouped_gemm: bad out_dtype %d", out_dtype);
  ALTO_REQUIRE((reinterpret_cast<uintptr_t>(out) & (out_dtype == ALTO_DT_F32 ? 3 : 1)) == 0, "grouped_gemm: out must be aligned to its element size");
  if (M_total == 0 || N == 0) return ALTO_MXFP4_OK;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  OperandView A{a, lda, a_scales, a_ss_r, ps ? M_total * 16 : a_ss_k, a_is_2d};
  // 256x256 tiles when the problem fills them and the layouts fit their loads (unit-stride scale rows, 32-bit buffer
  // offsets, 16-byte output chunks); otherwise the direct kernel below
  const bool tiled = M_total >= 128 && N >= 128 && K >= 512 && a_ss_k == 1 && ws_k == 1 && N % 8 == 0 && ldo % 8 == 0 &&
                     (reinterpret_cast<uintptr_t>(out) & 15) == 0 && product_below(1ll << 31, M_total, lda) && product_below(1ll << 31, N, ldw) &&
                     product_below(1ll << 31, M_total, a_ss_r) && product_below(1ll << 31, N, ws_r) &&
                     grouped_max_passes(M_total, num_groups) * ((N + GT_TN - 1) / GT_TN) < (1ll << 28);
  if (ps && !(tiled && out_dtype == ALTO_DT_BF16)) {
    set_error("grouped_gemm_ps: shape (%lld, %lld, %lld) is not served by the tile kernel; use plain scales", (long long)M_total, (long long)N, (long long)K);
    return ALTO_MXFP4_ENOTIMPL;
  }
  if (tiled) {
    const int64_t need = grouped_workspace_bytes(M_total, num_groups);
    ALTO_REQUIRE(plan != nullptr && plan_bytes >= need && (reinterpret_cast<uintptr_t>(plan) & 15) == 0,
                 "grouped_gemm: %s of %lld bytes is too small: M_total = %lld with %d groups needs %lld bytes (16-byte aligned)", plan_name,
                 (long long)plan_bytes, (long long)M_total, num_groups, (long long)need);
    const bool tail = (K / 32) % 16 != 0;
    int32_t* pl = reinterpret_cast<int32_t*>(plan);
    int rc = -1;
#define ALTO_GROUPED_LAUNCH(T, ...) launch_grouped_tiled<T, __VA_ARGS__>(A, w, w_stride_e, ldw, w_scales, ws_stride_e, ws_r, w_is_2d, offs, group_expert, num_groups, num_experts, M_total, N, K, out, ldo, pl, build_plan, st)
    if (ps) {
      int lms = -1, nst = 4;
      if (tail) gemm_tile_last_stage(K / 32, lms, nst);
      switch (tail ? lms * 4 + nst - 1 : -1) {
        case -1: rc = ALTO_GROUPED_LAUNCH(__bf16, false, -1, 4, true); break;
        case 0: rc = ALTO_GROUPED_LAUNCH(__bf16, true, 0, 1, true); break;
        case 1: rc = ALTO_GROUPED_LAUNCH(__bf16, true, 0, 2, true); break;
        case 2: rc = ALTO_GROUPED_LAUNCH(__bf16, true, 0, 3, true); break;
        case 3: rc = ALTO_GROUPED_LAUNCH(__bf16, true, 0, 4, true); break;
        case 4: rc = ALTO_GROUPED_LAUNCH(__bf16, true, 1, 1, true); break;
        case 5: rc = ALTO_GROUPED_LAUNCH(__bf16, true, 1, 2, true); break;
        case 6: rc = ALTO_GROUPED_LAUNCH(__bf16, true, 1, 3, true); break;
        default: rc = ALTO_GROUPED_LAUNCH(__bf16, true, 1, 4, true); break;
      }
    } else if (!tail) {
      rc = out_dtype == ALTO_DT_BF16 ? ALTO_GROUPED_LAUNCH(__bf16, false) : ALTO_GROUPED_LAUNCH(float, false);
    } else if (out_dtype != ALTO_DT_BF16) {
      rc = ALTO_GROUPED_LAUNCH(float, true);   // (fp32 output: the general ending)
    } else {
      // K is known here: the kernel that ends the reduction exactly where K ends
      int lms, nst;
      gemm_tile_last_stage(K / 32, lms, nst);
      switch (lms * 4 + nst - 1) {
        case 0: rc = ALTO_GROUPED_LAUNCH(__bf16, true, 0, 1); break;
        case 1: rc = ALTO_GROUPED_LAUNCH(__bf16, true, 0, 2); break;
        case 2: rc = ALTO_GROUPED_LAUNCH(__bf16, true, 0, 3); break;
        case 3: rc = ALTO_GROUPED_LAUNCH(__bf16, true, 0, 4); break;
        case 4: rc = ALTO_GROUPED_LAUNCH(__bf16, true, 1, 1); break;
        case 5: rc = ALTO_GROUPED_LAUNCH(__bf16, true, 1, 2); break;
        case 6: rc = ALTO_GROUPED_LAUNCH(__bf16, true, 1, 3); break;
        default: rc = ALTO_GROUPED_LAUNCH(__bf16, true, 1, 4); break;
      }
    }
#undef ALTO_GROUPED_LAUNCH
    if (rc != 0) {
      set_error("grouped_gemm: could not reserve %d bytes of LDS", GT_LDS_BYTES);
      return ALTO_MXFP4_ELAUNCH;
    }
    return check_launch("grouped_gemm");
  }
  // upper bound on row tiles: every expert (and the zero tail) may end with one partial tile
  const int64_t tiles = M_total / 64 + num_groups + 2;
  ALTO_REQUIRE(tiles <= 65535, "grouped_gemm: M_total too large for the fallback kernel");
  dim3 grid((unsigned)((N + 63) / 64), (unsigned)tiles);
  if (out_dtype == ALTO_DT_BF16)
    hipLaunchKernelGGL(grouped_simple_kernel<__bf16>, grid, dim3(256), 0, st, A, w, w_stride_e, ldw, w_scales, ws_stride_e, ws_r, ws_k, w_is_2d,
                       offs, group_expert, num_groups, num_experts, M_total, N, (int)(K / 32), (__bf16*)out, ldo);
  else
    hipLaunchKernelGGL(grouped_simple_kernel<float>, grid, dim3(256), 0, st, A, w, w_stride_e, ldw, w_scales, ws_stride_e, ws_r, ws_k, w_is_2d,
                       offs, group_expert, num_groups, num_experts, M_total, N, (int)(K / 32), (float*)out, ldo);
  return check_launch("grouped_gemm");
}

}  // namespace
}  // namespace alto

extern "C" int64_t alto_mxfp4_grouped_gemm_workspace_bytes(int64_t M_total, int num_groups) {
  if (M_total < 0 || M_total >= (1ll << 31) || num_groups < 0) return 0;   // sizes no grouped call accepts
  return alto::grouped_workspace_bytes(M_total, num_groups);
}

extern "C" int alto_mxfp4_grouped_gemm(const uint8_t* a, int64_t lda, const uint8_t* a_scales, int64_t a_ss_r, int64_t a_ss_k, int a_is_2d,
                                       const uint8_t* w, int64_t w_stride_e, int64_t ldw,
                                       const uint8_t* w_scales, int64_t ws_stride_e, int64_t ws_r, int64_t ws_k, int w_is_2d,
                                       const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts,
                                       int64_t M_total, int64_t N, int64_t K, void* out, int out_dtype, int64_t ldo,
                                       void* workspace, int64_t workspace_bytes, void* stream) {
  return alto::grouped_gemm_impl(a, lda, a_scales, a_ss_r, a_ss_k, a_is_2d, w, w_stride_e, ldw, w_scales, ws_stride_e, ws_r, ws_k, w_is_2d, offs, group_expert,
                                 num_groups, num_experts, M_total, N, K, out, out_dtype, ldo, workspace, workspace_bytes, "the workspace", true, stream);
}

extern "C" int alto_mxfp4_grouped_gemm_planned(const uint8_t* a, int64_t lda, const uint8_t* a_scales, int64_t a_ss_r, int64_t a_ss_k, int a_is_2d,
                                               const uint8_t* w, int64_t w_stride_e, int64_t ldw,
                                               const uint8_t* w_scales, int64_t ws_stride_e, int64_t ws_r, int64_t ws_k, int w_is_2d,
                                               const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts,
                                               int64_t M_total, int64_t N, int64_t K, void* out, int out_dtype, int64_t ldo,
                                               const void* workspace, int64_t workspace_bytes, void* stream) {
  return alto::grouped_gemm_impl(a, lda, a_scales, a_ss_r, a_ss_k, a_is_2d, w, w_stride_e, ldw, w_scales, ws_stride_e, ws_r, ws_k, w_is_2d, offs, group_expert,
                                 num_groups, num_experts, M_total, N, K, out, out_dtype, ldo, const_cast<void*>(workspace), workspace_bytes, "the workspace",
                                 false, stream);
}

extern "C" int alto_mxfp4_grouped_gemm_ps(const uint8_t* a, int64_t lda, const uint8_t* a_packed, const uint8_t* w, int64_t w_stride_e, int64_t ldw,
                                          const uint8_t* w_packed, int64_t wp_stride_e, const int32_t* offs, const int32_t* group_expert,
                                          int num_groups, int num_experts, int64_t M_total, int64_t N, int64_t K, void* out, int64_t ldo,
                                          void* workspace, int64_t workspace_bytes, int plan_built, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(((reinterpret_cast<uintptr_t>(a_packed) | reinterpret_cast<uintptr_t>(w_packed) | (uintptr_t)wp_stride_e) & 15) == 0,
               "grouped_gemm_ps: packed scales (and the stride between experts) must be 16-byte aligned");
  ALTO_REQUIRE(K >= 0 && K < (1ll << 31) && product_below(1ll << 31, (K / 32 + 15) / 16, M_total > N ? M_total : N, 16),
               "grouped_gemm_ps: packed scales beyond 2 GiB");
  // A: [blocks][M_total][16]; expert e's weights: [blocks][N][16] at w_packed + e * wp_stride_e
  return grouped_gemm_impl(a, lda, a_packed, 16, 1, 0, w, w_stride_e, ldw, w_packed, wp_stride_e, 16, 1, 0, offs, group_expert, num_groups, num_experts,
                           M_total, N, K, out, ALTO_DT_BF16, ldo, workspace, workspace_bytes, "the workspace", plan_built == 0, stream, true);
}

extern "C" int alto_mxfp4_grouped_gemm_plan(const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts, int64_t M_total,
                                            void* workspace, int64_t workspace_bytes, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(offs != nullptr, "grouped_gemm_plan: NULL offs");
  ALTO_REQUIRE(((reinterpret_cast<uintptr_t>(offs) | reinterpret_cast<uintptr_t>(group_expert)) & 3) == 0, "grouped_gemm_plan: offs and group_expert must be 4-byte aligned");
  ALTO_REQUIRE(num_groups > 0 && num_groups <= 65536, "grouped_gemm_plan: num_groups (%d) out of range", num_groups);
  ALTO_REQUIRE(group_expert != nullptr || num_groups == num_experts, "grouped_gemm_plan: without group_expert, num_groups must equal num_experts");
  ALTO_REQUIRE(num_experts > 0 && num_experts <= 4096, "grouped_gemm_plan: num_experts (%d) out of range", num_experts);
  ALTO_REQUIRE(M_total >= 0 && M_total < (1ll << 31), "grouped_gemm_plan: M_total out of range");
  const int64_t need = grouped_workspace_bytes(M_total, num_groups);
  ALTO_REQUIRE(workspace != nullptr && workspace_bytes >= need && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0,
               "grouped_gemm_plan: workspace of %lld bytes is too small: M_total = %lld with %d groups needs %lld bytes (16-byte aligned)",
               (long long)workspace_bytes, (long long)M_total, num_groups, (long long)need);
  if (M_total == 0) return ALTO_MXFP4_OK;
  PassWalk wk{offs, group_expert, num_groups, num_experts, M_total};
  hipLaunchKernelGGL(grouped_plan_kernel, dim3(1), dim3(PLAN_THREADS), 0, reinterpret_cast<hipStream_t>(stream), wk, (int)((M_total + GT_TM - 1) / GT_TM),
                     reinterpret_cast<int32_t*>(workspace), (int)grouped_max_passes(M_total, num_groups));
  return check_launch("grouped_gemm_plan");
}

namespace alto {
namespace {
constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[MAX_DEVICES] = {};

// device address of `scratch` on the current GPU, looked up once per device
int scratch_of_current_device(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    set_error("grouped_gemm_noalloc: no current HIP device (or device index beyond %d)", MAX_DEVICES - 1);
    return ALTO_MXFP4_ELAUNCH;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      set_error("grouped_gemm_noalloc: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      return ALTO_MXFP4_ELAUNCH;
    }
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return ALTO_MXFP4_OK;
}
}  // namespace
}  // namespace alto

extern "C" int alto_mxfp4_init(void) {
  using namespace alto;
  void* p = nullptr;
  return scratch_of_current_device(&p);
}

extern "C" int alto_mxfp4_grouped_gemm_noalloc(const uint8_t* a, int64_t lda, const uint8_t* a_scales, int64_t a_ss_r, int64_t a_ss_k, int a_is_2d,
                                               const uint8_t* w, int64_t w_stride_e, int64_t ldw,
                                               const uint8_t* w_scales, int64_t ws_stride_e, int64_t ws_r, int64_t ws_k, int w_is_2d,
                                               const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts,
                                               int64_t M_total, int64_t N, int64_t K, void* out, int out_dtype, int64_t ldo, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(M_total >= 0 && M_total < (1ll << 31) && num_groups > 0, "grouped_gemm_noalloc: bad sizes");
  ALTO_REQUIRE(grouped_workspace_bytes(M_total, num_groups) <= ALTO_NOALLOC_SCRATCH_BYTES,
               "grouped_gemm_noalloc: M_total = %lld rows in %d groups need a pass list of %lld bytes, more than the built-in %lld: use "
               "alto_mxfp4_grouped_gemm with a workspace", (long long)M_total, num_groups, (long long)grouped_workspace_bytes(M_total, num_groups),
               (long long)ALTO_NOALLOC_SCRATCH_BYTES);
  void* plan = nullptr;
  const int rc = scratch_of_current_device(&plan);
  if (rc != ALTO_MXFP4_OK) return rc;
  return grouped_gemm_impl(a, lda, a_scales, a_ss_r, a_ss_k, a_is_2d, w, w_stride_e, ldw, w_scales, ws_stride_e, ws_r, ws_k, w_is_2d, offs, group_expert,
                           num_groups, num_experts, M_total, N, K, out, out_dtype, ldo, plan, ALTO_NOALLOC_SCRATCH_BYTES, "the built-in scratch array", true, stream);
}

namespace alto {
namespace {
// ps: go_scales / x_scales are packed along the tokens ([ceil(M_total / 512)][N or K][16]); tile kernel and bf16 only
int grouped_dw_impl(const uint8_t* go, int64_t ld_go, const uint8_t* go_scales, int64_t gs_r, int64_t gs_k, int go_is_2d,
                    const uint8_t* x, int64_t ld_xq, const uint8_t* x_scales, int64_t xs_r, int64_t xs_k, int x_is_2d,
                    const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts,
                    int64_t M_total, int64_t N, int64_t K, void* dw, int dw_dtype, int64_t dw_stride_e, int64_t dw_stride_n, int64_t dw_stride_k,
                    float out_scale, void* stream, bool ps) {
  ALTO_REQUIRE(go && go_scales && x && x_scales && offs && dw, "grouped_gemm_dw: NULL pointer");
  ALTO_REQUIRE(((reinterpret_cast<uintptr_t>(offs) | reinterpret_cast<uintptr_t>(group_expert)) & 3) == 0, "grouped_gemm_dw: offs and group_expert must be 4-byte aligned");
  ALTO_REQUIRE((reinterpret_cast<uintptr_t>(dw) & (dw_dtype == ALTO_DT_F32 ? 3 : 1)) == 0, "grouped_gemm_dw: dw must be aligned to its element size");
  ALTO_REQUIRE(num_experts > 0 && num_experts <= 65535, "grouped_gemm_dw: num_experts (%d) out of range", num_experts);
  ALTO_REQUIRE(num_groups > 0 && num_groups <= 65536, "grouped_gemm_dw: num_groups (%d) out of range", num_groups);
  ALTO_REQUIRE(group_expert != nullptr || num_groups == num_experts, "grouped_gemm_dw: without group_expert, num_groups must equal num_experts");
  ALTO_REQUIRE(M_total >= 0 && M_total % 32 == 0, "grouped_gemm_dw: M_total (%lld) must be a multiple of 32", (long long)M_total);
  ALTO_REQUIRE(N >= 0 && K >= 0 && M_total < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), "grouped_gemm_dw: size out of range");
  ALTO_REQUIRE(ld_go >= M_total / 2 && ld_xq >= M_total / 2 && ld_go % 16 == 0 && ld_xq % 16 == 0,
               "grouped_gemm_dw: ld_go/ld_xq must be >= M_total/2 and multiples of 16 bytes");
  ALTO_REQUIRE(((reinterpret_cast<uintptr_t>(go) | reinterpret_cast<uintptr_t>(x)) & 15) == 0, "grouped_gemm_dw: go and x must be 16-byte aligned");
  ALTO_REQUIRE(dw_dtype == ALTO_DT_BF16 || dw_dtype == ALTO_DT_F32, "grouped_gemm_dw: bad dw_dtype %d", dw_dtype);
  ALTO_REQUIRE(gs_r >= 0 && gs_k >= 0 && xs_r >= 0 && xs_k >= 0 && dw_stride_e >= 0 && dw_stride_n >= 0 && dw_stride_k >= 0, "grouped_gemm_dw: negative stride");
  if (N == 0 || K == 0) return ALTO_MXFP4_OK;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  ALTO_REQUIRE((!go_is_2d || N % 32 == 0) && (!x_is_2d || K % 32 == 0), "grouped_gemm_dw: 2D scales need N (%lld) / K (%lld) %% 32 == 0", (long long)N, (long long)K);
  OperandView GO{go, ld_go, go_scales, gs_r, gs_k, go_is_2d ? 1 : 0};
  OperandView X{x, ld_xq, x_scales, xs_r, xs_k, x_is_2d ? 1 : 0};
  {
    // 256x256 tiles: the output's unit-stride dim becomes the GEMM's column dim, so the operands swap roles for dW stored [E, K, N]
    const bool n_major = dw_stride_k == 1;   // dW[e] is [N][K]
    const OperandView& P = n_major ? GO : X;
    const OperandView& Q = n_major ? X : GO;
    const int64_t NP = n_major ? N : K, NQ = n_major ? K : N;
    const int64_t ld = n_major ? dw_stride_n : dw_stride_k;
    const bool unit = n_major || dw_stride_n == 1;
    const bool tiled = unit && M_total >= 512 && N >= 128 && K >= 128 && (ps || (gs_k == 1 && xs_k == 1)) && NQ % 8 == 0 && ld % 8 == 0 && dw_stride_e % 8 == 0 &&
                       (reinterpret_cast<uintptr_t>(dw) & 15) == 0 && product_below(1ll << 31, N, ld_go) && product_below(1ll << 31, K, ld_xq) &&
                       product_below(1ll << 31, N, gs_r) && product_below(1ll << 31, K, xs_r) && num_groups <= GT_DW_MAX_GROUPS && num_experts <= 65535 &&
                       ((NP + GT_TM - 1) / GT_TM) * ((NQ + GT_TN - 1) / GT_TN) < (1ll << 28);
    if (ps && !(tiled && dw_dtype == ALTO_DT_BF16)) {
      set_error("grouped_gemm_dw_ps: shape (%lld tokens, %lld, %lld) is not served by the tile kernel; use plain scales", (long long)M_total, (long long)N, (long long)K);
      return ALTO_MXFP4_ENOTIMPL;
    }
    if (tiled) {
      const int rc = ps ? launch_dw_tiled<__bf16, true>(P, Q, NP, NQ, offs, group_expert, num_groups, num_experts, M_total, dw, dw_stride_e, ld, out_scale, st)
                     : dw_dtype == ALTO_DT_BF16
                         ? launch_dw_tiled<__bf16>(P, Q, NP, NQ, offs, group_expert, num_groups, num_experts, M_total, dw, dw_stride_e, ld, out_scale, st)
                         : launch_dw_tiled<float>(P, Q, NP, NQ, offs, group_expert, num_groups, num_experts, M_total, dw, dw_stride_e, ld, out_scale, st);
      if (rc != 0) {
        set_error("grouped_gemm_dw: could not reserve %d bytes of LDS", GT_DW_LDS_BYTES);
        return ALTO_MXFP4_ELAUNCH;
      }
      return check_launch("grouped_gemm_dw");
    }
  }
  dim3 grid((unsigned)((K + 63) / 64), (unsigned)((N + 63) / 64), (unsigned)num_experts);
  ALTO_REQUIRE(grid.y <= 65535u, "grouped_gemm_dw: N too large");
  if (dw_dtype == ALTO_DT_BF16)
    hipLaunchKernelGGL(grouped_dw_simple_kernel<__bf16>, grid, dim3(256), 0, st, GO, X, offs, group_expert, num_groups, M_total, N, K, (__bf16*)dw, dw_stride_e, dw_stride_n, dw_stride_k, out_scale);
  else
    hipLaunchKernelGGL(grouped_dw_simple_kernel<float>, grid, dim3(256), 0, st, GO, X, offs, group_expert, num_groups, M_total, N, K, (float*)dw, dw_stride_e, dw_stride_n, dw_stride_k, out_scale);
  return check_launch("grouped_gemm_dw");
}
}  // namespace
}  // namespace alto

extern "C" int alto_mxfp4_grouped_gemm_dw(const uint8_t* go, int64_t ld_go, const uint8_t* go_scales, int64_t gs_r, int64_t gs_k, int go_is_2d,
                                          const uint8_t* x, int64_t ld_xq, const uint8_t* x_scales, int64_t xs_r, int64_t xs_k, int x_is_2d,
                                          const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts,
                                          int64_t M_total, int64_t N, int64_t K, void* dw, int dw_dtype, int64_t dw_stride_e, int64_t dw_stride_n, int64_t dw_stride_k,
                                          float out_scale, void* stream) {
  return alto::grouped_dw_impl(go, ld_go, go_scales, gs_r, gs_k, go_is_2d, x, ld_xq, x_scales, xs_r, xs_k, x_is_2d, offs, group_expert, num_groups, num_experts,
                               M_total, N, K, dw, dw_dtype, dw_stride_e, dw_stride_n, dw_stride_k, out_scale, stream, false);
}

extern "C" int alto_mxfp4_grouped_gemm_dw_ps(const uint8_t* go, int64_t ld_go, const uint8_t* go_packed, const uint8_t* x, int64_t ld_xq, const uint8_t* x_packed,
                                             const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts,
                                             int64_t M_total, int64_t N, int64_t K, void* dw, int64_t dw_stride_e, int64_t dw_stride_n, int64_t dw_stride_k,
                                             float out_scale, void* stream) {
  using namespace alto;
  ALTO_REQUIRE(((reinterpret_cast<uintptr_t>(go_packed) | reinterpret_cast<uintptr_t>(x_packed)) & 15) == 0, "grouped_gemm_dw_ps: packed scales must be 16-byte aligned");
  ALTO_REQUIRE(M_total >= 0 && M_total < (1ll << 31) && N >= 0 && K >= 0 && product_below(1ll << 31, (M_total + 511) / 512, N > K ? N : K, 16),
               "grouped_gemm_dw_ps: negative size, or packed scales beyond 2 GiB");
  // go: [blocks][N][16], x: [blocks][K][16]; ss_k carries the bytes from block to block
  return grouped_dw_impl(go, ld_go, go_packed, 16, N * 16, 0, x, ld_xq, x_packed, 16, K * 16, 0, offs, group_expert, num_groups, num_experts,
                         M_total, N, K, dw, ALTO_DT_BF16, dw_stride_e, dw_stride_n, dw_stride_k, out_scale, stream, true);
}
