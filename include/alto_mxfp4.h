/*
 * C ABI of libalto_mxfp4.so: MXFP4 training kernels for AMD MI355X (gfx950).
 *
 * Every entry point takes raw device pointers, sizes and a HIP stream
 * (passed as void*; NULL = the default stream), launches on that stream and
 * returns immediately.  Nothing is allocated inside the library: the caller
 * owns inputs and outputs.  The return value is 0 on success or a negative
 * ALTO_MXFP4_E* code; alto_mxfp4_last_error() then describes the failure
 * (thread-local string).  Invalid shapes are rejected BEFORE any launch.
 * Common to all entry points: sizes, counts and strides are non-negative,
 * matrix dimensions stay below 2^31, and a pointer to 2-, 4- or 8-byte
 * elements (bf16 / fp32 outputs, int32 offsets, uint64 state) is aligned to
 * its element size; the stricter alignments are stated per function.
 *
 * Each function names the entry point of the reference (AMD-AGI/ALTO, paths
 * relative to its checkout) whose device work it replaces.
 */
#ifndef ALTO_MXFP4_H
#define ALTO_MXFP4_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ALTO_MXFP4_OK 0
#define ALTO_MXFP4_EINVAL (-1)   /* bad argument (shape, alignment, flag combination) */
#define ALTO_MXFP4_ELAUNCH (-2)  /* the HIP runtime reported an error at launch */
#define ALTO_MXFP4_ENOTIMPL (-3) /* valid request that this build does not implement */

#define ALTO_MXFP4_BLOCK 32 /* MX block size (BLOCK_SIZE_DEFAULT, mxfp_quantization.py:17) */
#define ALTO_MXFP4_ALIGN_M 128 /* group alignment of the grouped GEMM (autotune.py:13) */

/* element types of high-precision tensors */
#define ALTO_DT_BF16 0
#define ALTO_DT_F32 1

/* rounding */
#define ALTO_ROUND_RNE 0
#define ALTO_ROUND_SR 1 /* stochastic, needs rand_bits */

/* clip modes (mxfp_quantization.py:428-438) */
#define ALTO_CLIP_NONE 0
#define ALTO_CLIP_STATIC 1
#define ALTO_CLIP_DYNAMIC 2 /* std-based scale (:54-59,65-70): row output only, no Hadamard, no UOS */

int alto_mxfp4_version(void);
const char* alto_mxfp4_last_error(void);

/*
 * Fused quantizer.  Replaces _convert_to_mxfp4_kernel and its host wrapper
 * (alto/kernels/fp4/mxfp4/mxfp_quantization.py:257-339, 410-484) and, when
 * `hadamard` is set, the preceding HadamardTransform.__call__(left_mul=True)
 * (alto/kernels/hadamard_transform/transform.py:115-142).
 *
 * Input: `batch` row-major matrices x[b][M][C] (element stride 1 along C, `ld_x`
 * elements between rows, `bs_x` elements between matrices), dtype bf16 or f32.
 *
 * Row output (quantised along C, i.e. convert_to_mxfp4(x, axis=-1)); produced when row_codes != NULL:
 *   row_codes  [b][M][C/2]   bytes, even element in the low nibble
 *   row_scales 1D: [b][M][C/32]      2D: [b][M/32][C/32]
 * Column output (quantised along M, i.e. convert_to_mxfp4(x, axis=-2)); produced when col_codes != NULL:
 *   col_codes  [b][C][M/2]   (the memory layout behind the transposed view the reference returns)
 *   col_scales 1D: [b][C][M/32]      2D: [b][C/32][M/32]
 * All outputs are dense (no padding between rows or matrices).
 *
 * hadamard != 0: the column output quantises H.x instead of x, where H is the
 *   randomized 32-point Hadamard transform along M built from `signs` (32
 *   values, +1/-1) and `perm` (a permutation of 0..31; NULL = identity), result
 *   divided by float32(sqrt(32)) and rounded to the input dtype, with the fp32
 *   summation order: scatter z[perm[j]] = x[j], butterflies of stride 1,2,4,8,16.
 *   The row output never sees the transform (mxfp_linear.py:466-494).
 *   Requires is_2d == 0.
 * rounding == ALTO_ROUND_SR: `rand_bits` holds one uint32 per input element
 *   (same indexing as x with row stride ld_rand, matrix stride bs_rand); element
 *   x[i][j] consumes rand_bits[i][j] for the row AND the column output
 *   (rule of _quantize_e2m1, alto/kernels/fp4/fp4_common/triton_fp4_ops.py:49-61,79-80).
 * clip_mode applies to the column output when both outputs are requested (the
 *   reference clips only its axis=0 quantisations, mxfp_linear.py:390-396, 486-493)
 *   and to whichever single output is requested otherwise.
 *
 * Requirements: C % 32 == 0 for the row output; M % 32 == 0 for the column
 * output and for 2D blocks; C % 8 == 0; ld_x % 8 == 0 (bf16) / % 4 == 0 (f32);
 * 16-byte aligned x.
 */
int alto_mxfp4_quantize(const void* x, int dtype, int64_t batch, int64_t M, int64_t C, int64_t ld_x, int64_t bs_x,
                        uint8_t* row_codes, uint8_t* row_scales, uint8_t* col_codes, uint8_t* col_scales,
                        int is_2d, int rounding, const uint32_t* rand_bits, int64_t ld_rand, int64_t bs_rand,
                        int hadamard, const int8_t* signs, const uint8_t* perm,
                        int clip_mode, int use_uos, void* stream);

/*
 * The same quantizer with a row pitch for the code outputs: row_codes[b][M][ld_row_codes] and
 * col_codes[b][C][ld_col_codes] (bytes; 0 = dense, i.e. C/2 and M/2).  A GEMM operand whose rows start on
 * 128-byte boundaries loads whole cache lines; the host layer pads K = 2880-like shapes this way for its own
 * intermediate operands.  No counterpart in the reference (its outputs are always dense).
 */
int alto_mxfp4_quantize_pitched(const void* x, int dtype, int64_t batch, int64_t M, int64_t C, int64_t ld_x, int64_t bs_x,
                                uint8_t* row_codes, uint8_t* row_scales, uint8_t* col_codes, uint8_t* col_scales,
                                int64_t ld_row_codes, int64_t ld_col_codes,
                                int is_2d, int rounding, const uint32_t* rand_bits, int64_t ld_rand, int64_t bs_rand,
                                int hadamard, const int8_t* signs, const uint8_t* perm,
                                int clip_mode, int use_uos, void* stream);

/*
 * The same quantizer with stochastic rounding whose random words are made INSIDE the kernel: element x[b][i][j] consumes
 * word ((b * M + i) * C + j) of the stream that alto_mxfp4_random_bits(out, n, seed, offset) writes (Philox4x32-10,
 * key = seed, counter = offset + word / 4), for the row AND the column output.  Filling a dense [batch][M][C] tensor with
 * alto_mxfp4_random_bits and passing it to alto_mxfp4_quantize_pitched gives the same bytes; this entry point reads no
 * random tensor and needs no fill launch.  It stands for the in-kernel draw of the reference
 * (tl.randint4x in alto/kernels/fp4/fp4_common/triton_fp4_ops.py:11-21, used at mxfp_quantization.py:129,184-185).
 * philox_state: NULL, or DEVICE memory holding {uint64 key, uint64 counter}: the kernel then takes key and counter from
 * there and ignores seed / offset, so that a captured launch (HIP graph) draws fresh words on every replay once the
 * state is advanced between replays (alto_mxfp4_philox_advance).  clip_mode = dynamic is not offered here
 * (ALTO_MXFP4_ENOTIMPL).  C < 2^26.
 */
int alto_mxfp4_quantize_sr_philox(const void* x, int dtype, int64_t batch, int64_t M, int64_t C, int64_t ld_x, int64_t bs_x,
                                  uint8_t* row_codes, uint8_t* row_scales, uint8_t* col_codes, uint8_t* col_scales,
                                  int64_t ld_row_codes, int64_t ld_col_codes, int is_2d,
                                  uint64_t seed, uint64_t offset, const uint64_t* philox_state,
                                  int hadamard, const int8_t* signs, const uint8_t* perm,
                                  int clip_mode, int use_uos, void* stream);

/*
 * The same quantizer with the stochastic rounding of the gfx950 hardware converts: one v_cvt_scalef32_sr_pk_fp4_bf16
 * (or _f32) per PAIR of neighbouring elements along the quantisation axis, one random dword per pair.  This is what the
 * reference runs on gfx950 when use_asm is left at its default (alto/kernels/fp4/mxfp4/mxfp_quantization.py:133-182,
 * USE_ASM = is_cdna4() at :426-427).  The dwords are cut from the Philox4x32-10 stream (key = seed, 128-bit counter
 * starting at offset), made inside the kernel.  With nb = ceil(M / 32) and "call c" = the Philox block with counter
 * offset + c:
 *   row output, pair (elements 2p, 2p+1) of x[b][i][.], j = 2p:
 *     bf16: dword = word (i%32)/8 of call ((b nb + i/32) (C/8) + j/8) 8 + i%8, shifted left by 8 ((j%8)/2)
 *     fp32: dword = word (j%8)/2 of call (((b nb + i/32) (C/8) + j/8) 8 + i%8) 4 + (i%32)/8
 *   column output, pair (rows 2p, 2p+1 of the transformed matrix) of column j, band i/32 = 2p/32, R = batch nb C:
 *     bf16: dword = word (p%16)/4 of call R + (b nb + i/32) C + j, shifted left by 8 (p%4)
 *     fp32: dword = word p%4 of call 4 R + ((b nb + i/32) C + j) 4 + (p%16)/4
 *   (the instruction reads the top 7 bits of the dword for a bf16 pair and the top 23 for an fp32 pair, so four bf16 pairs
 *   share one Philox word).  With is_2d both packings hold the codes of the row rule.
 * A call consumes alto_mxfp4_quantize_sr_hw_words(dtype, batch, M, C) words of the stream whatever outputs it writes.
 * philox_state as in alto_mxfp4_quantize_sr_philox.  clip_mode = dynamic is not offered here (ALTO_MXFP4_ENOTIMPL).
 * Results differ from ALTO_ROUND_SR's (the software rule of triton_fp4_ops.py:49-61): the instruction never moves an
 * exactly representable value and looks at fewer random bits.
 */
int alto_mxfp4_quantize_sr_hw(const void* x, int dtype, int64_t batch, int64_t M, int64_t C, int64_t ld_x, int64_t bs_x,
                              uint8_t* row_codes, uint8_t* row_scales, uint8_t* col_codes, uint8_t* col_scales,
                              int64_t ld_row_codes, int64_t ld_col_codes, int is_2d,
                              uint64_t seed, uint64_t offset, const uint64_t* philox_state,
                              int hadamard, const int8_t* signs, const uint8_t* perm,
                              int clip_mode, int use_uos, void* stream);

/* Random words one alto_mxfp4_quantize_sr_hw call of these sizes takes from its stream (a multiple of 4). */
int64_t alto_mxfp4_quantize_sr_hw_words(int dtype, int64_t batch, int64_t M, int64_t C);

/*
 * The quantizer with every rounding mode behind one signature, plus output-layout flags.  sr_mode: 0 = nearest even
 * (alto_mxfp4_quantize_pitched with use_sr = 0), 1 = stochastic with the words in rand_bits (the same call with use_sr =
 * 1), 2 = alto_mxfp4_quantize_sr_philox, 3 = alto_mxfp4_quantize_sr_hw; arguments a mode does not use are ignored.
 * Codes, and scales where no flag asks otherwise, are those calls' bit for bit.
 * flags (clip_mode not dynamic; M % 32 == 0; M C < 2^36; ALTO_MXFP4_EINVAL otherwise; with is_2d a block's scale is
 * repeated for its 32 rows, as alto_mxfp4_pack_scales does; with batch > 1 the packed matrices follow one another):
 *   ALTO_QUANT_PACK_ROW_SCALES (1): row_scales receives the packed layout of alto_mxfp4_pack_scales for rows = M, K = C
 *     (alto_mxfp4_packed_scales_bytes(M, C) bytes), pads included, instead of [M][C/32];
 *   ALTO_QUANT_PACK_COL_SCALES (2): col_scales likewise for rows = C, K = M.
 * The GEMMs on packed scales (alto_mxfp4_gemm_ps, alto_mxfp4_grouped_gemm_ps) then take the quantizer's output as it is.
 * The reference has one layout only (mxfp_quantization.py:340-420 writes [M][C/32]); the flags have no counterpart there.
 */
#define ALTO_QUANT_PACK_ROW_SCALES 1
#define ALTO_QUANT_PACK_COL_SCALES 2
int alto_mxfp4_quantize_ex(const void* x, int dtype, int64_t batch, int64_t M, int64_t C, int64_t ld_x, int64_t bs_x,
                           uint8_t* row_codes, uint8_t* row_scales, uint8_t* col_codes, uint8_t* col_scales,
                           int64_t ld_row_codes, int64_t ld_col_codes, int is_2d, int sr_mode,
                           const uint32_t* rand_bits, int64_t ld_rand, int64_t bs_rand, uint64_t seed, uint64_t offset,
                           const uint64_t* philox_state, int hadamard, const int8_t* signs, const uint8_t* perm,
                           int clip_mode, int use_uos, int flags, void* stream);

/*
 * Moves the counter of a device-resident Philox state {key, counter} past `words` random words (counter += ceil(words / 4)),
 * enqueued on `stream` after the quantizer call that consumed them.  A one-thread kernel; it can be captured together
 * with that call.  No counterpart in the reference (its Philox offsets are host integers).
 */
int alto_mxfp4_philox_advance(uint64_t* philox_state, uint64_t words, void* stream);

/*
 * Standalone randomized Hadamard transform along M in blocks of 32 rows:
 *   y[32b + i][c] = cast((sum_j W[i][j] * fp32(x[32b + j][c])) / float32(sqrt(32)))
 * with W built from signs/perm as in alto_mxfp4_quantize (same summation order, so
 * quantising y along M equals the fused column output bit for bit).  Replaces
 * HadamardTransform.__call__(left_mul=True) (alto/kernels/hadamard_transform/transform.py:115-142).
 * x, y: row-major [M][C] of `dtype` with row strides ld_x, ld_y (elements); M % 32 == 0.
 * signs and perm are HOST arrays, read before the call returns (also in alto_mxfp4_quantize).
 */
int alto_mxfp4_hadamard(const void* x, int dtype, int64_t M, int64_t C, int64_t ld_x, void* y, int64_t ld_y,
                        const int8_t* signs, const uint8_t* perm, void* stream);

/*
 * The other three forms of HadamardTransform.__call__(value, inverse, left_mul) (transform.py:115-142), same
 * arithmetic (fixed butterfly order, one division by float32(sqrt(32)), one rounding to `dtype`):
 *   left_mul = 1: y[32b + i][c] = sum_j V[i][j] x[32b + j][c]      (M % 32 == 0)
 *   left_mul = 0: y[r][32b + j] = sum_i x[r][32b + i] V[i][j]      (C % 32 == 0)
 * with V = W, or V = W^T when `inverse` is set (W is orthogonal up to the factor 32, so W^T / sqrt(32) undoes
 * W / sqrt(32)).  alto_mxfp4_hadamard is the case inverse = 0, left_mul = 1.
 */
int alto_mxfp4_hadamard_apply(const void* x, int dtype, int64_t M, int64_t C, int64_t ld_x, void* y, int64_t ld_y,
                              const int8_t* signs, const uint8_t* perm, int inverse, int left_mul, void* stream);

/*
 * Dequantizer.  Replaces _convert_from_mxfp4_kernel
 * (alto/kernels/fp4/mxfp4/mxfp_quantization.py:342-407, 487-545).
 * codes [R][C/2] dense, scales [R][C/32] (1D) or [R/32][C/32] (2D) dense;
 * out element (r, c) is written at out[r * out_stride_r + c * out_stride_c]
 * (strides in elements) so that the caller can produce either orientation.
 */
int alto_mxfp4_dequantize(const uint8_t* codes, const uint8_t* scales, int64_t R, int64_t C, int is_2d,
                          void* out, int out_dtype, int64_t out_stride_r, int64_t out_stride_c,
                          int clip_mode, void* stream);

/*
 * Nibble transpose: codes packed along the columns of a [R][C] code matrix
 * (memory [R][C/2]) -> the same codes packed along the rows (memory [C][R/2]).
 * Used to turn an operand packed along the non-reduction dim (k_pack=False,
 * mxfp_linear.py:528) into the reduction-contiguous form the GEMM consumes.
 * R % 2 == 0, C % 2 == 0.
 */
int alto_mxfp4_transpose_codes(const uint8_t* in, int64_t R, int64_t C, uint8_t* out, void* stream);

/*
 * Block-scaled MXFP4 GEMM, C[M][N] = A[M][K] . B[N][K]^T with fp32 accumulation.
 * Replaces blockwise_mxfp4_gemm_kernel (alto/kernels/fp4/mxfp4/mxfp_linear.py:31-139);
 * the host side maps the reference's trans/k_pack flags onto this canonical form.
 *   a [M][K/2] bytes, row stride lda bytes;  b [N][K/2], row stride ldb bytes
 *   a_scales: 1D [M][K/32] or 2D [M/32][K/32]; element (i, g) at a_scales[i * a_ss_r + g * a_ss_k]
 *   b_scales likewise with (b_ss_r, b_ss_k)
 *   c: bf16 or f32, row stride ldc elements
 * K % 32 == 0; for 2D scales the respective row count % 32 == 0.
 * out_scale multiplies the result before the cast (1.0f normally; 16/9 for the
 * static-clip wgrad, mxfp_linear.py:543-544).
 */
int alto_mxfp4_gemm(const uint8_t* a, int64_t lda, const uint8_t* a_scales, int64_t a_ss_r, int64_t a_ss_k, int a_is_2d,
                    const uint8_t* b, int64_t ldb, const uint8_t* b_scales, int64_t b_ss_r, int64_t b_ss_k, int b_is_2d,
                    int64_t M, int64_t N, int64_t K, void* c, int c_dtype, int64_t ldc, float out_scale, void* stream);

/*
 * Packed scales: an internal layout of the scale bytes of one GEMM operand that the 256x256 tile kernels move into LDS
 * with one load per wave and 512-K block, without registers, fix-ups or LDS writes (2 to 5 % of a GEMM).  No counterpart
 * in the reference.  For an operand of `rows` rows and K / 32 groups:
 *   packed[(kb * rows + row) * 16 + 4 * (2 h + ms) + j] = scale of group 16 kb + 8 ms + 2 j + h of that row
 *   (kb < ceil(K / 512); h, ms in {0, 1}; j < 4), and 127 where that group lies beyond K.
 * alto_mxfp4_pack_scales builds it from plain scales (1D: element (row, g) at scales[row * ss_r + g * ss_k]; 2D: row / 32
 * instead of row); alto_mxfp4_packed_scales_bytes is its size.  The quantizers write it directly when asked to
 * (alto_mxfp4_quantize_ex, flags).
 */
int64_t alto_mxfp4_packed_scales_bytes(int64_t rows, int64_t K);
int alto_mxfp4_pack_scales(const uint8_t* scales, int64_t ss_r, int64_t ss_k, int is_2d, int64_t rows, int64_t K, uint8_t* packed, void* stream);

/*
 * alto_mxfp4_gemm on operands with packed scales, bf16 output: c[M][N] = a[M][K] . b[N][K]^T * out_scale.  Same results as
 * alto_mxfp4_gemm, bit for bit.  Serves the shapes of the tile kernel only (M, N >= 128, K >= 512, N % 8 == 0, ldc % 8 ==
 * 0, 16-byte aligned c): ALTO_MXFP4_ENOTIMPL otherwise, and the caller keeps plain scales for those.
 */
int alto_mxfp4_gemm_ps(const uint8_t* a, int64_t lda, const uint8_t* a_packed, const uint8_t* b, int64_t ldb, const uint8_t* b_packed,
                       int64_t M, int64_t N, int64_t K, void* c, int64_t ldc, float out_scale, void* stream);

/*
 * Ragged grouped GEMM for MoE experts.  Rows [offs[g], offs[g+1]) of A form group g and use
 * expert e(g) = group_expert ? group_expert[g] : g:
 *   out[r][:] = A[r][:] . W[e]^T,   W[e] = w + e * w_stride_e  ([N][K/2] bytes, row stride ldw),
 *   w_scales[e]: 1D [N][K/32] or 2D [N/32][K/32] at w_scales + e * ws_stride_e, strides (ws_r, ws_k).
 * Replaces _kernel_mxfp4_grouped_gemm_forward and, with the N-packed weight copy as W,
 * _kernel_mxfp4_grouped_gemm_backward_dx
 * (alto/kernels/fp4/mxfp4/mxfp_grouped_gemm/cg_forward.py:32-194, cg_backward.py:42-205).
 * `offs` is a DEVICE array of num_groups + 1 int32 row offsets, non-decreasing, offs[num_groups] <= M_total;
 * `group_expert` is a DEVICE array of num_groups int32 expert ids or NULL (then num_groups == num_experts:
 * the sorted-by-expert form of torch._grouped_mm).  Both are read by the kernel (no host sync).  The
 * reference's per-row expert index with 128-row groups maps to offs = 128 * g, group_expert = index[128 * g].
 * Groups need no alignment for 1D activation scales; rows outside every group (and groups whose expert id is
 * out of range) are written with zeros (the reference allocates zeros, cg_forward.py:260).
 * `workspace`: DEVICE memory of at least alto_mxfp4_grouped_gemm_workspace_bytes(M_total, num_groups) bytes, 16-byte
 * aligned, owned by the caller.  A one-workgroup kernel first writes the list of (256-row band, expert) passes there
 * (the reference scans the groups inside every program instead, cg_forward.py:120-140), the GEMM kernel reads it.  Its
 * contents need not be initialised and mean nothing after the call; two calls that overlap in time need two workspaces.
 */
int alto_mxfp4_grouped_gemm(const uint8_t* a, int64_t lda, const uint8_t* a_scales, int64_t a_ss_r, int64_t a_ss_k, int a_is_2d,
                            const uint8_t* w, int64_t w_stride_e, int64_t ldw,
                            const uint8_t* w_scales, int64_t ws_stride_e, int64_t ws_r, int64_t ws_k, int w_is_2d,
                            const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts,
                            int64_t M_total, int64_t N, int64_t K, void* out, int out_dtype, int64_t ldo,
                            void* workspace, int64_t workspace_bytes, void* stream);

/*
 * The two halves of alto_mxfp4_grouped_gemm for callers that run several grouped GEMMs over the same groups (the forward
 * and the input gradient of one layer share them): alto_mxfp4_grouped_gemm_plan writes the pass list for (offs,
 * group_expert, num_groups, num_experts, M_total) into `workspace` (the one-workgroup kernel only), and
 * alto_mxfp4_grouped_gemm_planned is alto_mxfp4_grouped_gemm without that kernel: it trusts `workspace` to hold the list
 * that a call of _plan -- or of alto_mxfp4_grouped_gemm itself -- wrote for exactly these five arguments, and only reads
 * it (N, K and the operands may differ from call to call).  Same results as alto_mxfp4_grouped_gemm, bit for bit.  No
 * counterpart in the reference, whose kernels scan the groups inside every program (cg_forward.py:120-140).
 */
int alto_mxfp4_grouped_gemm_plan(const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts, int64_t M_total,
                                 void* workspace, int64_t workspace_bytes, void* stream);
int alto_mxfp4_grouped_gemm_planned(const uint8_t* a, int64_t lda, const uint8_t* a_scales, int64_t a_ss_r, int64_t a_ss_k, int a_is_2d,
                                    const uint8_t* w, int64_t w_stride_e, int64_t ldw,
                                    const uint8_t* w_scales, int64_t ws_stride_e, int64_t ws_r, int64_t ws_k, int w_is_2d,
                                    const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts,
                                    int64_t M_total, int64_t N, int64_t K, void* out, int out_dtype, int64_t ldo,
                                    const void* workspace, int64_t workspace_bytes, void* stream);

/*
 * alto_mxfp4_grouped_gemm on operands with packed scales (alto_mxfp4_pack_scales), bf16 output: a_packed is the packed form
 * of the [M_total][K/32] activation scales, w_packed + e * wp_stride_e that of expert e's weight scales ([N] rows).
 * plan_built != 0: `workspace` already holds the pass list for these groups (alto_mxfp4_grouped_gemm_plan or an earlier
 * call), as in alto_mxfp4_grouped_gemm_planned.  Same results as alto_mxfp4_grouped_gemm, bit for bit; serves the tile
 * kernel's shapes only (ALTO_MXFP4_ENOTIMPL otherwise).  No counterpart in the reference.
 */
int alto_mxfp4_grouped_gemm_ps(const uint8_t* a, int64_t lda, const uint8_t* a_packed, const uint8_t* w, int64_t w_stride_e, int64_t ldw,
                               const uint8_t* w_packed, int64_t wp_stride_e, const int32_t* offs, const int32_t* group_expert,
                               int num_groups, int num_experts, int64_t M_total, int64_t N, int64_t K, void* out, int64_t ldo,
                               void* workspace, int64_t workspace_bytes, int plan_built, void* stream);

/*
 * Per-device set-up that the entry points otherwise do on first use: resolves, for the CURRENT device, the address of the
 * library's built-in pass-list array.  Call it once per device (with that device current) before capturing a HIP graph
 * that contains alto_mxfp4_grouped_gemm_noalloc.  Idempotent, thread-safe, allocates nothing.  No counterpart in the
 * reference.
 */
int alto_mxfp4_init(void);

/*
 * alto_mxfp4_grouped_gemm without the workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The pass list
 * lives in a 1 MiB array that is part of the library's device code (one copy per GPU, held until the process ends), so
 * the call allocates nothing; it serves M_total / 256 + num_groups + 2 <= 65535 and rejects larger problems with
 * ALTO_MXFP4_EINVAL.  Every call on a GPU shares that GPU's array: calls that overlap in time on one GPU (two streams,
 * two host threads) race on it and must use alto_mxfp4_grouped_gemm with separate workspaces instead.  Same results as
 * alto_mxfp4_grouped_gemm, bit for bit.  The array used is that of the CURRENT device, which must be the device `stream`
 * belongs to.  Its address is looked up on the first use on a device (a runtime query that may load the code object):
 * call alto_mxfp4_init() on every device beforehand when the first call would otherwise fall inside a stream capture.
 */
int alto_mxfp4_grouped_gemm_noalloc(const uint8_t* a, int64_t lda, const uint8_t* a_scales, int64_t a_ss_r, int64_t a_ss_k, int a_is_2d,
                                    const uint8_t* w, int64_t w_stride_e, int64_t ldw,
                                    const uint8_t* w_scales, int64_t ws_stride_e, int64_t ws_r, int64_t ws_k, int w_is_2d,
                                    const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts,
                                    int64_t M_total, int64_t N, int64_t K, void* out, int out_dtype, int64_t ldo, void* stream);

/* Bytes of workspace alto_mxfp4_grouped_gemm needs for M_total rows in num_groups groups (a bound, not a measurement). */
int64_t alto_mxfp4_grouped_gemm_workspace_bytes(int64_t M_total, int num_groups);

/*
 * Grouped weight gradient: dW[e][N][K] = sum over the rows r of every group of expert e of dY[r][:]^T . X[r][:],
 * operands packed along the token dim:  go [N][M_total/2], x [K][M_total/2] with
 * scales [N][M_total/32], [K][M_total/32] (1D along tokens; strides given), or with go_is_2d / x_is_2d one scale per
 * 32 x 32 block: [N/32][M_total/32], [K/32][M_total/32] (the use_2dblock_go / use_2dblock_x operands of cg_backward.py:398-497).
 * Replaces _kernel_mxfp4_grouped_gemm_backward_dw (cg_backward.py:213-395); with group_expert == NULL the
 * expert's row range comes from offs directly instead of a scan over all groups.  Every boundary between the
 * token ranges of two experts must be a multiple of 32 (the reference requires 128, cg_backward.py:443-447): an MX
 * block along the token dim cannot be split between experts.  The kernel checks this on the device (no host sync):
 * dW[e] of an expert with a misaligned boundary is written with NaN, never with a silently wrong gradient.
 * dW of experts with no tokens is written with zeros.  `offs` must be non-decreasing: every [offs[g], offs[g+1]) is
 * taken as given (empty when it runs backwards), so ranges that overlap would credit a token to two experts.
 * Element (e, n, k) lands at
 * dw[e * dw_stride_e + n * dw_stride_n + k * dw_stride_k].
 */
int alto_mxfp4_grouped_gemm_dw(const uint8_t* go, int64_t ld_go, const uint8_t* go_scales, int64_t gs_r, int64_t gs_k, int go_is_2d,
                               const uint8_t* x, int64_t ld_xq, const uint8_t* x_scales, int64_t xs_r, int64_t xs_k, int x_is_2d,
                               const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts,
                               int64_t M_total, int64_t N, int64_t K,
                               void* dw, int dw_dtype, int64_t dw_stride_e, int64_t dw_stride_n, int64_t dw_stride_k,
                               float out_scale, void* stream);

/*
 * alto_mxfp4_grouped_gemm_dw on operands whose scales are packed along the tokens (alto_mxfp4_pack_scales with rows = N
 * resp. K and the M_total tokens as the reduction: go_packed [ceil(M_total / 512)][N][16], x_packed [...][K][16] -- what
 * alto_mxfp4_quantize_ex writes as column scales with ALTO_QUANT_PACK_COL_SCALES), bf16 dW.  Same results bit for bit.
 * A run of tokens may start anywhere the plain call allows: the kernel starts at the 256-token line that holds the run's
 * first token, i.e. at the first or second half of a packed block, and reads its scale bytes from there.  Serves the shapes
 * of the tile kernel only (M_total >= 512, N, K >= 128, unit stride along the output's last dim, ...):
 * ALTO_MXFP4_ENOTIMPL otherwise, and the caller keeps plain scales for those.
 */
int alto_mxfp4_grouped_gemm_dw_ps(const uint8_t* go, int64_t ld_go, const uint8_t* go_packed, const uint8_t* x, int64_t ld_xq, const uint8_t* x_packed,
                                  const int32_t* offs, const int32_t* group_expert, int num_groups, int num_experts,
                                  int64_t M_total, int64_t N, int64_t K, void* dw, int64_t dw_stride_e, int64_t dw_stride_n, int64_t dw_stride_k,
                                  float out_scale, void* stream);

/*
 * Fused quantize -> dequantize: y = convert_from_mxfp4(convert_to_mxfp4(x, axis=-1, is_2d_block), output_dtype = dtype
 * of x), round to nearest even, no clipping, in one pass (no codes or scales are written).  Replaces the pair of
 * launches in the weight de-oscillation hook (alto/components/optimizer.py:123-158, which calls
 * mxfp_quantization.py:410-484 then :487-545).  x, y: `batch` row-major matrices [M][C] of bf16 or f32 with row
 * strides ld_x / ld_y and matrix strides bs_x / bs_y (elements).  With 2D blocks the result does not depend on the
 * quantisation axis; a 1D quantisation along the row dim is not offered here.
 */
int alto_mxfp4_qdq(const void* x, int dtype, int64_t batch, int64_t M, int64_t C, int64_t ld_x, int64_t bs_x,
                   void* y, int64_t ld_y, int64_t bs_y, int is_2d, int use_uos, void* stream);

/*
 * MXFP4 flash-attention forward (alto/kernels/fp4/mxfp4/triton_flash_attention_mxfp4.py:425-897, launched at :1031-1080
 * with BLOCK_N = 64, layout "bhsd", no bias / alibi / dropout / varlen): per key block of 64,
 *   S = (Q K^T) * sm_scale (FP4 x FP4, 2D-block scales), causal mask aligned bottom-right, m = running row max,
 *   P = exp2((S - m) * log2(e)) quantised to MXFP4 with one E8M0 scale per (row, 32 keys), round to nearest even,
 *   l = l * alpha + rowsum(dequantised P),  O = O * alpha + P V   (alpha = exp2((m_old - m) * log2(e))),
 * out = O / l as bf16 [B][Hq][Sq][Dv], lse = m + ln(l) as f32 [B][Hq][Sq].
 * q_codes [B][Hq][Sq][D/2], q_scales [B][Hq][Sq/32][D/32]; k_codes [B][Hk][Sk][D/2], k_scales [B][Hk][Sk/32][D/32]:
 * 2D-block quantisations of Q and K along D (mxfp_quantization.py:410-484, is_2d_block=True).  V is the same 2D-block
 * quantisation of [Sk][Dv], codes handed over packed along the keys (the column codes of alto_mxfp4_quantize):
 * vt_codes [B][Hk][Dv][Sk/2], v_scales [B][Hk][Sk/32][Dv/32].  K and V scale pointers 4-byte aligned, code pointers
 * 16-byte aligned.  Hq % Hk == 0 (grouped-query heads), D in {64,128,192,256}, Dv in {64,128}, Sq % 32 == 0,
 * Sk % 64 == 0.  Only the first Sk_used keys exist (Sk_used % 32 == 0, Sk - Sk_used < 64: a sequence of 32 (mod 64) keys is
 * padded with one block of zero rows before it is quantised); causal needs Sq <= Sk_used.  All tensors dense.
 */
int alto_mxfp4_attention_fwd(const void* q_codes, const void* q_scales, const void* k_codes, const void* k_scales,
                             const void* vt_codes, const void* v_scales, void* out, float* lse, int64_t B, int64_t Hq,
                             int64_t Hk, int64_t Sq, int64_t Sk, int64_t Sk_used, int64_t D, int64_t Dv, float sm_scale,
                             int causal, void* stream);

/*
 * The same with the additive terms of triton_flash_attention_mxfp4.py:288-299 on the scaled scores, after the causal mask
 * and before the running maximum:  S += bias[b][h][m][n]  (fp32; element at b bias_sb + h bias_sh + m bias_sm + n, strides
 * in elements, 0 to broadcast over batch or heads, bias_sm % 4 == 0, 16-byte aligned; NULL: none; a bias of -inf hides a
 * key) and the ALiBi term  S -= slope[b][h] * |m + Sk_used - Sq - n|  (fp32 slope at b alibi_sb + h alibi_sh; NULL: none).
 * (The reference's kernel drops the batch offset of the bias, :630; here the strides say what is meant.)
 */
int alto_mxfp4_attention_fwd_ex(const void* q_codes, const void* q_scales, const void* k_codes, const void* k_scales,
                                const void* vt_codes, const void* v_scales, void* out, float* lse, int64_t B, int64_t Hq,
                                int64_t Hk, int64_t Sq, int64_t Sk, int64_t Sk_used, int64_t D, int64_t Dv, float sm_scale,
                                int causal, const float* bias, int64_t bias_sb, int64_t bias_sh, int64_t bias_sm,
                                const float* alibi_slopes, int64_t alibi_sb, int64_t alibi_sh, void* stream);

/*
 * Fills out[0 .. n) with random 32-bit words for stochastic rounding: word 4 c + j is word j of Philox4x32-10 (Salmon et
 * al., SC'11) with the 128-bit counter c + offset and the 64-bit key `seed`.  The reference draws its bits inside its
 * kernel from the same generator family (tl.randint4x, alto/kernels/fp4/fp4_common/triton_fp4_ops.py:15-18) with
 * tile-local offsets; here they are a tensor so that the quantizer's result can be reproduced from its inputs.
 * out 16-byte aligned.
 */
int alto_mxfp4_random_bits(uint32_t* out, int64_t n, uint64_t seed, uint64_t offset, void* stream);

/*
 * Diagnostic, no counterpart in the reference: a register-only loop of FP4 scaled-MFMA instructions
 * (8 per iteration and wave, 8 waves per workgroup, `workgroups` workgroups; 2*32*32*64 FLOP each),
 * with constant (random_operands = 0) or pseudo-random FP4 operands.  bench.py times it to report
 * the rate the matrix pipe itself sustains on this part next to the published peak.
 * `sink` is device memory for 512 floats (practically never written).  `ticks` is NULL or device memory for two uint64:
 * the shader-clock cycles and the ticks of the constant 100 MHz counter that the loop of workgroup 0 took, whose ratio is
 * the clock the chip held under this load.
 */
int alto_mxfp4_probe_mfma(int random_operands, int iters, int workgroups, float* sink, uint64_t* ticks, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* ALTO_MXFP4_H */
