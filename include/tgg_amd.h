/* C ABI of the MI355X (gfx950) grouped-GEMM library, libtgg_amd.so.
 *
 * Every entry point takes raw device pointers, plain sizes and the HIP stream to
 * enqueue on (a hipStream_t passed as void*; NULL = the default stream).  Calls
 * are asynchronous: they validate their arguments on the host, launch, and
 * return.  Return value 0 = enqueued; 1 = rejected argument; 2 = HIP runtime
 * error.  tgg_last_error() gives the message of the calling thread's last
 * failure.  No entry point allocates, frees or synchronises.
 *
 * Each declaration cites the reference interface it stands in for
 * (paths relative to the DeepLink-org/Triton_Grouped_GEMM tree).
 */
#ifndef TGG_AMD_H_
#define TGG_AMD_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element type codes */
#define TGG_BF16 0
#define TGG_F16 1
#define TGG_E4M3 2 /* OCP float8_e4m3fn */
#define TGG_E5M2 3 /* OCP float8_e5m2 */

#define TGG_MAX_GROUPS 1024      /* tgg_m_grouped_gemm, tgg_k_grouped_gemm(_queued); the quantizer's and the sort's tables */
#define TGG_MAX_GROUPS_OTHER 512 /* every other GEMM entry point (padded, placed, masked, fused FP8 output, FP8): larger
                                  * group counts are rejected with return code 1 */

/* C[r,:] = A[r,:] . B[g(r)]^T (trans_b=1, B is [G,N,K]) or A[r,:] . B[g(r)] (trans_b=0, B is [G,K,N]);
 * rows of group g are the sizes[g] rows after those of groups < g; fp32 accumulate, output in `dtype`.
 * Replaces m_grouped_gemm / _m_grouped_gemm_launch + _build_m_grouped_metadata
 * (gemm/BF16/m_grouped_gemm_TMA.py:297-447; SM80 twin gemm/BF16/m_grouped_gemm.py:220-292). */
int tgg_m_grouped_gemm(const void* A, const void* B, void* C, const void* sizes, int sizes_i64, int G, int64_t M,
                       int N, int K, int trans_b, int dtype, int num_cu, void* stream);

/* Same contraction with A/C physically padded: group g starts at sum_{h<g} round_up(sizes[h], align).
 * Replaces deep_gemm.m_grouped_bf16_gemm_nt_contiguous as called from m_grouped_bf16_nt_contiguous
 * (gemm/deep_gemm_ops.py:24-57).  Pad rows of C are not written. */
int tgg_m_grouped_gemm_padded(const void* A, const void* B, void* C, const void* sizes, int sizes_i64, int G,
                              int64_t M, int N, int K, int align, int dtype, int num_cu, void* stream);

/* As tgg_m_grouped_gemm_padded, but group g's rows are [row_start[g], row_start[g] + sizes[g]): the groups'
 * regions may lie in any order (they must not overlap; a group has one region -- a caller whose expert owns several
 * passes one group per region, with B holding that expert's weights once per region).  What a per-row grouped_layout
 * that lists experts out of ascending order describes; the reference forwards any such layout to its backend
 * (gemm/deep_gemm_ops.py:24-57). */
int tgg_m_grouped_gemm_placed(const void* A, const void* B, void* C, const void* sizes, int sizes_i64,
                              const int32_t* row_start, int G, int64_t M, int N, int K, int dtype, int num_cu,
                              void* stream);

/* For each g and r < masked_m[g]: C[g*m_stride + r,:] = A[g*m_stride + r,:] . B[g]^T (trans_b=1, B [G,N,K]) or
 * . B[g] (trans_b=0, B [G,K,N]); other rows untouched.  Replaces m_grouped_gemm_masked
 * (gemm/BF16/m_grouped_gemm_masked_TMA.py:164-250); m_stride is its expected_m. */
int tgg_m_grouped_gemm_masked(const void* A, const void* B, void* C, const void* masked_m, int masked_i64, int G,
                              int64_t m_stride, int64_t M, int N, int K, int trans_b, int dtype, int num_cu,
                              void* stream);

/* C[g] = A[start[g]:end[g], :]^T . B[start[g]:end[g], :], A [Ktot,Mdim], B [Ktot,N], C [G,Mdim,N];
 * empty segments give zeros.  Replaces k_grouped_gemm (gemm/BF16/k_grouped_gemm_TMA.py:217-294;
 * SM80 twin gemm/BF16/k_grouped_gemm.py:142-216). */
int tgg_k_grouped_gemm(const void* A, const void* B, void* C, const int32_t* start, const int32_t* end, int G,
                       int Mdim, int N, int64_t Ktot, int dtype, int num_cu, void* stream);

/* tgg_k_grouped_gemm with a work queue (same reference function, gemm/BF16/k_grouped_gemm_TMA.py:217-294).  A
 * K-grouped tile costs what its group has tokens, so with ragged groups no fixed assignment of tiles to the
 * persistent workgroups is even.  `queue` points to TGG_QUEUE_WORDS int32 in device memory that are ZERO when the
 * kernel starts; the workgroups draw their tile ids from them (one counter per XCD), largest groups first, and a
 * workgroup that drew expensive tiles draws fewer.  Results are bit-identical to tgg_k_grouped_gemm.  The kernel
 * leaves the words ZERO again (the workgroup that finishes last clears them), so a caller clears them once, when it
 * allocates them, and may pass the same words to launch after launch on one stream -- also inside a captured graph,
 * with no fill node.  A launch must have the words to itself until it has finished (one queue per stream).
 * queue = NULL: the fixed assignment. */
#define TGG_QUEUE_WORDS 16 /* eight counters, the count of finished workgroups, seven spare */
int tgg_k_grouped_gemm_queued(const void* A, const void* B, void* C, const int32_t* start, const int32_t* end, int G,
                              int Mdim, int N, int64_t Ktot, int dtype, int num_cu, int32_t* queue, void* stream);

/* C = (Aq . Bq[g]^T) * a_scale[r] * b_scale[g*N+n].  Replaces gmm_fp8_act_per_channel_w_per_expert
 * (gemm/FP8/m_grouped_gemm_channel_expert.py:139-198). */
int tgg_m_grouped_gemm_fp8_channel(const void* Aq, const float* a_scale, const void* Bq, const float* b_scale,
                                   void* C, const void* sizes, int sizes_i64, int G, int64_t M, int N, int K,
                                   int fmt_a, int fmt_b, int out_dtype, int num_cu, void* stream);

/* out[g] = (x[:,seg_g] . y[:,seg_g]^T) * xs[g*M+m] * ys[g*N+n], x [M,Ktot], y [N,Ktot], segments =
 * prefix sums of tokens[g]; bf16 output [G,M,N].  Any token counts (the reference wants them padded to 128 with
 * zero data; here a segment ends where its count says); Ktot must be a multiple of 16.  Replaces matmul
 * (gemm/FP8/k_grouped_gemm_channel_expert.py:143-181). */
int tgg_k_grouped_gemm_fp8_channel(const void* x, const float* xs, const void* y, const float* ys, void* out,
                                   const int32_t* tokens, int G, int M, int N, int64_t Ktot, int fmt_a, int fmt_b,
                                   int num_cu, void* stream);

/* tgg_k_grouped_gemm_fp8_channel with a work queue (same reference function,
 * gemm/FP8/k_grouped_gemm_channel_expert.py:143-181); `queue` as in tgg_k_grouped_gemm_queued (zero before, zero
 * after).  Only the tuned kernel (token counts that are all multiples of 16) draws from it; the shape-agnostic
 * kernel leaves it untouched. */
int tgg_k_grouped_gemm_fp8_channel_queued(const void* x, const float* xs, const void* y, const float* ys, void* out,
                                          const int32_t* tokens, int G, int M, int N, int64_t Ktot, int fmt_a,
                                          int fmt_b, int num_cu, int32_t* queue, void* stream);

/* out[r,n] = sum_kb (sum_{k in kb} Aq[r,k] Bq[g,n,k]) * sa[r,kb] * sb[g,n/128,kb]; e4m3fn codes, A physically
 * padded per group to `align` rows, sb [G,ceil(N/128),ceil(K/128)], bf16 output.  sa holds M x ceil(K/128)
 * floats, row-major [M,KB] (sa_mn_major=0) or KB-major [KB,M] (sa_mn_major=1, the layout the tuned kernel
 * streams).  Replaces deep_gemm.m_grouped_fp8_gemm_nt_contiguous as called from m_grouped_fp8_nt_contiguous
 * (gemm/deep_gemm_ops.py:60-100). */
int tgg_m_grouped_gemm_fp8_block(const void* Aq, const float* sa, const void* Bq, const float* sb, void* C,
                                 const void* sizes, int sizes_i64, int G, int64_t M, int N, int K, int align,
                                 int sa_mn_major, int num_cu, void* stream);

/* As tgg_m_grouped_gemm_fp8_block with group g's rows at [row_start[g], row_start[g] + sizes[g]), regions in any
 * order (gemm/deep_gemm_ops.py:60-100 forwards any per-row layout). */
int tgg_m_grouped_gemm_fp8_block_placed(const void* Aq, const float* sa, const void* Bq, const float* sb, void* C,
                                        const void* sizes, int sizes_i64, const int32_t* row_start, int G, int64_t M,
                                        int N, int K, int sa_mn_major, int num_cu, void* stream);

/* bf16 x [M,N] -> codes [N,M_expand] (transposed, each group padded to 128 columns, zero tail) and
 * scales [N/128, M_expand/128].  Replaces trans_per_block_quant_expand_128x
 * (quant/trans_per_block_quant_expand_128x.py:135-208). */
int tgg_trans_per_block_quant_expand_128x(const void* x, void* codes, float* scales, const void* sizes,
                                          int sizes_i64, int G, int64_t M, int N, int64_t M_expand, int fmt,
                                          void* stream);

/* bf16 x [M,K] -> codes [M,K], scales [M,K/128] (scales_mn_major=0) or stored transposed [K/128,M]
 * (scales_mn_major=1); 1x128 recipe.  Replaces per_token_cast_to_fp8
 * (gemm/FP8/m_grouped_gemm_channel_expert.py:217-222). */
int tgg_per_token_cast_to_fp8(const void* x, void* codes, float* scales, int64_t M, int K, int fmt,
                              int scales_mn_major, void* stream);

/* bf16 x [batch,R,C] -> codes (same shape), scales [batch,ceil(R/128),ceil(C/128)]; 128x128 recipe.
 * Replaces per_block_cast_to_fp8 (gemm/FP8/m_grouped_gemm_channel_expert.py:237-245). */
int tgg_per_block_cast_to_fp8(const void* x, void* codes, float* scales, int batch, int R, int C, int fmt,
                              void* stream);

/* Element-wise fp32 -> fp8 code with the conversion the quantizers use (test hook for the
 * `.to(torch.float8_*)` casts of the recipes above). */
int tgg_cvt_f32_to_fp8(const float* in, void* out, int64_t n, int fmt, void* stream);

/* M-grouped GEMM whose output leaves as FP8 codes with one fp32 scale per row and 128 columns (the 1x128 activation
 * recipe), bit-identical to tgg_m_grouped_gemm followed by tgg_per_token_cast_to_fp8 on its 16-bit result but without
 * the round trip through memory.  codes [M, N] fp8 (fmt 2 = e4m3fn, 3 = e5m2); scales [M, N/128] fp32, or stored
 * [N/128, M] when scales_mn_major (what the block-scaled GEMM consumes).  N must be a multiple of 128.  Returns 1 with
 * a message for shapes the fused kernel does not take (more than 512 groups, very long rows); the two separate calls
 * give the same result.  No counterpart in the reference's Python API: it fuses m_grouped_gemm
 * (gemm/BF16/m_grouped_gemm_TMA.py:435) with per_token_cast_to_fp8 (gemm/FP8/m_grouped_gemm_channel_expert.py:217-222),
 * the step between the two expert GEMMs of an FP8 MoE layer. */
int tgg_m_grouped_gemm_fp8_out(const void* A, const void* B, void* codes, float* scales, const void* sizes,
                               int sizes_i64, int G, int64_t M, int N, int K, int trans_b, int dtype, int fmt,
                               int scales_mn_major, int num_cu, void* stream);

/* ---- MoE token permute / unpermute: the steps either side of the grouped GEMMs -----------------------------------
 * Replace moe_permute_topK_op / moe_recover_topK_op / moe_recover_topK_bwd_op of the reference's baseline extension
 * (grouped_gemm/csrc/permute.cu:504-690, kernels :40-297; Python side grouped_gemm/grouped_gemm/ops.py:52-257).
 * dtype codes: 0 bf16, 1 fp16, 2 e4m3fn, 3 e5m2 (row copy only), 4 fp32.  Rows must be multiples of 16 bytes.
 *
 * tgg_moe_permute_map: stable sort of the flattened [num_tokens, topk] expert assignment (expert ids in
 *   [0, num_experts), num_experts <= 1024; an id of -1 marks a dropped assignment).
 *   row_id_map[k * num_tokens + t] = destination row of assignment (t, k) in expert-major order, ties in flat order
 *   (what cub::DeviceRadixSort::SortPairs + moe_permute_topK_row_map produce, permute.cu:40-101, :541-548), or -1 when
 *   dropped or when the destination is >= num_out_tokens (0 = keep all).  tokens_per_expert (optional, int32 or int64
 *   [num_experts]) receives the per-expert row counts, i.e. the size_per_group argument of the grouped GEMMs.
 *   workspace: device memory of at least tgg_moe_sort_workspace_bytes(...) bytes, contents irrelevant before and after.
 * tgg_moe_permute_rows: permuted[row_id_map[k, t], :] = input[t, :] for every kept assignment.
 * tgg_moe_unpermute: output[t, :] = sum_k probs[t, k] * input[row_id_map[k, t], :] over kept assignments, fp32
 *   arithmetic, one rounding to the activation type (probs may be null: plain sum; also the backward of permute_rows).
 * tgg_moe_unpermute_bwd: act_grad[row_id_map[k, t], :] = probs[t, k] * grad_output[t, :];
 *   prob_grad[t, k] = <grad_output[t, :], fwd_input[row_id_map[k, t], :]> (0 for dropped); prob_grad may be null. */
int tgg_moe_sort_workspace_bytes(int64_t num_tokens, int topk, int num_experts, int64_t* bytes);
int tgg_moe_permute_map(const int32_t* indices, int64_t num_tokens, int topk, int num_experts, int64_t num_out_tokens,
                        int32_t* row_id_map, void* tokens_per_expert, int counts_i64, void* workspace,
                        int64_t workspace_bytes, void* stream);
/* tgg_moe_permute_map without the workspace argument, for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The
 * sort's temporaries live in a fixed 8 MiB + 8 KiB array inside the library's device code (one copy per GPU, held
 * until the process ends); the call allocates and frees nothing.  Same results as tgg_moe_permute_map.  Limit:
 * num_tokens * topk <= 1048576 (2^20) assignments, num_experts <= 1024; larger problems are rejected with return
 * code 1 and a message.  All calls on one GPU share the array: calls that overlap on one GPU (different streams, or
 * different threads) race; calls on one stream are ordered and safe. */
int tgg_moe_permute_map_static(const int32_t* indices, int64_t num_tokens, int topk, int num_experts,
                               int64_t num_out_tokens, int32_t* row_id_map, void* tokens_per_expert, int counts_i64,
                               void* stream);
int tgg_moe_permute_rows(const void* input, void* permuted, const int32_t* row_id_map, int64_t num_tokens, int topk,
                         int hidden, int dtype, void* stream);
int tgg_moe_unpermute(const void* input, void* output, const int32_t* row_id_map, const float* probs,
                      int64_t num_tokens, int topk, int hidden, int dtype, void* stream);
int tgg_moe_unpermute_bwd(const void* grad_output, const void* fwd_input, const int32_t* row_id_map, const float* probs,
                          void* act_grad, float* prob_grad, int64_t num_tokens, int topk, int hidden, int dtype,
                          void* stream);

/* Test hook, runs entirely on the host (no GPU needed): the order in which `grid` persistent workgroups walk
 * the output tiles of a launch, computed by the same scheduler functions the kernels execute.  It restates
 * what the reference's grouped_launch / m_indices_pad tile enumeration guarantees
 * (gemm/BF16/m_grouped_gemm_TMA.py:55-71, :297-326): every tile of the padded tile space exactly once.
 *   sizes  host array [G]; mode 0 M-grouped, 1 rows padded to `aux`, 2 masked with `aux` rows per group,
 *          4 K-grouped by token counts (`aux` = total tokens, m_total = rows of each output; the tile space lists
 *          the groups by decreasing token count, and what is reported is the fixed walk, not a queued launch's draws)
 *   tile   256 (tuned kernels) or 128 (shape-agnostic kernel); split as in the "tile_split" option
 *   out    [capacity][6] = workgroup, position in its walk, group, first row, valid rows, first column */
int tgg_debug_tile_order(const int64_t* sizes, int G, int mode, int64_t m_total, int64_t aux, int N, int tile,
                         int grid, int split, int64_t* out, int64_t capacity, int64_t* num_tiles);

/* Test hook, host only: the group table's row-tile lookup that the transposing quantizer and the GEMM schedulers share.
 * Row tile i (counted over the groups' ceil(size / tile) tiles in group order, as m_indices_pad does,
 * gemm/BF16/m_grouped_gemm_TMA.py:297-326; the quantizer's token_start / pad_start arithmetic,
 * quant/trans_per_block_quant_expand_128x.py:91-110) -> out[i] = {group, first row in A, valid rows}.
 * modes as in tgg_debug_tile_order (0, 1, 2); n_chunk is the tile-order option, which must not change the answer. */
int tgg_debug_row_tiles(const int64_t* sizes, int G, int mode, int64_t m_total, int64_t aux, int tile, int n_chunk,
                        int64_t* out, int64_t capacity, int64_t* num_row_tiles);

/* Test hook, host only: which elements of each operand the shape-agnostic kernel would touch for a launch of the
 * given entry point, found by walking every tile with the kernel's own scheduler and address arithmetic.  It guards
 * what the reference gets from Triton's masked loads and TMA bounds (e.g. gemm/BF16/m_grouped_gemm.py:83-116,
 * gemm/FP8/m_grouped_gemm_channel_expert.py:119-136): no access outside the tensors, whatever the group count.
 *   kind  0 / 1 tgg_m_grouped_gemm with trans_b = 1 / 0; 2 masked (aux = m_stride); 3 padded (aux = align);
 *         4 placed (row_start); 5 tgg_k_grouped_gemm (sizes = token counts, M = Mdim, aux = Ktot);
 *         6 FP8 per-channel M-grouped; 7 FP8 per-channel K-grouped (M = rows of x, aux = Ktot);
 *         8 / 9 FP8 block-scaled with sa stored [M, KB] / [KB, M] (aux = align); 10 the same, placed (row_start)
 *   out   [7][2] = lowest and highest element index touched in A, B, C, scale_m, scale_n, sa, sb
 *         ({INT64_MAX, -1} for an operand that is never touched) */
int tgg_debug_generic_extents(int kind, const int64_t* sizes, const int32_t* row_start, int G, int64_t M, int64_t aux,
                              int N, int K, int64_t* out);

/* Test hook, host only: the deal of the K-grouped kernels' work queue.  out[xq][n] (row-major, [8][draws]) = the tile
 * id behind the n-th draw from XCD xq's counter on a grid of `grid` workgroups (a multiple of 8; other grids use
 * one counter whose draws are the ids themselves).  The reference has no counterpart (its K-grouped kernels walk
 * tiles at a fixed stride, gemm/BF16/k_grouped_gemm_TMA.py:124-135); what must hold is that the eight sequences
 * together list every id once and each of them in growing order. */
int tgg_debug_queue_order(int grid, int draws, int32_t* out);

/* Library controls (process-wide test and tuning hooks, not a per-call interface: every launch reads each option
 * once, atomically, so a thread that changes one while another thread launches decides only which value that launch
 * sees; returns 1 for an unknown key):
 *   "force_generic" 0/1  route every GEMM through the shape-agnostic kernel
 *   "variant"       int  tile configuration of the tuned kernels (16-bit, and FP8 M-grouped): 0 (default) = chosen per launch on the
 *                        device from the group sizes -- 256x128 when all such tiles fit one round of the persistent
 *                        workgroups; otherwise, for 16-bit M-grouped / masked and FP8 M-grouped launches, the
 *                        weight-streaming configuration (128x256 tiles, three weight slab buffers) when its rounds of
 *                        the persistent workgroups, at 0.7 of a 256-row tile's cost each, are no more than those of
 *                        the 256x256 tiles (groups of up to about 200 rows on average); 256x256 otherwise; 1 = always 256x128; 2 = always 256x256; 4 = always the weight-streaming
 *                        configuration (16-bit NT / NN, FP8 M-grouped)
 *   "four_wave"     int  16-bit M-grouped / masked NT (or NN with N a multiple of 256), K a multiple of 128 (at least 256): 1 (default) = the four-wave
 *                        kernel (128x128 per wave) on large launches (more than four rounds of 256x128 tiles; masked
 *                        launches and M-grouped ones with fewer than 512 rows per group on average enqueue both
 *                        kernels, which decide on the device from the sizes which of them runs), 0 = eight-wave
 *                        kernels only, 2 = the four-wave kernel on every launch it can take, whatever the sizes
 *   "tile_split"    0/1  M-grouped tuned kernels: per-XCD contiguous tile ranges (default 1) or interleaved sweeps
 *   "n_chunk"       int  column tiles per chunk of the tile order (0 = automatic, at most eight)
 *   "store_nt"      0/1  write the output with non-temporal stores (default 1)
 *   "kg_second_launch" 0/1  tgg_k_grouped_gemm_fp8_channel enqueues the tuned kernel and the shape-agnostic kernel, and
 *                        each decides on the device from the token counts whether it runs (tuned: all counts multiples
 *                        of 16); 0 leaves the second one out, so a test can see what the tuned kernel does alone */
int tgg_set_option(const char* key, int value);
const char* tgg_last_error(void);
int tgg_version(void);

#ifdef __cplusplus
}
#endif
#endif /* TGG_AMD_H_ */
