/* C-ABI of libmortar_hip.so: the MI355X (gfx950) implementation of the MORTAR sparse-MLP path.
 *
 * Every entry point takes plain pointers and sizes.  Device pointers are raw HIP device
 * addresses, `stream` is a hipStream_t passed as void* (NULL = the null stream).  All entry
 * points return 0 on success and a negative code on failure; mortar_last_error() returns the
 * message of the calling thread's last failure.  Nothing here allocates device memory: the
 * caller owns inputs, outputs and the workspaces named below.
 *
 * Reference interfaces replaced (paths relative to the reference checkout):
 *   stk_dds(lhs, data, offsets, row_indices, column_indices, ..., shape0, shape1, True)
 *       morph/sparse/stk/backend/custom_ops.py:35-56 (forward use block_sparse.py:956-965).  Restriction: the
 *       reference multiplies whatever bf16 values `data` holds; this runtime multiplies TERNARY blocks only
 *       (every value of block j is 0 or +-s_j).  Other data is reported as an error (mortar_requantize,
 *       ternary_tol), never multiplied approximately.
 *   _SwiGLUMortar.forward                      morph/model/transformer.py:402-431
 *   TileRouter.forward steps 5-8               morph/model/routing.py:232-284
 *   route_flags                                morph/kernels/triton/fused_decode_step.py:1913-1927
 *   mortar_pack_strips / mortar_gemv           morph/kernels/triton/fused_decode_step.py:1465-1547
 *   rmsnorm_rows / attention.RMSNorm           fused_decode_step.py:305-321, morph/model/attention.py:133-141
 *   pack_mortar_ternary                        morph/inference/deploy_quant.py:344-374
 */
#ifndef MORTAR_HIP_H
#define MORTAR_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MORTAR_BLK 16            /* carved block edge (carve(blocking=16)) */

enum {
    MORTAR_OK = 0,
    MORTAR_ERR_ARG = -1,       /* bad argument / shape / alignment */
    MORTAR_ERR_SCALE = -2,     /* scale outside the representable window */
    MORTAR_ERR_HIP = -3,       /* HIP runtime error (message has hipGetErrorString) */
    MORTAR_ERR_LIMIT = -4      /* size beyond a stated maximum */
};

/* One carved matrix W [Rb*16, Cb*16] in device memory.
 *   codes   [nnz*16] uint32: block j, output row n -> one dword holding its 16 ternary codes in the
 *           device bit layout produced by mortar_encode_blocks_host
 *   sdup    [nnz] uint32: per-block scale pattern produced by mortar_encode_blocks_host
 *   col     [nnz] the reference's mortar_column_indices (int16, unchanged)
 *   row_ptr [Rb+1] the reference's mortar_offsets (int32, unchanged)
 * Octet stream (the copy every SpMM kernel reads, prefill and decode; from mortar_octet_layout_host): the block-columns are cut
 * into nseg = ceil(Cb / seg_cb) K segments, and every (segment, row) run of blocks into groups of 8 blocks
 * (the last one padded with all-zero blocks) so that one 16-byte load per lane fetches the lane's code dwords
 * of four consecutive block pairs:
 *   row_desc [nseg*Rb*4] int32 per (segment, row): {first group, end group, number of blocks, 0}
 *   col_o holds block-columns relative to the segment start
 *   codes_o [ngroups*2*16*4] uint32: ((group*2 + s)*16 + n)*4 + t = row n of block 8*g + 2*t + s of the row
 *   sd_o    [ngroups*2*4] uint32 and col_o [ngroups*2*4] int32: (group*2 + s)*4 + t, same block
 * Optional 4-bit copy of the code stream for prefill-sized launches (M > 64), from mortar_fp4_stream_host; NULL =
 * prefill unpacks the 2-bit stream.  Same octets, every ternary code as the FP4 (E2M1) nibble the unpack feeds the
 * hardware conversion with (0 -> 0x0, +1 -> 0x4, -1 -> 0xC), which saves the shift and mask of the 2-bit unpack:
 *   codes4_o [ngroups*4*16*4] uint32: ((group*4 + 2*s + h)*16 + n)*4 + t = columns 8h .. 8h+7 of row n of block
 *            8*g + 2*t + s, column 8h + q in bits [4q, 4q+3]
 * Decode-sized launches always read the 2-bit stream (half the bytes).                                          */
typedef struct {
    const uint32_t *codes;
    const uint32_t *sdup;
    const int16_t *col;
    const int32_t *row_ptr;
    const int32_t *row_desc;
    const uint32_t *codes_o;
    const uint32_t *sd_o;
    const int32_t *col_o;
    const uint32_t *codes4_o;
    int32_t Rb, Cb, nnz;
    int32_t seg_cb;   /* block-columns per K segment of the octet stream (>= Cb: one segment) */
    float uniform_scale;   /* != 0: every block has this (bf16-representable) scale, the reference's per-tensor
                              mortar_scale (deploy_quant.py:344-374); from mortar_uniform_scale_host.  The kernels then
                              multiply +-2 / 0 blocks and scale the fp32 sums once, as the reference's decode kernel
                              does (fused_decode_step.py:1441-1443), instead of scaling every block's weights.
                              0: per-block scales (always valid, also for a uniform matrix). */
    int32_t reserved_;
} mortar_bcsr_t;

const char *mortar_last_error(void);
int mortar_abi_version(void);

/* ---- host-side packing (no GPU needed) ------------------------------------------------------- */

/* Re-encode the reference's flat 2-bit pack (pack_ternary_codes: 4 codes/byte, u=code+1, row-major over
 * [nnz,16,16]; deploy_quant.py:56-71) into the device layout, and turn fp32 scales (scale_count = 1 for
 * the reference's per-tensor scale, or nnz for per-block scales) into the per-block pattern.
 * packed: host [nnz*64] bytes; codes_out host [nnz*16] uint32; sdup_out host [nnz] uint32.
 * Fails with MORTAR_ERR_SCALE when bf16(scale) is non-finite or its magnitude is outside [2^-100, 2^100]
 * (0 is allowed and zeroes the block). */
int mortar_encode_blocks_host(const uint8_t *packed, int64_t nnz, const float *scale, int64_t scale_count,
                              uint32_t *codes_out, uint32_t *sdup_out);

/* The scale shared by all blocks, from the sdup patterns of mortar_encode_blocks_host: *scale_out = that bf16 value
 * as float, or 0 if the blocks differ (or the scale is 0).  Put it into mortar_bcsr_t.uniform_scale. */
int mortar_uniform_scale_host(const uint32_t *sdup, int64_t nnz, float *scale_out);

/* Inverse of the code part (for tests): device-layout dwords -> int8 codes [nnz,16,16]. */
int mortar_decode_blocks_host(const uint32_t *codes, int64_t nnz, int8_t *codes_out);

/* Validates a BCSR (offsets start at 0 and never decrease, columns in range and strictly ascending in a row). */
int mortar_validate_bcsr_host(const int32_t *row_ptr, const int16_t *col, int32_t Rb, int32_t Cb);

/* Octet stream of one matrix (see mortar_bcsr_t).  row_desc_out host [Rb*4] is always written; the return
 * value is the number of groups.  With codes_o_out == NULL only row_desc_out is filled (size query);
 * otherwise codes_o_out [ngroups*128], sd_o_out [ngroups*8], col_o_out [ngroups*8] are filled from the
 * encoded codes / sdup and the column indices. */
int64_t mortar_octet_layout_host(const int32_t *row_ptr, int32_t Rb, int32_t Cb, int32_t seg_cb,
                                 const uint32_t *codes, const uint32_t *sdup, const int16_t *col,
                                 int32_t *row_desc_out, uint32_t *codes_o_out, uint32_t *sd_o_out,
                                 int32_t *col_o_out);

/* 4-bit copy of an octet code stream: codes_o host [ngroups*128] (from mortar_octet_layout_host) ->
 * codes4_o_out host [ngroups*256], layout as described at mortar_bcsr_t.  No counterpart in the reference. */
int mortar_fp4_stream_host(const uint32_t *codes_o, int64_t ngroups, uint32_t *codes4_o_out);

/* Position of every block in the octet streams (the index the device-side re-pack scatters to):
 * pos_out host [nnz], pos_out[j] = (group*2 + s)*4 + t of block j, for the same seg_cb as mortar_octet_layout_host. */
int mortar_octet_positions_host(const int32_t *row_ptr, int32_t Rb, int32_t Cb, int32_t seg_cb, const int16_t *col,
                                int32_t *pos_out);

/* Topology of W^T (reference: stk matrix.py:107-125 `_transpose`, which yields mortar_offsets_t,
 * mortar_column_indices_t and mortar_block_offsets_t): offsets_t_out host [Cb+1], col_t_out host [nnz] = block-row
 * of each block in transposed order, src_block_out host [nnz] = its index in the original order.  Blocks of one
 * column keep ascending row order (the reference leaves that order to the sort backend).  A pack built over
 * (offsets_t, col_t) and filled by mortar_requantize(..., src_block, transpose = 1) multiplies by W^T: the dX
 * product stk_dds(..., transpose_b=False) (custom_ops.py:35-56). */
int mortar_transpose_topology_host(const int32_t *row_ptr, const int16_t *col, int32_t Rb, int32_t Cb,
                                   int32_t *offsets_t_out, int16_t *col_t_out, int32_t *src_block_out);

/* Largest K segment (in block-columns) whose 32-token activation tile fits in LDS; a matrix with
 * Cb <= this runs the single-segment prefill kernel.  Use seg_cb = ceil(Cb / ceil(Cb / max)). */
int mortar_prefill_max_seg_cb(void);

/* Largest K segment whose 4-token (rows <= 4) or 16-token (rows <= 16) tile fits in LDS.  A second stream of a matrix laid
 * out with segments that wide (same codes; fewer, longer row parts, so less padding to octets and fewer barrier pairs:
 * one segment instead of three for a `down` of 5632 inputs at up to 4 rows, two at up to 16) serves calls of up to that
 * many rows only: the layer-batched decode launches run 9 % faster on it.  Calls with more rows on such a stream are
 * refused.  No counterpart in the reference. */
int mortar_decode_max_seg_cb(int32_t rows);

/* Row-unit order for uneven nnz: units sorted by descending block count and dealt into groups of `group`
 * consecutive positions with similar totals (longest-processing-time first); use group = 16, the number of
 * wavefronts of a prefill workgroup.  rows_per_unit = 1 (plain) or 2 (gate row u and up row u + Rb/2).
 * Every group lists its units heaviest first; with snake != 0 the odd groups are reversed.  Use snake = 1 for
 * matrices with several K segments (their prefill kernel gives wave w the positions w, w + group, ... of its window:
 * without the reversal wave 0 would collect the heaviest unit of every group) and snake = 0 for single-segment
 * matrices, whose kernels let the waves of a workgroup draw positions one after another (the last draws of a window
 * should be its lightest units).
 * order_out host [n_units]: the unit at each schedule position.  Uniform rows keep the natural order. */
int mortar_unit_order_host(const int32_t *row_ptr, int32_t Rb, int32_t rows_per_unit, int32_t group, int32_t snake,
                           int32_t *order_out);

/* Second pass over a unit order for matrices with several K segments (nseg > 1).  The K-segmented prefill
 * kernel ends every segment with a workgroup barrier, so a workgroup waits in each segment for the wave whose
 * units hold the most blocks IN THAT SEGMENT.  Within every window of waves * units_per_wave consecutive
 * positions (one workgroup; wave w owns positions w, w + waves, ...) the units are dealt again so that the sum
 * over the segments of the heaviest wave is small (greedy by heaviest segment, then pairwise exchanges).  Which
 * units a window holds does not change.  The prefill kernels run waves = 16 with units_per_wave = 4 for plain
 * units and 2 for gate/up units.  row_desc: host [nseg*Rb*4] from mortar_octet_layout_host.  order: host
 * [n_units], in and out (start from mortar_unit_order_host).  A no-op for nseg == 1 or units_per_wave == 1.
 * No counterpart in the reference, whose Triton grid has one program per output tile. */
int mortar_unit_order_segments_host(const int32_t *row_desc, int32_t Rb, int32_t nseg, int32_t rows_per_unit,
                                    int32_t waves, int32_t units_per_wave, int32_t *order);

/* Part descriptors in schedule order, the form the kernels walk: for position pos, K segment sg and row a of
 * the unit, sched_out[((pos*nseg + sg)*rows_per_unit + a)*4 ..] = {first octet, end octet, blocks, unit}, taken
 * from row_desc (mortar_octet_layout_host) of row unit + a*n_units.  order: host [n_units] from
 * mortar_unit_order_host, or NULL for the natural order.  sched_out host [n_units*nseg*rows_per_unit*4]. */
int mortar_schedule_host(const int32_t *row_desc, int32_t Rb, int32_t nseg, int32_t rows_per_unit,
                         const int32_t *order, int32_t *sched_out);

/* Decode work list.  Splits every row unit into entries of <= max_blocks blocks inside one K segment of
 * kseg block-columns.  Each entry is 8 int32: {rowA, pA, cntA, rowB, pB, cntB, slot, seg}; rowB = -1 for
 * plain units.  Call with entries_out = NULL to get the entry count (return value >= 0), then again with
 * a buffer.  nslots_out = max partial slots per row; row_slots_out host [Rb] = slots of each row (optional).
 * Entries are grouped by segment and padded with null entries (rowA = -1) to a multiple of 4 per segment,
 * because one workgroup serves 4 consecutive entries of one segment. */
int64_t mortar_decode_worklist_host(const int32_t *row_ptr, const int16_t *col, int32_t Rb, int32_t Cb,
                                    int32_t rows_per_unit, int32_t kseg, int32_t max_blocks,
                                    int32_t *entries_out, int32_t *nslots_out, int32_t *row_slots_out);

/* ---- SpMM on bf16 MFMA, fp32 accumulate (any M) -------------------------------------------------- */

/* y[M, Rb*16] = x[M, Cb*16] @ W^T (bf16 in, bf16 out).  Replaces stk_dds(..., transpose_b=True)
 * (morph/sparse/stk/backend/custom_ops.py:35-56).
 * sched: device copy of mortar_schedule_host(rows_per_unit = 1), or NULL for the natural row order.
 * ldx / ldy in elements; x and y 16-byte aligned, ldx % 8 == 0, ldy % 4 == 0. */
int mortar_spmm_bf16(const mortar_bcsr_t *W, const int32_t *sched, const uint16_t *x, int64_t M, int64_t ldx,
                     uint16_t *y, int64_t ldy, void *stream);

/* h[M, d_ff] = silu(gate) * up [* gates per cluster], gate_up = W [2*d_ff, d_model] with gate rows
 * [0, d_ff) and up rows [d_ff, 2*d_ff) (transformer.py:335-336,403-405).  Intermediates are rounded to
 * bf16 where the reference materialises a bf16 tensor.  gates: device fp32 [M, n_clusters] or NULL;
 * d_ff % n_clusters == 0.  sched: mortar_schedule_host(rows_per_unit = 2) or NULL.
 * Routed skipping (optional): tok_cnt/tok_list from mortar_remoe_route with tile = mortar_route_tile(Cb, M); when
 * given (requires cluster_size % 16 == 0 and mortar_route_tile != 0) only active (token, block-row) tiles are
 * computed and written; inactive entries of h are left untouched and must be masked by the consumer
 * (mortar_spmm_bf16_masked).  Without the lists, calls of M <= 64 rows with gates and cluster_size % 16 == 0 still
 * leave out every unit whose cluster has no positive gate among the tokens of its 4- or 16-token tile, and write
 * zeros for it (the value the gates produce), so h is fully written. */
int mortar_gateup_swiglu_bf16(const mortar_bcsr_t *W, const int32_t *sched, const uint16_t *x, int64_t M,
                              int64_t ldx, uint16_t *h, int64_t ldh, const float *gates, int32_t n_clusters,
                              const int32_t *tok_cnt, const uint8_t *tok_list, void *stream);

/* As mortar_spmm_bf16, but input element (m, c) is read as 0 when active[m, c / cluster_size] == 0
 * (active: device uint8 [M, n_clusters]); used for `down` after a routed mortar_gateup_swiglu_bf16. */
int mortar_spmm_bf16_masked(const mortar_bcsr_t *W, const int32_t *sched, const uint16_t *x, int64_t M,
                            int64_t ldx, uint16_t *y, int64_t ldy, const uint8_t *active, int32_t n_clusters,
                            void *stream);

/* `down` with the hyper-connection POST write fused into its epilogue, for decode batches (M <= 64): the MLP output
 * y = x W^T never goes to memory.  Reference: engine._hc calls the MLP and then _hc_post_fwd_kernel
 * (morph/inference/engine.py:996-1001, 1052-1060; morph/kernels/triton/fused_hyper_connection.py:927-970; wide carriers
 * hc_post_wide, morph/kernels/triton/fused_decode_step.py:1725-1739):
 *   out[t, i, :] = sum_j hres[t, i, j] * carrier[t, j, :] + hpost[t, i] * y[t, :] (+ term[t, :])
 * fp32 arithmetic in that order; y enters rounded to bf16 (what mortar_spmm_bf16 would have stored).
 *   carrier, out  [M, n_streams, Rb*16] contiguous, bf16 (carrier_f32 = 0; 8-byte aligned) or fp32 (1; 16-byte aligned);
 *                 1 <= n_streams <= 4;  hres fp32 [M, n, n], hpost fp32 [M, n];  term [M, Rb*16] of the carrier's type or NULL
 *   active / n_clusters  as mortar_spmm_bf16_masked (NULL: no input mask)
 * MORTAR_ERR_LIMIT for M > 64: prefill-sized calls store y (mortar_spmm_bf16) and combine in a second pass. */
int mortar_spmm_hc_post(const mortar_bcsr_t *W, const int32_t *sched, const uint16_t *x, int64_t M, int64_t ldx,
                        const void *carrier, int32_t carrier_f32, int32_t n_streams, const float *hres,
                        const float *hpost, const void *term, void *out, const uint8_t *active, int32_t n_clusters,
                        void *stream);

/* Token tile of routed mortar_gateup_swiglu_bf16 for M rows against a matrix with Cb block-columns: the tile
 * size mortar_remoe_route must be called with.  4 for M <= 4, 16 for M <= 64, otherwise 32 or 64
 * depending on Cb; 0 when in_features is too wide for routed skipping (one LDS tile must hold a row of x). */
int mortar_route_tile(int32_t Cb, int64_t M);

/* ---- ReMoE gating --------------------------------------------------------------------------- */

/* TileRouter steps 5-8: kth = k-th largest logit per token; g0 = relu(logit - kth) (threshold only when
 * k < n); gates = g0 * (k / max(sum g0, 1e-6)); active = gates > 0.  logits/gates fp32 [M, n], active uint8
 * [M, n] (may be NULL).  n <= 1024. */
int mortar_remoe_gates(const float *logits, int64_t M, int32_t n, int32_t k, float *gates, uint8_t *active,
                       void *stream);

/* Wavefront-ballot compaction of active tokens per (token tile, cluster):
 * tok_cnt[t*n + c] = number of tokens of tile t (tile tokens each: 4 or a multiple of 16, <= 256) with active[m, c] != 0,
 * tok_list[(t*n + c)*tile + i] = tile-local index of the i-th such token, ascending. */
int mortar_remoe_route(const uint8_t *active, int64_t M, int32_t n, int32_t tile, int32_t *tok_cnt,
                       uint8_t *tok_list, void *stream);

/* route_flags: row_act[b, r] (int32 [B, 2*d_ff/16], gate half then up half) and col_act[b, c]
 * (int32 [B, d_ff/16]) = gate[b, lo] > 0 or gate[b, hi] > 0 with lo = (r*16)/cls, hi = (r*16+15)/cls.
 * ld* = row strides in elements. */
int mortar_route_flags(const float *gates, int64_t B, int32_t n_clusters, int64_t ldg, int32_t d_ff,
                       int32_t *row_act, int64_t ldr, int32_t *col_act, int64_t ldc, void *stream);

/* Decode-side router front end + gating tail in two launches, for 1..64 tokens: TileRouter.forward steps 1-8
 * (morph/model/routing.py:181-284); the reference's fused form is morph/kernels/triton/fused_router.py:43-140
 * (projection GEMV + one tail kernel, B == 1).
 *   qv = x Wq^T + iter_vec;  q = LayerNorm(qv; ln_w, ln_b, ln_eps);  sa = q[:d/2] Ka^T;  sb = q[d/2:] Kb^T
 *   logits[g] = sa[p / nsk] + sb[p % nsk] + bias[g],  p = g mod nsk^2   (nsk^2 == n: the 1:1 product map of
 *   fused_router.py; nsk^2 < n: the reference's wrap, routing.py:227-230)
 *   nsk^2 > n: logits[g] = (g-th largest of the nsk^2 product scores) + bias[g], the reference's
 *   topk(product_scores, n).values (routing.py:212-222; e.g. 352 groups under 19 x 19 keys); nsk^2 <= 2048
 *   gates / active as mortar_remoe_gates.
 * x: [B, d] bf16 (x_is_f32 = 0) or fp32 (1), row stride ldx; wq fp32 [d, d] row-major (query_proj.weight);
 * iter_vec fp32 [d] (iter_embed[it]) or NULL; ln_w, ln_b fp32 [d]; ka, kb fp32 [nsk, d/2]; bias fp32 [n].
 * qv: caller workspace fp32 [B, d].  logits_out fp32 [B, n] or NULL; gates fp32 [B, n]; active uint8 [B, n] or NULL.
 * All arithmetic fp32 (the deploy router stays fp32, fused_router.py:26-28); sums are ordered differently from a
 * library GEMM, so gates agree with the eager path to rounding (the reference's own gate: active mismatch 0,
 * max gate error 2e-6, away from exact ties at the threshold). */
int mortar_router_bf16(const void *x, int32_t x_is_f32, int64_t B, int32_t d, int64_t ldx, const float *wq,
                       const float *iter_vec, const float *ln_w, const float *ln_b, float ln_eps, const float *ka,
                       const float *kb, int32_t nsk, const float *bias, int32_t n, int32_t k, float *qv,
                       float *logits_out, float *gates, uint8_t *active, void *stream);

/* The router behind a library GEMM, for prefill-sized calls: TileRouter.forward steps 2-8 (morph/model/routing.py:188-284)
 * on the projected query qv = x Wq^T (fp32 [N, d], row stride ldq; the dense projection of step 1, routing.py:181-186,
 * is a plain GEMM and stays with the caller's BLAS).  q = LayerNorm(qv + iter_vec), sub-key scores, product-key logits
 * (direct, wrapped or ranked exactly as in mortar_router_bf16), gating tail as mortar_remoe_gates: one launch instead
 * of the reference's layer_norm, two matmuls, broadcast add, topk, bias add, topk, relu, sum, divide.
 * iter_vec fp32 [d] or NULL; ln_w, ln_b fp32 [d]; ka, kb fp32 [nsk, d/2]; bias fp32 [n]; all 16-byte aligned.
 * logits_out fp32 [N, n] or NULL; gates fp32 [N, n]; active uint8 [N, n] or NULL.  d a multiple of 8 up to 8192,
 * n <= 1024; the ranked branch (nsk^2 > n) takes up to 1024 product keys (sorted in a wavefront's registers).  Sums are ordered differently from the library routines, so gates agree with the eager path
 * to fp32 rounding (the active set exactly, away from logits within rounding of the threshold). */
int mortar_router_tail_f32(const float *qv, int64_t N, int32_t d, int64_t ldq, const float *iter_vec, const float *ln_w,
                           const float *ln_b, float ln_eps, const float *ka, const float *kb, int32_t nsk,
                           const float *bias, int32_t n, int32_t k, float *logits_out, float *gates, uint8_t *active,
                           void *stream);

/* ---- decode (M <= 64) ------------------------------------------------------------------------ */

/* mortar_spmm_bf16 / mortar_gateup_swiglu_bf16 / mortar_spmm_bf16_masked serve decode batches directly: for
 * M <= 64 they run small-tile variants (4- or 16-token tiles, small workgroups) that read every weight block
 * from HBM once per launch.  That path replaces mortar_gemv (fused_decode_step.py:1502-1547, kernels :1341-1459)
 * for the MLP pair as the engine calls it (morph/inference/engine.py:980-986).
 *
 * Layer-batched form for M <= 64 (one to four 16-token tiles per layer): ONE launch runs the same operation on n_layers independent
 * (matrix, input, output) triples of identical shape (Rb, Cb, seg_cb).  No counterpart in the reference, which
 * issues one mortar_gemv per matrix (morph/inference/engine.py:980-986); this is for callers that hold many weight
 * sets whose inputs are known (several models, a stack probed for bandwidth).
 *   mortar_stack_table_bytes  bytes of device memory the parameter table needs
 *   mortar_stack_prepare      validates the layers, writes the table (synchronous host-to-device copy);
 *                             W: host array [n_layers] of descriptors with device pointers, x / y: host arrays
 *                             of device pointers, sched: host array of device schedules or NULL; swiglu = 0: y_l = x_l W_l^T, 1: y_l = silu(g) * u of gate_up W_l
 *   mortar_stack_run          launches the prepared table (any number of times); W0 = &W[0], same swiglu,
 *                             n_layers and M as prepared */
int64_t mortar_stack_table_bytes(int32_t n_layers);
int mortar_stack_prepare(int32_t swiglu, int32_t n_layers, const mortar_bcsr_t *W, const int32_t *const *sched,
                         const uint16_t *const *x, uint16_t *const *y, int64_t M, int64_t ldx, int64_t ldy,
                         void *table_dev, void *stream);
int mortar_stack_run(int32_t swiglu, int32_t n_layers, const mortar_bcsr_t *W0, int64_t M, const void *table_dev,
                     void *stream);

/* Generic decode GEMV over a work list (mortar_decode_worklist_host; entries on the device).
 * x bf16 [B, Cb*16]; B <= 64.
 *   mode 0: y bf16 [B, Rb*16] = x W^T
 *   mode 1: W = gate_up; y = h bf16 [B, Rb*8] = silu(g)*u [* gates[b, n/cls]]
 * nslots = 1: entries write the result directly.  nslots > 1: partial sums go to `part`
 * (fp32 [nslots, B, Rb*16], caller workspace) and a second kernel combines them in slot order, reading
 * row_slots (device copy of the work list's row_slots_out).
 * row_act / col_act (int32, may be NULL): ReMoE flags (mortar_route_flags), applied per stream as the reference's
 * kernel does (fused_decode_step.py:1378-1393): the sum of output block-row r is zero for stream b when
 * row_act[b, r] == 0 (gate_up: r runs over gate rows then up rows, Rb entries), and the blocks of input block-column c
 * contribute nothing to stream b when col_act[b, c] == 0.  Work is skipped where ALL B streams agree: a unit none of
 * whose rows is active for any stream, a block whose input column is off for every stream. */
int mortar_gemv_bf16(const mortar_bcsr_t *W, const int32_t *entries, int64_t n_entries, int32_t nslots,
                     const int32_t *row_slots, int32_t kseg, int32_t mode, const uint16_t *x, int32_t B, int64_t ldx,
                     uint16_t *y, int64_t ldy, float *part,
                     const float *gates, int32_t n_clusters, int64_t ldg,
                     const int32_t *row_act, int64_t ldr, const int32_t *col_act, int64_t ldc,
                     void *stream);

/* The same work-list GEMV in the reference engine's arithmetic (fused_decode_step.py:1335, 1341-1459, 1502-1547; the
 * engine runs fp32, morph/inference/engine.py:156-160): fp32 activations in, exact +-x / 0 products, fp32 sums, the
 * block's fp32 scale applied to the block sum (scale-after-sum; with scale_count = 1 the reference's one mortar_scale),
 * SwiGLU as g * sigmoid(g) * u and gates in fp32, fp32 out.  Internally an fp32 activation is split exactly into three
 * bf16 terms and a block is contracted with +-2 / 0 codes on the bf16 MFMA, so no product is rounded.
 *   scale      device fp32 [scale_count], scale_count = 1 or nnz (NOT rounded to bf16)
 *   swiglu_x   != 0: x is the gate_up output [B, 2 * in_features] and the input is silu(g) * u computed on load
 *              (the reference's down call form, fused_decode_step.py:1410-1414)
 *   x fp32 [B, ldx]; y fp32 [B, Rb*16] (mode 0) or [B, Rb*8] (mode 1), 16-byte aligned, ldy % 4 == 0
 *   kseg       block-columns per K segment of the work list; 3 * 2 * kseg * (16 * ceil(B / 16) + 1) * 16 bytes of LDS
 *   sched      the plain-product schedule of the pack (mortar_schedule_host with one row per unit, device), or NULL
 *   part       device workspace of part_bytes >= mortar_gemv_f32_workspace_bytes(W, B, nslots) bytes, 16-byte aligned
 *              (may be NULL when nslots == 1; then only the work-list kernel runs)
 *   other arguments as mortar_gemv_bf16.  Agreement with a float64 evaluation: fp32 rounding of the sums only.
 * With one scale (scale_count = 1, the reference's format), a schedule and the workspace, the product runs on
 * the bandwidth-bound SpMM kernels instead of the work list: the three bf16 terms of the B rows become 3 * B bf16 rows,
 * the one-scale SpMM kernels contract them with the +-2 / 0 blocks and keep the fp32 sums unrounded, and a last pass
 * adds the three sums of a row and applies the scale and the epilogue - the same exact products and fp32 sums, in
 * another order of addition (2 to 3 times faster at the headline shapes).  Flags keep their per-stream meaning there: a chunk of x
 * whose column is off for its stream enters as zeros, and the sum of a row that is off for a stream is written as
 * zero; no weight is skipped, which is still faster than the work list with skipping (17 against 25 us per MLP at
 * one row, 21 against 49 us at 16 rows). */
int64_t mortar_gemv_f32_workspace_bytes(const mortar_bcsr_t *W, int32_t B, int32_t nslots);
int mortar_gemv_f32(const mortar_bcsr_t *W, const float *scale, int64_t scale_count, const int32_t *sched,
                    const int32_t *entries,
                    int64_t n_entries, int32_t nslots, const int32_t *row_slots, int32_t kseg, int32_t mode,
                    int32_t swiglu_x, const float *x, int32_t B, int64_t ldx, float *y, int64_t ldy, float *part,
                    int64_t part_bytes, const float *gates, int32_t n_clusters, int64_t ldg,
                    const int32_t *row_act, int64_t ldr, const int32_t *col_act, int64_t ldc, void *stream);

/* mortar_gemv_bf16 for callers that cannot allocate device memory or hand in a workspace: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments and
 * results (bit for bit) as mortar_gemv_bf16 minus `part`: the fp32 partial sums of split rows (nslots > 1) go to a
 * buffer of MORTAR_GEMV_NOALLOC_MAX_FLOATS floats (4 MiB) that lives inside the library, one copy per GPU, held
 * until the process ends.  nslots * B * Rb*16 floats beyond that size are refused with MORTAR_ERR_LIMIT.  The call
 * allocates nothing, neither on the device nor on the host side of HIP.  All calls on one GPU share that GPU's buffer:
 * calls that may overlap there (different streams, different threads) race on it and must be ordered by the caller;
 * calls on one stream are ordered by the stream.  The first call on a device looks up the buffer's address
 * (hipGetSymbolAddress): make one call outside a graph capture before capturing. */
#define MORTAR_GEMV_NOALLOC_MAX_FLOATS (1 << 20)
int64_t mortar_gemv_noalloc_max_floats(void);
int mortar_gemv_bf16_noalloc(const mortar_bcsr_t *W, const int32_t *entries, int64_t n_entries, int32_t nslots,
                             const int32_t *row_slots, int32_t kseg, int32_t mode, const uint16_t *x, int32_t B,
                             int64_t ldx, uint16_t *y, int64_t ldy,
                             const float *gates, int32_t n_clusters, int64_t ldg,
                             const int32_t *row_act, int64_t ldr, const int32_t *col_act, int64_t ldc,
                             void *stream);

/* ---- product over stored bf16 block values (the operator-level drop-in) ------------------------ */

/* y = x W^T with W given by the reference's BCSR arrays as they are: stk_dds(lhs, data, offsets, row_indices,
 * column_indices, ..., transpose_b = True), morph/sparse/stk/backend/custom_ops.py:35-56 (kernel
 * triton_kernels.py:170-230): bf16 operands, fp32 accumulation, bf16 store, for ANY bf16 block values -- no ternary
 * restriction, nothing is quantised.  (The ternary entry points above stream 2- / 4-bit codes and are the fast path of
 * the modules; this one is what the stk_dds operator calls.)
 *   row_ptr  device int32 [Rb+1] (mortar_offsets);  col device int16 [nnz] (mortar_column_indices), ascending in a row
 *   data     device bf16 [nnz,16,16] (mortar_data, element [j, lr, c] = W[row_j*16+lr, col_j*16+c]), 16-byte aligned
 *   seg_ptr  device int32 [Rb, nseg+1] from mortar_segment_ptr_host with seg_cb = mortar_values_seg_cb(Cb), nseg =
 *            ceil(Cb / seg_cb); needed when nseg > 1 (in_features too wide for one 32-token LDS tile), else may be NULL
 *   x bf16 [M, ldx] 16-byte aligned, ldx % 8 == 0;  y bf16 [M, ldy] 8-byte aligned, ldy % 4 == 0
 * The dX product (transpose_b = False) is the same call on the transposed topology (mortar_transpose_topology_host)
 * with the blocks gathered in that order and transposed. */
int32_t mortar_values_seg_cb(int32_t Cb);
int mortar_segment_ptr_host(const int32_t *row_ptr, const int16_t *col, int32_t Rb, int32_t Cb, int32_t seg_cb,
                            int32_t *seg_ptr_out);
int mortar_dds_values_bf16(const int32_t *row_ptr, const int16_t *col, const int32_t *seg_ptr, const uint16_t *data,
                           int32_t Rb, int32_t Cb, int64_t nnz, const uint16_t *x, int64_t M, int64_t ldx, uint16_t *y,
                           int64_t ldy, void *stream);

/* ---- RMSNorm ---------------------------------------------------------------------------------- */

/* mortar_gateup_swiglu_bf16 with the RMSNorm in front of the MLP (attention.RMSNorm, morph/model/attention.py:133-141,
 * called as mlp(norm_mlp(x)) in morph/model/mhc.py:249-250) applied to the rows of x while they are staged: the
 * normalised activations never go to memory.  norm_w: bf16 [in_features], 16-byte aligned, or NULL for no weight.
 * Same bits as mortar_rmsnorm_bf16 followed by mortar_gateup_swiglu_bf16.  The reference fuses the same norm into
 * its dense ternary GEMV (X_MODE = 1, morph/kernels/triton/fused_decode_step.py:1149-1169).
 * Available when mortar_norm_fusable(Cb) != 0 (in_features <= 2048 in one K segment); otherwise MORTAR_ERR_LIMIT. */
int mortar_norm_gateup_swiglu_bf16(const mortar_bcsr_t *W, const int32_t *sched, const uint16_t *x, int64_t M,
                                   int64_t ldx, const uint16_t *norm_w, float norm_eps, uint16_t *h, int64_t ldh,
                                   const float *gates, int32_t n_clusters, const int32_t *tok_cnt,
                                   const uint8_t *tok_list, void *stream);
int mortar_norm_fusable(int32_t Cb);

/* The carved SwiGLU MLP as one call: y = down(silu(gate) * up [* gates per cluster]) with gate_up applied to x or to
 * RMSNorm(x) -- _SwiGLUMortar.forward, morph/model/transformer.py:402-431 (called as mlp(norm_mlp(x)),
 * morph/model/mhc.py:249-250).  Two launches (gate_up with the SwiGLU in its epilogue, then down), same arithmetic and
 * same bits as mortar_[norm_]gateup_swiglu_bf16 followed by mortar_spmm_bf16.  What the call adds: the hidden
 * activations between the launches live in `hidden`, a caller workspace of mortar_mlp_hidden_bytes(M, d_ff) bytes
 * (16-byte aligned) whose layout belongs to the library.  From 513 rows up (both launches then run 32-token tiles) it is
 * tile order -- the 32 tokens x 16 features of a (token tile, block-column) in 1 KB of contiguous memory -- so that
 * gate_up stores whole result tiles as contiguous runs and down copies its K segments asynchronously into LDS without
 * passing through registers; below, and for matrices without the 4-bit stream, it is row-major [M, d_ff].
 *   norm != 0: RMS-normalise the rows of x on the way in (norm_w bf16 [in_features] or NULL, norm_eps), needs
 *              mortar_norm_fusable(Wgu->Cb) != 0
 *   gates      fp32 [M, n_clusters] or NULL, multiplied per cluster of d_ff / n_clusters hidden features (in bf16)
 *   phase      0: both launches; 1: gate_up only (fills `hidden`); 2: down only (reads `hidden` as phase 1 of the same
 *              M left it) -- for callers that time or interleave the two launches
 * Token lists (routed skipping) and input masks keep their own entry points. */
int64_t mortar_mlp_hidden_bytes(int64_t M, int32_t d_ff);
int mortar_mlp_bf16(const mortar_bcsr_t *Wgu, const int32_t *sched_gu, const mortar_bcsr_t *Wdn, const int32_t *sched_dn,
                    const uint16_t *x, int64_t M, int64_t ldx, int32_t norm, const uint16_t *norm_w, float norm_eps,
                    const float *gates, int32_t n_clusters, void *hidden, uint16_t *y, int64_t ldy, int32_t phase,
                    void *stream);

/* y = bf16(bf16(x * rsqrt(mean(x^2) + eps)) * w) per row; x, y bf16 [M, d]; w bf16 [d] or NULL (= 1). */
int mortar_rmsnorm_bf16(const uint16_t *x, int64_t M, int32_t d, int64_t ldx, const uint16_t *w, float eps,
                        uint16_t *y, int64_t ldy, void *stream);

/* ---- device-side re-pack ------------------------------------------------------------------------ */

/* Ternarise block values on the device and rewrite the matrix's value arrays (codes, sdup, codes_o, sd_o and,
 * when present, codes4_o) in place; the topology arrays are not touched.  One launch (two with scale_mode 0)
 * replaces the reference's per-forward torch ternarisation of mortar_data (block_sparse.py:909-919) and its
 * deploy pack (deploy_quant.py:81-95, 344-374) followed by a host re-pack.
 *   values     device [nnz,16,16], bf16 (values_f32 = 0) or fp32 (1), 16-byte aligned: the reference's mortar_data
 *   pos        device int32 [nnz] from mortar_octet_positions_host
 *   src_block  device int32 [nnz] or NULL: block j of W takes the values of block src_block[j] (NULL: block j)
 *   transpose  != 0: the source block is read transposed.  src_block + transpose fill the W^T pack of
 *              mortar_transpose_topology_host from the values of W.
 *   scale_mode 0: one scale per matrix, mean|w| over all values clamped to >= 1e-8 (deploy_quant.py:91)
 *              1: one scale per block, mean|w| of the (source) block clamped to >= 1e-6 (block_sparse.py:397)
 *              2: scale_in device fp32 [1];  3: scale_in device fp32 [nnz], indexed by source block
 *   code = sign(w/s) where |w/s| > threshold (fp32 division, strict compare), else 0; means are summed in fp64
 *   in a fixed order.  The kernels multiply by bf16(s) (round to nearest even), as the reference's bf16 autocast does.
 *   scale_out  device fp32, [1] for modes 0 and 2, [nnz] for 1 and 3 (order of W's blocks), or NULL
 *   status     device int32 [2] or NULL.  Both words are set to 0 first (unless flags bit 0 is set), then
 *              status[0] = 1 if bf16(s) of some block lies outside [2^-100, 2^100] (that block is zeroed; the host
 *              packer returns MORTAR_ERR_SCALE for it), status[1] = 1 if the ternary check below fails
 *   flags      bit 0: do not clear status first, so that it accumulates over several calls (a caller that reads it
 *              only now and then still sees every failure)
 *   ternary_tol  > 0 (scale_mode 2 or 3 only): the values are expected to be ternary already, 0 or +-s of the given
 *              scale; status[1] = 1 if some value is neither, |v| <= tol * s or ||v| - s| <= tol * s.  This is how the
 *              stk_dds operator states its restriction: the runtime multiplies ternary blocks only, and data that the
 *              reference's stk_dds would multiply as arbitrary bf16 values is reported instead of silently quantised.
 *   workspace  device, mortar_requantize_workspace_bytes() bytes, 8-byte aligned; needed for scale_mode 0 only
 * mortar_bcsr_t.uniform_scale is host state: after modes 0 / 2 the caller may set it to bf16(s) to select the
 * scale-after-sum kernels, or leave it 0 (per-block kernels, always valid). */
int64_t mortar_requantize_workspace_bytes(void);
int mortar_requantize(const mortar_bcsr_t *W, const void *values, int32_t values_f32, const int32_t *pos,
                      const int32_t *src_block, int32_t transpose, int32_t scale_mode, float threshold,
                      const float *scale_in, float *scale_out, int32_t *status, int32_t flags, float ternary_tol,
                      void *workspace, void *stream);

/* Makes a result unusable when a re-pack reported an error: if status[0] | status[1] != 0 (the words of
 * mortar_requantize, read on the device, no host synchronisation) every 4 bytes of out[0..bytes) become 0x7FC07FC0,
 * NaN both as bf16 pairs and as fp32; otherwise out is not touched.  The stk_dds operator enqueues it behind its
 * product, so data the reference's stk_dds (custom_ops.py:35-56) would multiply as arbitrary bf16 values never yields
 * finite numbers of a silently re-quantised matrix, also in calls that do not wait for the status words.
 *   out device, 4-byte aligned, bytes a multiple of 4; status device int32 [2]. */
int mortar_poison_on_status(void *out, int64_t bytes, const int32_t *status, void *stream);

/* ---- SwiGLU between the two matrices, training form ------------------------------------------------ */

/* h = bf16(bf16(silu(gate)) * up) from a stored gate_up output gu [M, 2*d_ff] (gate = columns [0, d_ff), up =
 * [d_ff, 2*d_ff)), and its derivative dgu [M, 2*d_ff] from gu and dh [M, d_ff]: the eager path of
 * _SwiGLUMortar.forward (morph/model/transformer.py:411-413: gu.chunk(2), F.silu(gate) * up) and what torch autograd
 * derives from it, each in one launch.  Inference uses the fused epilogue of mortar_gateup_swiglu_bf16 instead; training
 * keeps gu for the backward.  All bf16, d_ff and leading dimensions multiples of 8, rows 16-byte aligned. */
int mortar_swiglu_bf16(const uint16_t *gu, int64_t ldg, int64_t M, int32_t d_ff, uint16_t *h, int64_t ldh, void *stream);
int mortar_swiglu_backward_bf16(const uint16_t *gu, int64_t ldg, const uint16_t *dh, int64_t ldh, int64_t M, int32_t d_ff,
                                uint16_t *dgu, int64_t ldo, void *stream);

/* ---- weight gradient on the topology ------------------------------------------------------------ */

/* out[j] = a[:, 16 rows of block j]^T @ b[:, 16 columns of block j] for every kept block: the dW product of the
 * carved linear, the reference's stk_sdd_at_b(a, b, data, offsets, row_indices, column_indices) -> [nnz, blk, blk]
 * (morph/sparse/stk/backend/custom_ops.py:78-96; forward y = x W^T: a = dY [M, out], b = x [M, in]).  bf16 operands,
 * fp32 accumulation over the M tokens, bf16 result (round to nearest even).
 *   mortar_sdd_blocks_per_wave_host: how many kept blocks one wavefront of a workgroup accumulates (8, 10, ... 22;
 *     a workgroup of 16 wavefronts owns 16 times as many blocks of a few consecutive block-rows of one K segment),
 *     chosen for this topology at M tokens: smaller groups fill the chip with fewer token ranges, larger ones stage
 *     fewer bytes per block.  Any built size gives the same results.
 *   mortar_sdd_plan_host: the work partition for a topology and a group size (host, once per pair).  plan_out = NULL
 *     returns the number of int32 words needed; otherwise fills plan_out (plan_words = its capacity) and returns the
 *     words used; plan_out[0] = n_wg.  Upload the plan to the device.
 *   mortar_sdd_bf16: plan device int32, with the n_wg and blocks_per_wave it was made for (workgroup ids are laid
 *     out per XCD as runs of (token range, row group x K segment) so that the readers of one slice share an L2); a bf16
 *     [M, lda >= Rb*16], b bf16 [M, ldb >= Cb*16], 16-byte aligned with leading dimensions multiples of 8; acc device
 *     workspace of mortar_sdd_workspace_bytes(n_wg, nnz, blocks_per_wave, M) bytes, 16-byte aligned (every token range
 *     writes its fp32 sums to a slab of its own, and a last pass adds the slabs in a fixed order: results are
 *     reproducible); out device bf16 [nnz,16,16], 16-byte aligned.  M = 0 gives zeros. */
int32_t mortar_sdd_blocks_per_wave_host(const int32_t *row_ptr, const int16_t *col, int32_t Rb, int32_t Cb, int64_t M);
int64_t mortar_sdd_plan_host(const int32_t *row_ptr, const int16_t *col, int32_t Rb, int32_t Cb, int32_t blocks_per_wave,
                             int32_t *plan_out, int64_t plan_words);
int64_t mortar_sdd_workspace_bytes(int32_t n_wg, int32_t nnz, int32_t blocks_per_wave, int64_t M);
int mortar_sdd_bf16(const int32_t *plan, int32_t n_wg, int32_t blocks_per_wave, int32_t Rb, int32_t Cb,
                    int32_t nnz, const uint16_t *a, int64_t lda, const uint16_t *b, int64_t ldb, int64_t M, float *acc,
                    uint16_t *out, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MORTAR_HIP_H */
