/*
 * shareprefill_hip.h -- C ABI of libshareprefill_hip.so (MI355X / gfx950).
 *
 * The library is the device side of the SharePrefill prefill-attention layer: block average
 * pooling, last-block vertical/slash scoring, cumulative-mass block selection, cross-head
 * pattern sharing and the GQA causal block-sparse flash attention.  The reference implements
 * this path in Python + Triton; each entry point below names the reference code it replaces
 * (paths relative to the reference checkout).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless the comment says "host";
 *   - batch size is 1 (shareprefill/attn/attention_sharing.py:42-44);
 *   - q/k/v are bf16 with explicit element strides for the token and head axes and a
 *     contiguous head_dim axis, so both [N,H,D] and [H,N,D] storage are accepted as is;
 *   - all work is enqueued on `stream` (a hipStream_t; NULL = the default stream), nothing
 *     synchronises the stream, nothing allocates;
 *   - return value 0 = ok, negative = error (SP_ERR_*), text from sp_last_error();
 *   - block masks are bit matrices: mask[h][r][w] is a uint64 word, bit (c & 63) of word
 *     (c >> 6) is block (r, c); nbw = ceil(nb / 64) words per row.  Flat block id of the
 *     reference = r * nb + c (shareprefill/attn/shareprefill_attn.py:491-492).
 */
#ifndef SHAREPREFILL_HIP_H
#define SHAREPREFILL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SP_OK 0
#define SP_ERR_INVALID_ARGUMENT (-1)
#define SP_ERR_UNSUPPORTED (-2)
#define SP_ERR_HIP (-3)
#define SP_ERR_WORKSPACE (-4)

/* per-head decision written by sp_share_decide (attention_sharing.py:182-190 use_dense/use_share/use_query_aware) */
#define SP_DEC_VS 0
#define SP_DEC_DENSE 1
#define SP_DEC_SHARE 2
#define SP_DEC_QA 3

/* flags */
#define SP_FLAG_LOGITS_BF16 1u /* round pooled / last-block logits to bf16 as the reference's bf16 einsum does */
/* Bits 8..15 of flags: the head_dim, in units of 8, that the selection's 1/sqrt(head_dim) scale
 * (attention_sharing.py:127, 197, 357) is formed from, for q / k whose head_dim axis has been zero-padded to a width
 * the kernels are built for (the padding changes no dot product).  0 = the tensors' own d. */
#define SP_FLAG_SCALE_DIM(head_dim) ((((uint32_t)(head_dim)) / 8u) << 8)

/* tail handling of sp_pool_avg_bf16 */
#define SP_POOL_TAIL_TRUE_LENGTH 0 /* divide the ragged last block by its length (attn/utils.py:171,187) */
#define SP_POOL_TAIL_RESCALE 1     /* mean over bs, then *bs/(bs-pad) in bf16 (attention_sharing.py:350-356) */

typedef void* sp_stream_t;

/* Cross-layer sharing state, one slot per SHARED cluster (attention_sharing.py:41-78).
 * The struct itself lives in host memory; every member pointer is device memory owned by the caller. */
typedef struct sp_cluster_state {
  int32_t n_clusters;
  int32_t nb;  /* blocks per side the slabs are sized for */
  int32_t nbw; /* ceil(nb/64) */
  int32_t struct_bytes; /* sizeof(sp_cluster_state) as the caller was compiled.  0 or SP_CLUSTER_STATE_V1_BYTES = the
                           first layout of this struct, which ended with `accum`: no member behind it is read */
  int32_t* info;     /* [C][8]: 0 pivot head (-1 none), 1 has_pattern, 2 pivot nv, 3 pivot ns, 4 pivot layer,
                        5 rows counted by a running sp_pivot_update (zero between calls) */
  double* ratio;     /* [C]     vs_ratio of the pivot (valid once has_pattern) */
  float* vert;       /* [C][nb] pivot's pooled last-row vertical vector */
  float* slash;      /* [C][nb] pivot's pooled last-row slash vector */
  uint8_t* cols;     /* [C][nb] 1 = block column in the pivot's own vertical set */
  uint8_t* dists;    /* [C][nb] 1 = block distance in the pivot's own slash set */
  uint64_t* pattern; /* [C][nb][nbw] pivot block pattern */
  uint64_t* accum;   /* [C][2]  scratch of sp_pivot_update (covered / total mass, fixed point); zero on entry, and
                        every completed call leaves it zero again: allocate it zero-filled */
  float* avg_map;    /* [C][nb][nb] or NULL: the pivot's block-average attention map, kept by sp_pivot_update for
                        AttentionSharing.get_pivotal_attn (attention_sharing.py:87-99); valid once has_pattern
                        (since library version 2; read only when struct_bytes >= sizeof(sp_cluster_state)) */
} sp_cluster_state;
#define SP_CLUSTER_STATE_V1_BYTES 80 /* 4 x int32 + 8 pointers */

/* ---- library info ------------------------------------------------------------------------- */
int sp_version(void);
const char* sp_arch(void);       /* "gfx950" */
const char* sp_last_error(void); /* host string, valid until the next failing call on this thread */

/* pool types of sp_pool_bf16, numbered as in the reference's kernel (attn/utils.py:135, 255) */
#define SP_POOL_AVG 0
#define SP_POOL_MAX 1
#define SP_POOL_MIN 2
#define SP_POOL_MAXABS 3 /* max of absolute values */
#define SP_POOL_SUM 4

/* ---- (a) block average pooling --------------------------------------------------------------
 * Replaces triton_bnhd_pool / bnhd_pool_kernel (attn/utils.py:131-261, "avg" mode) and the torch
 * .mean used for Q (attention_sharing.py:350-356).
 * x: bf16 [n][h][d] with strides; y: bf16 [nb][h][d] contiguous.  fp32 accumulation.
 * head_enable: optional int32[h]; heads with 0 are skipped (their rows of y are left untouched). */
int sp_pool_avg_bf16(const void* x, void* y, int64_t n, int32_t h, int32_t d, int64_t x_stride_n,
                     int64_t x_stride_h, int32_t bs, int32_t tail_mode, const int32_t* head_enable,
                     sp_stream_t stream);
/* The other pool types of bnhd_pool_kernel (attn/utils.py:180-191; nothing in the selection uses them): per block of
 * bs tokens the maximum, the minimum, the maximum of the absolute values or the sum (SP_POOL_*; SP_POOL_AVG = the
 * call above with SP_POOL_TAIL_TRUE_LENGTH).  As in the reference's kernel, tokens of a ragged last block that lie
 * beyond the sequence count as zeros (its masked load, utils.py:168-179): that block's maximum is at least 0 and its
 * minimum at most 0.  Sums accumulate in fp32 and are rounded to bf16 once. */
int sp_pool_bf16(const void* x, void* y, int64_t n, int32_t h, int32_t d, int64_t x_stride_n, int64_t x_stride_h,
                 int32_t bs, int32_t pool_type, sp_stream_t stream);

/* ---- last-block scores -> vertical / slash --------------------------------------------------
 * Replaces attention_sharing.py:127-167 + sum_all_diagonal_matrix (attn/utils.py:79-86) +
 * torch_bhn_sumpool (attn/utils.py:33-44): softmax over all keys of the last bs queries
 * (scaled by 1/sqrt(d), causal inside the last bs columns), column mean -> vert_tok[hq][n],
 * anti-diagonal mean -> slash_tok[hq][n], and their block sums vert_blk / slash_blk [hq][nb].
 * bs: 16, 32, 64 or 128 (attention_sharing.py:127 takes any; shareprefill_attn.py:509-516 allows these); d 128;
 * n >= bs (the kernels work on the last 128 token positions' queries and drop the rows a smaller block, or a
 * shorter prompt, lacks).
 * workspace: sp_lastq_scores_workspace_bytes(...) bytes of device scratch. */
size_t sp_lastq_scores_workspace_bytes(int64_t n, int32_t hq, int32_t bs);
int sp_lastq_scores_bf16(const void* q, const void* k, int64_t n, int32_t hq, int32_t hkv, int32_t d,
                         int64_t q_stride_n, int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                         int32_t bs, uint32_t flags, void* workspace, size_t workspace_bytes,
                         float* vert_tok, float* slash_tok, float* vert_blk, float* slash_blk,
                         sp_stream_t stream);

/* ---- cumulative-mass primitives (attn/utils.py:47-76) --------------------------------------
 * Canonical arithmetic: entries ordered by (value desc, index asc); running sums are exact
 * sums of the values truncated to unsigned 2^-48 fixed point.  Inputs: finite, >= 0, row sum < 2^14.
 *
 * sp_cover_count: score_cover_topk (utils.py:47-50): out[v] = count(cumsum <= thr) + 1 for each of
 * n_vec vectors of length len (row stride = len).
 * workspace (both functions): sp_cover_select_workspace_bytes(n_vec resp. 2*hq) bytes of device scratch, 8-byte
 * aligned. */
int sp_cover_count(const float* x, int32_t n_vec, int64_t len, float thr, int32_t* out, void* workspace,
                   size_t workspace_bytes, sp_stream_t stream);

/* budgets of attention_sharing.py:169-176: clamp(cover_count(.)/bs + 1, minb, maxb) for both vectors */
int sp_cover_budgets(const float* vert_tok, const float* slash_tok, int32_t hq, int64_t n, int32_t bs,
                     float pattern_threshold, int32_t min_blocks, int32_t max_blocks, int32_t* nv, int32_t* ns,
                     void* workspace, size_t workspace_bytes, sp_stream_t stream);

/* ---- query-aware test (attention_sharing.py:193-202) ----------------------------------------
 * avg_qk[h] = softmax_fp32(mean_i(last_q[h]) . kbar[:, h/g]); js_qa[h] = sqrt_JS(avg_qk[h], vert_blk[h]);
 * use_qa[h] = js_qa[h] < queryaware_threshold (NaN compares false).  kbar: bf16 [nb][hkv][d]. */
int sp_queryaware_test_bf16(const void* q, const void* kbar, const float* vert_blk, int64_t n, int32_t hq,
                            int32_t hkv, int32_t d, int64_t q_stride_n, int64_t q_stride_h, int32_t bs,
                            uint32_t flags, float queryaware_threshold, float* avg_qk, float* js_qa,
                            int32_t* use_qa, sp_stream_t stream);

/* ---- pivot election / share test (attention_sharing.py:204-301) -----------------------------
 * Walks the heads in ascending order.  head_cluster[h] = slot of the head's cluster in `state`
 * for this layer, or -1 when the head is in no shared cluster.  Writes decision[h] (SP_DEC_*),
 * js_v / js_s (NaN where no share test ran) and the final budgets (min_blocks for QA / sharing heads).
 * A newly elected pivot stores its pooled vectors, its budgets and its own vertical / slash sets. */
int sp_share_decide(const sp_cluster_state* state /* host */, const int32_t* head_cluster, int32_t layer_idx,
                    int32_t hq, const float* vert_blk, const float* slash_blk, const int32_t* use_qa,
                    const int32_t* nv, const int32_t* ns, int32_t min_blocks, float similarity_threshold,
                    double fallback_threshold, int32_t* decision, float* js_v, float* js_s, int32_t* nv_final,
                    int32_t* ns_final, sp_stream_t stream);

/* ---- mask construction (attention_sharing.py:303-337, attn/utils.py:99-128) -----------------
 * mask[h] = vertical-slash blocks (sink column and main diagonal forced, top-nv columns, top-ns
 * distances) | all lower-triangular blocks (DENSE) | the cluster pivot's pattern (SHARE).
 * Overwrites mask[hq][nb][nbw]. */
int sp_build_mask(const sp_cluster_state* state /* host */, const int32_t* head_cluster, const int32_t* decision,
                  const float* vert_blk, const float* slash_blk, const int32_t* nv_final, const int32_t* ns_final,
                  int32_t hq, int32_t nb, uint64_t* mask, sp_stream_t stream);

/* ---- query-aware block selection (attention_sharing.py:339-364, attn/utils.py:53-57) --------
 * For heads with decision == SP_DEC_QA: probs[h] = softmax rows of (qbar[h]/sqrt(d)) . kbar^T with the
 * block-causal mask ([nb][nb] fp32, caller scratch [hq][nb][nb]); then the global cumulative-mass
 * selection at pattern_threshold * nb (crossing entry excluded) is OR-ed into mask[h].  pattern_threshold is a
 * double because the reference forms that product from the Python float before the comparison takes it to fp32:
 * score = fp32(pattern_threshold * nb) (attention_sharing.py:361, attn/utils.py:56).
 * qbar: bf16 [nb][hq][d] (sp_pool_avg_bf16 of q), kbar: bf16 [nb][hkv][d]. */
float sp_queryaware_select_score(double pattern_threshold, int32_t nb); /* host arithmetic only: the score above */
int sp_queryaware_select_bf16(const void* qbar, const void* kbar, const int32_t* decision, int32_t hq,
                              int32_t hkv, int32_t d, int32_t nb, uint32_t flags, double pattern_threshold,
                              float* probs, uint64_t* mask, void* workspace, size_t workspace_bytes,
                              sp_stream_t stream);

/* the selection alone, on caller-supplied probabilities: mask[v] |= kept entries of x[v] ([nb][nb] each),
 * restricted to the lower triangle (entries above the diagonal are ignored; they are exactly zero in the
 * reference's maps); vectors with enable[v] == 0 are skipped (enable may be NULL).
 * workspace: sp_cover_select_workspace_bytes(n_vec) bytes of device scratch, 8-byte aligned (also needed by
 * sp_queryaware_select_bf16, with n_vec = hq). */
size_t sp_cover_select_workspace_bytes(int32_t n_vec);
int sp_cover_select_global(const float* x, const int32_t* enable, int32_t n_vec, int32_t nb, float score,
                           uint64_t* mask, void* workspace, size_t workspace_bytes, sp_stream_t stream);

/* ---- GQA causal block-sparse flash attention ------------------------------------------------
 * Replaces triton_block_wise_prefill_attention / block_wise_prefill_attention_kernel /
 * count_kernel (shareprefill_attn.py:187-620).  out: bf16 [n][hq][d] contiguous.  Only blocks set in
 * mask (and c <= r) are computed.  For heads with decision == SP_DEC_DENSE the block-averaged attention
 * map avg_attn[h][nb][nb] (fp32, pre-zeroed by the caller) is written as well (:425-457); decision and
 * avg_attn may both be NULL.
 * bs: 16, 32, 64 or 128 (:509-516); mask [hq][nb][ceil(nb / 64)] and avg_attn are on the grid nb = ceil(n / bs) <= 4096.
 * The kernels are built on 128-token blocks: for a smaller bs they visit every 128-token block that holds a kept
 * block and drop the others' keys per 16 x 16 sub-tile, like the keys the causal predicate hides (exact; the work is
 * that of the 128-token blocks), the maps of DENSE heads come from the recomputing pass only, and
 * SP_ATTN_HALF_CHANNELS is accepted and ignored (all 128 channels of out are written).
 * workspace: sp_attn_workspace_bytes(...) bytes of device scratch (key-major repack of V, a work counter and
 * the pivot heads' softmax row statistics).
 * sp_attn_repack_v_bf16 fills it; sp_block_sparse_attn_fwd_bf16 calls it first unless flags has
 * SP_ATTN_V_REPACKED (the caller already repacked this v into this workspace). */
#define SP_ATTN_V_REPACKED 1u
#define SP_ATTN_PAIR_ROWS 2u /* skip the per-call analysis of how to pair query blocks into work items and pair rows
                                2p, 2p+1 of every head: what a dense mask wants; the result never depends on it */
#define SP_ATTN_HALF_CHANNELS 4u /* q, k and v are zero beyond channel 64 (a head_dim of 16 / 32 / 64 zero-padded to the
                                    kernel's 128, shareprefill_attn.py:503-508): the products skip those channels and
                                    channels 64..127 of out are NOT written */
size_t sp_attn_workspace_bytes(int64_t n, int32_t hq, int32_t hkv, int32_t d, int32_t bs);
/* Optional extra workspace per pivot head (decision == SP_DEC_DENSE with avg_attn requested): with
 * sp_attn_workspace_bytes rounded up to 256 bytes + p * sp_attn_pivot_scratch_bytes(n, bs) bytes of workspace, the
 * first p pivot heads (ascending head index) are processed in a launch of their own that keeps per-query block sums,
 * and their block-average maps (shareprefill_attn.py:425-457) are made from those instead of a second pass over
 * Q.K^T; further pivots, or all of them with the base size, take that second pass.  Same results to rounding. */
size_t sp_attn_pivot_scratch_bytes(int64_t n, int32_t bs);
int sp_attn_repack_v_bf16(const void* v, int64_t n, int32_t hkv, int32_t d, int64_t v_stride_n, int64_t v_stride_h,
                          int32_t bs, void* workspace, size_t workspace_bytes, sp_stream_t stream);
int sp_block_sparse_attn_fwd_bf16(const void* q, const void* k, const void* v, int64_t n, int32_t hq, int32_t hkv,
                                  int32_t d, int64_t q_stride_n, int64_t q_stride_h, int64_t k_stride_n,
                                  int64_t k_stride_h, int64_t v_stride_n, int64_t v_stride_h, int32_t bs,
                                  float softmax_scale, const uint64_t* mask, const int32_t* decision, void* out,
                                  float* avg_attn, void* workspace, size_t workspace_bytes, uint32_t flags,
                                  sp_stream_t stream);

/* ---- decode step -------------------------------------------------------------------------------
 * Replaces the flash_attn_func call of the decode branch (shareprefill_attn.py:146-155): one query token per
 * head against the whole KV cache, no mask.  q: bf16 [hq][d] (head stride in elements), k / v: bf16
 * [hkv][n][d] with token and head strides, out: bf16 [hq][d] contiguous.  d a multiple of 8 up to 128 (built for
 * 128; a smaller head is zero-padded to 128 on its way into LDS and reads only its own bytes), hq / hkv <= 32; q, k, v
 * 16-byte aligned with strides that are multiples of 8 elements.
 * workspace: sp_decode_workspace_bytes(n, hq, hkv) bytes of device scratch, 8-byte aligned. */
size_t sp_decode_workspace_bytes(int64_t n, int32_t hq, int32_t hkv);
int sp_decode_attn_bf16(const void* q, const void* k, const void* v, int64_t n, int32_t hq, int32_t hkv, int32_t d,
                        int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h, int64_t v_stride_n,
                        int64_t v_stride_h, float softmax_scale, void* out, void* workspace,
                        size_t workspace_bytes, sp_stream_t stream);

/* The same decode step for callers that cannot allocate (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): no counterpart in the reference.  Identical arguments and results, but the chunk
 * partials live in a device array built into the library (SP_DECODE_STATIC_SCRATCH_BYTES = 8 MiB per GPU, held
 * until the process ends) instead of a caller's workspace; nothing is allocated or freed, here or in any routine it
 * calls.  Shapes whose partials exceed the array (sp_decode_workspace_bytes(n, hq, hkv) > 8 MiB, e.g. more than about
 * 16000 (chunk, head) pairs) are refused with SP_ERR_WORKSPACE.  All calls on one GPU share that GPU's array: calls
 * that overlap in time on one GPU (two streams, two threads) race; calls ordered on one stream are safe, and
 * nothing needs clearing between them.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress); make that call outside graph capture. */
#define SP_DECODE_STATIC_SCRATCH_BYTES (8u << 20)
int sp_decode_attn_static_bf16(const void* q, const void* k, const void* v, int64_t n, int32_t hq, int32_t hkv,
                               int32_t d, int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                               int64_t v_stride_n, int64_t v_stride_h, float softmax_scale, void* out,
                               sp_stream_t stream);

/* ---- rotary position embedding in front of the attention function ---------------------------------
 * The reference's patched model produces (cos, sin) per position (model_patch.py:121) and leaves the rotation to
 * the Hugging Face attention layer, which evaluates  x*cos + rotate_half(x)*sin  (rotate_half(x) =
 * cat(-x[d/2:], x[:d/2])) with five elementwise bf16 kernels per tensor.  This entry point rotates q and k in
 * place in one pass with the same roundings (each product and the sum rounded to bf16, nearest even): the result
 * is bit-identical to that expression for finite inputs.
 * q: bf16 [n][hq][d], k: bf16 [n][hkv][d] (token and head strides in elements), cos_t / sin_t: bf16 [n][d] with
 * row stride cs_stride_n.  d a multiple of 16; pointers and strides 16-byte aligned.  hq or hkv may be 0. */
int sp_rope_inplace_bf16(void* q, void* k, const void* cos_t, const void* sin_t, int64_t n, int32_t hq, int32_t hkv,
                         int32_t d, int64_t q_stride_n, int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                         int64_t cs_stride_n, sp_stream_t stream);

/* ---- pivot state update (attention_sharing.py:94-103, attn/utils.py:60-76) ------------------
 * For each head with decision == SP_DEC_DENSE: per-row cumulative-mass selection (>= threshold,
 * crossing entry included) of avg_attn[h] -> state.pattern, the pivot's vs_ratio
 * (attention_sharing.py:278-286, duplicates counted) -> state.ratio, has_pattern = 1.  When several DENSE heads name
 * the same cluster, the highest head's map is the one kept (the reference stores them in ascending order). */
int sp_pivot_update(const sp_cluster_state* state /* host */, const int32_t* head_cluster, const int32_t* decision,
                    const float* avg_attn, int32_t hq, int32_t nb, float pattern_threshold, sp_stream_t stream);

/* per-row selection alone: pattern[r] = kept entries of row r of x[nb][nb] (lower triangle, (0,0) set) */
int sp_cover_select_rows(const float* x, int32_t nb, float thr, uint64_t* pattern, sp_stream_t stream);

/* ---- helpers ----------------------------------------------------------------------------------
 * CSR row pointers of a mask (triton_column_count_cumsum, shareprefill_attn.py:226-269):
 * row_ptr[h][r+1] = number of set blocks in rows 0..r of head h; row_ptr[h][0] = 0. */
int sp_mask_row_pointers(const uint64_t* mask, int32_t hq, int32_t nb, int32_t* row_ptr, sp_stream_t stream);

/* The reference's block_idx form of a selection (the argument of triton_block_wise_prefill_attention,
 * shareprefill_attn.py:484-486, 528-540, and the first return value of get_active_blocks, attention_sharing.py:366):
 * block_idx[h][0..k) = flat block ids row * nb + col in any order, row stride idx_stride_h elements, padded with any
 * value outside [0, nb * nb) (the reference pads with nb * (nb + 1)).
 * sp_block_idx_to_mask: mask[hq][nb][ceil(nb/64)] = the bit mask the attention entry point takes; ids above the
 *   diagonal are dropped (the reference's kernel masks every element of such a block, shareprefill_attn.py:401-406).
 * sp_block_idx_row_pointers: triton_column_count_cumsum (shareprefill_attn.py:187-269) on the ids themselves:
 *   row_ptr[h][r+1] = number of ids with id / nb <= r (duplicates counted, as by the reference's histogram);
 *   row_ptr[h][0] = 0.  nb <= 4096. */
int sp_block_idx_to_mask(const int64_t* block_idx, int64_t idx_stride_h, int64_t k, int32_t hq, int32_t nb,
                         uint64_t* mask, sp_stream_t stream);
int sp_block_idx_row_pointers(const int64_t* block_idx, int64_t idx_stride_h, int64_t k, int32_t hq, int32_t nb,
                              int32_t* row_ptr, sp_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* SHAREPREFILL_HIP_H */
