/*
 * C ABI of the MI355X (gfx950) sparse-attention library: dense / block-sparse /
 * column-sparse flash-attention forward and the colsum kernel.
 *
 * Every entry point takes raw device pointers, sizes and element strides, launches
 * asynchronously on the HIP stream it is given (a hipStream_t passed as void*, NULL =
 * the default stream) and returns 0 or a negative LVAR_E* code.  No entry point
 * allocates, frees or synchronises; scratch memory, where an entry point uses any, is a
 * workspace argument.  Tensors are bf16 with unit stride on the head
 * dimension; "strides" are in elements for (batch, head, row).
 *
 * Base-2 softmax statistics follow the reference kernels: M = max_n(q.k*scale*log2e),
 * L = sum_n exp2(q.k*scale*log2e - M); both fp32, contiguous [B,H,Lq].
 */
#ifndef LVAR_SPARSE_ATTN_H
#define LVAR_SPARSE_ATTN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LVAR_OK 0
#define LVAR_EINVAL (-1)      /* bad size / null pointer / misaligned pointer or stride */
#define LVAR_EUNSUPPORTED (-2) /* head_dim, block shape or query-group size not built */
#define LVAR_ELAUNCH (-3)      /* HIP reported a launch error */
#define LVAR_ETOOBIG (-4)      /* lvar_block_sparse_attn_static_fwd: more query tiles than its scratch buffer holds */

/* Tensor view: base pointer plus element strides of a [B,H,rows,d] bf16 tensor (d stride 1). */
typedef struct {
  const void* ptr;
  int64_t stride_b;
  int64_t stride_h;
  int64_t stride_row;
} lvar_tensor_t;

/*
 * Partial-result workspace of the balanced launches (the *_ws_fwd entry points): device memory owned by the
 * caller, 256-byte aligned; its contents need no preparation (a balanced launch clears the arrival counters it is
 * going to use with a small kernel ahead of the attention kernel, and leaves them zero when it ends).  With it, a launch whose plain grid would fill the chip unevenly (at most 1024 query tiles
 * and fewer than four rounds of workgroups: the middle scales of a next-scale-prediction schedule, few query tiles
 * with long or ragged lists) picks a share of about (all list entries) / (resident workgroup slots), cuts every
 * query tile whose list is long enough into round(entries / share) pieces of equal length and runs one workgroup
 * per whole tile or piece.  The pieces of a tile are parked in the workspace and added up, in list order, by the
 * workgroup that arrives last, so results are deterministic (they differ from the plain launch in the last bits
 * of fp32 partial sums only).  For tile lists the item table of the launch is built on the device from the list
 * lengths by a one-workgroup kernel ahead of the attention kernel; dense attention needs no table.  A null ptr,
 * a workspace too small for a slot pair per compute unit, or sizes that leave every query tile whole give the
 * plain launch.  Launches that share a workspace must not overlap in time (one workspace per stream).
 * min_share_tiles / min_piece_tiles (0 = defaults 8 / 4, in 64-key tiles): the smallest share, and the
 * smallest piece a query tile may be cut into.
 * The reference has no counterpart: its kernels launch one program per 64-row query tile
 * (kernels/sparse_attn/triton/attn_dense.py:205-206, attn_csp.py:236-237).
 */
typedef struct {
  void* ptr;
  int64_t bytes;
  int min_share_tiles;
  int min_piece_tiles;
} lvar_workspace_t;

/* Bytes of a workspace that lets every balanced launch of the current device use all its slots
 * (head_dim 64 or 128; head_dim 256 has no balanced launch and gets the 4 KiB minimum), or a negative LVAR_E* code. */
int64_t lvar_attn_workspace_bytes(int head_dim);

/* Shares (resident workgroup slots) that a *_ws_fwd launch of these sizes is planned for as a balanced launch on the
 * current device, 0 if it would run as the plain launch.  For dense attention (kind 0) the answer is the launch's own
 * decision; for tile lists (kinds 1 and 2) it is an upper bound: the kernel looks at the real list lengths and leaves
 * every query tile whole (the plain launch's work split) when no list is long enough to cut.  kind 0 = dense, 1 = block list (block_k 64, 128 or 256, list_len = nk_max; group_rows is only looked at for the value 64: query blocks of 64 rows always run as the plain launch),
 * 2 = token list (group_rows, list_len = idx_row_stride).  Pure planning: nothing is launched. */
int lvar_attn_balanced_workgroups(int kind, int group_rows, int block_k, int B, int H, int Lq, int Lk, int list_len,
                                  int head_dim, lvar_workspace_t workspace);

/* Library version (major*10000 + minor*100 + patch) and the gfx target it was built for. */
int lvar_version(void);
const char* lvar_target_arch(void);
const char* lvar_status_string(int status);

/*
 * Dense flash-attention forward, o = softmax(q k^T scale) v, plus (M, L).
 * Replaces torch.ops.chipmunk.dense_attn (kernels/chipmunk/csrc/chipmunk.cu:57,
 * kernels/chipmunk/csrc/attn/dense_attn.cu:248-372) and sattn_triton.dense_attn
 * (kernels/sparse_attn/triton/attn_dense.py:186-231).
 * LSE2, if not NULL, receives the base-2 log-sum-exp M + log2(L) (fp32 [B,H,Lq]), the form the
 * colsum entry point consumes.  o may be NULL (statistics only); M, L and LSE2 may each be NULL.
 * head_dim in {64, 128, 256} (256: one wave per SIMD with 512 registers and 128 KiB of LDS per workgroup, always
 * the plain launch; built for coverage of the reference's Triton range, kernels/sparse_attn/triton/
 * attn_dense_colsum.py:246, not tuned).  This holds for every attention, colsum and window-score entry point
 * below except the static-scratch one.  Grouped-query attention: k and v hold kv_heads heads, H a multiple of it, and query
 * head h reads K/V head h / (H / kv_heads) (the layout of the reference's expansion, kernels/sparse_attn/
 * sparse_attn_ops.py:228-233; kernels/chipmunk/csrc/attn/dense_colsum_attn.cu:386-387); kv_heads = H otherwise.
 */
int lvar_dense_attn_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o,
                        float* M, float* L, float* LSE2,
                        int B, int H, int kv_heads, int Lq, int Lk, int head_dim,
                        float scale, void* stream);

/* lvar_dense_attn_fwd with a partial-result workspace (see lvar_workspace_t); o must not be NULL for the
 * workspace to be used. */
int lvar_dense_attn_ws_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o,
                           float* M, float* L, float* LSE2,
                           int B, int H, int kv_heads, int Lq, int Lk, int head_dim,
                           float scale, lvar_workspace_t workspace, void* stream);

/*
 * Dense flash-attention forward returning the per-row constant of the reference's native op:
 * rcp[b,h,i] = 1 / (2^M * L) (fp32 contiguous [B,H,Lq]), the `l_vec` that torch.ops.chipmunk.dense_attn
 * returns beside o (kernels/chipmunk/csrc/attn/dense_attn.cu:227-230, schema at chipmunk.cu:57) and that
 * torch.ops.chipmunk.dense_colsum_attn takes as its fourth argument.  o and rcp must not be NULL.
 */
int lvar_dense_attn_rcp_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o, float* rcp,
                            int B, int H, int kv_heads, int Lq, int Lk, int head_dim,
                            float scale, void* stream);

/*
 * Colsum given the row statistics: cs[b,h,g,n] = sum_{i in group g} exp2(q_i.k_n*scale*log2e - lse2_i),
 * lse2 = M + log2(L) (fp32 contiguous [B,H,Lq], as written by lvar_dense_attn_fwd), groups of
 * q_group_size consecutive query rows (a multiple of 32), rows >= Lq add zero.
 * cs is fp32 contiguous [B,H,G,Lk], G = ceil(Lq/q_group_size); every element is written exactly once
 * (no atomics, no pre-zeroing, deterministic).  block_sums, if not NULL, receives the sums of cs over
 * blocks of 64 consecutive keys, fp32 contiguous [B,H,G,ceil(Lk/64)] (ragged last block).
 * Replaces pass 2 of _full_attn_fwd (kernels/sparse_attn/triton/attn_dense_colsum.py:216-231)
 * and torch.ops.chipmunk.dense_colsum_attn (kernels/chipmunk/csrc/chipmunk.cu:58,
 * kernels/chipmunk/csrc/attn/dense_colsum_attn.cu:355-522), which takes the same precomputed
 * per-row constant as its fourth argument.  k holds kv_heads heads (grouped-query attention as in
 * lvar_dense_attn_fwd; the column sums stay per query head).
 */
int lvar_colsum_fwd(lvar_tensor_t q, lvar_tensor_t k, const float* lse2, float* cs, float* block_sums,
                    int B, int H, int kv_heads, int Lq, int Lk, int head_dim, int q_group_size,
                    float scale, void* stream);

/*
 * Column-sparse (token-list) attention:
 *   o[b,h,i,:] = o_accum[b,h,i,:] + o_scale * softmax(q_i k[idx]^T scale) v[idx],
 *   idx = indices[b,h,g,0:counts[b,h,g]],  g = i / group_rows,
 * with multiset semantics (a repeated index is attended twice).  indices is int32
 * [B,H,G,idx_row_stride] (row stride in elements, >= max count), counts int32 [B,H,G]
 * contiguous, clamped to [0, idx_row_stride].  Indices outside [0,Lk) are clamped.  count == 0 leaves o = o_accum,
 * M = -inf, L = 1.  o_accum may be NULL (treated as zero) and may alias o.
 * group_rows (query rows sharing one list; the reference uses 192) must be a multiple of 64 or of 96, else
 * LVAR_EUNSUPPORTED.  Gathered rows are addressed with a 24-bit multiply: Lk <= 2^24 and K/V row strides
 * below 2^23 elements, else LVAR_EUNSUPPORTED.  A count that is not a multiple of 64 is honoured exactly:
 * the last tile is masked at the count (the reference attends whole 64-entry tiles, attn_csp.py:53-70,
 * and therefore requires counts that are multiples of 64).
 * Replaces sattn_triton.csp_attn (kernels/sparse_attn/triton/attn_csp.py:215-265) and
 * torch.ops.chipmunk.csp_attn (kernels/chipmunk/csrc/chipmunk.cu:59,
 * kernels/chipmunk/csrc/attn/csp_attn.cu:318-433).
 */
int lvar_csp_attn_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v,
                      lvar_tensor_t o_accum, lvar_tensor_t o, float* M, float* L,
                      const int32_t* indices, const int32_t* counts,
                      int G, int64_t idx_row_stride, int group_rows,
                      int B, int H, int Lq, int Lk, int head_dim,
                      float o_scale, float scale, void* stream);

/* lvar_csp_attn_fwd with a partial-result workspace (see lvar_workspace_t). */
int lvar_csp_attn_ws_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v,
                         lvar_tensor_t o_accum, lvar_tensor_t o, float* M, float* L,
                         const int32_t* indices, const int32_t* counts,
                         int G, int64_t idx_row_stride, int group_rows,
                         int B, int H, int Lq, int Lk, int head_dim,
                         float o_scale, float scale, lvar_workspace_t workspace, void* stream);

/*
 * Token-list attention of a sparse step with the O-cache resampled in the epilogue:
 *   o[b,h,i,:] = bilinear(o_cache[b,h])(y_i, x_i) + o_scale * softmax(q_i k[idx]^T scale) v[idx],
 * where o_cache [B,H,src_side*src_side,head_dim] (bf16) is the cached attention output of a coarser
 * src_side x src_side token grid, the Lq = dst_side*dst_side queries form a dst_side x dst_side grid
 * (i = y_i*dst_side + x_i), and the resampling uses half-pixel centres with edge clamp
 * (source coordinate max(0, (t+0.5)*src_side/dst_side - 0.5): torch's bilinear, align_corners=False).
 * The four taps are read in the attention epilogue and combined in fp32, so the upsampled cache
 * is never written to memory and o is rounded once.  Other arguments as lvar_csp_attn_fwd.
 * Replaces upsample_Ocache(...).to(v.dtype) followed by csp_attn(q,k,v,scale,inds,counts,o,1)
 * (models/sparvar/sparse_attn.py:324-362, 1129-1142).
 */
int lvar_csp_attn_upsample_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v,
                               lvar_tensor_t o_cache, int src_side, int dst_side,
                               lvar_tensor_t o, float* M, float* L,
                               const int32_t* indices, const int32_t* counts,
                               int G, int64_t idx_row_stride, int group_rows,
                               int B, int H, int Lq, int Lk, int head_dim,
                               float o_scale, float scale, void* stream);

/* lvar_csp_attn_upsample_fwd with a partial-result workspace (see lvar_workspace_t). */
int lvar_csp_attn_upsample_ws_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v,
                                  lvar_tensor_t o_cache, int src_side, int dst_side,
                                  lvar_tensor_t o, float* M, float* L,
                                  const int32_t* indices, const int32_t* counts,
                                  int G, int64_t idx_row_stride, int group_rows,
                                  int B, int H, int Lq, int Lk, int head_dim,
                                  float o_scale, float scale, lvar_workspace_t workspace, void* stream);

/*
 * Block-sparse attention over a compacted per-query-block list of key blocks in the flex
 * BlockMask layout consumed by SparseFlexAttn (models/sparvar/basic_sparvar.py:55-72,187-194):
 * kv_num_blocks int32 [B,H,nQ] (stride_nb_b, stride_nb_h, 1), kv_indices int32
 * [B,H,nQ,nk_max] (stride_ki_b, stride_ki_h, stride_ki_q, 1); a stride of 0 broadcasts.
 * kv_num_blocks entries are clamped to [0, nk_max].
 * block_q = 64 or a multiple of 128, block_k in {64, 128, 256}; edge blocks are clipped to Lq / Lk.  Query blocks of
 * 128 rows are the fast shape (one 4-wave workgroup per block); 64-row blocks run as 2-wave workgroups (the 64 x 64
 * blocks of the reference's small configurations), larger ones as several 128-row workgroups that share a list.
 * A query block with no key block yields o = 0, M = -inf, L = 1.
 */
int lvar_block_sparse_attn_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o,
                               float* M, float* L,
                               const int32_t* kv_num_blocks, int64_t stride_nb_b, int64_t stride_nb_h,
                               const int32_t* kv_indices, int64_t stride_ki_b, int64_t stride_ki_h,
                               int64_t stride_ki_q, int nk_max,
                               int block_q, int block_k,
                               int B, int H, int Lq, int Lk, int head_dim,
                               float scale, void* stream);

/* lvar_block_sparse_attn_fwd with a partial-result workspace (see lvar_workspace_t). */
int lvar_block_sparse_attn_ws_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o,
                                  float* M, float* L,
                                  const int32_t* kv_num_blocks, int64_t stride_nb_b, int64_t stride_nb_h,
                                  const int32_t* kv_indices, int64_t stride_ki_b, int64_t stride_ki_h,
                                  int64_t stride_ki_q, int nk_max,
                                  int block_q, int block_k,
                                  int B, int H, int Lq, int Lk, int head_dim,
                                  float scale, lvar_workspace_t workspace, void* stream);

/*
 * lvar_block_sparse_attn_ws_fwd without the workspace argument: the partial-result workspace is a buffer of
 * LVAR_STATIC_SCRATCH_BYTES that lives inside the library (one copy per GPU, held until the process ends), so this
 * entry point allocates nothing and takes no memory beyond the inputs and outputs from the caller.  It has no
 * counterpart in the reference; it is for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  Same arguments, results and balanced-launch
 * rule as lvar_block_sparse_attn_ws_fwd given a workspace of LVAR_STATIC_SCRATCH_BYTES; arguments are checked before the
 * buffer is looked at, so a refused call has not touched it.
 * Limits: B * H * ceil(Lq / 128) (ceil(Lq / 64) for 64-row query blocks) <= LVAR_STATIC_MAX_QUERY_TILES and head_dim <= 128, else LVAR_ETOOBIG (larger
 * launches have enough query tiles to fill the chip: use lvar_block_sparse_attn_fwd).  All calls on one GPU share
 * that GPU's buffer: calls that overlap in time on one GPU (different streams or threads) race.
 */
#define LVAR_STATIC_SCRATCH_BYTES (34ll << 20)
#define LVAR_STATIC_MAX_QUERY_TILES 1024
int lvar_block_sparse_attn_static_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o,
                                      float* M, float* L,
                                      const int32_t* kv_num_blocks, int64_t stride_nb_b, int64_t stride_nb_h,
                                      const int32_t* kv_indices, int64_t stride_ki_b, int64_t stride_ki_h,
                                      int64_t stride_ki_q, int nk_max,
                                      int block_q, int block_k,
                                      int B, int H, int Lq, int Lk, int head_dim,
                                      float scale, void* stream);

/*
 * Block-list build: for every (batch, head, query block) row of block_scores (fp32 contiguous
 * [B,H,nQ,nK], e.g. the block sums of lvar_colsum_fwd with q_group_size = block_q) keep the blocks set
 * in base_mask (uint8 [nQ,nK], shared by all batches and heads, may be NULL) plus the best-scoring
 * other blocks until `target` blocks are kept (all base blocks are kept even beyond target), and
 * write the ascending compacted list: kv_num_blocks int32 [B,H,nQ], kv_indices int32 [B,H,nQ,nK]
 * (unused tail zero).  Ties go to the smaller block index (stable descending order), so the lists are
 * a pure function of the scores.  nK <= 2048.
 * Does on the GPU what the reference does with torch.topk plus list padding
 * (models/sparvar/sparse_attn.py:1012-1036) and what its unused mask_to_indices / topk_indices
 * helpers compact (kernels/chipmunk/csrc/indexed_io/mask_to_indices.cu:21-97, topk_indices.cu:26-145).
 */
int lvar_block_topk_lists(const float* block_scores, const uint8_t* base_mask,
                          int32_t* kv_num_blocks, int32_t* kv_indices,
                          int B, int H, int nQ, int nK, int target, void* stream);

/*
 * Exact top-k key selection per row: for each of `rows` rows of `scores` (fp32, row stride
 * score_row_stride >= Lk elements; e.g. the [B*H*G, Lk] view of the column sums) write the columns
 * of the k largest values, in ASCENDING column order, to indices[row, 0:k] (row stride
 * idx_row_stride >= k; columns [k, zero_to) are set to 0, zero_to <= idx_row_stride, the rest is left untouched)
 * and, if counts is not NULL, k to counts[row].
 * Ties at the k-th value go to the smaller column, so the selected SET equals that of a stable
 * descending sort and is a pure function of the scores (-0.0 and +0.0 tie; NaN scores are not supported).
 * Radix select, no sort: rows of up to 16384 columns are read once and held in registers, longer ones
 * are re-read from L2 in every pass.  Replaces `torch.topk(bs, k=indices_count, dim=-1).indices` of the full step
 * (models/sparvar/sparse_attn.py:1012-1036), which returns the same set ordered by value, and the
 * reference's unused quantile kernel (kernels/chipmunk/csrc/indexed_io/topk_indices.cu:26-145).
 */
int lvar_topk_token_lists(const float* scores, int64_t score_row_stride,
                          int32_t* indices, int64_t idx_row_stride, int32_t* counts,
                          int rows, int Lk, int k, int zero_to, void* stream);

/*
 * Sparse-step key list in one launch: for every (batch*head) slice bh < BH and query group g < Gk of
 * the current scale,
 *   out[bh,g, j]         = clamp(src[bh, gS(g), j / rep], 0, Lk-1)      for j < count
 *   out[bh,g, count + j] = local_indices[g, j]                            for j < local_count
 *   out_counts[bh,g]     = count + local_count                            (if out_counts != NULL)
 * where gS(g) = clamp(rint((g + 0.5) / Gk * Gs - 0.5), 0, Gs-1) in fp32 with round-half-to-even,
 * rep = 1 if src_len >= count else ceil(count / src_len).  src_indices is int32 [BH, Gs, src_row_stride]
 * (first src_len columns valid), local_indices int64 [Gk, local_row_stride] (may be NULL with
 * local_count = 0), out_indices int32 [BH*Gk, out_row_stride >= count + local_count]; columns
 * [count + local_count, zero_to) of every output row are set to 0 (zero_to <= out_row_stride, 0 = untouched).
 * Replaces map_inds_counts_across_scales (models/sparvar/sparse_attn.py:366-421) followed by the
 * top-k-then-local concatenation and padding of the sparse step (models/sparvar/sparse_attn.py:1096-1121).
 */
int lvar_remap_concat_lists(const int32_t* src_indices, int64_t src_row_stride, int src_len,
                            const int64_t* local_indices, int64_t local_row_stride, int local_count,
                            int32_t* out_indices, int64_t out_row_stride, int32_t* out_counts,
                            int BH, int Gs, int Gk, int count, int Lk, int zero_to, void* stream);

/*
 * Mask compaction: for each of `rows` rows of a uint8 mask (row stride mask_row_stride >= n) write the
 * ascending columns of its non-zero entries to indices[row, :] (row stride idx_row_stride >= n), round
 * the count up to a multiple of `multiple_of` (capped at n) by appending the lowest zero columns, zero
 * the rest of the n columns, and store the padded count in counts[row].  With multiple_of = 1 and a
 * block mask this yields flex BlockMask lists (kv_num_blocks / kv_indices).  Counterpart of the
 * reference's mask_to_indices (kernels/chipmunk/csrc/indexed_io/mask_to_indices.cu:21-97) with two
 * stated differences: the list is in ascending column order (the reference writes a thread-strided order;
 * the SET is the same), and the padded count is capped at n (the reference's rounded count can exceed the
 * row, mask_to_indices.cu:62,93).
 */
int lvar_mask_to_lists(const uint8_t* mask, int64_t mask_row_stride,
                       int32_t* indices, int64_t idx_row_stride, int32_t* counts,
                       int rows, int n, int multiple_of, void* stream);

/*
 * Window-query key scores: for every (batch, head)
 *   s[n]      = scale * sum_{i < n_window} q[row(window_keys[i])] . k[n],   row(x) = clamp(x - (Lk - Lq), 0, Lq-1),
 *   s[n]      = -inf at the window's own keys n in window_keys,
 *   scores[n] = pool_{|m - n| <= pool_kernel_size/2} s[m]   (average with zero padding, or maximum),
 *   scores[n] = -inf again at the window's own keys.
 * q [B,H,Lq,d] holds the queries of the newest Lq of the Lk keys; window_keys is int64 [B,H,n_window]
 * (key positions, repeats count twice), scores fp32 contiguous [B,H,Lk]; pool_kernel_size odd, <= 33.
 * One pass over K with the summed window query (fp32).  Replaces the query gather, the
 * [n_window x Lk] matmul, masking, sum and pooling of ScaleKV's cache selection
 * (models/scalekv/scale_kv.py:233-262), which rounds every logit to bf16 before summing.
 */
int lvar_window_key_scores(lvar_tensor_t q, lvar_tensor_t k, const int64_t* window_keys, int n_window,
                           float* scores, int B, int H, int Lq, int Lk, int head_dim,
                           int pool_kernel_size, int max_pool, float scale, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LVAR_SPARSE_ATTN_H */
