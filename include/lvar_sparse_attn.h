/*
 * C ABI of the MI355X (gfx950) sparse-attention library: dense / block-sparse /
 * column-sparse flash-attention forward and the colsum kernel.
 *
 * Every entry point takes raw device pointers, sizes and element strides, launches
 * asynchronously on the HIP stream it is given (a hipStream_t passed as void*, NULL =
 * the default stream) and returns 0 or a negative LVAR_E* code.  No entry point
 * allocates, frees or synchronises.  Tensors are bf16 with unit stride on the head
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
#define LVAR_EUNSUPPORTED (-2) /* head_dim or block shape not built */
#define LVAR_ELAUNCH (-3)      /* HIP reported a launch error */

/* Tensor view: base pointer plus element strides of a [B,H,rows,d] bf16 tensor (d stride 1). */
typedef struct {
  const void* ptr;
  int64_t stride_b;
  int64_t stride_h;
  int64_t stride_row;
} lvar_tensor_t;

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
 * head_dim in {64, 128}.
 */
int lvar_dense_attn_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o,
                        float* M, float* L, float* LSE2,
                        int B, int H, int Lq, int Lk, int head_dim,
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
 * per-row constant as its fourth argument.
 */
int lvar_colsum_fwd(lvar_tensor_t q, lvar_tensor_t k, const float* lse2, float* cs, float* block_sums,
                    int B, int H, int Lq, int Lk, int head_dim, int q_group_size,
                    float scale, void* stream);

/*
 * Column-sparse (token-list) attention:
 *   o[b,h,i,:] = o_accum[b,h,i,:] + o_scale * softmax(q_i k[idx]^T scale) v[idx],
 *   idx = indices[b,h,g,0:counts[b,h,g]],  g = i / group_rows,
 * with multiset semantics (a repeated index is attended twice).  indices is int32
 * [B,H,G,idx_row_stride] (row stride in elements, >= max count), counts int32 [B,H,G]
 * contiguous, clamped to [0, idx_row_stride].  Indices outside [0,Lk) are clamped.  count == 0 leaves o = o_accum,
 * M = -inf, L = 1.  o_accum may be NULL (treated as zero) and may alias o.
 * group_rows must be a multiple of 32 (the reference uses 192).
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

/*
 * Block-sparse attention over a compacted per-query-block list of key blocks in the flex
 * BlockMask layout consumed by SparseFlexAttn (models/sparvar/basic_sparvar.py:55-72,187-194):
 * kv_num_blocks int32 [B,H,nQ] (stride_nb_b, stride_nb_h, 1), kv_indices int32
 * [B,H,nQ,nk_max] (stride_ki_b, stride_ki_h, stride_ki_q, 1); a stride of 0 broadcasts.
 * kv_num_blocks entries are clamped to [0, nk_max].
 * block_q in {128}, block_k in {64, 128}; edge blocks are clipped to Lq / Lk.
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

#ifdef __cplusplus
}
#endif
#endif /* LVAR_SPARSE_ATTN_H */
