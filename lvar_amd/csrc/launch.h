// Host-side launch interface shared by the kernel translation units and the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <atomic>
#include "common.h"
#include "../../include/lvar_sparse_attn.h"

namespace lvar {

enum { MODE_BLOCK = 1, MODE_GATHER = 2 };  // dense attention = MODE_BLOCK with a null list

struct AttnParams {
  const bf16_t *q, *k, *v;
  bf16_t* o;
  const bf16_t* o_accum;
  float *M, *L, *LSE2;
  float* RCP;     // optional per-row constant 1 / (2^M * L)
  int64_t q_sb, q_sh, q_sr;
  int64_t k_sb, k_sh, k_sr;
  int64_t v_sb, v_sh, v_sr;
  int64_t o_sb, o_sh, o_sr;
  int64_t oa_sb, oa_sh, oa_sr;
  int B, H, Lq, Lk;
  int kv_group;   // query heads per key/value head (1 = as many K/V heads as query heads)
  float c;        // softmax scale * log2(e)
  float o_scale;  // epilogue factor of the token-list variant
  // key-tile list: kv_indices / kv_num_blocks (block list) or indices / counts (token list)
  const int32_t* list;
  const int32_t* cnt;
  int64_t list_sb, list_sh, list_sg;
  int64_t cnt_sb, cnt_sh;
  int list_len;    // entries available per list row; counts are clamped to it
  int group_rows;  // query rows sharing one list
  int sub_shift;   // log2(64-key tiles per key block)
  int up_src, up_dst;  // token-list variant: o_accum is an up_src x up_src token grid, bilinearly
                       // resampled to the up_dst x up_dst grid of the queries (0 = o_accum has Lq rows)
  int nqt, total_wg;
  // balanced launch: workspace handed in by the caller (null = plain launch).  The launch code fills in sk_wgs
  // (0 = plain launch after all), sk_counters (per-query-tile arrival counters, all zero between launches) and
  // sk_slots (2 * sk_wgs slots of partial results).
  void* sk_ws;
  int64_t sk_ws_bytes;
  int* sk_counters;
  float* sk_slots;
  int sk_wgs;        // shares of the balanced launch (resident workgroup slots it is planned for)
  const int* sk_plan;  // item table (plan_kernel), from the caller or built in the workspace; unused for dense attention
  int sk_uniform_n;  // dense attention: pieces per query tile (0 = use the table)
  int sk_min_share;  // list entries a workgroup should at least get (fewer workgroups take part otherwise)
  int sk_min_piece;  // a cut closer than this many list entries to a query-tile boundary is moved onto it
};

struct ColsumParams {
  const bf16_t *q, *k;
  const float* lse2;  // base-2 log-sum-exp per query row, M + log2(L)
  float* cs;
  float* bs;          // optional per-64-key block sums [B,H,G,ceil(Lk/64)]
  int64_t q_sb, q_sh, q_sr;
  int64_t k_sb, k_sh, k_sr;
  int B, H, Lq, Lk, G;
  int kv_group;   // query heads per key head
  int group_rows;
  float c;
  int nkt, nkb, total_wg;
  int q_splits, split_rows;   // ranges of query groups per key tile, rows per range (set at launch)
};

struct MaskListParams {
  const float* scores;     // [rows, nK]
  const uint8_t* base;     // [nQ, nK] or null
  int32_t* kv_num_blocks;  // [rows]
  int32_t* kv_indices;     // [rows, nK]
  int rows, nQ, nK, target;
};

struct TopkListParams {
  const float* scores;  // [rows, n] with row stride score_stride
  int32_t* indices;     // [rows, >= k] with row stride out_stride
  int32_t* counts;      // [rows] or null
  int64_t score_stride, out_stride;
  int rows, n, k;
  int zero_to;          // columns [k, zero_to) of every index row are set to 0 (0 = left untouched)
};

struct RemapListParams {
  const int32_t* src;    // [BH, Gs, src_stride]
  const int64_t* local;  // [Gk, local_stride] or null
  int32_t* out;          // [BH*Gk, out_stride]
  int32_t* counts;       // [BH*Gk] or null
  int64_t src_stride, local_stride, out_stride;
  int rows, Gs, Gk, cnt, rep, L, Lk;
  int zero_to;           // columns [cnt + L, zero_to) of every output row are set to 0 (0 = left untouched)
};

struct MaskCompactParams {
  const uint8_t* mask;  // [rows, n] with row stride mask_stride
  int32_t* indices;     // [rows, out_len] with row stride out_stride
  int32_t* counts;      // [rows]
  int64_t mask_stride, out_stride;
  int rows, n, out_len, multiple_of, zero_tail;
};

// Raises a kernel's dynamic-LDS limit once per device (the attribute is kept per device); `done` is a
// per-kernel bit set of the devices already handled.  Safe to call from several host threads.
inline bool ensure_lds_limit(const void* kernel, int bytes, std::atomic<uint64_t>& done) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return false;
  const uint64_t bit = 1ull << (dev & 63);
  if (done.load(std::memory_order_acquire) & bit) return true;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) return false;
  done.fetch_or(bit, std::memory_order_release);
  return true;
}

struct WinScoreParams {
  const bf16_t *q, *k;
  const int64_t* window;  // [B*H, W] key positions of the window tokens
  float* out;             // [B*H, Lk]
  int64_t q_sb, q_sh, q_sr, k_sb, k_sh, k_sr;
  int B, H, Lq, Lk, W, ksize, maxpool, nchunks, total_wg;
  float scale;
};

int launch_window_scores(const WinScoreParams& p, int head_dim, hipStream_t s);
int launch_topk_token_lists(const TopkListParams& p, hipStream_t s);
int launch_remap_concat_lists(const RemapListParams& p, hipStream_t s);
int launch_mask_to_lists(const MaskCompactParams& p, hipStream_t s);
int launch_block_topk_lists(const MaskListParams& p, hipStream_t s);
int launch_attn(const AttnParams& p, int head_dim, int mode, bool accum, bool lse_only, int nwaves, hipStream_t s);
int launch_colsum(const ColsumParams& p, int head_dim, hipStream_t s);
int sk_slot_floats(int head_dim, int mode, int nwaves);
int sk_plan(int total_wg, int nwaves, int slot_floats, int64_t per_tile, int sub, int64_t ws_bytes, int& min_share, int& min_piece);
int sk_dense_pieces(int total_wg, int T, int sk_wgs, int min_share, int min_piece);   // dense attention: pieces per query tile, 0 = plain launch
int device_cus();   // compute units of the current device (cached), 0 on error
constexpr int64_t SK_COUNTER_BYTES = 4096;   // head of the workspace: one int32 arrival counter per query tile
int64_t sk_plan_bytes(int P);                // then the item table, then 2 * P slots

}  // namespace lvar
