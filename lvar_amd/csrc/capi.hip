// extern "C" entry points declared in include/lvar_sparse_attn.h: argument validation and
// parameter packing; all device work is in attn_fwd.hip / colsum.hip.
#include <cmath>
#include "../../include/lvar_sparse_attn.h"
#include "launch.h"

using namespace lvar;

// Scratch of lvar_block_sparse_attn_static_fwd: arrival counters, item table and partial-result slots of a balanced
// launch with one share per compute unit of a 256-CU part at head_dim 128 (4 KiB + 41 KiB + 2 * 256 * 67 KiB).
// Every GPU the library runs on holds its own copy, at its own address, until the process ends.  In host code the
// name is only a handle for hipGetSymbolAddress: the address that kernels and fills take is looked up per device.
constexpr int64_t kStaticScratchBytes = 34ll << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

// Device address of this GPU's copy of `scratch`, looked up once per device with that device current.
void* static_scratch() {
  static std::atomic<void*> ptrs[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  void* ptr = ptrs[dev].load(std::memory_order_acquire);
  if (ptr) return ptr;
  if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return nullptr;
  ptrs[dev].store(ptr, std::memory_order_release);
  return ptr;
}

constexpr float kLog2e = 1.4426950408889634f;

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// rows are read/written with 16-byte vector accesses: base and every stride must keep them aligned
bool view_ok(const lvar_tensor_t& t) {
  return t.ptr && aligned16(t.ptr) && t.stride_b % 8 == 0 && t.stride_h % 8 == 0 && t.stride_row % 8 == 0;
}

// K/V rows are addressed with 32-bit byte offsets inside one (batch, head) slice.  The fills of a ragged last tile
// (or of the last tiles of a 256-key block) form offsets of up to 319 rows beyond the last key before the buffer
// descriptor's bound turns them into zeros: those offsets must not wrap either.
// (Token lists clamp every gathered row to the last key: pad_rows = 0.)
bool kv_span_ok(const lvar_tensor_t& t, int Lk, int head_dim, int pad_rows = 320) {
  return t.stride_row > 0 && (double)t.stride_row * 2.0 * ((double)Lk + pad_rows) + head_dim * 2.0 < 2147483647.0;
}

bool shape_ok(int B, int H, int Lq, int Lk, float scale) {
  return B > 0 && H > 0 && Lq > 0 && Lk > 0 && std::isfinite(scale) && scale > 0.f;
}

// Waves per workgroup of the token-list kernel, by the number of query rows that share a list.  A multiple
// of 192 rows (the reference's group size) runs as one 8-wave workgroup per 192 rows: six computing waves
// and two waves that only read the list and issue the K/V fills (they take the two wave slots that six
// 256-register waves leave free on a CU).  Other multiples of 96 or 64 rows run as 3- or 2-wave workgroups
// that each fetch for themselves.  0 = unsupported group size.
int gather_waves(int group_rows) {
  if (group_rows % 192 == 0) return 8;
  if (group_rows % 96 == 0) return 3;
  if (group_rows % 64 == 0) return 2;
  return 0;
}

void fill_qkv(AttnParams& p, const lvar_tensor_t& q, const lvar_tensor_t& k, const lvar_tensor_t& v) {
  p.q = (const bf16_t*)q.ptr; p.q_sb = q.stride_b; p.q_sh = q.stride_h; p.q_sr = q.stride_row;
  p.k = (const bf16_t*)k.ptr; p.k_sb = k.stride_b; p.k_sh = k.stride_h; p.k_sr = k.stride_row;
  p.v = (const bf16_t*)v.ptr; p.v_sb = v.stride_b; p.v_sh = v.stride_h; p.v_sr = v.stride_row;
}

// A workspace makes the launch eligible for the balanced grid; alignment and size are checked here, whether
// it is used is decided at launch (launch_one in attn_fwd.hip).
bool attach_workspace(AttnParams& p, const lvar_workspace_t* ws) {
  if (!ws || !ws->ptr) return true;
  if ((reinterpret_cast<uintptr_t>(ws->ptr) & 255u) != 0 || ws->bytes < 0 || ws->min_share_tiles < 0 || ws->min_piece_tiles < 0) return false;
  p.sk_ws = ws->ptr; p.sk_ws_bytes = ws->bytes;
  p.sk_min_share = ws->min_share_tiles; p.sk_min_piece = ws->min_piece_tiles;
  return true;
}

}  // namespace

extern "C" {

int lvar_version(void) { return 200; }
const char* lvar_target_arch(void) { return "gfx950"; }

const char* lvar_status_string(int status) {
  switch (status) {
    case LVAR_OK: return "ok";
    case LVAR_EINVAL: return "invalid argument (size, null/misaligned pointer, stride or scale)";
    case LVAR_EUNSUPPORTED: return "unsupported head_dim, block shape or query-group size";
    case LVAR_ELAUNCH: return "HIP launch failed";
    case LVAR_ETOOBIG: return "problem larger than the static scratch buffer allows (use the workspace entry point)";
    default: return "unknown status";
  }
}

static int dense_common(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o, float* M, float* L,
                        float* LSE2, float* RCP, int B, int H, int kv_heads, int Lq, int Lk, int head_dim, float scale,
                        const lvar_workspace_t* ws, void* stream) {
  if (!shape_ok(B, H, Lq, Lk, scale) || !view_ok(q) || !view_ok(k)) return LVAR_EINVAL;
  if (kv_heads <= 0 || H % kv_heads != 0) return LVAR_EINVAL;
  const bool lse_only = (o.ptr == nullptr);
  if (!kv_span_ok(k, Lk, head_dim) || (!lse_only && !kv_span_ok(v, Lk, head_dim))) return LVAR_EINVAL;
  if (!lse_only && (!view_ok(v) || !view_ok(o) || o.stride_row <= 0)) return LVAR_EINVAL;
  if (lse_only && !((M && L) || LSE2 || RCP)) return LVAR_EINVAL;
  AttnParams p{};
  fill_qkv(p, q, k, lse_only ? k : v);
  p.o = (bf16_t*)o.ptr; p.o_sb = o.stride_b; p.o_sh = o.stride_h; p.o_sr = o.stride_row;
  p.M = M; p.L = L; p.LSE2 = LSE2; p.RCP = RCP;
  p.B = B; p.H = H; p.Lq = Lq; p.Lk = Lk; p.kv_group = H / kv_heads;
  p.c = scale * kLog2e; p.o_scale = 1.f;
  p.list = nullptr; p.cnt = nullptr; p.group_rows = 128; p.sub_shift = 0;
  if (!attach_workspace(p, ws)) return LVAR_EINVAL;
  return launch_attn(p, head_dim, MODE_BLOCK, false, lse_only, 4, (hipStream_t)stream);
}

int lvar_dense_attn_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o, float* M, float* L,
                        float* LSE2, int B, int H, int kv_heads, int Lq, int Lk, int head_dim, float scale, void* stream) {
  return dense_common(q, k, v, o, M, L, LSE2, nullptr, B, H, kv_heads, Lq, Lk, head_dim, scale, nullptr, stream);
}

int lvar_dense_attn_ws_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o, float* M, float* L,
                           float* LSE2, int B, int H, int kv_heads, int Lq, int Lk, int head_dim, float scale,
                           lvar_workspace_t workspace, void* stream) {
  return dense_common(q, k, v, o, M, L, LSE2, nullptr, B, H, kv_heads, Lq, Lk, head_dim, scale, &workspace, stream);
}

int lvar_dense_attn_rcp_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o, float* rcp,
                            int B, int H, int kv_heads, int Lq, int Lk, int head_dim, float scale, void* stream) {
  if (!o.ptr || !rcp) return LVAR_EINVAL;
  return dense_common(q, k, v, o, nullptr, nullptr, nullptr, rcp, B, H, kv_heads, Lq, Lk, head_dim, scale, nullptr, stream);
}

int lvar_colsum_fwd(lvar_tensor_t q, lvar_tensor_t k, const float* lse2, float* cs, float* block_sums,
                    int B, int H, int kv_heads, int Lq, int Lk, int head_dim, int q_group_size, float scale, void* stream) {
  if (!shape_ok(B, H, Lq, Lk, scale) || !view_ok(q) || !view_ok(k) || !lse2 || !cs) return LVAR_EINVAL;
  if (kv_heads <= 0 || H % kv_heads != 0) return LVAR_EINVAL;
  if (q_group_size <= 0 || q_group_size % 32 != 0) return LVAR_EINVAL;
  if (!kv_span_ok(q, Lq, head_dim, 0)) return LVAR_EINVAL;
  ColsumParams p{};
  p.q = (const bf16_t*)q.ptr; p.q_sb = q.stride_b; p.q_sh = q.stride_h; p.q_sr = q.stride_row;
  p.k = (const bf16_t*)k.ptr; p.k_sb = k.stride_b; p.k_sh = k.stride_h; p.k_sr = k.stride_row;
  p.lse2 = lse2; p.cs = cs; p.bs = block_sums;
  p.B = B; p.H = H; p.Lq = Lq; p.Lk = Lk; p.kv_group = H / kv_heads;
  p.group_rows = q_group_size;
  p.G = (Lq + q_group_size - 1) / q_group_size;
  p.c = scale * kLog2e;
  return launch_colsum(p, head_dim, (hipStream_t)stream);
}

static int csp_common(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o_accum, int up_src, int up_dst,
                      lvar_tensor_t o, float* M, float* L, const int32_t* indices, const int32_t* counts, int G,
                      int64_t idx_row_stride, int group_rows, int B, int H, int Lq, int Lk, int head_dim,
                      float o_scale, float scale, const lvar_workspace_t* ws, void* stream) {
  if (!shape_ok(B, H, Lq, Lk, scale) || !view_ok(q) || !view_ok(k) || !view_ok(v) || !view_ok(o)) return LVAR_EINVAL;
  if (o.stride_row <= 0 || (o_accum.ptr && (!view_ok(o_accum) || o_accum.stride_row <= 0))) return LVAR_EINVAL;
  if (!kv_span_ok(k, Lk, head_dim, 0) || !kv_span_ok(v, Lk, head_dim, 0)) return LVAR_EINVAL;
  // gathered rows are addressed with a 24-bit multiply: token index and row stride in bytes below 2^24
  if (Lk > (1 << 24) || k.stride_row * 2 >= (1 << 24) || v.stride_row * 2 >= (1 << 24)) return LVAR_EUNSUPPORTED;
  if (!indices || !counts || G <= 0 || idx_row_stride <= 0) return LVAR_EINVAL;
  if (group_rows <= 0 || (int64_t)G * group_rows < Lq) return LVAR_EINVAL;
  AttnParams p{};
  fill_qkv(p, q, k, v);
  p.o = (bf16_t*)o.ptr; p.o_sb = o.stride_b; p.o_sh = o.stride_h; p.o_sr = o.stride_row;
  p.o_accum = (const bf16_t*)o_accum.ptr; p.oa_sb = o_accum.stride_b; p.oa_sh = o_accum.stride_h; p.oa_sr = o_accum.stride_row;
  p.M = M; p.L = L;
  p.B = B; p.H = H; p.Lq = Lq; p.Lk = Lk;
  p.c = scale * kLog2e; p.o_scale = o_scale;
  p.list = indices; p.cnt = counts;
  p.list_sg = idx_row_stride; p.list_sh = (int64_t)G * idx_row_stride; p.list_sb = (int64_t)H * p.list_sh;
  p.cnt_sh = G; p.cnt_sb = (int64_t)H * G;
  p.list_len = (int)(idx_row_stride > 0x7fffffff ? 0x7fffffff : idx_row_stride);
  p.group_rows = group_rows;
  p.up_src = up_src; p.up_dst = up_dst;
  const int nw = gather_waves(group_rows);
  if (nw == 0) return LVAR_EUNSUPPORTED;
  if (!attach_workspace(p, ws)) return LVAR_EINVAL;
  return launch_attn(p, head_dim, MODE_GATHER, true, false, nw, (hipStream_t)stream);
}

int lvar_csp_attn_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o_accum, lvar_tensor_t o,
                      float* M, float* L, const int32_t* indices, const int32_t* counts, int G,
                      int64_t idx_row_stride, int group_rows, int B, int H, int Lq, int Lk, int head_dim,
                      float o_scale, float scale, void* stream) {
  return csp_common(q, k, v, o_accum, 0, 0, o, M, L, indices, counts, G, idx_row_stride, group_rows, B, H, Lq, Lk,
                    head_dim, o_scale, scale, nullptr, stream);
}

int lvar_csp_attn_ws_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o_accum, lvar_tensor_t o,
                         float* M, float* L, const int32_t* indices, const int32_t* counts, int G,
                         int64_t idx_row_stride, int group_rows, int B, int H, int Lq, int Lk, int head_dim,
                         float o_scale, float scale, lvar_workspace_t workspace, void* stream) {
  return csp_common(q, k, v, o_accum, 0, 0, o, M, L, indices, counts, G, idx_row_stride, group_rows, B, H, Lq, Lk,
                    head_dim, o_scale, scale, &workspace, stream);
}

static bool upsample_ok(lvar_tensor_t o_cache, int src_side, int dst_side, int Lq) {
  return o_cache.ptr && src_side > 0 && dst_side > 0 && src_side <= 32768 && dst_side <= 32768 &&
         (int64_t)dst_side * dst_side == Lq;
}

int lvar_csp_attn_upsample_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o_cache,
                               int src_side, int dst_side, lvar_tensor_t o, float* M, float* L,
                               const int32_t* indices, const int32_t* counts, int G, int64_t idx_row_stride,
                               int group_rows, int B, int H, int Lq, int Lk, int head_dim,
                               float o_scale, float scale, void* stream) {
  if (!upsample_ok(o_cache, src_side, dst_side, Lq)) return LVAR_EINVAL;
  return csp_common(q, k, v, o_cache, src_side, dst_side, o, M, L, indices, counts, G, idx_row_stride, group_rows,
                    B, H, Lq, Lk, head_dim, o_scale, scale, nullptr, stream);
}

int lvar_csp_attn_upsample_ws_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o_cache,
                                  int src_side, int dst_side, lvar_tensor_t o, float* M, float* L,
                                  const int32_t* indices, const int32_t* counts, int G, int64_t idx_row_stride,
                                  int group_rows, int B, int H, int Lq, int Lk, int head_dim,
                                  float o_scale, float scale, lvar_workspace_t workspace, void* stream) {
  if (!upsample_ok(o_cache, src_side, dst_side, Lq)) return LVAR_EINVAL;
  return csp_common(q, k, v, o_cache, src_side, dst_side, o, M, L, indices, counts, G, idx_row_stride, group_rows,
                    B, H, Lq, Lk, head_dim, o_scale, scale, &workspace, stream);
}

// argument checks of the block-list entry points (everything but the workspace)
static int block_sparse_check(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o, const int32_t* kv_num_blocks,
                              const int32_t* kv_indices, int nk_max, int block_q, int block_k, int B, int H, int Lq, int Lk,
                              int head_dim, float scale) {
  if (!shape_ok(B, H, Lq, Lk, scale) || !view_ok(q) || !view_ok(k) || !view_ok(v) || !view_ok(o)) return LVAR_EINVAL;
  if (!kv_span_ok(k, Lk, head_dim) || !kv_span_ok(v, Lk, head_dim)) return LVAR_EINVAL;
  if (!kv_num_blocks || !kv_indices || nk_max <= 0 || o.stride_row <= 0) return LVAR_EINVAL;
  // query blocks of 64 rows (two-wave workgroups) or a multiple of 128 rows (128-row workgroups that share a list)
  if ((block_q != 64 && (block_q <= 0 || block_q % 128 != 0)) || (block_k != 64 && block_k != 128 && block_k != 256)) return LVAR_EUNSUPPORTED;
  if (head_dim != 64 && head_dim != 128 && head_dim != 256) return LVAR_EUNSUPPORTED;
  return LVAR_OK;
}

static int block_sparse_common(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o, float* M, float* L,
                               const int32_t* kv_num_blocks, int64_t stride_nb_b, int64_t stride_nb_h,
                               const int32_t* kv_indices, int64_t stride_ki_b, int64_t stride_ki_h,
                               int64_t stride_ki_q, int nk_max, int block_q, int block_k, int B, int H, int Lq, int Lk,
                               int head_dim, float scale, const lvar_workspace_t* ws, void* stream) {
  const int chk = block_sparse_check(q, k, v, o, kv_num_blocks, kv_indices, nk_max, block_q, block_k, B, H, Lq, Lk, head_dim, scale);
  if (chk != LVAR_OK) return chk;
  AttnParams p{};
  fill_qkv(p, q, k, v);
  p.o = (bf16_t*)o.ptr; p.o_sb = o.stride_b; p.o_sh = o.stride_h; p.o_sr = o.stride_row;
  p.M = M; p.L = L;
  p.B = B; p.H = H; p.Lq = Lq; p.Lk = Lk;
  p.c = scale * kLog2e; p.o_scale = 1.f;
  p.list = kv_indices; p.cnt = kv_num_blocks;
  p.list_sb = stride_ki_b; p.list_sh = stride_ki_h; p.list_sg = stride_ki_q;
  p.cnt_sb = stride_nb_b; p.cnt_sh = stride_nb_h;
  p.list_len = nk_max;
  p.group_rows = block_q;
  p.sub_shift = (block_k == 256) ? 2 : (block_k == 128) ? 1 : 0;
  if (!attach_workspace(p, ws)) return LVAR_EINVAL;
  return launch_attn(p, head_dim, MODE_BLOCK, false, false, block_q == 64 ? 2 : 4, (hipStream_t)stream);
}

int lvar_block_sparse_attn_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o, float* M, float* L,
                               const int32_t* kv_num_blocks, int64_t stride_nb_b, int64_t stride_nb_h,
                               const int32_t* kv_indices, int64_t stride_ki_b, int64_t stride_ki_h,
                               int64_t stride_ki_q, int nk_max, int block_q, int block_k, int B, int H, int Lq, int Lk,
                               int head_dim, float scale, void* stream) {
  return block_sparse_common(q, k, v, o, M, L, kv_num_blocks, stride_nb_b, stride_nb_h, kv_indices, stride_ki_b, stride_ki_h,
                             stride_ki_q, nk_max, block_q, block_k, B, H, Lq, Lk, head_dim, scale, nullptr, stream);
}

int lvar_block_sparse_attn_ws_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o, float* M, float* L,
                                  const int32_t* kv_num_blocks, int64_t stride_nb_b, int64_t stride_nb_h,
                                  const int32_t* kv_indices, int64_t stride_ki_b, int64_t stride_ki_h,
                                  int64_t stride_ki_q, int nk_max, int block_q, int block_k, int B, int H, int Lq, int Lk,
                                  int head_dim, float scale, lvar_workspace_t workspace, void* stream) {
  return block_sparse_common(q, k, v, o, M, L, kv_num_blocks, stride_nb_b, stride_nb_h, kv_indices, stride_ki_b, stride_ki_h,
                             stride_ki_q, nk_max, block_q, block_k, B, H, Lq, Lk, head_dim, scale, &workspace, stream);
}

int lvar_attn_balanced_workgroups(int kind, int group_rows, int block_k, int B, int H, int Lq, int Lk, int list_len,
                                  int head_dim, lvar_workspace_t workspace) {
  if (B <= 0 || H <= 0 || Lq <= 0 || Lk <= 0 || (head_dim != 64 && head_dim != 128 && head_dim != 256) || kind < 0 || kind > 2) return LVAR_EINVAL;
  if (!workspace.ptr || head_dim == 256) return 0;   // head_dim 256 always takes the plain launch
  int nwaves = 4, mode = MODE_BLOCK, sub = 0;
  int64_t per_tile = (Lk + 63) / 64;
  if (kind == 1) {
    if (block_k != 64 && block_k != 128 && block_k != 256) return LVAR_EUNSUPPORTED;
    if (group_rows == 64) return 0;   // 64-row query blocks always take the plain launch; any other value: 128-row workgroups
    sub = block_k == 256 ? 2 : block_k == 128 ? 1 : 0;
    per_tile = list_len;
  } else if (kind == 2) {
    nwaves = gather_waves(group_rows);
    if (nwaves == 0) return LVAR_EUNSUPPORTED;
    mode = MODE_GATHER;
    per_tile = (list_len + 63) / 64;
  }
  const int rows = (nwaves == 8 ? 6 : nwaves) * 32;
  const int64_t tiles = (int64_t)B * H * ((Lq + rows - 1) / rows);
  if (tiles > 0x7fffffff) return 0;
  int share = workspace.min_share_tiles, piece = workspace.min_piece_tiles;
  const int P = sk_plan((int)tiles, nwaves, sk_slot_floats(head_dim, mode, nwaves), per_tile, sub, workspace.bytes, share, piece);
  // dense attention: the launch code takes the plain launch when the tiles stay whole (the same decision, shared)
  if (kind == 0 && P > 0 && sk_dense_pieces((int)tiles, (int)per_tile, P, share, piece) == 0) return 0;
  return P;
}

int lvar_block_sparse_attn_static_fwd(lvar_tensor_t q, lvar_tensor_t k, lvar_tensor_t v, lvar_tensor_t o, float* M, float* L,
                                      const int32_t* kv_num_blocks, int64_t stride_nb_b, int64_t stride_nb_h,
                                      const int32_t* kv_indices, int64_t stride_ki_b, int64_t stride_ki_h,
                                      int64_t stride_ki_q, int nk_max, int block_q, int block_k, int B, int H, int Lq, int Lk,
                                      int head_dim, float scale, void* stream) {
  // arguments first: a call that is refused must not have touched the scratch that a launch in flight may be using
  const int st = block_sparse_check(q, k, v, o, kv_num_blocks, kv_indices, nk_max, block_q, block_k, B, H, Lq, Lk, head_dim, scale);
  if (st != LVAR_OK) return st;
  // the scratch holds the counters and the item table of at most LVAR_STATIC_MAX_QUERY_TILES query tiles
  const int wg_rows = block_q == 64 ? 64 : 128;
  const int64_t tiles = (int64_t)B * H * ((Lq + wg_rows - 1) / wg_rows);
  if (tiles > LVAR_STATIC_MAX_QUERY_TILES || head_dim > 128) return LVAR_ETOOBIG;
  void* ptr = static_scratch();
  if (!ptr) return LVAR_ELAUNCH;
  // The array keeps what the last call left; a balanced launch clears the arrival counters it is going to use
  // itself (table kernel or fill kernel ahead of the attention kernel), a plain launch never touches the array.
  lvar_workspace_t ws{};
  ws.ptr = ptr;
  ws.bytes = kStaticScratchBytes;
  return block_sparse_common(q, k, v, o, M, L, kv_num_blocks, stride_nb_b, stride_nb_h, kv_indices, stride_ki_b, stride_ki_h,
                             stride_ki_q, nk_max, block_q, block_k, B, H, Lq, Lk, head_dim, scale, &ws, stream);
}

int64_t lvar_attn_workspace_bytes(int head_dim) {
  if (head_dim == 256) return SK_COUNTER_BYTES;   // never balanced: the smallest workspace the entry points accept
  if (head_dim != 64 && head_dim != 128) return LVAR_EUNSUPPORTED;
  const int cus = device_cus();
  if (cus <= 0) return LVAR_ELAUNCH;
  // the larger of: two slots per share with two 4-wave workgroups per CU, or with one 8-wave workgroup per CU
  const int64_t a = sk_plan_bytes(2 * cus) + 2ll * (2 * cus) * sk_slot_floats(head_dim, MODE_BLOCK, 4) * 4;
  const int64_t b = sk_plan_bytes(cus) + 2ll * cus * sk_slot_floats(head_dim, MODE_GATHER, 8) * 4;
  return SK_COUNTER_BYTES + (a > b ? a : b);
}

int lvar_block_topk_lists(const float* block_scores, const uint8_t* base_mask, int32_t* kv_num_blocks,
                          int32_t* kv_indices, int B, int H, int nQ, int nK, int target, void* stream) {
  if (!block_scores || !kv_num_blocks || !kv_indices || B <= 0 || H <= 0 || nQ <= 0 || nK <= 0 || target < 0)
    return LVAR_EINVAL;
  MaskListParams p{};
  p.scores = block_scores; p.base = base_mask; p.kv_num_blocks = kv_num_blocks; p.kv_indices = kv_indices;
  p.rows = B * H * nQ; p.nQ = nQ; p.nK = nK; p.target = target;
  return launch_block_topk_lists(p, (hipStream_t)stream);
}

int lvar_topk_token_lists(const float* scores, int64_t score_row_stride, int32_t* indices, int64_t idx_row_stride,
                          int32_t* counts, int rows, int Lk, int k, int zero_to, void* stream) {
  if (!scores || !indices || rows < 0 || Lk <= 0 || k < 0 || k > Lk || score_row_stride < Lk || idx_row_stride < k ||
      zero_to < 0 || zero_to > idx_row_stride)
    return LVAR_EINVAL;
  TopkListParams p{};
  p.scores = scores; p.indices = indices; p.counts = counts;
  p.score_stride = score_row_stride; p.out_stride = idx_row_stride;
  p.rows = rows; p.n = Lk; p.k = k; p.zero_to = zero_to;
  return launch_topk_token_lists(p, (hipStream_t)stream);
}

int lvar_remap_concat_lists(const int32_t* src_indices, int64_t src_row_stride, int src_len,
                            const int64_t* local_indices, int64_t local_row_stride, int local_count,
                            int32_t* out_indices, int64_t out_row_stride, int32_t* out_counts,
                            int BH, int Gs, int Gk, int count, int Lk, int zero_to, void* stream) {
  if (!src_indices || !out_indices || BH < 0 || Gs <= 0 || Gk <= 0 || count < 0 || Lk <= 0 || src_len <= 0 ||
      src_row_stride < src_len || local_count < 0 || (local_count > 0 && (!local_indices || local_row_stride < local_count)) ||
      out_row_stride < (int64_t)count + local_count || zero_to < 0 || zero_to > out_row_stride)
    return LVAR_EINVAL;
  RemapListParams p{};
  p.src = src_indices; p.local = local_count > 0 ? local_indices : nullptr; p.out = out_indices; p.counts = out_counts;
  p.src_stride = src_row_stride; p.local_stride = local_row_stride; p.out_stride = out_row_stride;
  p.rows = BH * Gk; p.Gs = Gs; p.Gk = Gk; p.cnt = count; p.L = local_count; p.Lk = Lk; p.zero_to = zero_to;
  p.rep = (src_len >= count) ? 1 : (count + src_len - 1) / src_len;
  return launch_remap_concat_lists(p, (hipStream_t)stream);
}

int lvar_mask_to_lists(const uint8_t* mask, int64_t mask_row_stride, int32_t* indices, int64_t idx_row_stride,
                       int32_t* counts, int rows, int n, int multiple_of, void* stream) {
  if (!mask || !indices || !counts || rows < 0 || n <= 0 || multiple_of <= 0 || mask_row_stride < n || idx_row_stride < n)
    return LVAR_EINVAL;
  MaskCompactParams p{};
  p.mask = mask; p.indices = indices; p.counts = counts;
  p.mask_stride = mask_row_stride; p.out_stride = idx_row_stride;
  p.rows = rows; p.n = n; p.out_len = n; p.multiple_of = multiple_of; p.zero_tail = 1;
  return launch_mask_to_lists(p, (hipStream_t)stream);
}

int lvar_window_key_scores(lvar_tensor_t q, lvar_tensor_t k, const int64_t* window_keys, int n_window,
                           float* scores, int B, int H, int Lq, int Lk, int head_dim,
                           int pool_kernel_size, int max_pool, float scale, void* stream) {
  if (!view_ok(q) || !view_ok(k) || !scores || B <= 0 || H <= 0 || Lq <= 0 || Lk <= 0 || Lq > Lk || n_window < 0 ||
      (n_window > 0 && !window_keys) || !std::isfinite(scale))
    return LVAR_EINVAL;
  WinScoreParams p{};
  p.q = (const bf16_t*)q.ptr; p.q_sb = q.stride_b; p.q_sh = q.stride_h; p.q_sr = q.stride_row;
  p.k = (const bf16_t*)k.ptr; p.k_sb = k.stride_b; p.k_sh = k.stride_h; p.k_sr = k.stride_row;
  p.window = window_keys; p.out = scores;
  p.B = B; p.H = H; p.Lq = Lq; p.Lk = Lk; p.W = n_window; p.ksize = pool_kernel_size; p.maxpool = max_pool ? 1 : 0;
  p.scale = scale;
  return launch_window_scores(p, head_dim, (hipStream_t)stream);
}

}  // extern "C"
