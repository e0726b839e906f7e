// Window-query key scores (the scoring step of a ScaleKV-style cache selection): the logits of a small
// set of "window" queries against every key are summed over the queries, smoothed by a 1-D pool
// along the key axis and masked at the window's own keys.  Since sum_i (q_i . k_n) = (sum_i q_i) . k_n
// the work is one pass over K with a single summed query: HBM-bound (2 bytes x d per key), no MFMA.
#include "common.h"
#include "launch.h"

namespace lvar {

constexpr int WS_KEYS = 512;   // keys per workgroup (every workgroup sums the window queries for itself: the more keys, the less that weighs)
constexpr int WS_MAXR = 16;    // largest pool radius (kernel_size <= 33)

template <int D>
__global__ __launch_bounds__(256) void window_scores_kernel(const WinScoreParams p) {
  constexpr int LPR = D / 8;          // lanes that share one key row (8 bf16 = 16 bytes each)
  constexpr int RPP = 256 / LPR;      // key rows per pass of the workgroup
  __shared__ float qs[D];
  __shared__ float part[RPP][D];
  __shared__ float sc[WS_KEYS + 2 * WS_MAXR];
  __shared__ uint8_t wm[WS_KEYS + 2 * WS_MAXR];
  const int tid = threadIdx.x;
  // Workgroup ids are dealt round-robin to the 8 XCDs, each with an L2 of its own; remapped so that one XCD walks a
  // contiguous range of (batch, head, chunk), the window queries of a (batch, head) are fetched from memory by one
  // XCD instead of by all eight (they are read by every workgroup of the slice: as many bytes as 256 keys).
  const int per_xcd = gridDim.x >> 3;
  const int w = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (w >= p.total_wg) return;
  const int bh = w / p.nchunks, chunk = w - bh * p.nchunks;
  const int b = bh / p.H, h = bh - b * p.H;
  const int r = p.ksize >> 1;
  const int n0 = chunk * WS_KEYS - r;  // key of sc[0]
  const int span = WS_KEYS + 2 * r;
  const int64_t* win = p.window + (int64_t)bh * p.W;
  const bf16_t* qb = p.q + b * p.q_sb + h * p.q_sh;
  const bf16_t* kb = p.k + b * p.k_sb + h * p.k_sh;

  // summed window query, fp32; a window key n is the query row clamp(n - (Lk - Lq), 0, Lq-1).
  // Row group g (LPR lanes, 16 bytes each) adds up the window rows g, g + RPP, ...; the RPP partial
  // sums meet in LDS.
  const int g = tid / LPR, l = tid - g * LPR;
  constexpr int UN = 8;   // rows in flight per lane: the loads of a batch are issued together, not one per round trip
  {
    float a[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int i0 = g; i0 < p.W; i0 += RPP * UN) {
      int rows[UN];
#pragma unroll
      for (int u = 0; u < UN; u++) {
        const int i = i0 + u * RPP;
        rows[u] = (int)win[min(i, p.W - 1)];
      }
      u32x4 qv4[UN];
#pragma unroll
      for (int u = 0; u < UN; u++) {
        const int row = max(0, min(p.Lq - 1, rows[u] - (p.Lk - p.Lq)));
        qv4[u] = *(const u32x4*)(qb + (int64_t)row * p.q_sr + l * 8);
      }
#pragma unroll
      for (int u = 0; u < UN; u++) {
        if (i0 + u * RPP < p.W) {
#pragma unroll
          for (int e = 0; e < 4; e++) { a[2 * e] += bf16_lo(qv4[u][e]); a[2 * e + 1] += bf16_hi(qv4[u][e]); }
        }
      }
    }
#pragma unroll
    for (int e = 0; e < 8; e++) part[g][l * 8 + e] = a[e];
  }
  __syncthreads();
  for (int c = tid; c < D; c += 256) {
    float acc = 0.f;
    for (int gg = 0; gg < RPP; gg++) acc += part[gg][c];
    qs[c] = acc;
  }
  __syncthreads();

  float qv[8];
#pragma unroll
  for (int e = 0; e < 8; e++) qv[e] = qs[l * 8 + e];
  const float pad = p.maxpool ? -INFINITY : 0.f;
  for (int j0 = g; j0 < span; j0 += RPP * UN) {
    u32x4 kv[UN];
#pragma unroll
    for (int u = 0; u < UN; u++) {
      const int n = max(0, min(p.Lk - 1, n0 + j0 + u * RPP));   // clamped: the load is unconditional, its use is not
      kv[u] = *(const u32x4*)(kb + (int64_t)n * p.k_sr + l * 8);
    }
#pragma unroll
    for (int u = 0; u < UN; u++) {
      const int j = j0 + u * RPP, n = n0 + j;
      float dot = 0.f;
#pragma unroll
      for (int e = 0; e < 4; e++) dot += bf16_lo(kv[u][e]) * qv[2 * e] + bf16_hi(kv[u][e]) * qv[2 * e + 1];
      dot = group_sum<LPR>(dot);
      if (l == 0 && j < span) {
        sc[j] = (n >= 0 && n < p.Lk) ? dot * p.scale : pad;
        wm[j] = 0;
      }
    }
  }
  __syncthreads();
  // the window's own keys do not compete: -inf before the pool (it spreads to their neighbours under
  // an average) and again after it
  for (int i = tid; i < p.W; i += 256) {
    const int j = (int)win[i] - n0;
    if (j >= 0 && j < span) { sc[j] = -INFINITY; wm[j] = 1; }
  }
  __syncthreads();
  for (int t = tid; t < WS_KEYS; t += 256) {
    const int n = chunk * WS_KEYS + t;
    if (n < p.Lk) {
      float acc = p.maxpool ? -INFINITY : 0.f;
      for (int e = 0; e <= 2 * r; e++) acc = p.maxpool ? fmaxf(acc, sc[t + e]) : acc + sc[t + e];
      if (!p.maxpool) acc = acc / (float)p.ksize;
      p.out[(int64_t)bh * p.Lk + n] = wm[t + r] ? -INFINITY : acc;
    }
  }
}

int launch_window_scores(const WinScoreParams& p0, int head_dim, hipStream_t stream) {
  WinScoreParams p = p0;
  if ((p.ksize & 1) == 0 || p.ksize < 1 || (p.ksize >> 1) > WS_MAXR) return LVAR_EUNSUPPORTED;
  p.nchunks = (p.Lk + WS_KEYS - 1) / WS_KEYS;
  p.total_wg = p.B * p.H * p.nchunks;
  const dim3 grid((p.total_wg + 7) / 8 * 8);
  if (head_dim == 128) hipLaunchKernelGGL(window_scores_kernel<128>, grid, dim3(256), 0, stream, p);
  else if (head_dim == 64) hipLaunchKernelGGL(window_scores_kernel<64>, grid, dim3(256), 0, stream, p);
  else if (head_dim == 256) hipLaunchKernelGGL(window_scores_kernel<256>, grid, dim3(256), 0, stream, p);
  else return LVAR_EUNSUPPORTED;
  return hipGetLastError() == hipSuccess ? LVAR_OK : LVAR_ELAUNCH;
}

}  // namespace lvar
