// Key-list build on the GPU for the token-list attention path: exact per-row top-k selection of the
// column sums, the cross-scale query-group remap fused with the local-run append, and the
// compaction of a boolean mask into index lists.  All three are HBM/L2-bound integer work: one pass
// (or a few L2-resident passes) over the rows, ballot/prefix compaction, no sorting.
#include <utility>
#include "common.h"
#include "launch.h"

namespace lvar {

__device__ __forceinline__ int lanes_below(unsigned long long bal, int lane) {
  return __builtin_popcountll(bal & ((1ull << lane) - 1ull));
}

// Inclusive scan over the 64 lanes of a wave with data-parallel-primitive moves (row shifts by 1, 2, 4, 8 inside the rows
// of 16 lanes, then the last lane of row 0 / 2 broadcast into row 1 / 3 and the last lane of row 1 into rows 2 and 3):
// six dependent vector instructions instead of six round trips through the LDS crossbar.  Lanes that a move does not
// reach take the identity.  Lane 63 ends up with the reduction over the wave.
template <class Op>
__device__ __forceinline__ int wave_scan(int v, const int identity, Op op) {
  v = op(v, __builtin_amdgcn_update_dpp(identity, v, 0x111, 0xf, 0xf, false));   // row_shr:1
  v = op(v, __builtin_amdgcn_update_dpp(identity, v, 0x112, 0xf, 0xf, false));   // row_shr:2
  v = op(v, __builtin_amdgcn_update_dpp(identity, v, 0x114, 0xf, 0xf, false));   // row_shr:4
  v = op(v, __builtin_amdgcn_update_dpp(identity, v, 0x118, 0xf, 0xf, false));   // row_shr:8
  v = op(v, __builtin_amdgcn_update_dpp(identity, v, 0x142, 0xa, 0xf, false));   // row_bcast:15 into rows 1 and 3
  v = op(v, __builtin_amdgcn_update_dpp(identity, v, 0x143, 0xc, 0xf, false));   // row_bcast:31 into rows 2 and 3
  return v;
}
__device__ __forceinline__ uint32_t wave_umax(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_readlane(wave_scan((int)v, 0, [](int a, int b) { return (int)max((uint32_t)a, (uint32_t)b); }), 63);
}
__device__ __forceinline__ uint32_t wave_umin(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_readlane(wave_scan((int)v, -1, [](int a, int b) { return (int)min((uint32_t)a, (uint32_t)b); }), 63);
}

// ---------------------------------------------------------------------------------------------
// Exact top-k per row by radix select.  One 512-thread workgroup per row; wave w owns the w-th
// contiguous eighth of the (padded) row and every thread keeps its KPT keys in registers (KPT = 0:
// rows too long for that are re-read from L2 in every pass).
//   a histogram pass (11 bits, starting below the bits that all keys of the row share; LDS atomics)
//   finds the bin of the k-th largest key; the keys of that bin are compared with each other directly
//   (or, if they are too many, go through up to two more histogram passes), which gives the exact
//   value T of the k-th largest key and the number `need` of keys equal to T that belong to the
//   selection (ties go to the smaller column);
//   a counting pass gives every wave its number of selected keys, the last pass writes the selected
//   columns in ascending order (ballot compaction into an LDS ring, full-width stores).
// ---------------------------------------------------------------------------------------------
constexpr int TOPK_BINS = 2048;
constexpr int TOPK_CAND = 256;   // keys of the first pass's bin that are resolved by direct comparison

template <int KPT, int NT>
__global__ __launch_bounds__(NT, (KPT >= 1 && KPT <= 24) ? 6 : 1) void topk_token_lists_kernel(const TopkListParams p) {
  constexpr int NW = NT / 64;
  __shared__ int hist[TOPK_BINS];
  __shared__ __attribute__((aligned(16))) uint32_t cand[TOPK_CAND];
  __shared__ int wsum[NW];
  __shared__ int sel[2];  // chosen bin, keys still wanted inside it
  __shared__ int ncand;
  __shared__ int wgt[NW], weq[NW];
  const int row = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float* s = p.scores + (int64_t)row * p.score_stride;
  int32_t* out = p.indices + (int64_t)row * p.out_stride;
  const int n = p.n;
  int want = min(max(p.k, 0), n);  // keys still to be found among those matching the prefix
  if (tid == 0 && p.counts) p.counts[row] = want;
  // columns [k, zero_to) of the list row: defined (zero) instead of whatever the buffer held
  for (int t = want + tid; t < p.zero_to; t += NT) out[t] = 0;
  if (want == 0) return;

  // chunk c of wave w covers columns (w * cpw + c) * 64 .. +63
  const int cpw = KPT ? KPT : ((n + NT - 1) / NT);
  const int col0 = wave * cpw * 64 + lane;
  uint32_t keys[KPT ? KPT : 1];
  uint32_t kmax = 0u, kmin = 0xffffffffu;   // over the real columns of this thread
  if (KPT) {
    // All KPT loads are issued back to back (a branch around each would make them KPT dependent round trips):
    // buffer loads bounded to the row, so that columns beyond n read as zero instead of reaching past the row.
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)s, 0, n * 4, 0x00020000);
    uint32_t raw[KPT ? KPT : 1];
#pragma unroll
    for (int c = 0; c < KPT; c++) raw[c] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, col0 * 4, c * 256, 0);
#pragma unroll
    for (int c = 0; c < KPT; c++) {
      const bool real = col0 + c * 64 < n;
      keys[c] = real ? real_key(__builtin_bit_cast(float, raw[c])) : 0u;
      kmax = max(kmax, keys[c]);
      kmin = min(kmin, real ? keys[c] : 0xffffffffu);
    }
  } else {
    for (int c = 0; c < cpw; c++) {
      const int j = col0 + c * 64;
      if (j < n) { const uint32_t key = real_key(s[j]); kmax = max(kmax, key); kmin = min(kmin, key); }
    }
  }
  // visit(f): f(column, key) for every chunk of this wave (all 64 lanes call it together); padding columns have key 0.
  // The column numbers are formed from a copy of col0 that the compiler cannot relate to the ones of the loads:
  // kept alive from there they would be spilled, and their reloads would wait for every store in flight.
  int c0 = col0;
  asm volatile("" : "+v"(c0));
  auto visit = [&](auto&& f) {
    if (KPT) {
#pragma unroll
      for (int c = 0; c < KPT; c++) f(c0 + c * 64, keys[c]);
    } else {
      for (int c = 0; c < cpw; c++) {
        const int j = c0 + c * 64;
        f(j, (j < n) ? real_key(s[j]) : 0u);
      }
    }
  };

  // Column sums of one row sit in a narrow range: with the digits taken from the top of the key nearly every key
  // would fall into a handful of bins of the first pass and the LDS atomics of a wave would serialise on them.  The
  // bits that the largest and the smallest key of the row have in common are therefore taken as known, and the
  // digits start at the first bit in which keys differ: `top` low bits are left to resolve, 11 at a time.
  kmax = wave_umax(kmax);
  kmin = wave_umin(kmin);
  if (lane == 0) { wgt[wave] = (int)kmax; weq[wave] = (int)kmin; }
  if (tid == 0) ncand = 0;
  __syncthreads();
#pragma unroll
  for (int w = 0; w < NW; w++) { kmax = max(kmax, (uint32_t)wgt[w]); kmin = min(kmin, (uint32_t)weq[w]); }
  const int top = 32 - __builtin_clz((kmax ^ kmin) | 1u) + (((kmax ^ kmin) == 0u) ? -1 : 0);   // 0 when all keys are equal
  uint32_t pmask = (top >= 32) ? 0u : ~((1u << top) - 1u);
  uint32_t prefix = kmax & pmask;
  if (top == 0) __syncthreads();   // no pass below to separate these reads of wgt / weq from their reuse
  bool first = true;
  for (int hi = top; hi > 0;) {
    const int shift = max(0, hi - 11);
    const int bits = hi - shift;
    hi = shift;
    const int nbins = 1 << bits;
    for (int t = tid; t < nbins; t += NT) hist[t] = 0;
    __syncthreads();
    visit([&](int j, uint32_t key) {
      if ((key & pmask) == prefix) atomicAdd(&hist[(key >> shift) & (nbins - 1)], 1);
    });
    __syncthreads();
    // thread t owns the bpt bins nbins-1 - t*bpt .. (descending); find the bin holding the want-th key from the top
    const int bpt = (nbins + NT - 1) / NT;   // 1 when there are as many threads as bins (then every thread owns one)
    const int btop = nbins - 1 - tid * bpt;
    int mine = 0;
    for (int e = 0; e < bpt; e++) mine += (btop - e >= 0) ? hist[btop - e] : 0;
    const int incl = wave_scan(mine, 0, [](int a, int b) { return a + b; });
    if (lane == 63) wsum[wave] = incl;
    __syncthreads();
    int before = incl - mine;
    for (int w = 0; w < wave; w++) before += wsum[w];
    if (before < want && want <= before + mine) {  // exactly one thread
      int acc = before, bin = btop;
      for (int e = 0; e < bpt; e++) {
        const int h = (btop - e >= 0) ? hist[btop - e] : 0;
        if (acc + h >= want) { bin = btop - e; break; }
        acc += h;
      }
      sel[0] = bin;
      sel[1] = want - acc;
    }
    __syncthreads();
    prefix |= (uint32_t)sel[0] << shift;
    pmask |= (uint32_t)(nbins - 1) << shift;
    want = sel[1];
    // (the next write of `sel` lies behind three more barriers: no barrier needed after these reads)
    if (first && hi > 0) {
      // After the first pass the chosen bin usually holds a few dozen keys.  They are copied to LDS, and if they
      // fit, every one of them counts the candidates above it: the one with fewer than `want` above and at least
      // `want` at or above is the threshold, and the other passes are not needed.
      first = false;
      visit([&](int j, uint32_t key) {
        const bool m = (key & pmask) == prefix;
        const unsigned long long bm = __builtin_amdgcn_ballot_w64(m);
        if (bm != 0ull) {
          int base = 0;
          if (lane == 0) base = atomicAdd(&ncand, __builtin_popcountll(bm));
          base = __builtin_amdgcn_readfirstlane(base);
          const int at = base + lanes_below(bm, lane);
          if (m && at < TOPK_CAND) cand[at] = key;
        }
      });
      __syncthreads();
      const int nc = ncand;
      if (nc <= TOPK_CAND) {
        if (tid < nc) {
          const uint32_t kt = cand[tid];
          int above = 0, at_or_above = 0;
          // four candidates per LDS read (all lanes read the same address): the loop is bound by the latency of its reads
          for (int u = 0; u < nc; u += 4) {
            const u32x4 ku = *(const u32x4*)(cand + u);
#pragma unroll
            for (int e = 0; e < 4; e++) {
              const bool in = u + e < nc;
              above += in && ku[e] > kt;
              at_or_above += in && ku[e] >= kt;
            }
          }
          if (above < want && want <= at_or_above) { sel[0] = (int)kt; sel[1] = want - above; }   // equal keys write equal values
        }
        __syncthreads();
        prefix = (uint32_t)sel[0];
        want = sel[1];
        break;
      }
    }
  }
  const uint32_t T = prefix;  // key of the k-th largest element
  const int need = want;      // selected keys equal to T (the first `need` of them by column)

  int gt = 0, eq = 0;
  visit([&](int j, uint32_t key) {
    gt += __builtin_popcountll(__builtin_amdgcn_ballot_w64(key > T));
    eq += __builtin_popcountll(__builtin_amdgcn_ballot_w64(key == T));
  });
  if (lane == 0) { wgt[wave] = gt; weq[wave] = eq; }
  __syncthreads();
  int pos = 0, eq_before = 0;
  for (int w = 0; w < wave; w++) {
    pos += wgt[w] + max(0, min(weq[w], need - eq_before));
    eq_before += weq[w];
  }
  int eq_left = max(0, need - eq_before);
  // The selected columns of a wave are collected in a 128-entry ring in LDS (the histogram is no longer needed: the
  // barrier above lies between its last read and these writes) and leave in full 64-entry, 256-byte stores instead
  // of one partial store per chunk.  LDS operations of one wave complete in order, so the ring needs no barrier.
  int* ring = hist + wave * 128;
  int head = 0, fill = 0;   // wave-uniform
  visit([&](int j, uint32_t key) {
    unsigned long long bk = __builtin_amdgcn_ballot_w64(key > T);
    const unsigned long long beq = __builtin_amdgcn_ballot_w64(key == T);
    if (beq != 0ull && eq_left > 0) {   // keys equal to the threshold: the first eq_left of them by column
      bk |= __builtin_amdgcn_ballot_w64(key == T && lanes_below(beq, lane) < eq_left);
      eq_left = max(0, eq_left - __builtin_popcountll(beq));
    }
    if ((bk >> lane) & 1ull) ring[(head + fill + lanes_below(bk, lane)) & 127] = j;
    fill += __builtin_popcountll(bk);
    if (fill >= 64) {
      out[pos + lane] = ring[(head + lane) & 127];
      head = (head + 64) & 127;
      pos += 64;
      fill -= 64;
    }
  });
  if (lane < fill) out[pos + lane] = ring[(head + lane) & 127];
}

// Keys per thread: every value up to 24 (a row of n keys takes ceil(n / 512) of them: no pass walks more than one
// chunk of padding per wave), then 28 and 32; longer rows are re-read from L2 in every pass.
template <int KPT>
static bool topk_try(const TopkListParams& p, hipStream_t stream) {
  if (p.n > 512 * KPT) return false;
  hipLaunchKernelGGL((topk_token_lists_kernel<KPT, 512>), dim3(p.rows), dim3(512), 0, stream, p);
  return true;
}
template <int... KPT>
static bool topk_dispatch(const TopkListParams& p, hipStream_t stream, std::integer_sequence<int, KPT...>) {
  return (topk_try<KPT + 1>(p, stream) || ...);
}

int launch_topk_token_lists(const TopkListParams& p, hipStream_t stream) {
  if (p.rows == 0) return LVAR_OK;
  // 512 threads per row keep a row of up to 16384 keys in registers (KPT keys per thread)
  if (!topk_dispatch(p, stream, std::make_integer_sequence<int, 24>{}) && !topk_try<28>(p, stream) && !topk_try<32>(p, stream))
    hipLaunchKernelGGL((topk_token_lists_kernel<0, 512>), dim3(p.rows), dim3(512), 0, stream, p);
  return hipGetLastError() == hipSuccess ? LVAR_OK : LVAR_ELAUNCH;
}

// ---------------------------------------------------------------------------------------------
// Sparse-step list: out[b,h,g, 0:cnt]       = clamp(src[b,h,gS(g), j / rep], 0, Lk-1)
//                   out[b,h,g, cnt:cnt+L]   = local[g, 0:L]
//                   counts[b,h,g]           = cnt + L
// with gS(g) = clamp(rint((g + 0.5) / Gk * Gs - 0.5), 0, Gs-1) in fp32 (round half to even).
// One workgroup per output row.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void remap_concat_lists_kernel(const RemapListParams p) {
  const int row = blockIdx.x;  // bh * Gk + g
  const int g = row % p.Gk, bh = row / p.Gk;
  // three separately rounded fp32 operations (no fused multiply-add), as an eager tensor expression does
  const float pos = __fsub_rn(__fmul_rn(__fdiv_rn((float)g + 0.5f, (float)p.Gk), (float)p.Gs), 0.5f);
  const int gs = max(0, min(p.Gs - 1, (int)__builtin_rintf(pos)));
  const int32_t* src = p.src + ((int64_t)bh * p.Gs + gs) * p.src_stride;
  int32_t* out = p.out + (int64_t)row * p.out_stride;
  for (int j = threadIdx.x; j < p.cnt; j += 256) out[j] = max(0, min(p.Lk - 1, src[j / p.rep]));
  if (p.local) {
    const int64_t* loc = p.local + (int64_t)g * p.local_stride;
    for (int j = threadIdx.x; j < p.L; j += 256) out[p.cnt + j] = (int32_t)loc[j];
  }
  const int total = p.cnt + (p.local ? p.L : 0);
  for (int j = total + threadIdx.x; j < p.zero_to; j += 256) out[j] = 0;   // the rest of the row: defined (zero)
  if (threadIdx.x == 0 && p.counts) p.counts[row] = total;
}

int launch_remap_concat_lists(const RemapListParams& p, hipStream_t stream) {
  if (p.rows == 0) return LVAR_OK;
  hipLaunchKernelGGL(remap_concat_lists_kernel, dim3(p.rows), dim3(256), 0, stream, p);
  return hipGetLastError() == hipSuccess ? LVAR_OK : LVAR_ELAUNCH;
}

// ---------------------------------------------------------------------------------------------
// Mask compaction: ascending columns of the set entries of a uint8 row, count rounded up to a
// multiple with the lowest unset columns as padding.  One 256-thread workgroup per row: every wave
// owns a contiguous quarter of the 64-column chunks, counts its set entries (mask bytes loaded eight
// chunks at a time), learns its output offset from the counts of the waves before it, and writes
// its columns on a second sweep; wave 0 then appends the padding.
// ---------------------------------------------------------------------------------------------
constexpr int MASKLIST_T = 256;

__global__ __launch_bounds__(MASKLIST_T) void mask_to_lists_kernel(const MaskCompactParams p) {
  constexpr int NW = MASKLIST_T / 64, UN = 8;
  __shared__ int wcnt[NW];
  const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint8_t* m = p.mask + (int64_t)row * p.mask_stride;
  int32_t* out = p.indices + (int64_t)row * p.out_stride;
  const int n = p.n;
  const int chunks = (n + 63) >> 6;
  const int cpw = (chunks + NW - 1) / NW;
  const int c_lo = min(chunks, wave * cpw), c_hi = min(chunks, c_lo + cpw);
  // sweep(f): f(first column of the chunk, ballot of the set entries) for every chunk of this wave, ascending
  auto sweep = [&](auto&& f) {
    for (int c0 = c_lo; c0 < c_hi; c0 += UN) {
      uint8_t v[UN];
#pragma unroll
      for (int u = 0; u < UN; u++) {
        const int j = (c0 + u) * 64 + lane;
        v[u] = m[min(j, n - 1)];          // clamped: the load is unconditional, its use is not
      }
#pragma unroll
      for (int u = 0; u < UN; u++) {
        const int j = (c0 + u) * 64 + lane;
        if (c0 + u < c_hi) f((c0 + u) * 64, __builtin_amdgcn_ballot_w64(j < n && v[u] != 0));
      }
    }
  };
  int mine = 0;
  sweep([&](int, unsigned long long bal) { mine += __builtin_popcountll(bal); });
  if (lane == 0) wcnt[wave] = mine;
  __syncthreads();
  int pos = 0, total = 0;
#pragma unroll
  for (int w = 0; w < NW; w++) {
    pos += (w < wave) ? wcnt[w] : 0;
    total += wcnt[w];
  }
  sweep([&](int col0, unsigned long long bal) {
    if ((bal >> lane) & 1ull) out[pos + lanes_below(bal, lane)] = col0 + lane;
    pos += __builtin_popcountll(bal);
  });
  const int mult = max(1, p.multiple_of);
  const int padded = min(n, (total + mult - 1) / mult * mult);
  if (wave == 0) {
    // padding: the lowest unset columns, in ascending order (fewer than `multiple_of` of them)
    int filled = total;
    for (int c = 0; c < chunks && filled < padded; c++) {
      const int j = c * 64 + lane;
      const bool off = j < n && m[j] == 0;
      const unsigned long long bal = __builtin_amdgcn_ballot_w64(off);
      const int at = filled + lanes_below(bal, lane);
      if (off && at < padded) out[at] = j;
      filled = min(padded, filled + __builtin_popcountll(bal));
    }
  }
  if (p.zero_tail)
    for (int t = padded + tid; t < p.out_len; t += MASKLIST_T) out[t] = 0;
  if (tid == 0) p.counts[row] = padded;
}

int launch_mask_to_lists(const MaskCompactParams& p, hipStream_t stream) {
  if (p.rows == 0) return LVAR_OK;
  hipLaunchKernelGGL(mask_to_lists_kernel, dim3(p.rows), dim3(MASKLIST_T), 0, stream, p);
  return hipGetLastError() == hipSuccess ? LVAR_OK : LVAR_ELAUNCH;
}

}  // namespace lvar
