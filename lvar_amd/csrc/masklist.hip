// Block-list build on the GPU: per (batch, head, query block) row, keep the always-on blocks of a
// static base mask plus the best-scoring remaining blocks up to a target count, and emit the
// compacted ascending block list (flex BlockMask layout: count + indices, unused tail zero).
//
// One 256-thread workgroup per row.  Selection is by exact rank: block j is kept if fewer than `extra`
// non-base blocks beat it, where "beats" is (score greater) or (score equal and index smaller), i.e. the
// order of a stable descending sort, so the result is a pure function of the scores.  Score and index are
// packed into one 64-bit key (score key in the high word, complement of the index in the low word; base
// blocks get the key 0, which beats nothing), the keys of the row sit in LDS, and a thread counts the keys
// above its own with one compare per key: no global memory access inside the rank loop.
#include "common.h"
#include "launch.h"

namespace lvar {

constexpr int MASKLIST_MAX_NK = 2048;  // blocks per row held in LDS
constexpr int MASKLIST_NT = 256;

__global__ __launch_bounds__(MASKLIST_NT) void block_topk_lists_kernel(const MaskListParams p) {
  constexpr int NT = MASKLIST_NT, NW = NT / 64;
  __shared__ uint64_t key[MASKLIST_MAX_NK];
  __shared__ int wcnt[NW];
  __shared__ int nbase_s;
  const int row = blockIdx.x;               // (b*H + h)*nQ + i
  const int i = row % p.nQ;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float* s = p.scores + (int64_t)row * p.nK;
  const uint8_t* base = p.base ? p.base + (int64_t)i * p.nK : nullptr;
  const int nK = p.nK;

  if (tid == 0) nbase_s = 0;
  __syncthreads();
  int mybase = 0;
  for (int j = tid; j < nK; j += NT) {
    const bool isb = base && base[j];
    key[j] = isb ? 0ull : (((uint64_t)real_key(s[j]) << 32) | (uint64_t)(0xffffffffu - (uint32_t)j));
    mybase += isb ? 1 : 0;
  }
  if (mybase) atomicAdd(&nbase_s, mybase);
  __syncthreads();
  const int extra = max(0, min(p.target, nK) - nbase_s);

  int32_t* out = p.kv_indices + (int64_t)row * nK;
  int written = 0;   // kept blocks of the chunks before this one (the same in every thread)
  for (int c0 = 0; c0 < nK; c0 += NT) {
    const int j = c0 + tid;
    bool keep = false;
    if (j < nK) {
      const uint64_t mine = key[j];
      if (mine == 0ull) {
        keep = true;                         // base block
      } else if (extra > 0) {
        int rank = 0;
        int t = 0;
        for (; t + 4 <= nK; t += 4) {        // broadcast reads
          rank += (key[t] > mine) + (key[t + 1] > mine) + (key[t + 2] > mine) + (key[t + 3] > mine);
        }
        for (; t < nK; t++) rank += key[t] > mine;
        keep = rank < extra;
      }
    }
    const unsigned long long bal = __builtin_amdgcn_ballot_w64(keep);
    if (lane == 0) wcnt[wave] = __builtin_popcountll(bal);
    __syncthreads();
    int before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < NW; w++) {
      const int n = wcnt[w];
      before += (w < wave) ? n : 0;
      total += n;
    }
    if (keep) out[written + before + __builtin_popcountll(bal & ((1ull << lane) - 1ull))] = j;
    written += total;
    __syncthreads();   // wcnt is rewritten by the next chunk
  }
  for (int t = written + tid; t < nK; t += NT) out[t] = 0;
  if (tid == 0) p.kv_num_blocks[row] = written;
}

int launch_block_topk_lists(const MaskListParams& p, hipStream_t stream) {
  if (p.nK > MASKLIST_MAX_NK) return LVAR_EUNSUPPORTED;
  hipLaunchKernelGGL(block_topk_lists_kernel, dim3(p.rows), dim3(MASKLIST_NT), 0, stream, p);
  return hipGetLastError() == hipSuccess ? LVAR_OK : LVAR_ELAUNCH;
}

}  // namespace lvar
