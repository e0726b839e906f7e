// Block-list build on the GPU: per (batch, head, query block) row, keep the always-on blocks of a
// static base mask plus the best-scoring remaining blocks up to a target count, and emit the
// compacted ascending block list (flex BlockMask layout: count + indices, unused tail zero).
//
// One wave per row.  Selection is by exact rank: block j is kept if fewer than `extra` non-base
// blocks beat it, where "beats" is (score greater) or (score equal and index smaller), i.e. the
// order of a stable descending sort, so the result is a pure function of the scores.
#include "common.h"
#include "launch.h"

namespace lvar {

constexpr int MASKLIST_MAX_NK = 2048;  // blocks per row held in LDS

__global__ __launch_bounds__(64) void block_topk_lists_kernel(const MaskListParams p) {
  __shared__ float sc[MASKLIST_MAX_NK];
  const int row = blockIdx.x;               // (b*H + h)*nQ + i
  const int i = row % p.nQ;
  const int lane = threadIdx.x;
  const float* s = p.scores + (int64_t)row * p.nK;
  const uint8_t* base = p.base ? p.base + (int64_t)i * p.nK : nullptr;
  const int chunks = (p.nK + 63) >> 6;

  // stage scores; base blocks get +inf so they never compete, count them on the way
  int nbase = 0;
  for (int c = 0; c < chunks; c++) {
    const int j = c * 64 + lane;
    bool isb = false;
    if (j < p.nK) {
      isb = base && base[j];
      sc[j] = isb ? INFINITY : s[j];
    }
    nbase += __builtin_popcountll(__builtin_amdgcn_ballot_w64(isb));
  }
  __syncthreads();
  const int extra = max(0, min(p.target, p.nK) - nbase);

  int32_t* out = p.kv_indices + (int64_t)row * p.nK;
  int written = 0;
  for (int c = 0; c < chunks; c++) {
    const int j = c * 64 + lane;
    bool keep = false;
    if (j < p.nK) {
      const float mine = sc[j];
      if (mine == INFINITY && base && base[j]) {
        keep = true;
      } else if (extra > 0) {
        int rank = 0;
        for (int t = 0; t < p.nK; t++) {
          const float o = sc[t];  // broadcast read
          const bool other_base = (o == INFINITY) && base && base[t];
          rank += (!other_base && (o > mine || (o == mine && t < j))) ? 1 : 0;
        }
        keep = rank < extra;
      }
    }
    const unsigned long long bal = __builtin_amdgcn_ballot_w64(keep);
    if (keep) out[written + __builtin_popcountll(bal & ((1ull << lane) - 1ull))] = j;
    written += __builtin_popcountll(bal);
  }
  for (int t = written + lane; t < p.nK; t += 64) out[t] = 0;
  if (lane == 0) p.kv_num_blocks[row] = written;
}

int launch_block_topk_lists(const MaskListParams& p, hipStream_t stream) {
  if (p.nK > MASKLIST_MAX_NK) return LVAR_EUNSUPPORTED;
  hipLaunchKernelGGL(block_topk_lists_kernel, dim3(p.rows), dim3(64), 0, stream, p);
  return hipGetLastError() == hipSuccess ? LVAR_OK : LVAR_ELAUNCH;
}

}  // namespace lvar
