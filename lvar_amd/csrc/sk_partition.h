// Work partition of the balanced ("stream") launch of the attention kernel.
//
// The query tiles of a launch, in launch order, form one sequence of work units (a unit = one entry of a
// tile list: a 64-key tile, or a key block of a block list); query tile w owns the positions
// [pfx[w], pfx[w+1]) of that sequence, with a weight of max(units, 1) so that a tile with an empty list still
// has an owner.  The sequence is cut into P nearly equal ranges, one per workgroup; a cut closer than
// `min_piece` units to a query-tile boundary is moved onto the boundary, so that no workgroup pays the
// prologue and epilogue of a query tile for a sliver of work.  A query tile cut into several pieces is
// finished by the workgroup whose piece completes last: every piece goes to a slot of the partial-result
// workspace and the finisher adds the pieces up in launch order, so the result does not depend on timing.
//
// Everything here is integer arithmetic shared by the device code and by a host-side test.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__) || defined(__CUDACC__)
#define LVAR_HD __host__ __device__ __forceinline__
#else
#define LVAR_HD inline
#endif

namespace lvar {

constexpr int SK_MAX_QTILES = 2048;   // query tiles per balanced launch (prefix table held in LDS)

struct SkPartition {
  const int* pfx;   // [N + 1] prefix sums of the weights, pfx[0] = 0
  int N;            // query tiles
  int U;            // pfx[N]
  int P;            // workgroups that take part (P >= 1)
  int min_piece;    // >= 1

  // query tile whose range holds position x (0 <= x < U)
  LVAR_HD int find(int x) const {
    int lo = 0, hi = N - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (pfx[mid] <= x) lo = mid; else hi = mid - 1;
    }
    return lo;
  }
  // start of the range of workgroup j (= end of the range of workgroup j-1)
  LVAR_HD int bound(int j) const {
    if (j <= 0) return 0;
    if (j >= P) return U;
    const int a = (int)(((int64_t)U * j) / P);
    const int w = find(a);
    const int lo = pfx[w], hi = pfx[w + 1];
    if (a - lo < min_piece) return lo;
    if (hi - a < min_piece) return hi;
    return a;
  }
  // Cuts strictly inside query tile w: workgroup boundaries j_first .. j_first + n_inside - 1.  The pieces of
  // the tile are then owned by the workgroups j_first - 1 + k, k = 0 .. n_inside.
  LVAR_HD void cuts_inside(int w, int& j_first, int& n_inside) const {
    const int64_t lo = pfx[w], hi = pfx[w + 1];
    // a_j = floor(U j / P) lies in [lo + min_piece, hi - min_piece]
    const int64_t x = lo + min_piece, y = hi - min_piece;
    if (y < x) { j_first = 0; n_inside = 0; return; }
    const int64_t jf = (x * P + U - 1) / U;             // smallest j with a_j >= x
    const int64_t jl = ((y + 1) * P + U - 1) / U - 1;   // largest j with a_j <= y
    const int64_t jf_c = jf < 1 ? 1 : jf;
    const int64_t jl_c = jl > P - 1 ? P - 1 : jl;
    j_first = (int)jf_c;
    n_inside = jl_c >= jf_c ? (int)(jl_c - jf_c + 1) : 0;
  }
};

// Slot of the partial-result workspace for the piece of workgroup `wg` that starts at unit `u0` of its query
// tile: a workgroup has at most one piece that starts a query tile and is cut at its end (slot 1) and at most
// one that continues a query tile begun by an earlier workgroup (slot 0).
LVAR_HD int sk_slot(int wg, bool piece_starts_tile) { return 2 * wg + (piece_starts_tile ? 1 : 0); }

}  // namespace lvar
