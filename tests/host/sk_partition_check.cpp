// Host-side check of the work partition of the balanced attention launch (lvar_amd/csrc/sk_partition.h):
// walks the ranges exactly as the kernel does and verifies, for random weight tables, that
//   * the ranges of the P workgroups tile the whole sequence without gap or overlap,
//   * every piece of a cut query tile has at least min_piece units, as has what is cut off beside it,
//   * the finisher's enumeration (cuts_inside) names exactly the workgroups that own the pieces, in order,
//   * no two pieces share a workspace slot, and a workgroup uses at most its two slots.
// Prints "ok <cases>" or the first violation.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <random>
#include <set>
#include <vector>
#include "../../lvar_amd/csrc/sk_partition.h"

using namespace lvar;

struct Piece { int wg, u0, u1; };

static bool check(const std::vector<int>& weights, int P, int min_piece, const char** why) {
  const int N = (int)weights.size();
  std::vector<int> pfx(N + 1, 0);
  for (int i = 0; i < N; i++) pfx[i + 1] = pfx[i] + weights[i];
  SkPartition part{pfx.data(), N, pfx[N], P, min_piece};
  std::map<int, std::vector<Piece>> pieces;   // query tile -> pieces in workgroup order
  std::set<int> slots;
  int covered = 0;
  for (int me = 0; me < P; me++) {
    int x0 = part.bound(me);
    const int x1 = part.bound(me + 1);
    if (x0 != covered) { *why = "ranges do not abut"; return false; }
    if (x1 < x0) { *why = "range ends before it starts"; return false; }
    covered = x1;
    if (x0 >= x1) continue;
    int wq = part.find(x0);
    int used = 0;
    while (x0 < x1) {
      const int lo = pfx[wq], hi = pfx[wq + 1];
      if (x0 < lo || x0 >= hi) { *why = "item outside its query tile"; return false; }
      const int e = x1 < hi ? x1 : hi;
      const bool whole = (x0 == lo && e == hi);
      if (!whole) {
        if (e - x0 < min_piece) { *why = "piece smaller than min_piece"; return false; }
        pieces[wq].push_back(Piece{me, x0 - lo, e - lo});
        const int slot = sk_slot(me, x0 == lo);
        if (!slots.insert(slot).second) { *why = "workspace slot used twice"; return false; }
        if (++used > 2) { *why = "more than two pieces in one workgroup"; return false; }
      }
      x0 = e;
      wq++;
    }
  }
  if (covered != pfx[N]) { *why = "sequence not covered"; return false; }
  for (int w = 0; w < N; w++) {
    int j_first, n_inside;
    part.cuts_inside(w, j_first, n_inside);
    auto it = pieces.find(w);
    if (it == pieces.end()) {
      if (n_inside != 0) { *why = "finisher expects pieces of an uncut tile"; return false; }
      continue;
    }
    const auto& ps = it->second;
    if ((int)ps.size() != n_inside + 1) { *why = "piece count differs from cuts_inside"; return false; }
    int at = 0;
    for (int k = 0; k <= n_inside; k++) {
      if (ps[k].wg != j_first - 1 + k) { *why = "piece owner differs from cuts_inside"; return false; }
      if (ps[k].u0 != at) { *why = "pieces of a tile do not abut"; return false; }
      if ((k == 0) != (ps[k].u0 == 0)) { *why = "first piece does not start the tile"; return false; }
      at = ps[k].u1;
    }
    if (at != weights[w]) { *why = "pieces do not cover the tile"; return false; }
  }
  return true;
}

int main() {
  std::mt19937 rng(12345);
  int cases = 0;
  for (int iter = 0; iter < 4000; iter++) {
    const int N = 1 + rng() % (iter % 7 == 0 ? 2048 : 300);
    const int kind = rng() % 5;
    std::vector<int> w(N);
    for (int i = 0; i < N; i++) {
      switch (kind) {
        case 0: w[i] = 1 + rng() % 3; break;                       // tiny lists
        case 1: w[i] = 21; break;                                  // equal lists
        case 2: w[i] = 1 + rng() % 165; break;                     // ragged
        case 3: w[i] = (rng() % 10 == 0) ? 165 : 1; break;          // a few long lists among empty ones
        default: w[i] = 1 + (rng() % 2 ? rng() % 40 : 0); break;
      }
    }
    const int Ps[] = {1, 2, 8, 256, 512, 37};
    const int mp = 1 + rng() % 6;
    const int min_share = mp + rng() % 8;     // the launch code keeps min_share >= min_piece
    int U = 0;
    for (int x : w) U += x;
    // as the kernel: no more workgroups than shares of min_share units
    const int P = std::max(1, std::min(Ps[rng() % 6], U / min_share));
    const char* why = "";
    if (!check(w, P, mp, &why)) {
      std::printf("FAIL iter %d N %d kind %d P %d min_piece %d: %s\n", iter, N, kind, P, mp, why);
      return 1;
    }
    cases++;
  }
  std::printf("ok %d\n", cases);
  return 0;
}
