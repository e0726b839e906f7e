// Host-side check of the work partition of the balanced attention launch (lvar_amd/csrc/sk_partition.h), with
// the arithmetic the device code uses, on random list-length tables:
//   * the pieces of every query tile abut and cover it, and no piece of a cut tile is smaller than min_piece,
//   * pieces of one tile differ by at most one unit, and a cut tile's pieces are between 2/3 and 2 shares long
//     (longer only when the tile already has the maximum number of pieces),
//   * a launch of N + P workgroups has one for every item, and 2 * P workspace slots hold every piece.
// Prints "ok <cases>" or the first violation.
#include <algorithm>
#include <cstdio>
#include <random>
#include <vector>
#include "../../lvar_amd/csrc/sk_partition.h"

using namespace lvar;

static bool check(const std::vector<int>& units, int P, int min_share, int min_piece, const char** why) {
  const int N = (int)units.size();
  int U = 0;
  for (int t : units) U += std::max(t, 1);
  const int S = sk_share(U, P, min_share);
  const bool cut = sk_worth_cutting(U, S, N, P);
  long items = 0, slots = 0;
  for (int w = 0; w < N; w++) {
    const int T = units[w];
    const int n = cut ? sk_pieces(T, S, min_piece) : 1;
    if (n < 1) { *why = "no piece"; return false; }
    items += n;
    if (n > 1) slots += n;
    int at = 0, lo = 1 << 30, hi = 0;
    for (int kp = 0; kp < n; kp++) {
      int u0, u1;
      sk_piece(T, n, kp, u0, u1);
      if (u0 != at) { *why = "pieces of a tile do not abut"; return false; }
      if (n > 1 && u1 - u0 < min_piece) { *why = "piece smaller than min_piece"; return false; }
      lo = std::min(lo, u1 - u0);
      hi = std::max(hi, u1 - u0);
      at = u1;
    }
    if (at != T) { *why = "pieces do not cover the tile"; return false; }
    if (n > 1 && hi - lo > 1) { *why = "pieces of unequal length"; return false; }
    if (n > SK_MAX_PIECES) { *why = "too many pieces"; return false; }
    if (n > 1 && (3 * lo < 2 * S - 3 || (hi > 2 * S && n < SK_MAX_PIECES))) { *why = "piece far from the share"; return false; }
  }
  if (items > N + P) { *why = "more items than workgroups"; return false; }
  if (slots > 2 * P) { *why = "more pieces than slots"; return false; }
  return true;
}

int main() {
  std::mt19937 rng(12345);
  int cases = 0;
  for (int iter = 0; iter < 6000; iter++) {
    const int N = 1 + rng() % (iter % 7 == 0 ? 1024 : 300);
    const int kind = rng() % 5;
    std::vector<int> t(N);
    for (int i = 0; i < N; i++) {
      switch (kind) {
        case 0: t[i] = rng() % 4; break;                           // tiny and empty lists
        case 1: t[i] = 21; break;                                  // equal lists
        case 2: t[i] = rng() % 166; break;                         // ragged
        case 3: t[i] = (rng() % 10 == 0) ? 165 : 0; break;          // a few long lists among empty ones
        default: t[i] = (rng() % 2 ? rng() % 40 : 0); break;
      }
    }
    const int Ps[] = {8, 16, 256, 512, 40, 304};
    const int P = Ps[rng() % 6];
    const int mp = 1 + rng() % 6;
    const int min_share = mp + rng() % 8;     // the launch code keeps min_share >= min_piece
    const char* why = "";
    if (!check(t, P, min_share, mp, &why)) {
      std::printf("FAIL iter %d N %d kind %d P %d min_share %d min_piece %d: %s\n", iter, N, kind, P, min_share, mp, why);
      return 1;
    }
    cases++;
  }
  std::printf("ok %d\n", cases);
  return 0;
}
