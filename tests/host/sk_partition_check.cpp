// Host-side check of the work partition of the balanced attention launch (lvar_amd/csrc/sk_partition.h), with
// the arithmetic the kernel uses, on random weight tables:
//   * the pieces of every query tile abut and cover it, and none is smaller than min_piece units,
//   * no item is larger than a share plus what dropped cuts can add (2 * min_piece),
//   * there are fewer cuts than shares, so a launch of N + P workgroups has one for every item,
//   * no two pieces share a workspace slot and every slot index is below 2 * P.
// Prints "ok <cases>" or the first violation.
#include <algorithm>
#include <cstdio>
#include <random>
#include <set>
#include <vector>
#include "../../lvar_amd/csrc/sk_partition.h"

using namespace lvar;

static bool check(const std::vector<int>& weights, int P, int min_share, int min_piece, const char** why) {
  const int N = (int)weights.size();
  std::vector<int> pfx(N + 1, 0);
  for (int i = 0; i < N; i++) pfx[i + 1] = pfx[i] + weights[i];
  const int U = pfx[N];
  int S = sk_share(U, P, min_share);
  if (2 * ((U + S - 1) / S) < 3 * N && N <= P) S = U;   // as the kernel: tiles stay whole
  std::set<int> slots;
  int cuts = 0;
  for (int w = 0; w < N; w++) {
    int jf, ni;
    sk_cuts_inside(pfx[w], pfx[w + 1], S, min_piece, jf, ni);
    if (ni < 0) { *why = "negative cut count"; return false; }
    cuts += ni;
    int at = 0;
    for (int kp = 0; kp <= ni; kp++) {
      int u0, u1;
      sk_piece(pfx[w], pfx[w + 1], S, jf, ni, kp, u0, u1);
      if (u0 != at) { *why = "pieces of a tile do not abut"; return false; }
      if (u1 <= u0) { *why = "empty piece"; return false; }
      if (ni > 0 && u1 - u0 < min_piece) { *why = "piece smaller than min_piece"; return false; }
      if (u1 - u0 > S + 2 * min_piece && ni > 0) { *why = "piece larger than a share"; return false; }
      if (ni > 0) {
        // a cut is a multiple of the share
        if (kp > 0 && (pfx[w] + u0) % S != 0) { *why = "cut off the share grid"; return false; }
        const int slot = sk_slot(jf, kp);
        if (slot < 0 || slot >= 2 * P) { *why = "slot index out of range"; return false; }
        if (!slots.insert(slot).second) { *why = "workspace slot used twice"; return false; }
      }
      at = u1;
    }
    if (at != weights[w]) { *why = "pieces do not cover the tile"; return false; }
  }
  if (cuts >= std::max(P, 1)) { *why = "as many cuts as shares"; return false; }
  return true;
}

int main() {
  std::mt19937 rng(12345);
  int cases = 0;
  for (int iter = 0; iter < 6000; iter++) {
    const int N = 1 + rng() % (iter % 7 == 0 ? 1024 : 300);
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
    const int Ps[] = {8, 16, 256, 512, 40, 304};
    const int P = Ps[rng() % 6];
    const int mp = 1 + rng() % 6;
    const int min_share = mp + rng() % 8;     // the launch code keeps min_share >= min_piece
    const char* why = "";
    if (!check(w, P, min_share, mp, &why)) {
      std::printf("FAIL iter %d N %d kind %d P %d min_share %d min_piece %d: %s\n", iter, N, kind, P, min_share, mp, why);
      return 1;
    }
    cases++;
  }
  std::printf("ok %d\n", cases);
  return 0;
}
