// Work partition of the balanced launch of the attention kernel.
//
// A unit of work is one entry of a query tile's list: a 64-key tile (dense and token lists) or a key block
// (block lists).  A launch with U units in N query tiles picks a share S of about U / (resident workgroup slots)
// units, cuts every query tile whose list is long enough into n = round(T / S) pieces of (nearly) equal length,
// and runs one workgroup per item (a whole query tile, or one piece).  A query tile cut into pieces is finished
// by the workgroup whose piece completes last: every piece is parked in a slot of the partial-result workspace
// and the finisher adds the pieces up in list order, so the result does not depend on timing.
//
// The item table of a launch ("plan") is built on the device from the list lengths (plan_kernel in attn_fwd.hip);
// dense attention, where all lists have the same length, needs no table.  Everything here is integer arithmetic
// shared by the device code and by a host-side test.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define LVAR_HD __host__ __device__ __forceinline__
#else
#define LVAR_HD inline
#endif

namespace lvar {

constexpr int SK_MAX_QTILES = 1024;    // query tiles per balanced launch
constexpr int SK_PLAN_HEADER = 8;      // ints: {magic, items, N, S, slots used, 0, 0, 0}
constexpr int SK_PLAN_ITEM = 8;        // ints per item: {tile, u0, u1, first slot or -1, pieces, piece, tile units, 0}
constexpr int SK_PLAN_MAGIC = 0x4c564b53;

// Share for U units over at most P workgroups, none smaller than min_share units.
LVAR_HD int sk_share(int U, int P, int min_share) {
  const int s = (U + P - 1) / (P > 0 ? P : 1);
  return s > min_share ? s : min_share;
}

constexpr int SK_MAX_PIECES = 8;       // pieces of one query tile (the finisher reads all their statistics at once)

// Pieces of a query tile with T units: round(T / S), but no piece below min_piece units and at most SK_MAX_PIECES.
LVAR_HD int sk_pieces(int T, int S, int min_piece) {
  int n = (T + S / 2) / S;
  const int cap = T / (min_piece > 0 ? min_piece : 1);
  if (n > cap) n = cap;
  if (n > SK_MAX_PIECES) n = SK_MAX_PIECES;
  return n < 1 ? 1 : n;
}

// Unit range of piece kp of n: [T*kp/n, T*(kp+1)/n)
LVAR_HD void sk_piece(int T, int n, int kp, int& u0, int& u1) {
  u0 = (int)(((int64_t)T * kp) / n);
  u1 = (int)(((int64_t)T * (kp + 1)) / n);
}

// With at most as many query tiles as workgroup slots the plain launch already runs them all at once; cutting
// only pays if it makes the longest walk clearly shorter: at least one and a half shares per tile on average.
LVAR_HD bool sk_worth_cutting(int U, int S, int N, int P) { return !(N <= P && 2 * ((U + S - 1) / S) < 3 * N); }

}  // namespace lvar
