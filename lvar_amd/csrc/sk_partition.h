// Work partition of the balanced launch of the attention kernel.
//
// The query tiles of a launch, in launch order, form one sequence of work units (a unit = one entry of a
// tile list: a 64-key tile, or a key block of a block list); query tile w owns the positions
// [pfx[w], pfx[w+1]) of that sequence, with a weight of max(units, 1) so that a tile with an empty list still
// has an owner.  The sequence is cut at the multiples of the share S (chosen so that there are about as many
// shares as the chip has resident workgroup slots); a cut closer than `min_piece` units to a query-tile boundary
// is dropped, so that no workgroup pays the prologue and epilogue of a query tile for a sliver of work.  What
// lies between two neighbouring breakpoints (tile boundaries and kept cuts) is an item, and every workgroup of
// the launch runs exactly one item: a whole query tile, or a piece of one.  A query tile cut into pieces is
// finished by the workgroup whose piece completes last: every piece goes to a slot of the partial-result
// workspace and the finisher adds the pieces up in list order, so the result does not depend on timing.
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

constexpr int SK_MAX_QTILES = 1024;   // query tiles per balanced launch (two prefix tables held in LDS)

// Share for U units over at most P workgroups, none smaller than min_share units.
LVAR_HD int sk_share(int U, int P, int min_share) {
  const int s = (U + P - 1) / (P > 0 ? P : 1);
  return s > min_share ? s : min_share;
}

// Kept cuts strictly inside the query tile that owns [lo, hi): the multiples j*S with lo + min_piece <= j*S
// <= hi - min_piece, j = j_first .. j_first + n_inside - 1.
LVAR_HD void sk_cuts_inside(int lo, int hi, int S, int min_piece, int& j_first, int& n_inside) {
  const int x = lo + min_piece, y = hi - min_piece;
  j_first = (int)(((unsigned)x + (unsigned)S - 1u) / (unsigned)S);
  const int j_last = y >= 0 ? (int)((unsigned)y / (unsigned)S) : -1;
  n_inside = (y >= x && j_last >= j_first) ? j_last - j_first + 1 : 0;
}

// Piece kp (0 .. n_inside) of a tile with kept cuts j_first ..: its unit range inside the tile.
LVAR_HD void sk_piece(int lo, int hi, int S, int j_first, int n_inside, int kp, int& u0, int& u1) {
  u0 = kp == 0 ? 0 : (j_first + kp - 1) * S - lo;
  u1 = kp == n_inside ? hi - lo : (j_first + kp) * S - lo;
}

// Workspace slot of piece kp of a tile whose first kept cut is j_first: the piece that starts the tile ends at
// cut j_first and takes the odd slot of that cut, a later piece starts at cut j_first + kp - 1 and takes its even slot.
// Cuts are numbered 1 .. ceil(U / S) - 1, so 2 * ceil(U / S) slots suffice.
LVAR_HD int sk_slot(int j_first, int kp) { return kp == 0 ? 2 * j_first - 1 : 2 * (j_first + kp - 1); }

}  // namespace lvar
