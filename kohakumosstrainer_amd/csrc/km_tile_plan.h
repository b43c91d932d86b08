// Which tile a work-group computes and how a launch is cut into tile shapes: integer arithmetic
// with no HIP dependency, compiled for the device (hipcc) and for the host (g++), where the CPU
// tests check that every tile is handed out exactly once.
#pragma once
#include "km_numeric.h"

namespace km {

// Work-group id -> (tile_m, tile_n). Work-groups are dealt round-robin to the 8 XCDs, each
// with its own L2; first give every XCD a contiguous run of tiles, then walk that run in
// bands of group_m row-tiles so that neighbours in time share A rows and B rows in L2. The 32
// tiles that an XCD's compute units work on at a time are group_m tile rows by 32 / group_m tile
// columns, and what they fetch is group_m row panels of A and 32 / group_m row panels of B: 8 x 4
// or 4 x 8 where the operands' elements are the same size, 4 x 8 where A's are twice B's
// (16-bit activations against 8-bit codes: 4 x 2 + 8 = 16 panel units against 8 x 2 + 4 = 20).
constexpr int kXcds = 8;
constexpr int kGroupM = 8;
constexpr int kGroupMWideA = 4;
KM_HD void tile_of(int pid, int tiles_m, int tiles_n, int& tm, int& tn, int group_m = kGroupM) {
  const int total = tiles_m * tiles_n;
  const int xcd = pid % kXcds, local = pid / kXcds;
  const int tall = total / kXcds, rem = total % kXcds;
  int p = xcd < rem ? xcd * (tall + 1) + local : rem * (tall + 1) + (xcd - rem) * tall + local;
  const int per_group = group_m * tiles_n;
  const int first_m = (p / per_group) * group_m;
  const int rows = tiles_m - first_m < group_m ? tiles_m - first_m : group_m;
  const int in_group = p % per_group;
  tm = first_m + in_group % rows;
  tn = in_group / rows;
}

// A tiles_m x tiles_n grid of large tiles on a card that runs `units` of them at a time (one per
// compute unit): the leading tile columns whose tiles fill whole rounds. The columns after them
// would be a last, partly empty round; a launch of smaller tiles takes them. All columns when
// the grid is whole rounds already.
KM_HD int whole_round_columns(int tiles_m, int tiles_n, int units) {
  const long long total = (long long)tiles_m * tiles_n;
  if (tiles_m <= 0 || tiles_n <= 0 || units <= 0 || total % units == 0) return tiles_n > 0 ? tiles_n : 0;
  return (int)(total / units * units / tiles_m);
}

}  // namespace km
