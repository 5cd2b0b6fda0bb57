// Launch index -> output tile, shared by the kernels and by the host (sd_tile_of_block, which tests use to check
// that the map is a bijection onto the tile grid).
#pragma once

#include <hip/hip_runtime.h>

namespace sd {

// Maps the launch index to an output tile so that the workgroups resident on one XCD (the hardware
// deals consecutive workgroup ids round-robin over the 8 XCDs, each with its own L2) cover a compact
// patch of the tile grid: each XCD gets a contiguous run of the tile order, and the order walks
// GROUP_M tile rows at a time (column by column inside a group).
// tile rows walked together: 8 for the DSD kernels (their row panels are the sparse, smaller operand),
// 4 for SDD (8 measured 25 % slower there)
constexpr int DSD_GROUP_M = 8, SDD_GROUP_M = 4;
template <int GROUP_M>
__host__ __device__ inline void tile_of_block(int bid, int tiles_m, int tiles_n, int& tm, int& tn) {
  constexpr int XCDS = 8;
  const int total = tiles_m * tiles_n;
  const int per = total / XCDS, rem = total % XCDS;
  const int x = bid % XCDS, i = bid / XCDS;
  const int lin = x * per + (x < rem ? x : rem) + i;
  const int group = lin / (GROUP_M * tiles_n);
  const int first_m = group * GROUP_M;
  const int gm = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
  const int in_group = lin - group * GROUP_M * tiles_n;
  tm = first_m + in_group % gm;
  tn = in_group / gm;
}

}  // namespace sd
