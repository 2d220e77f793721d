// Which query tile a workgroup of the 16x16x32 attention kernels computes: the arithmetic alone, kept apart from the
// kernels so that the same functions can be compiled for the host and every workgroup of a grid checked to land on a
// tile of its own (tests/host/fa16_work_cover.cpp does that).  Plain C++: no HIP types.
#pragma once

#if defined(__HIPCC__)
#define FA16_HD __host__ __device__ __forceinline__
#else
#define FA16_HD inline
#endif

namespace msd {
namespace fa16 {

// A tile of `groups` (batch, head) pairs x `tiles` query tiles each.  group < 0: the workgroup has nothing to do.
struct Work {
  int group;  // (batch, head) index, or the head alone with the packed numbering
  int tile;
};

// Runs: workgroups are dealt round-robin to the 8 XCDs; XCD x takes the x-th eighth of the tiles in (group, tile)
// order, so consecutive tiles of a head share an XCD's L2.  The grid may be larger than 8 * ceil(total / 8).
FA16_HD Work runs(int block, int groups, int tiles) {
  const int total = groups * tiles;
  const int per_xcd = (total + 7) / 8;
  const int j = block >> 3;
  const int work = (block & 7) * per_xcd + j;
  if (work >= total || j >= per_xcd) return Work{-1, 0};
  const int group = work / tiles;
  return Work{group, work - group * tiles};
}
inline long long runs_grid(long long groups, long long tiles) { return (groups * tiles + 7) / 8 * 8; }

// Units of one heavy and one light tile (u and tiles - 1 - u; heavy_first_index: the heavy one is the lower index,
// as with pairs numbered by descending length, or the higher one, as with causal tiles).  An XCD takes a run of units,
// starts all its heavy halves first and its light halves last, in reverse.
FA16_HD Work units(int block, int groups, int tiles, bool heavy_is_low) {
  const int units_per_group = (tiles + 1) / 2;
  const int n_units = groups * units_per_group;
  const int per_xcd = (n_units + 7) / 8;
  const int j = block >> 3;
  if (j >= 2 * per_xcd) return Work{-1, 0};
  const bool heavy = j < per_xcd;
  const int unit = (block & 7) * per_xcd + (heavy ? j : 2 * per_xcd - 1 - j);
  if (unit >= n_units) return Work{-1, 0};
  const int group = unit / units_per_group;
  const int u = unit - group * units_per_group;
  if (!heavy && 2 * u == tiles - 1) return Work{-1, 0};  // odd count: the middle tile is its own partner
  return Work{group, heavy == heavy_is_low ? u : tiles - 1 - u};
}
inline long long units_grid(long long groups, long long tiles) { return 16 * ((groups * ((tiles + 1) / 2) + 7) / 8); }

// Spread: workgroup i takes tile i in (tile descending, group) order - or, with the packed numbering (one group per
// head, tiles numbered through the sequences), in (tile, head) order - so that consecutive workgroups, which go to
// consecutive XCDs, are tiles of the same weight.
FA16_HD Work spread(int block, int groups, int tiles, bool packed) {
  if (block >= groups * tiles) return Work{-1, 0};
  const int t = block / groups;
  return Work{block - t * groups, packed ? t : tiles - 1 - t};
}

}  // namespace fa16
}  // namespace msd
