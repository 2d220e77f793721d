// Host check of the tile numbering of the 16x16x32 attention kernels (mindie-sd_amd/csrc/fa16_work.hpp, the functions
// the kernels themselves call): every workgroup of a grid lands on a tile of its own, every tile is taken exactly
// once, and - for the numbering in units of a heavy and a light tile - the work of the busiest XCD stays close to the
// mean.  usage: fa16_work_cover <groups> <tiles>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "fa16_work.hpp"

using namespace msd::fa16;

static long long checks = 0;

static void fail(const char* what, int groups, int tiles, int block) {
  std::printf("FAILED %s groups %d tiles %d block %d\n", what, groups, tiles, block);
  std::exit(1);
}

template <class F>
static void cover(const char* name, int groups, int tiles, long long grid, F&& f, bool weigh_causal) {
  std::vector<int> seen((size_t)groups * tiles, 0);
  double xcd_work[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (long long block = 0; block < grid; ++block) {
    const Work w = f((int)block);
    if (w.group < 0) continue;
    if (w.group >= groups || w.tile < 0 || w.tile >= tiles) fail(name, groups, tiles, (int)block);
    if (seen[(size_t)w.group * tiles + w.tile]++) fail(name, groups, tiles, (int)block);
    xcd_work[block & 7] += weigh_causal ? w.tile + 1 : 1;
    ++checks;
  }
  for (size_t i = 0; i < seen.size(); ++i)
    if (seen[i] != 1) fail(name, groups, tiles, -1);
  if (weigh_causal && (long long)groups * tiles >= 2048) {  // enough tiles for the balance to mean something
    double mx = 0, sum = 0;
    for (double x : xcd_work) {
      mx = x > mx ? x : mx;
      sum += x;
    }
    if (mx > 1.05 * sum / 8) {
      std::printf("FAILED balance %s groups %d tiles %d: busiest XCD %.3f of the mean\n", name, groups, tiles, mx / (sum / 8));
      std::exit(1);
    }
  }
}

int main(int argc, char** argv) {
  if (argc != 3) return 2;
  const int groups = std::atoi(argv[1]), tiles = std::atoi(argv[2]);
  cover("runs", groups, tiles, runs_grid(groups, tiles), [&](int b) { return runs(b, groups, tiles); }, false);
  // a grid sized for more tiles than exist (the packed numbering's upper bound)
  cover("runs, larger grid", groups, tiles, runs_grid(groups, tiles + 3) + 64, [&](int b) { return runs(b, groups, tiles); },
        false);
  cover("units, heavy = high index", groups, tiles, units_grid(groups, tiles),
        [&](int b) { return units(b, groups, tiles, false); }, true);
  cover("units, heavy = low index", groups, tiles, units_grid(groups, tiles),
        [&](int b) { return units(b, groups, tiles, true); }, false);
  cover("spread", groups, tiles, units_grid(groups, tiles), [&](int b) { return spread(b, groups, tiles, false); }, false);
  cover("spread, runs grid", groups, tiles, runs_grid(groups, tiles), [&](int b) { return spread(b, groups, tiles, false); },
        false);
  cover("spread, packed", groups, tiles, runs_grid(groups, tiles + 5), [&](int b) { return spread(b, groups, tiles, true); },
        false);
  std::printf("%lld checks passed\n", checks);
  return 0;
}
