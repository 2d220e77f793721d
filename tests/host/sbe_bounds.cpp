// Host build of the index arithmetic of the block-mask estimate kernels (mindie-sd_amd/csrc/sbe_index.hpp, shared
// with sparse_estimate.hip): the loops of sbe_scores_kernel and sbe_select_kernel are walked for every workgroup,
// wave and lane of a launch with each memory access replaced by a bounds assertion, and the LDS layout the DMA
// writes is compared with the one the operand reads expect.
//   usage: sbe_bounds S heads N layout(0 = BNSD, 1 = BSND) causal ws_heads
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "sbe_index.hpp"

using namespace msd::sbe;
typedef long long ll;

static ll n_checks = 0;
#define CHECK(cond, ...)                                  \
  do {                                                    \
    ++n_checks;                                           \
    if (!(cond)) {                                        \
      std::printf("VIOLATION %s:%d: ", __FILE__, __LINE__); \
      std::printf(__VA_ARGS__);                           \
      std::printf("\n");                                  \
      std::exit(1);                                       \
    }                                                     \
  } while (0)

int main(int argc, char** argv) {
  if (argc != 7) return 2;
  const int S = std::atoi(argv[1]), heads_total = std::atoi(argv[2]), N = std::atoi(argv[3]);
  const int layout = std::atoi(argv[4]), causal = std::atoi(argv[5]), ws_heads = std::atoi(argv[6]);
  const int B = heads_total / N;
  const Geom g = make_geom(S);
  // element strides of a contiguous [B][N][S][128] (BNSD) or [B][S][N][128] (BSND) tensor
  const ll ss = layout == 0 ? 128 : (ll)N * 128, sn = layout == 0 ? (ll)S * 128 : 128, sb = (ll)N * S * 128;
  const ll tensor_bytes = (ll)B * N * S * 128 * 2;
  const ll range = dma_range(S, ss);
  CHECK(range > 0 && range < (1ll << 31), "descriptor range %lld", range);
  const int col_cap = std::max(1, S / kStride);
  const ll ws_floats = (ll)ws_heads * ws_floats_per_head(g);
  const ll part_floats = (ll)ws_heads * part_floats_per_head(g);  // mused starts here
  const ll ml_start = part_floats + (ll)ws_heads * mused_floats_per_head(g);  // group maxima / sums start here
  const ll score_floats = (ll)heads_total * g.NB * g.NB;
  std::vector<int> lds_owner(kOperandBytes / 16);  // which (row, logical chunk) each 16-byte LDS slot received

  // the entry point goes through the heads in groups of ws_heads
  for (int head0 = 0; head0 < heads_total; head0 += ws_heads) {
    const int heads = std::min(ws_heads, heads_total - head0);
    const int wph = work_per_head(g), ng = col_groups(g);
    const int total = heads * wph, per_xcd = (total + 7) / 8, grid = (total + 7) / 8 * 8;
    std::vector<char> seen(total, 0);
    std::vector<char> pair_seen((size_t)heads * g.tiles * ng, 0);          // (head, row tile, column group)
    std::vector<char> tile_done((size_t)heads * g.tiles * g.tiles, 0);     // (head, row tile, column tile) walked
    std::vector<char> group_ran((size_t)heads * g.tiles * kColGroups, 0);
    for (int bid = 0; bid < grid; ++bid) {
      const int work = (bid & 7) * per_xcd + (bid >> 3);
      if ((bid >> 3) >= per_xcd || work >= total) continue;
      CHECK(!seen[work], "work item %d taken twice", work);
      seen[work] = 1;
      const int hl = work / wph;
      int rt, cg;
      decode_work(g, work - hl * wph, rt, cg);
      CHECK(rt >= 0 && rt < g.tiles && cg >= 0 && cg < ng, "work item %d decodes to row tile %d, group %d", work, rt, cg);
      CHECK(!pair_seen[((size_t)hl * g.tiles + rt) * ng + cg], "(row tile, group) taken twice");
      pair_seen[((size_t)hl * g.tiles + rt) * ng + cg] = 1;
      if (causal) rt = g.tiles - 1 - rt;
      const int head = head0 + hl, b = head / N, n = head - b * N;
      {
        const int t_begin = group_begin(g, cg);
        const int t_end = std::min(group_begin(g, cg + 1), wg_col_tiles(g, causal, col_cap, rt * kTile));
        CHECK(t_begin >= 0 && group_begin(g, cg + 1) <= g.tiles && group_begin(g, cg + 1) > t_begin, "group %d bounds", cg);
        for (int t = t_begin; t < t_end; ++t) {
          CHECK(!tile_done[((size_t)hl * g.tiles + rt) * g.tiles + t], "column tile walked twice");
          tile_done[((size_t)hl * g.tiles + rt) * g.tiles + t] = 1;
        }
        if (t_begin < t_end) group_ran[((size_t)hl * g.tiles + rt) * kColGroups + cg] = 1;
      }
      // only the first and the last head of a group and the first, second and last row tile are walked lane by
      // lane (the arithmetic is affine in both); every work item is still checked for its mapping above
      if ((hl != 0 && hl != heads - 1) || (rt > 1 && rt < g.tiles - 2)) continue;
      const int i0 = rt * kTile;
      const ll slab = (b * sb + n * sn) * 2;  // byte offset of the (batch, head) slab inside the tensor
      const int n_tiles = wg_col_tiles(g, causal, col_cap, i0);
      CHECK(n_tiles >= 1 && n_tiles <= g.tiles, "n_tiles %d", n_tiles);
      const int t_begin = group_begin(g, cg), t_end = std::min(group_begin(g, cg + 1), n_tiles);
      if (t_begin >= t_end) continue;  // the workgroup returns before its first request
      for (int wave = 0; wave < kWaves; ++wave) {
        const int my_cols = wave_cols(g, causal, col_cap, i0 + 32 * wave);
        CHECK(my_cols >= 1 && my_cols <= g.Sr, "my_cols %d", my_cols);
        CHECK((my_cols + kTile - 1) / kTile <= n_tiles, "wave sees more tiles than the workgroup walks");
        CHECK(my_cols > 0, "tile 0 must be visible");
      }
      for (int t = t_begin; t < t_end; ++t)
        for (int s = 0; s < kStride; ++s)
          for (int dh = 0; dh < 2; ++dh) {
            // only the first two and the last tile of the group lane by lane
            if (t > t_begin + 1 && t < t_end - 1) continue;
            for (int operand = 0; operand < 2; ++operand) {  // 0: query rows, 1: key columns
              std::fill(lds_owner.begin(), lds_owner.end(), -1);
              for (int wave = 0; wave < kWaves; ++wave)
                for (int i = 0; i < 4; ++i)
                  for (int lane = 0; lane < 64; ++lane) {
                    const int r0 = operand == 0 ? i0 : t * kTile;
                    const int tok = operand == 0 ? kStride - 1 - s : s;
                    const ll voff = dma_voffset(wave, lane, ss), soff = dma_soffset(r0, i, tok, dh, ss);
                    CHECK(voff >= 0 && soff >= 0 && voff + soff + 16 < (1ll << 31), "offset overflow %lld %lld", voff, soff);
                    const ll off = voff + soff;
                    const int row = dma_row(i, wave, lane), chunk = dma_logical_chunk(row, lane);
                    // what the request names: token 8 * (r0 + row) + tok, bytes 128 dh + 16 chunk .. + 16 of its row
                    const ll token = (ll)kStride * (r0 + row) + tok;
                    CHECK(off == token * ss * 2 + dh * kChunkBytes + chunk * 16, "offset names the wrong bytes");
                    if (off + 16 <= range) {
                      CHECK(token < S, "in-range request for token %lld >= S", token);
                      CHECK(slab + off + 16 <= tensor_bytes, "read past the tensor");
                    } else {
                      CHECK(token >= S, "token %lld < S is cut off by the descriptor range", token);
                    }
                    const int lds = dma_lds(i, wave) + lane * 16;
                    CHECK(lds >= 0 && lds + 16 <= kOperandBytes, "LDS destination %d", lds);
                    CHECK(lds_owner[lds / 16] == -1, "LDS slot written twice");
                    lds_owner[lds / 16] = row * 8 + chunk;
                  }
              // every slot filled, and the operand reads find logical chunk 2 ks + h of row `row` where they look
              for (int row = 0; row < kTile; ++row)
                for (int ks = 0; ks < 4; ++ks)
                  for (int h = 0; h < 2; ++h) {
                    const int a = frag_lds(row, ks, h);
                    CHECK(a >= 0 && a + 16 <= kOperandBytes && a % 16 == 0, "operand read at %d", a);
                    CHECK(lds_owner[a / 16] == row * 8 + 2 * ks + h, "operand read finds the wrong chunk");
                  }
            }
          }
      // epilogue stores and the read-back
      for (int wave = 0; wave < kWaves; ++wave)
        for (int l32 = 0; l32 < 32; ++l32)
          for (int h = 0; h < 2; ++h) {
            const int my_row = i0 + 32 * wave + l32;
            CHECK(my_row < g.Rp, "row %d", my_row);
            {
              const ll li = ml_start + ml_index(g, hl, my_row, cg);
              CHECK(li >= ml_start && li + 2 <= ws_floats && li % 2 == 0, "group maximum / sum store %lld of %lld", li, ws_floats);
            }
            for (int t = t_begin; t < t_end; ++t) {
              const ll pi = part_index(g, hl, my_row, 0) + t * kBlocksPerTile + 8 * h;
              CHECK(pi >= 0 && pi + 8 <= part_floats && pi % 4 == 0, "part store %lld of %lld", pi, part_floats);
              const ll mi = part_floats + mused_index(g, hl, my_row, 0) + t;
              CHECK(mi >= part_floats && mi < ml_start, "mused store %lld of %lld", mi, ml_start);
            }
          }
    }
    // every (row tile, column tile) a row tile sees was walked by exactly one workgroup
    for (int hl = 0; hl < heads; ++hl)
      for (int rt = 0; rt < g.tiles; ++rt) {
        const int n_tiles = wg_col_tiles(g, causal, col_cap, rt * kTile);
        for (int t = 0; t < g.tiles; ++t)
          CHECK(tile_done[((size_t)hl * g.tiles + rt) * g.tiles + t] == (t < n_tiles ? 1 : 0), "row tile %d column tile %d", rt, t);
      }
    // sbe_finalize_kernel: 64 lanes per (head, block row)
    for (int hl = 0; hl < heads; hl += std::max(1, heads - 1))
      for (int brow = 0; brow < g.NB; ++brow) {
        const int head = head0 + hl, row0 = 16 * brow, rows = std::min(16, g.Sr - row0);
        CHECK(rows >= 1, "block row %d without rows", brow);
        const int i0 = row0 / kTile * kTile, rt = i0 / kTile;
        const int n_tiles = wg_col_tiles(g, causal, col_cap, i0);
        for (int lane = 0; lane < rows; ++lane)
          for (int c = 0; c < ng && group_begin(g, c) < n_tiles; ++c) {
            const ll li = ml_start + ml_index(g, hl, row0 + lane, 0) + 2 * c;
            CHECK(li >= ml_start && li + 2 <= ws_floats, "group maximum / sum read %lld", li);
            CHECK(group_ran[((size_t)hl * g.tiles + rt) * kColGroups + c], "reads a group that never ran");
          }
        const int blocks_done = n_tiles * kBlocksPerTile;
        for (int J0 = 0; J0 < g.NB; J0 += 64)
          for (int lane = 0; lane < 64; ++lane) {
            const int J = J0 + lane;
            const bool live = J < g.NB && J < blocks_done;
            for (int i = 0; i < rows; ++i) {
              const ll pi = part_index(g, hl, row0, live ? J : 0) + (ll)i * g.NBp;
              const ll mi = part_floats + mused_index(g, hl, row0, live ? J >> 4 : 0) + (ll)i * g.tiles;
              CHECK(pi >= 0 && pi < part_floats, "part read %lld", pi);
              CHECK(mi >= part_floats && mi < ml_start, "mused read %lld", mi);
              CHECK(tile_done[((size_t)hl * g.tiles + rt) * g.tiles + (live ? J >> 4 : 0)], "reads a tile never written");
            }
            if (J < g.NB) {
              const ll si = score_index(g, head, brow, 0) + J;
              CHECK(si >= 0 && si < score_floats, "score store %lld of %lld", si, score_floats);
            }
          }
      }
    for (int w = 0; w < total; ++w) CHECK(seen[w], "work item %d never taken", w);
  }

  // ---- sbe_select_kernel: one workgroup of 256 threads per (head, block row) ---------------------------------------
  const int NB = g.NB, pitch = (NB + 31) / 32 * 32;
  int n2 = 8;
  while (n2 < NB) n2 <<= 1;
  const int sorted0 = (NB + 3) & ~3, prefix0 = sorted0 + n2;
  const ll mask_bytes = (ll)heads_total * NB * pitch, lds_floats = sorted0 + 2 * n2;
  for (int by = 0; by < heads_total; by += std::max(1, heads_total - 1))
    for (int bx = 0; bx < NB; ++bx)
      for (int tid = 0; tid < 256; ++tid) {
        const ll r = (ll)by * NB + bx;
        const int L = causal ? bx + 1 : NB;
        for (int j = tid; j < L; j += 256) CHECK(j < NB && r * NB + j < score_floats, "score read");
        int l2 = 8;
        while (l2 < L) l2 <<= 1;
        CHECK(l2 <= n2, "sort width %d", l2);
        for (int e = tid; e < l2; e += 256) CHECK(sorted0 + e < prefix0, "sort slot");
        if (tid == 0) {
          for (int j = 0; j < L; j += 8) {  // 8 values per step, the next 8 requested ahead
            CHECK(sorted0 + j + 8 <= prefix0 && prefix0 + j + 8 <= lds_floats, "running sums %d", j);
            if (j + 8 < L) CHECK(sorted0 + j + 16 <= prefix0, "read ahead %d", j);
          }
          CHECK(sorted0 + L - 1 < prefix0 && prefix0 + L - 1 < lds_floats, "guard read");  // positions are within [0, L - 1]
        }
        for (int j = tid; j < pitch; j += 256) CHECK(r * pitch + j < mask_bytes, "mask store");
        CHECK(r < (ll)heads_total * NB, "count store");
      }
  std::printf("S %d heads %d layout %s causal %d groups of %d: %lld checks passed (Sr %d, NB %d, tiles %d, workspace %lld MiB)\n", S,
              heads_total, layout ? "BSND" : "BNSD", causal, ws_heads, n_checks, g.Sr, g.NB, g.tiles,
              ws_floats * 4 >> 20);
  return 0;
}
