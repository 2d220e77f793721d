// Index arithmetic of the block-mask estimate kernels (sparse_estimate.hip), kept apart from the kernels so that
// the same functions can be compiled for the host and driven through every (workgroup, wave, lane, tile, chunk)
// of a launch with bounds assertions (tests/host/sbe_bounds.cpp does that at the long-sequence shapes).
// Plain C++: no HIP types.
#pragma once

#if defined(__HIPCC__)
#define SBE_HD __host__ __device__ __forceinline__
#else
#define SBE_HD inline
#endif

namespace msd {
namespace sbe {

// Geometry.  A strided row / column stands for 8 consecutive tokens; a workgroup owns kTile strided rows and walks
// a group of strided-column tiles of kTile; the head_dim x 8 contraction is walked in 16 chunks of 64 elements
// (chunk c: token s = c / 2 of the group of 8, head_dim half dh = c % 2).
constexpr int kStride = 8;
constexpr int kTile = 256;                     // strided rows per workgroup = strided columns per tile
constexpr int kWaves = 8;                      // 32 strided rows each
constexpr int kChunkBytes = 128;               // bytes of one row of a chunk (64 16-bit elements)
constexpr int kOperandBytes = kTile * kChunkBytes;   // 32 KiB: one chunk of the query rows or of the key columns
constexpr int kStageBytes = 2 * kOperandBytes;       // query chunk + key chunk
constexpr int kLdsBytes = 2 * kStageBytes;           // two stages
constexpr int kBlocksPerTile = kTile / 16;     // 16 mask blocks (128 tokens = 16 strided columns) per tile

struct Geom {
  int S;        // tokens
  int Sr;       // strided rows = ceil(S / 8)
  int NB;       // mask blocks = ceil(S / 128)
  int tiles;    // ceil(Sr / kTile): row tiles of a head = column tiles of a full row
  int Rp;       // tiles * kTile: rows of the workspace arrays per head
  int NBp;      // tiles * kBlocksPerTile: row pitch of `part`
};

SBE_HD Geom make_geom(int S) {
  Geom g;
  g.S = S;
  g.Sr = (S + kStride - 1) / kStride;
  g.NB = (S + 127) / 128;
  g.tiles = (g.Sr + kTile - 1) / kTile;
  g.Rp = g.tiles * kTile;
  g.NBp = g.tiles * kBlocksPerTile;
  return g;
}

// A row tile's column tiles are split over up to kColGroups workgroups (column groups of nearly equal size), and
// the workgroups of kRowBlock consecutive row tiles x all column groups are numbered consecutively: the 32
// workgroups an XCD runs at a time then share 4 query panels (2 MB) and 8 key streams through its L2, where one
// workgroup per row tile walking all columns had 32 query panels (16 MB) in flight and re-read them from the fabric
// for every column tile.
constexpr int kColGroups = 8;
constexpr int kRowBlock = 4;
SBE_HD int col_groups(const Geom& g) { return g.tiles < kColGroups ? g.tiles : kColGroups; }
SBE_HD int group_begin(const Geom& g, int cg) { return (int)((long long)cg * g.tiles / col_groups(g)); }  // cg <= groups
SBE_HD int work_per_head(const Geom& g) { return g.tiles * col_groups(g); }
// work item w of a head (0 .. work_per_head - 1) -> row tile and column group
SBE_HD void decode_work(const Geom& g, int w, int& rt, int& cg) {
  const int ng = col_groups(g);
  const int rb = w / (kRowBlock * ng);
  const int rows_in_block = g.tiles - rb * kRowBlock < kRowBlock ? g.tiles - rb * kRowBlock : kRowBlock;
  const int within = w - rb * kRowBlock * ng;
  rt = rb * kRowBlock + within % rows_in_block;
  cg = within / rows_in_block;
}

// Workspace per head (floats): partial block sums [Rp][NBp], the reference maxima they were taken against
// [Rp][tiles], and per row and column group the final maximum and row sum of that group [Rp][kColGroups][2].
SBE_HD long long part_floats_per_head(const Geom& g) { return (long long)g.Rp * g.NBp; }
SBE_HD long long mused_floats_per_head(const Geom& g) { return (long long)g.Rp * g.tiles; }
SBE_HD long long ml_floats_per_head(const Geom& g) { return (long long)g.Rp * kColGroups * 2; }
SBE_HD long long ws_floats_per_head(const Geom& g) {
  return part_floats_per_head(g) + mused_floats_per_head(g) + ml_floats_per_head(g);
}

// Strided columns that the rows of one wave see: all of them, or (causal, the reference's rule
// tests/plugin/test_sparseblockestimate.py:71-78) those below the end of the wave's step of 1024 query tokens, cut
// down to whole groups of 8 tokens (col_cap = S / 8).
SBE_HD int wave_cols(const Geom& g, int causal, int col_cap, int row0_of_wave) {
  if (!causal) return g.Sr;
  const int lim = 128 * (row0_of_wave / 128 + 1);
  return lim < col_cap ? lim : col_cap;
}
// Column tiles a workgroup walks: up to the largest limit of its waves.
SBE_HD int wg_col_tiles(const Geom& g, int causal, int col_cap, int i0) {
  const int cols = wave_cols(g, causal, col_cap, i0 + kTile - 32);
  return (cols + kTile - 1) / kTile;
}

// ---- LDS-DMA of one chunk of one operand: 32 instructions of 8 rows x 128 bytes, 4 per wave -----------------------
// Instruction i of wave w fills rows 8 * (8 * i + w) .. + 8 of the operand; lane L fills the physical 16-byte chunk
// L % 8 of row L / 8 of those, fetching the logical chunk (L % 8) ^ ((row >> 1) & 7).
SBE_HD int dma_row(int i, int wave, int lane) { return 8 * (8 * i + wave) + (lane >> 3); }
SBE_HD int dma_logical_chunk(int row, int lane) { return (lane & 7) ^ ((row >> 1) & 7); }
// per-lane byte offset (the part that does not depend on i, tile or chunk)
SBE_HD int dma_voffset(int wave, int lane, long long ss) {
  const int row = dma_row(0, wave, lane);
  return (int)((long long)kStride * row * ss * 2) + dma_logical_chunk(row, lane) * 16;
}
// wave-uniform byte offset: first strided row/column r0 of the tile, instruction i, token `tok` (0..7) of the
// groups, head_dim half dh
SBE_HD long long dma_soffset(int r0, int i, int tok, int dh, long long ss) {
  return ((long long)kStride * (r0 + 64 * i) + tok) * ss * 2 + dh * kChunkBytes;
}
// bytes of one (batch, head) slab that the buffer descriptor exposes; offsets at or beyond read as zeros
SBE_HD long long dma_range(int S, long long ss) { return ((long long)(S - 1) * ss + 128) * 2; }
// LDS byte offset (inside an operand) that instruction i of wave w writes: 1 KiB per instruction
SBE_HD int dma_lds(int i, int wave) { return (8 * i + wave) * 1024; }

// ---- operand reads of the matrix instruction (32x32x16): lane (l32, h), k step ks of the chunk --------------------
SBE_HD int frag_lds(int row, int ks, int h) { return row * kChunkBytes + ((((2 * ks + h)) ^ ((row >> 1) & 7)) << 4); }

// ---- workspace and output indices ---------------------------------------------------------------------------------
SBE_HD long long part_index(const Geom& g, int head_local, int row, int blk) {
  return ((long long)head_local * g.Rp + row) * g.NBp + blk;
}
SBE_HD long long mused_index(const Geom& g, int head_local, int row, int tile) {
  return ((long long)head_local * g.Rp + row) * g.tiles + tile;
}
SBE_HD long long ml_index(const Geom& g, int head_local, int row, int cg) {
  return (((long long)head_local * g.Rp + row) * kColGroups + cg) * 2;
}
SBE_HD long long score_index(const Geom& g, int head, int brow, int bcol) {
  return ((long long)head * g.NB + brow) * g.NB + bcol;
}

}  // namespace sbe
}  // namespace msd
