// Block mask estimation for adaptive block-sparse attention (XAttention style) on gfx950 (MI355X).
//
// Takes the place of the reference's in-tree AscendC kernel SparseBlockEstimate
// (csrc/ops/sparse_block_estimate/op_kernel/sparse_block_estimate.h, host wrapper
// csrc/plugin/sparse_block_estimate.cpp:27-85; numpy statement of the algorithm in
// tests/plugin/test_sparseblockestimate.py:49-145):
//   1. anti-diagonal strided scores: with stride 8, P'[i][j] = scale * sum_{s<8} q[8i+7-s] . k[8j+s]
//      (one eighth of the work of the full score matrix);
//   2. row softmax of P' summed over 16 x 16 blocks: the share of the (estimated) attention mass that 128-token
//      query block I puts on 128-token key block J;
//   3. per query block, sort the key blocks by mass, keep the smallest prefix whose mass reaches `threshold` of
//      the total (capped at row_sparse * blocks), always keep the first block (attention sink) and the last one.
// sbe_scores_kernel + sbe_finalize_kernel do 1 and 2 (P' is never written), sbe_select_kernel does 3.
#include <type_traits>

#include "common.hpp"
#include "sbe_index.hpp"

namespace msd {

// the float that lane `idx` (wave-uniform) holds in v
__device__ __forceinline__ float lane_value(float v, int idx) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), idx));
}

struct SbeParams {
  const void* q;
  const void* k;
  long long q_sb, q_sn, q_ss;  // element strides of batch, head, token (head_dim 128 contiguous)
  long long k_sb, k_sn, k_ss;
  int N, Nkv;
  int head0;     // first (batch * N + head) of this launch
  int heads;     // heads of this launch
  float scale_log2;
  int causal, col_cap;
  float* part;   // [heads][Rp][NBp]   block sums of exp2(score - reference), per strided row
  float* mused;  // [heads][Rp][tiles] the reference each column tile's sums were taken against
  float* ml;     // [heads][Rp][kColGroups][2] final maximum and row sum of every column group
  float* scores; // [all heads][NB][NB]
  sbe::Geom g;
};

// P' as a matrix product: Q' [Sr][8 x 128] (row i = tokens 8i+7, 8i+6, ..., 8i side by side) times K' [Sr][8 x 128]^T
// (row j = tokens 8j .. 8j+7), i.e. two row-major views of q and k whose 128-wide K chunks are paired in opposite
// order.  One workgroup (8 waves) owns 256 strided rows (2048 query tokens) of one head and walks one group of
// strided-column tiles of 256 (a row tile's columns are split over up to 8 workgroups, sbe_index.hpp); a wave owns 32 rows x 256 columns (8 accumulators of the 32x32x16 instruction, computed
// transposed: keys are the rows of the accumulator, so a softmax row lives in one lane pair).  The contraction
// runs in 16 chunks of 64 elements; a chunk of both operands (2 x 32 KiB) is staged in LDS by LDS-DMA, double
// buffered, one barrier per chunk.  Tokens past the end of the sequence are outside the buffer descriptors' range
// and read as zeros, as the reference pads them.
// After the last chunk of a tile the wave holds the 32 x 256 scores: running row maximum and sum, exp2, sums over
// the 16 columns of every mask block (8 in-lane additions and one exchange between the wave halves), stored per
// strided row together with the maximum they refer to.  When its tiles are done the workgroup stores the maximum and
// row sum its column group ended with; sbe_finalize_kernel combines the groups, rescales the stored sums to the final
// maximum, divides by the row sum and adds up the 16 rows of each mask block.
template <int DT>
__global__ __launch_bounds__(512, 1) void sbe_scores_kernel(const SbeParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  using E = Elem<DT>;
  using T = typename E::type;
  using X8 = typename E::x8;
  using namespace sbe;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  MSD_LDS char* smem = (MSD_LDS char*)smem_raw;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, h = lane >> 5;
  const Geom g = p.g;

  // consecutive work items stay on one XCD: 4 row tiles x 8 column groups of one head at a time (decode_work)
  const int wph = work_per_head(g);
  const int total = p.heads * wph;
  const int per_xcd = (total + 7) / 8;
  const int work = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if ((int)(blockIdx.x >> 3) >= per_xcd || work >= total) return;
  const int hl = work / wph;                           // head inside this launch
  int rt, cg;
  decode_work(g, work - hl * wph, rt, cg);
  if (p.causal) rt = g.tiles - 1 - rt;                 // the row tiles with the most columns start first
  const int head = p.head0 + hl;
  const int b = head / p.N, n = head - b * p.N;
  const int nkv = n / (p.N / p.Nkv);
  const int i0 = rt * kTile;

  const T* qg = (const T*)p.q + b * p.q_sb + n * p.q_sn;
  const T* kg = (const T*)p.k + b * p.k_sb + nkv * p.k_sn;
  const __amdgpu_buffer_rsrc_t q_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)qg, 0, (int)dma_range(g.S, p.q_ss), 0x00020000);
  const __amdgpu_buffer_rsrc_t k_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)kg, 0, (int)dma_range(g.S, p.k_ss), 0x00020000);
  const int q_voff = dma_voffset(wave, lane, p.q_ss), k_voff = dma_voffset(wave, lane, p.k_ss);

  const int my_cols = wave_cols(g, p.causal, p.col_cap, i0 + 32 * wave);  // strided columns this wave's rows see
  // this workgroup's column tiles: its group, cut at the last tile any of its rows sees
  const int t_begin = group_begin(g, cg);
  const int t_end = min(group_begin(g, cg + 1), wg_col_tiles(g, p.causal, p.col_cap, i0));
  if (t_begin >= t_end) return;

  // chunk c of column tile t into LDS stage `stage`: query rows i0.., token 7 - s; key columns 256 t.., token s
  auto load_chunk = [&](int t, int s, int dh, int stage) {
    MSD_LDS char* qb = smem + stage * kStageBytes;
    MSD_LDS char* kb = qb + kOperandBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(q_rsrc, (MSD_LDS void*)(qb + dma_lds(i, wave)), 16, q_voff,
                                               (int)dma_soffset(i0, i, kStride - 1 - s, dh, p.q_ss), 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(k_rsrc, (MSD_LDS void*)(kb + dma_lds(i, wave)), 16, k_voff,
                                               (int)dma_soffset(t * kTile, i, s, dh, p.k_ss), 0, 0);
    }
  };

  // operand read addresses: the lane's row of the query operand, row l32 of key block 0
  int q_rd[4], k_rd[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    q_rd[ks] = frag_lds(32 * wave + l32, ks, h);
    k_rd[ks] = kOperandBytes + frag_lds(l32, ks, h);
  }

  f32x16_t acc[8];
  float m_run = -INFINITY, l_run = 0.f;  // running row maximum (log2 units) and this lane's part of the row sum
  const int my_row = i0 + 32 * wave + l32;
  float* part_row = p.part + part_index(g, hl, my_row, 0);
  float* mused_row = p.mused + mused_index(g, hl, my_row, 0);

  load_chunk(t_begin, 0, 0, 0);
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  __syncthreads();

  auto chunk_step = [&](auto stage_c, int t, int s, bool has_next, int nt, int ns) {
    constexpr int stage = decltype(stage_c)::value;
    if (has_next) load_chunk(nt, ns, stage ^ 1, stage ^ 1);  // the next chunk is the other head_dim half
    MSD_LDS const char* base = smem + stage * kStageBytes;
    X8 qf[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) qf[ks] = *(MSD_LDS const X8*)(base + q_rd[ks]);
    X8 kf[2][8];
#pragma unroll
    for (int kb = 0; kb < 8; ++kb) kf[0][kb] = *(MSD_LDS const X8*)(base + k_rd[0] + kb * 32 * kChunkBytes);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      if (ks + 1 < 4) {
#pragma unroll
        for (int kb = 0; kb < 8; ++kb)
          kf[(ks + 1) & 1][kb] = *(MSD_LDS const X8*)(base + k_rd[ks + 1] + kb * 32 * kChunkBytes);
      }
#pragma unroll
      for (int kb = 0; kb < 8; ++kb) acc[kb] = E::mfma32(kf[ks & 1][kb], qf[ks], acc[kb]);
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's part of the next chunk has landed
    __syncthreads();
  };

  for (int t = t_begin; t < t_end; ++t) {
#pragma unroll
    for (int kb = 0; kb < 8; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[kb][r] = 0.f;
    for (int s = 0; s < kStride; ++s) {
      chunk_step(std::integral_constant<int, 0>{}, t, s, true, t, s);
      const bool more = s + 1 < kStride || t + 1 < t_end;
      chunk_step(std::integral_constant<int, 1>{}, t, s, more, s + 1 < kStride ? t : t + 1, s + 1 < kStride ? s + 1 : 0);
    }

    // ---- the tile's scores: accumulator kb register r = key 256 t + 32 kb + 8 (r / 4) + 4 h + r % 4 of row l32 ----
    const int j0 = t * kTile;
    float bs[16];  // this lane's part of the sum of block j (columns 16 j .. 16 j + 15 of the tile)
#pragma unroll
    for (int j = 0; j < 16; ++j) bs[j] = 0.f;
    if (j0 < my_cols) {  // otherwise (causal) nothing of this tile is visible to this wave's rows
      const bool cut = j0 + kTile > my_cols;  // the limit runs through this tile: test every column
      float mx = -INFINITY;
      if (cut) {
#pragma unroll
        for (int kb = 0; kb < 8; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = j0 + 32 * kb + 8 * (r >> 2) + 4 * h + (r & 3);
            if (key >= my_cols) acc[kb][r] = -INFINITY;
          }
      }
#pragma unroll
      for (int kb = 0; kb < 8; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, acc[kb][r]);
      mx = half_max(mx) * p.scale_log2;  // at least one column of the tile is visible, so this is finite
      const float m_new = fmaxf(m_run, mx);
      l_run *= fast_exp2(m_run - m_new);  // first visible tile: exp2(-inf) = 0
      m_run = m_new;
#pragma unroll
      for (int kb = 0; kb < 8; ++kb) {
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int r = 0; r < 8; ++r) s0 += fast_exp2(acc[kb][r] * p.scale_log2 - m_new);
#pragma unroll
        for (int r = 8; r < 16; ++r) s1 += fast_exp2(acc[kb][r] * p.scale_log2 - m_new);
        l_run += s0 + s1;
        bs[2 * kb] = s0;
        bs[2 * kb + 1] = s1;
      }
    }
    // lanes of half h receive and store the totals of blocks 8 h .. 8 h + 7 of their row (the workspace rows are
    // padded, no row test needed)
    f32x4_t lo, hi;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      lo[j] = half_pair_sum(bs[j], bs[8 + j]);
      hi[j] = half_pair_sum(bs[4 + j], bs[12 + j]);
    }
    *(f32x4_t*)(part_row + t * kBlocksPerTile + 8 * h) = lo;
    *(f32x4_t*)(part_row + t * kBlocksPerTile + 8 * h + 4) = hi;
    if (h == 0) mused_row[t] = m_run;
  }

  // ---- the group's final maximum and row sum (-inf and 0 for rows that saw none of its columns) ---------------------
  const float l_tot = half_sum(l_run);
  if (h == 0) *(f32x2_t*)(p.ml + ml_index(g, hl, my_row, cg)) = f32x2_t{m_run, l_tot};
#endif
}

// Second step of the block scores: one workgroup of 64 lanes per (head, mask block row).  For each of its (up to)
// 16 strided rows the final maximum and row sum are put together from the column groups, then lane J adds up the
// rows' sums of block J, each brought from the reference it was taken against to the final one and divided by the
// row sum.  Columns past the last tile the row tile walked (causal) are zero.
__global__ __launch_bounds__(64) void sbe_finalize_kernel(const SbeParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  using namespace sbe;
  const Geom g = p.g;
  const int lane = threadIdx.x;
  const int brow = blockIdx.x, hl = blockIdx.y;
  const int head = p.head0 + hl;
  const int row0 = 16 * brow;
  const int rows = min(16, g.Sr - row0);  // > 0 because brow < NB
  const int i0 = row0 / kTile * kTile;
  const int n_tiles = wg_col_tiles(g, p.causal, p.col_cap, i0);
  const int ng = col_groups(g);
  // lane i < rows: final maximum and reciprocal row sum of row row0 + i
  float m_fin = -INFINITY, inv_l = 0.f;
  if (lane < rows) {
    const float* ml = p.ml + ml_index(g, hl, row0 + lane, 0);
    for (int c = 0; c < ng && group_begin(g, c) < n_tiles; ++c) m_fin = fmaxf(m_fin, ml[2 * c]);
    float l = 0.f;
    for (int c = 0; c < ng && group_begin(g, c) < n_tiles; ++c) l += ml[2 * c + 1] * fast_exp2(ml[2 * c] - m_fin);
    inv_l = 1.0f / l;
  }
  const int blocks_done = n_tiles * kBlocksPerTile;
  float* out = p.scores + score_index(g, head, brow, 0);
  for (int J0 = 0; J0 < g.NB; J0 += 64) {
    const int J = J0 + lane;
    const bool live = J < g.NB && J < blocks_done;
    const float* pr = p.part + part_index(g, hl, row0, live ? J : 0);
    const float* mr = p.mused + mused_index(g, hl, row0, live ? J >> 4 : 0);
    float v = 0.f;
#pragma unroll 1
    for (int i = 0; i < rows; ++i) {  // wave-uniform trip count and lane index
      const float mf = lane_value(m_fin, i);
      const float w = lane_value(inv_l, i);
      v += pr[(long long)i * g.NBp] * fast_exp2(mr[i * g.tiles] - mf) * w;
    }
    if (J < g.NB) out[J] = live ? v : 0.f;
  }
#endif
}

// scores [BN][NB][NB] -> mask int8 [BN][NB][pitch] (pitch >= NB, padding zero) + count int32 [BN][NB].
// One workgroup per block row.  The rules are those of the reference kernel
// (csrc/ops/sparse_block_estimate/op_kernel/sparse_block_estimate.h:947-1078); its numpy statement
// (tests/plugin/test_sparseblockestimate.py:121-143) agrees with them for the default switches up to the handling
// of the first block, which the kernel leaves out of the ranking and of the total when keep_sink is set.
//   L = columns that take part: all NB, or (causal) the first brow + 1;  causal rows with L <= 2 keep all L.
//   Left out of the ranking (score 0): the last of the L columns if keep_recent or not causal; column 0 if keep_sink.
//   total = sum of the ranked scores;  descending stable sort;  guard = the first sorted score at which the
//   sequential fp32 running sum reaches threshold * total (threshold >= 1: guard = 0 and every column is kept);
//   if more than row_sparse * L columns would be kept and L >= 10, guard = sorted[int(row_sparse * L) - 1];
//   guard -= 1e-5;  column 0 is forced if keep_sink, the last one if keep_recent or not causal;
//   keep[j] = score[j] > guard;  column 0 is always kept.
constexpr float kSbeEps = 1e-5f;
// smallest power of two that is >= n and >= 8
__host__ __device__ inline int n2_of(int n) {
  int n2 = 8;
  while (n2 < n) n2 <<= 1;
  return n2;
}
__global__ __launch_bounds__(256) void sbe_select_kernel(const float* scores, signed char* mask, int* count, int NB,
                                                         int pitch, float threshold, float row_sparse, int keep_sink,
                                                         int keep_recent, int causal) {
#if defined(__HIP_DEVICE_COMPILE__)
  extern __shared__ __attribute__((aligned(16))) float sh[];  // [NB] row, [n2] sorted, [n2] running sums (n2: NB rounded up to a power of two, at least 8)
  float* row = sh;
  float* sorted = sh + ((NB + 3) & ~3);  // 16-byte aligned
  float* prefix = sorted + n2_of(NB);
  __shared__ float guard_s;
  __shared__ int first_s;
  __shared__ int cnt_s[4];
  const int tid = threadIdx.x;
  const long long r = (long long)blockIdx.y * NB + blockIdx.x;
  const float* src = scores + r * NB;
  const int L = causal ? (int)blockIdx.x + 1 : NB;  // columns that take part
  const bool whole_prefix = causal && L <= 2;
  const bool last_out = keep_recent || !causal;
  for (int j = tid; j < L; j += 256) row[j] = ((j == L - 1 && last_out) || (j == 0 && keep_sink)) ? 0.f : src[j];
  __syncthreads();
  // descending bitonic sort of the L values, padded with -inf to a power of two (only the sorted values are used,
  // so the order among equal ones does not matter)
  const int n2 = n2_of(L);
  for (int e = tid; e < n2; e += 256) sorted[e] = e < L ? row[e] : -INFINITY;
  __syncthreads();
  for (int k = 2; k <= n2; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int i = tid; i < (n2 >> 1); i += 256) {
        const int lo = ((i & ~(j - 1)) << 1) | (i & (j - 1)), hi = lo | j;
        const float a = sorted[lo], b = sorted[hi];
        const bool desc = (lo & k) == 0;
        if (desc ? a < b : a > b) {
          sorted[lo] = b;
          sorted[hi] = a;
        }
      }
      __syncthreads();
    }
  }
  // Sequential fp32 running sums of the sorted values (the reference kernel's order of additions), written over
  // them: one lane, eight values per step from two 16-byte reads that are requested one step ahead (the padding
  // up to a multiple of 8 holds -inf and only reaches sums past the end, which nobody reads).
  if (tid == 0 && threshold < 1.0f) {
    float run = 0.f;
    f32x4_t a = *(const f32x4_t*)(sorted), b4 = *(const f32x4_t*)(sorted + 4);
    for (int j = 0; j < L; j += 8) {
      f32x4_t na = a, nb = b4;
      if (j + 8 < L) {
        na = *(const f32x4_t*)(sorted + j + 8);
        nb = *(const f32x4_t*)(sorted + j + 12);
      }
      f32x4_t pa, pb;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        run += a[i];
        pa[i] = run;
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        run += b4[i];
        pb[i] = run;
      }
      *(f32x4_t*)(prefix + j) = pa;
      *(f32x4_t*)(prefix + j + 4) = pb;
      a = na;
      b4 = nb;
    }
  }
  if (tid == 0) first_s = L - 1;
  __syncthreads();
  // first position whose running sum reaches threshold * total (total = the last running sum)
  if (threshold < 1.0f) {
    const float lim = threshold * prefix[L - 1];
    int mine_first = L - 1;
    for (int j = tid; j < L; j += 256)
      if (prefix[j] >= lim) {
        mine_first = j;
        break;
      }
    if (mine_first < L - 1) atomicMin(&first_s, mine_first);
  }
  __syncthreads();
  if (tid == 0) {
    float guard = 0.f;
    int cnt = L;
    if (threshold < 1.0f) {
      cnt = first_s;
      guard = sorted[cnt];
    }
    if ((float)cnt > (float)L * row_sparse && L >= 10) {
      const int kk = max(1, (int)((float)L * row_sparse));
      guard = sorted[min(kk, L) - 1];
    }
    guard_s = guard - kSbeEps;
  }
  __syncthreads();
  const float guard = guard_s;
  int mine = 0;
  signed char* mrow = mask + r * pitch;
  for (int j = tid; j < pitch; j += 256) {
    int keep = 0;
    if (j < L) {
      float v = row[j];
      if (j == 0 && keep_sink) v = guard + 1.f;
      if (j == L - 1 && last_out) v = guard + 1.f;
      keep = (v > guard || whole_prefix || j == 0) ? 1 : 0;
    }
    mrow[j] = (signed char)keep;
    mine += keep;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mine += __shfl_xor(mine, o, 64);
  if ((tid & 63) == 0) cnt_s[tid >> 6] = mine;
  __syncthreads();
  if (tid == 0) count[r] = cnt_s[0] + cnt_s[1] + cnt_s[2] + cnt_s[3];
#endif
}

}  // namespace msd

using namespace msd;

extern "C" {

// Scratch of mindiesd_sbe_scores for `heads` (batch x head) pairs of S tokens, in bytes.  The call works with any
// workspace that holds at least one head and then goes through the heads in groups.
size_t mindiesd_sbe_scores_workspace_size(int heads, int S) {
  if (heads <= 0 || S <= 0) return 0;
  return (size_t)heads * (size_t)sbe::ws_floats_per_head(sbe::make_geom(S)) * sizeof(float);
}

// q, k [B][N | Nkv][S][128] (16-bit, element strides) -> block scores [B * N][NB][NB] fp32, NB = ceil(S / 128):
// scores[bn][I][J] = sum over the 16 x 16 block (I, J) of softmax_j(scale * P'), P'[i][j] = sum_{s<8} q[8i+7-s] . k[8j+s].
int mindiesd_sbe_scores(const void* q, const void* k, float* scores, int dtype, int B, int N, int Nkv, int S, int D,
                        long long q_sb, long long q_sn, long long q_ss, long long k_sb, long long k_sn, long long k_ss,
                        float scale, int causal, void* workspace, size_t ws_bytes, hipStream_t stream) {
  if (!q || !k || !scores || !workspace || B <= 0 || N <= 0 || Nkv <= 0 || S <= 0 || N % Nkv != 0) return MSD_ERR_BAD_ARG;
  if (D != 128 || !(scale > 0.f)) return MSD_ERR_UNSUPPORTED;
  if (dtype != MSD_DTYPE_BF16 && dtype != MSD_DTYPE_F16) return MSD_ERR_BAD_ARG;
  if ((((uintptr_t)q | (uintptr_t)k | (uintptr_t)workspace) & 15) || ((uintptr_t)scores & 3)) return MSD_ERR_BAD_ARG;
  if ((q_sb | q_sn | q_ss | k_sb | k_sn | k_ss) & 7) return MSD_ERR_BAD_ARG;
  if (q_ss < 128 || k_ss < 128) return MSD_ERR_BAD_ARG;
  const sbe::Geom g = sbe::make_geom(S);
  // 32-bit buffer offsets: the furthest byte a (zero-filled) request can name must stay below 2^31
  const long long far_rows = (long long)sbe::kStride * g.Rp + sbe::kStride;
  if (far_rows * q_ss * 2 + 512 >= (1ll << 31) || far_rows * k_ss * 2 + 512 >= (1ll << 31)) return MSD_ERR_UNSUPPORTED;
  const long long per_head = sbe::ws_floats_per_head(g) * (long long)sizeof(float);
  const long long fit = (long long)(ws_bytes / (size_t)per_head);
  if (fit < 1) return MSD_ERR_WORKSPACE;
  const long long BN = (long long)B * N;
  if (BN * g.NB * g.NB >= (1ll << 40)) return MSD_ERR_UNSUPPORTED;
  auto kern = dtype == MSD_DTYPE_BF16 ? sbe_scores_kernel<MSD_DTYPE_BF16> : sbe_scores_kernel<MSD_DTYPE_F16>;
  if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, sbe::kLdsBytes) != hipSuccess)
    return MSD_ERR_LAUNCH;
  const int group = (int)(fit < BN ? fit : BN);
  for (long long h0 = 0; h0 < BN; h0 += group) {
    SbeParams p{};
    p.q = q; p.k = k;
    p.q_sb = q_sb; p.q_sn = q_sn; p.q_ss = q_ss; p.k_sb = k_sb; p.k_sn = k_sn; p.k_ss = k_ss;
    p.N = N; p.Nkv = Nkv;
    p.head0 = (int)h0;
    p.heads = (int)(BN - h0 < group ? BN - h0 : group);
    p.scale_log2 = scale * 1.4426950408889634f;
    p.causal = causal ? 1 : 0;
    p.col_cap = S / sbe::kStride > 0 ? S / sbe::kStride : 1;
    p.part = (float*)workspace;
    p.mused = p.part + (long long)p.heads * sbe::part_floats_per_head(g);
    p.ml = p.mused + (long long)p.heads * sbe::mused_floats_per_head(g);
    p.scores = scores;
    p.g = g;
    const long long total = (long long)p.heads * sbe::work_per_head(g);
    if (total > (1ll << 30) || p.heads > 65535) return MSD_ERR_UNSUPPORTED;
    const unsigned grid = (unsigned)((total + 7) / 8 * 8);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(512), sbe::kLdsBytes, stream, p);
    hipLaunchKernelGGL(sbe_finalize_kernel, dim3(g.NB, p.heads), dim3(64), 0, stream, p);
    if (hipGetLastError() != hipSuccess) return MSD_ERR_LAUNCH;
  }
  return MSD_OK;
}

// Block scores -> int8 mask [BN][NB][pitch] and int32 counts [BN][NB] (the sparse_mask /
// sparse_count_table pair of the reference, csrc/plugin/sparse_block_estimate.cpp:69-78).
int mindiesd_sbe_select(const float* scores, signed char* mask, int* count, int BN, int NB, int pitch, float threshold,
                        float row_sparse, int keep_sink, int keep_recent, int causal, hipStream_t stream) {
  if (!scores || !mask || !count || BN <= 0 || NB <= 0 || pitch < NB) return MSD_ERR_BAD_ARG;
  const int lds = (((NB + 3) & ~3) + 2 * n2_of(NB)) * 4;
  if (BN > 65535 || lds > 60000) return MSD_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(sbe_select_kernel, dim3(NB, BN), dim3(256), lds, stream, scores, mask, count, NB, pitch,
                     threshold, row_sparse, keep_sink ? 1 : 0, keep_recent ? 1 : 0, causal ? 1 : 0);
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

}  // extern "C"
