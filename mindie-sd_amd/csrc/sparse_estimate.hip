// Block mask estimation for adaptive block-sparse attention (XAttention style) on gfx950 (MI355X).
//
// Takes the place of the reference's in-tree AscendC kernel SparseBlockEstimate
// (csrc/ops/sparse_block_estimate/op_kernel/sparse_block_estimate.h, host wrapper
// csrc/plugin/sparse_block_estimate.cpp:27-85; numpy statement of the algorithm in
// tests/plugin/test_sparseblockestimate.py:49-145):
//   1. anti-diagonal strided scores: with stride 8, P'[i][j] = scale * sum_{s<8} q[8i+7-s] . k[8j+s]
//      (one eighth of the work of the full score matrix) - a plain [S/8, 8D] x [8D, S/8] product that
//      the host side hands to the GEMM library;
//   2. sbe_block_scores_kernel: row softmax of P' and summation over 16 x 16 blocks: the share of the
//      (estimated) attention mass that 128-token query block I puts on 128-token key block J;
//   3. sbe_select_kernel: per query block, sort the key blocks by mass, keep the smallest prefix whose mass
//      reaches `threshold` of the total (capped at row_sparse * blocks), always keep the first block
//      (attention sink) and the last one.
#include "common.hpp"

namespace msd {

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// P' [BN][Sr][ldp] 16-bit (raw products, ldp % 8 == 0) -> scores [BN][NB][NB] fp32.
// One workgroup = one block row (16 strided rows); a wave owns 4 of the rows, a lane 8 consecutive
// columns at a time, i.e. half a column block.  Two passes over the rows (the second one hits L2).
// Causal (the reference's rule, tests/plugin/test_sparseblockestimate.py:71-78): the rows of one step of 1024
// query tokens (8 block rows) see the keys up to the end of that step, cut down to whole groups of 8 tokens:
// strided columns < min(col_cap, 128 * (step + 1)), col_cap = S / 8.
template <int DT>
__global__ __launch_bounds__(256) void sbe_block_scores_kernel(const void* pm_, float* scores, int Sr, int ldp,
                                                               int NB, float scale_log2, int causal, int col_cap) {
#if defined(__HIP_DEVICE_COMPILE__)
  using T = typename Elem<DT>::type;
  extern __shared__ float blk[];  // [NB] column-block sums of this block row
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int brow = blockIdx.x, bn = blockIdx.y;
  const T* pm = (const T*)pm_ + (long long)bn * Sr * ldp;
  for (int j = tid; j < NB; j += 256) blk[j] = 0.f;
  __syncthreads();
  const int cols = causal ? min(col_cap, 128 * ((brow >> 3) + 1)) : Sr;  // columns this block row sees
  const int chunks = (cols + 7) / 8;
  for (int rr = 0; rr < 4; ++rr) {
    const int row = brow * 16 + wave * 4 + rr;
    if (row >= Sr) break;  // wave-uniform
    const T* prow = pm + (long long)row * ldp;
    // pass 1: maximum and sum of exponentials (log2 domain)
    float mx = -INFINITY;
    for (int c = lane; c < chunks; c += 64) {
      union { i32x4_t v; T e[8]; } u;
      u.v = *(const i32x4_t*)(prow + c * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (c * 8 + j < cols) mx = fmaxf(mx, (float)u.e[j]);
    }
    mx = wave_max(mx) * scale_log2;
    float sum = 0.f;
    for (int c = lane; c < chunks; c += 64) {
      union { i32x4_t v; T e[8]; } u;
      u.v = *(const i32x4_t*)(prow + c * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (c * 8 + j < cols) sum += fast_exp2((float)u.e[j] * scale_log2 - mx);
    }
    sum = wave_sum(sum);
    const float inv = 1.0f / sum;
    // pass 2: probabilities summed per column block (two neighbouring lanes share a block)
    for (int c0 = 0; c0 < chunks; c0 += 64) {
      const int c = c0 + lane;
      float part = 0.f;
      if (c < chunks) {
        union { i32x4_t v; T e[8]; } u;
        u.v = *(const i32x4_t*)(prow + c * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (c * 8 + j < cols) part += fast_exp2((float)u.e[j] * scale_log2 - mx);
      }
      part += __shfl_xor(part, 1, 64);
      if (c < chunks && (lane & 1) == 0) atomicAdd(&blk[c >> 1], part * inv);
    }
  }
  __syncthreads();
  float* out = scores + ((long long)bn * NB + brow) * NB;
  for (int j = tid; j < NB; j += 256) out[j] = blk[j];
#endif
}

// scores [BN][NB][NB] -> mask int8 [BN][NB][pitch] (pitch >= NB, padding zero) + count int32 [BN][NB].
// One workgroup per block row.  Follows the statement in tests/plugin/test_sparseblockestimate.py:121-143
// (non-causal): the last column is left out of the ranking, the ranking is a stable descending sort, the
// prefix length is counted on a sequential fp32 running sum.
// Causal (:121-125): row i ranks its first i + 1 columns only (the diagonal block is the "last" one), rows 0
// and 1 keep their whole prefix, and the diagonal block is forced only when keep_recent is set.
__global__ __launch_bounds__(256) void sbe_select_kernel(const float* scores, signed char* mask, int* count, int NB,
                                                         int pitch, float threshold, float row_sparse, int keep_sink,
                                                         int keep_recent, int causal) {
#if defined(__HIP_DEVICE_COMPILE__)
  extern __shared__ float sh[];  // [NB] row, [NB] sorted
  float* row = sh;
  float* sorted = sh + NB;
  __shared__ float guard_s;
  __shared__ int cnt_s[4];
  const int tid = threadIdx.x;
  const long long r = (long long)blockIdx.y * NB + blockIdx.x;
  const float* src = scores + r * NB;
  const int L = causal ? (int)blockIdx.x + 1 : NB;  // columns that take part
  const bool whole_prefix = causal && blockIdx.x <= 1;
  for (int j = tid; j < L; j += 256) row[j] = j == L - 1 ? 0.f : src[j];
  __syncthreads();
  // stable descending rank sort
  for (int e = tid; e < L; e += 256) {
    const float x = row[e];
    int rank = 0;
    for (int j = 0; j < L; ++j) {
      const float y = row[j];
      rank += (y > x || (y == x && j < e)) ? 1 : 0;
    }
    sorted[rank] = x;
  }
  __syncthreads();
  if (tid == 0) {
    float total = 0.f;
    for (int j = 0; j < L; ++j) total += sorted[j];
    const float lim = threshold * total;
    int cnt = 1;
    float run = 0.f;
    for (int j = 0; j < L; ++j) {
      run += sorted[j];
      if (run < lim) ++cnt;
    }
    if (row_sparse > 0.f && (float)cnt > row_sparse * (float)L) cnt = (int)(row_sparse * (float)L);
    cnt = max(1, min(cnt, L));
    guard_s = sorted[cnt - 1];
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
      if (j == L - 1 && keep_recent) v = guard + 1.f;
      keep = (v >= guard || whole_prefix) ? 1 : 0;
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

// P' = raw strided products [BN][Sr][ldp] (16-bit, ldp % 8 == 0, 16-byte aligned) -> block scores
// [BN][NB][NB] fp32, NB = ceil(Sr / 16): softmax(scale * P') over the Sr columns of a row, summed over
// 16 x 16 blocks.
int mindiesd_sbe_block_scores(const void* pmat, float* scores, int dtype, int BN, int Sr, int ldp, float scale,
                              int causal, int col_cap, hipStream_t stream) {
  if (!pmat || !scores || BN <= 0 || Sr <= 0 || ldp < Sr) return MSD_ERR_BAD_ARG;
  if (causal && (col_cap < 1 || col_cap > Sr)) return MSD_ERR_BAD_ARG;
  if ((ldp & 7) || ((uintptr_t)pmat & 15)) return MSD_ERR_BAD_ARG;
  if (dtype != MSD_DTYPE_BF16 && dtype != MSD_DTYPE_F16) return MSD_ERR_BAD_ARG;
  if (!(scale > 0.f)) return MSD_ERR_UNSUPPORTED;
  const int NB = (Sr + 15) / 16;
  if (BN > 65535 || NB * 4 > 60000) return MSD_ERR_UNSUPPORTED;
  const dim3 grid(NB, BN);
  const float sl2 = scale * 1.4426950408889634f;
  if (dtype == MSD_DTYPE_BF16)
    hipLaunchKernelGGL(sbe_block_scores_kernel<MSD_DTYPE_BF16>, grid, dim3(256), NB * 4, stream, pmat, scores, Sr, ldp,
                       NB, sl2, causal ? 1 : 0, col_cap);
  else
    hipLaunchKernelGGL(sbe_block_scores_kernel<MSD_DTYPE_F16>, grid, dim3(256), NB * 4, stream, pmat, scores, Sr, ldp,
                       NB, sl2, causal ? 1 : 0, col_cap);
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

// Block scores -> int8 mask [BN][NB][pitch] and int32 counts [BN][NB] (the sparse_mask /
// sparse_count_table pair of the reference, csrc/plugin/sparse_block_estimate.cpp:69-78).
int mindiesd_sbe_select(const float* scores, signed char* mask, int* count, int BN, int NB, int pitch, float threshold,
                        float row_sparse, int keep_sink, int keep_recent, int causal, hipStream_t stream) {
  if (!scores || !mask || !count || BN <= 0 || NB <= 0 || pitch < NB) return MSD_ERR_BAD_ARG;
  if (BN > 65535 || NB * 8 > 60000) return MSD_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(sbe_select_kernel, dim3(NB, BN), dim3(256), NB * 8, stream, scores, mask, count, NB, pitch,
                     threshold, row_sparse, keep_sink, keep_recent, causal ? 1 : 0);
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

}  // extern "C"
