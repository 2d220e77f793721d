// RainFusion2.0 block-mask pipeline on the GPU (gfx950): window permutation + block mean pooling,
// pooled block scores -> softmax -> top-k threshold -> forced blocks -> int8 mask / index lists,
// inverse permutation.  HBM-bound byte/index work plus one small exact reduction per block.
//
// Replaces the torch/einops host pipeline of the reference:
//   rearrange_with_remaining      mindiesd/layers/flash_attn/sparse_flash_attn_rf_v2.py:137-196
//   avgpool                       sparse_flash_attn_rf_v2.py:24-73
//   do_tensor_rearrange_pooling   sparse_flash_attn_rf_v2.py:292-317
//   get_blockwise_mask            sparse_flash_attn_rf_v2.py:94-134
//   get_mask_index                sparse_flash_attn_rf_v2.py:76-91
//   inv_rearrange_with_remaining  sparse_flash_attn_rf_v2.py:199-289 (and rf_v3.py:22-97)
//
// Arithmetic: the reference evaluates the mask in the input dtype; every rounding point is kept
// (block mean: sum -> fp32 -> divide -> 16-bit; scores: dot -> 16-bit, * scale -> 16-bit,
// softmax -> 16-bit) but each sum is accumulated in fp64, where sums of products of 16-bit
// values are exact, so the result does not depend on the order of summation.
#include "common.hpp"

namespace msd {

struct Grid3 {
  int t, h, w;
};

// Source token (t,h,w)-flattened index of position i of the window-ordered image sequence.
__device__ __forceinline__ int window_source(int i, Grid3 g) {
  if (g.t == 0) return i;  // identity (plain pooling of an already ordered sequence)
  const int hw = g.h * g.w;
  const int hr = g.h & 7, wr = g.w & 7;
  if (hr == 0 && wr == 0) {
    // (f hn wn hb wb) -> (f hn hb wn wb)
    const int f = i / hw, r = i - f * hw;
    const int wn_cnt = g.w >> 3;
    const int win = r >> 6, in = r & 63;
    const int hn = win / wn_cnt, wn = win - hn * wn_cnt;
    return f * hw + (hn * 8 + (in >> 3)) * g.w + wn * 8 + (in & 7);
  }
  if (i < hw) return i;  // the first frame keeps its order
  const int j = i - hw;
  const int f = 1 + j / hw, r = j % hw;
  const int h8 = g.h - hr, w8 = g.w - wr;
  const int main_cnt = h8 * w8;
  int row, col;
  if (r < main_cnt) {
    const int wn_cnt = w8 >> 3;
    const int win = r >> 6, in = r & 63;
    const int hn = win / wn_cnt, wn = win - hn * wn_cnt;
    row = hn * 8 + (in >> 3);
    col = wn * 8 + (in & 7);
  } else if (r < main_cnt + hr * g.w) {
    const int r2 = r - main_cnt;  // bottom rows, all columns
    row = h8 + r2 / g.w;
    col = r2 % g.w;
  } else {
    const int r3 = r - main_cnt - hr * g.w;  // right columns of the aligned rows
    row = r3 / wr;
    col = w8 + r3 % wr;
  }
  return f * hw + row * g.w + col;
}

template <int DT>
__device__ __forceinline__ float round16(float f) {
  return (float)Elem<DT>::from_float(f);
}

struct RearrangeParams {
  const void* src[3];
  void* dst[3];
  void* pool;  // [3][B][N][NB][D] element strides below (may be null: rearrange only)
  long long s_sb, s_sn, s_ss;  // source strides (elements)
  long long d_sb, d_sn, d_ss;  // destination strides
  long long p_st, p_sb, p_sn, p_sblk;
  int B, N, S, txt_len;
  Grid3 g;
  int nb_img, nb_txt;
  int inverse;  // 1: dst[source(i)] = src[i] (undo the permutation, text back to the front)
};

// One workgroup = one 128-token block of one (tensor, batch, head): 16 lanes move one 256-byte row.
template <int DT>
__global__ __launch_bounds__(256) void rf_rearrange_pool_kernel(const RearrangeParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  using T = typename Elem<DT>::type;
  __shared__ double part[16][128];
  const int blk = blockIdx.x, bn = blockIdx.y, which = blockIdx.z;
  const int b = bn / p.N, n = bn - b * p.N;
  const int s_img = p.S - p.txt_len;
  const bool is_txt = blk >= p.nb_img;
  const int seg_blk = is_txt ? blk - p.nb_img : blk;
  const int seg_len = is_txt ? p.txt_len : s_img;
  const int cnt = min(128, seg_len - seg_blk * 128);
  const int c16 = threadIdx.x & 15, rgrp = threadIdx.x >> 4;
  const T* src = (const T*)p.src[which] + b * p.s_sb + n * p.s_sn + c16 * 8;
  T* dst = p.dst[which] ? (T*)p.dst[which] + b * p.d_sb + n * p.d_sn + c16 * 8 : nullptr;
  double acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = 0.0;
  for (int r = rgrp; r < cnt; r += 16) {
    const int i = seg_blk * 128 + r;  // position inside the segment
    // permuted sequence = [image in window order | text]; original = [text | image]
    const int pos_perm = is_txt ? s_img + i : i;
    const int pos_orig = is_txt ? i : p.txt_len + window_source(i, p.g);
    const int from = p.inverse ? pos_perm : pos_orig;
    const int to = p.inverse ? pos_orig : pos_perm;
    const i32x4_t raw = *(const i32x4_t*)(src + (long long)from * p.s_ss);
    if (dst) *(i32x4_t*)(dst + (long long)to * p.d_ss) = raw;
    if (p.pool) {
      union { i32x4_t v; T e[8]; } u;
      u.v = raw;
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] += (double)(float)u.e[j];
    }
  }
  if (!p.pool) return;
#pragma unroll
  for (int j = 0; j < 8; ++j) part[rgrp][c16 * 8 + j] = acc[j];
  __syncthreads();
  if (threadIdx.x < 128) {
    double s = 0.0;
#pragma unroll
    for (int r = 0; r < 16; ++r) s += part[r][threadIdx.x];
    // torch mean of a 16-bit tensor: cast_fp32 -> sum -> div -> cast
    const float mean = __fdiv_rn((float)s, (float)cnt);
    T* pool = (T*)p.pool + which * p.p_st + b * p.p_sb + n * p.p_sn + (long long)blk * p.p_sblk;
    pool[threadIdx.x] = Elem<DT>::from_float(mean);
  }
#endif
}

struct MaskParams {
  const void* q_pool;  // [B][N][NB][D]
  const void* k_pool;
  long long p_sb, p_sn, p_sblk;
  signed char* mask;  // [B][N][NB][NB] (may be null)
  int* blk_idx;       // [B][N][NB][kb_stride] ascending selected blocks, -1 padded (may be null)
  int* blk_cnt;       // [B][N][NB]
  long long* idx64;   // optional [NB][N][NB] int64, -1 padded: the reference's select_idx (batch 0)
  long long* cnt64;   // optional [NB][N]
  int B, N, NB, kb_stride;
  int keep_len, txt_blocks, ff_blocks, keep_diag;
  float scale;
};

constexpr int kMaxBlocks = 2048;

// One workgroup = kMaskRows consecutive query-block rows of one (batch, head): the pooled keys of the head are read
// once for all of them (with one row per workgroup the kernel was bound by those reads: 150 KiB from L2 per row),
// then the rows are finished one after the other.
constexpr int kMaskRows = 4;

template <int DT>
__global__ __launch_bounds__(256) void rf_block_mask_kernel(const MaskParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  using T = typename Elem<DT>::type;
  __shared__ float qrow[kMaskRows][128];
  __shared__ double red[256];
  // per key block (dynamic LDS, 14 + 4 * kMaskRows bytes per block: a row of 591 blocks leaves room for 8
  // workgroups per CU):
  extern __shared__ __attribute__((aligned(16))) char mask_lds[];
  const int NBp = (p.NB + 3) & ~3;
  double* ex = (double*)mask_lds;                                  // exp(score - maximum)
  unsigned short* key = (unsigned short*)(mask_lds + (size_t)NBp * 8);   // 16-bit pattern of the rounded probabilities
  float* xs_all = (float*)(mask_lds + (size_t)NBp * 12);           // [kMaskRows][NBp] scaled scores, rounded to 16 bit
  __shared__ int hist[256];
  __shared__ int suf[257];
  __shared__ int wave_cnt[4];
  __shared__ int sel_bin, sel_rem, run_base;
  const int row0 = blockIdx.x * kMaskRows, bn = blockIdx.y;
  const int b = bn / p.N, n = bn - b * p.N;
  const int tid = threadIdx.x;
  const int NB = p.NB;
  const int nrows = min(kMaskRows, NB - row0);
  const T* kp = (const T*)p.k_pool + b * p.p_sb + n * p.p_sn;
  for (int i = tid; i < kMaskRows * 128; i += 256) {
    const int r = i >> 7;
    const T* qp = (const T*)p.q_pool + b * p.p_sb + n * p.p_sn + (long long)(row0 + min(r, nrows - 1)) * p.p_sblk;
    qrow[r][i & 127] = (float)qp[i & 127];
  }
  __syncthreads();

  // ---- scores: exact dot -> fp32 -> 16 bit; * scale (fp32) -> 16 bit -----------------------------
  // 4 lanes share one key block: lane `sub` reads the 16-byte chunks sub, sub + 4, sub + 8, sub + 12 of its pooled
  // row (the four lanes of a block read 64 contiguous bytes per request) and the 4 partial sums are added with two
  // lane exchanges.  Every product and sum is exact in fp64, so the order of summation does not matter.
  const int sub = tid & 3, grp4 = tid >> 2;
  for (int c0 = 0; c0 < NB; c0 += 64) {
    const int c = c0 + grp4;
    double acc[kMaskRows];
#pragma unroll
    for (int r = 0; r < kMaskRows; ++r) acc[r] = 0.0;
    if (c < NB) {
      union { i32x4_t v; T e[8]; } u[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) u[i].v = *(const i32x4_t*)(kp + (long long)c * p.p_sblk + (sub + 4 * i) * 8);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const double kv = (double)(float)u[i].e[j];
#pragma unroll
          for (int r = 0; r < kMaskRows; ++r) acc[r] = fma((double)qrow[r][(sub + 4 * i) * 8 + j], kv, acc[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < kMaskRows; ++r) {
#pragma unroll
      for (int o = 2; o > 0; o >>= 1) acc[r] += __shfl_xor(acc[r], o, 64);
      if (c < NB && sub == 0) {
        const float s16 = round16<DT>((float)acc[r]);
        xs_all[r * NBp + c] = round16<DT>(__fmul_rn(s16, p.scale));
      }
    }
  }
  __syncthreads();

  for (int rr = 0; rr < nrows; ++rr) {
  const int row = row0 + rr;
  const float* xs = xs_all + rr * NBp;
  float lmax = -INFINITY;
  for (int c = tid; c < NB; c += 256) lmax = fmaxf(lmax, xs[c]);
  red[tid] = (double)lmax;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if (tid < s) red[tid] = fmax(red[tid], red[tid + s]);
    __syncthreads();
  }
  const double mx = red[0];
  __syncthreads();

  // ---- softmax in fp64, rounded to fp32 and then to 16 bit --------------------------------------
  // (the exponentials are kept in LDS between the sum and the division: fp64 exp is the longest chain here)
  double lsum = 0.0;
  for (int c = tid; c < NB; c += 256) {
    const double e = exp((double)xs[c] - mx);
    ex[c] = e;
    lsum += e;
  }
  red[tid] = lsum;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if (tid < s) red[tid] += red[tid + s];
    __syncthreads();
  }
  const double denom = red[0];
  for (int c = tid; c < NB; c += 256) {
    const float pr = (float)(ex[c] / denom);
    const T p16 = Elem<DT>::from_float(pr);
    key[c] = __builtin_bit_cast(unsigned short, p16);  // probabilities are >= 0: bit order == value order
  }
  hist[tid] = 0;
  __syncthreads();

  // ---- keep_len-th largest value: two-level radix select on the 16-bit patterns -------------------
  // Per level: histogram of one byte, suffix sums over the 256 bins (one bin per thread, a scan inside the
  // waves and a combine over the four of them), and the bin in which the wanted rank falls: the one with
  // suffix(bin) >= need > suffix(bin + 1); the rank inside it is need - suffix(bin + 1).
  const int lane = tid & 63, wv = tid >> 6;
  auto pick_bin = [&](int need) {
    int v = hist[tid];
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int t = __shfl_down(v, o, 64);
      if (lane + o < 64) v += t;
    }
    if (lane == 0) wave_cnt[wv] = v;
    __syncthreads();
    for (int w2 = wv + 1; w2 < 4; ++w2) v += wave_cnt[w2];
    suf[tid] = v;
    if (tid == 0) suf[256] = 0;
    __syncthreads();
    // bin 0 also takes what no other bin takes (the scan it replaces stopped there)
    const bool mine = tid == 0 ? suf[1] < need : (suf[tid] >= need && suf[tid + 1] < need);
    if (mine) {
      sel_bin = tid;
      sel_rem = need - suf[tid + 1];
    }
    __syncthreads();
  };
  for (int c = tid; c < NB; c += 256) atomicAdd(&hist[key[c] >> 8], 1);
  __syncthreads();
  pick_bin(p.keep_len);
  const int hi_bin = sel_bin;
  const int rem = sel_rem;
  hist[tid] = 0;
  __syncthreads();
  for (int c = tid; c < NB; c += 256)
    if ((key[c] >> 8) == hi_bin) atomicAdd(&hist[key[c] & 255], 1);
  __syncthreads();
  pick_bin(rem);
  if (tid == 0) run_base = 0;
  __syncthreads();
  const unsigned thr = ((unsigned)hi_bin << 8) | (unsigned)sel_bin;

  // ---- mask row (score >= threshold, forced rows / columns), ordered compaction -------------------
  const bool row_forced = row < p.ff_blocks || row >= NB - p.txt_blocks;
  const long long row_lin = ((long long)bn * NB + row);
  signed char* mrow = p.mask ? p.mask + row_lin * NB : nullptr;
  int* irow = p.blk_idx ? p.blk_idx + row_lin * p.kb_stride : nullptr;
  long long* irow64 = (p.idx64 && b == 0) ? p.idx64 + ((long long)row * p.N + n) * NB : nullptr;
  for (int c0 = 0; c0 < NB; c0 += 256) {
    const int c = c0 + tid;
    bool keep = false;
    if (c < NB) {
      keep = key[c] >= thr || row_forced || c < p.ff_blocks || c >= NB - p.txt_blocks || (p.keep_diag && c == row);
      if (mrow) mrow[c] = keep ? 1 : 0;
    }
    const unsigned long long bal = __builtin_amdgcn_ballot_w64(keep);
    if (lane == 0) wave_cnt[wv] = __builtin_popcountll(bal);
    __syncthreads();
    int off = run_base;
    for (int w2 = 0; w2 < wv; ++w2) off += wave_cnt[w2];
    off += __builtin_popcountll(bal & ((1ull << lane) - 1ull));
    if (keep) {
      if (irow) irow[off] = c;
      if (irow64) irow64[off] = c;
    }
    __syncthreads();
    if (tid == 0) run_base += wave_cnt[0] + wave_cnt[1] + wave_cnt[2] + wave_cnt[3];
    __syncthreads();
  }
  const int total = run_base;
  if (irow)
    for (int c = total + tid; c < p.kb_stride; c += 256) irow[c] = -1;
  if (irow64)
    for (int c = total + tid; c < NB; c += 256) irow64[c] = -1;
  if (tid == 0) {
    if (p.blk_cnt) p.blk_cnt[row_lin] = total;
    if (p.cnt64 && b == 0) p.cnt64[(long long)row * p.N + n] = total;
  }
  __syncthreads();
  }  // rows of the workgroup
#endif
}

// tok[i] = row of the original [text | image] sequence that holds the token at position i of the permuted
// [image in window order | text] sequence: the table the gather mode of the attention kernel reads.
__global__ __launch_bounds__(256) void rf_token_order_kernel(int* tok, int S, int txt_len, Grid3 g) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= S) return;
  const int s_img = S - txt_len;
  tok[i] = i < s_img ? txt_len + window_source(i, g) : i - s_img;
}

// int8 mask rows -> ascending index lists + counts (used when a caller supplies the mask).
__global__ __launch_bounds__(256) void mask_to_index_kernel(const signed char* mask, int* blk_idx, int* blk_cnt,
                                                            int QB, int KB, int kb_stride) {
  __shared__ int wave_cnt[4];
  __shared__ int run_base;
  const long long row_lin = (long long)blockIdx.y * QB + blockIdx.x;
  const signed char* mrow = mask + row_lin * KB;
  int* irow = blk_idx + row_lin * kb_stride;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  if (tid == 0) run_base = 0;
  __syncthreads();
  for (int c0 = 0; c0 < KB; c0 += 256) {
    const int c = c0 + tid;
    const bool keep = c < KB && mrow[c] != 0;
    const unsigned long long bal = __builtin_amdgcn_ballot_w64(keep);
    if (lane == 0) wave_cnt[wv] = __builtin_popcountll(bal);
    __syncthreads();
    int off = run_base;
    for (int w2 = 0; w2 < wv; ++w2) off += wave_cnt[w2];
    off += __builtin_popcountll(bal & ((1ull << lane) - 1ull));
    if (keep) irow[off] = c;
    __syncthreads();
    if (tid == 0) run_base += wave_cnt[0] + wave_cnt[1] + wave_cnt[2] + wave_cnt[3];
    __syncthreads();
  }
  const int total = run_base;
  for (int c = total + tid; c < kb_stride; c += 256) irow[c] = -1;
  if (tid == 0) blk_cnt[row_lin] = total;
}

}  // namespace msd

using namespace msd;

extern "C" {

int mindiesd_rf_rearrange_pool(const void* q, const void* k, const void* v, void* q_out, void* k_out, void* v_out,
                               void* pool, int dtype, int B, int N, int S, int D, long long s_sb, long long s_sn,
                               long long s_ss, long long d_sb, long long d_sn, long long d_ss, long long p_st,
                               long long p_sb, long long p_sn, long long p_sblk, int t, int h, int w, int txt_len,
                               int inverse, int n_tensors, hipStream_t stream) {
  if (!q || B <= 0 || N <= 0 || S <= 0) return MSD_ERR_BAD_ARG;
  if (n_tensors < 1 || n_tensors > 3 || (n_tensors > 1 && !k) || (n_tensors > 2 && !v)) return MSD_ERR_BAD_ARG;
  if (!pool && !q_out) return MSD_ERR_BAD_ARG;  // nothing to produce
  if (D != 128) return MSD_ERR_UNSUPPORTED;
  if (dtype != MSD_DTYPE_BF16 && dtype != MSD_DTYPE_F16) return MSD_ERR_BAD_ARG;
  // t == 0 selects the identity order (pooling only); otherwise t*h*w image tokens + txt_len text tokens
  if (txt_len < 0 || t < 0) return MSD_ERR_BAD_ARG;
  if (t > 0 && (h < 8 || w < 8 || (long long)t * h * w + txt_len != S)) return MSD_ERR_BAD_ARG;
  if (t == 0 && txt_len > S) return MSD_ERR_BAD_ARG;
  if ((s_sb | s_sn | s_ss | d_sb | d_sn | d_ss) & 7) return MSD_ERR_BAD_ARG;
  RearrangeParams p{};
  p.src[0] = q; p.src[1] = k; p.src[2] = v;
  p.dst[0] = q_out; p.dst[1] = k_out; p.dst[2] = v_out;
  p.pool = pool;
  p.s_sb = s_sb; p.s_sn = s_sn; p.s_ss = s_ss;
  p.d_sb = d_sb; p.d_sn = d_sn; p.d_ss = d_ss;
  p.p_st = p_st; p.p_sb = p_sb; p.p_sn = p_sn; p.p_sblk = p_sblk;
  p.B = B; p.N = N; p.S = S; p.txt_len = txt_len;
  p.g = Grid3{t, h, w};
  p.nb_img = (S - txt_len + 127) / 128;
  p.nb_txt = (txt_len + 127) / 128;
  p.inverse = inverse;
  dim3 grid(p.nb_img + p.nb_txt, B * N, n_tensors);
  if (dtype == MSD_DTYPE_BF16)
    hipLaunchKernelGGL(rf_rearrange_pool_kernel<MSD_DTYPE_BF16>, grid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL(rf_rearrange_pool_kernel<MSD_DTYPE_F16>, grid, dim3(256), 0, stream, p);
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

int mindiesd_rf_token_order(int* token_order, int S, int t, int h, int w, int txt_len, hipStream_t stream) {
  if (!token_order || S <= 0 || txt_len < 0 || t <= 0 || h < 8 || w < 8) return MSD_ERR_BAD_ARG;
  if ((long long)t * h * w + txt_len != S) return MSD_ERR_BAD_ARG;
  hipLaunchKernelGGL(rf_token_order_kernel, dim3((S + 255) / 256), dim3(256), 0, stream, token_order, S, txt_len,
                     Grid3{t, h, w});
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

int mindiesd_rf_block_mask(const void* q_pool, const void* k_pool, int dtype, int B, int N, int NB, int D,
                           long long p_sb, long long p_sn, long long p_sblk, float scale, int keep_len,
                           int txt_blocks, int ff_blocks, int keep_diag, signed char* mask, int* blk_idx,
                           int* blk_cnt, int kb_stride, long long* select_idx, long long* select_num,
                           hipStream_t stream) {
  if (!q_pool || !k_pool || B <= 0 || N <= 0 || NB <= 0) return MSD_ERR_BAD_ARG;
  if (D != 128 || NB > kMaxBlocks) return MSD_ERR_UNSUPPORTED;
  if (dtype != MSD_DTYPE_BF16 && dtype != MSD_DTYPE_F16) return MSD_ERR_BAD_ARG;
  if (keep_len < 1 || keep_len > NB) return MSD_ERR_BAD_ARG;
  if (blk_idx && kb_stride < NB) return MSD_ERR_BAD_ARG;
  if ((p_sb | p_sn | p_sblk) & 7) return MSD_ERR_BAD_ARG;
  MaskParams p{};
  p.q_pool = q_pool; p.k_pool = k_pool;
  p.p_sb = p_sb; p.p_sn = p_sn; p.p_sblk = p_sblk;
  p.mask = mask; p.blk_idx = blk_idx; p.blk_cnt = blk_cnt; p.idx64 = select_idx; p.cnt64 = select_num;
  p.B = B; p.N = N; p.NB = NB; p.kb_stride = kb_stride;
  p.keep_len = keep_len; p.txt_blocks = txt_blocks; p.ff_blocks = ff_blocks; p.keep_diag = keep_diag;
  p.scale = scale;
  dim3 grid((NB + kMaskRows - 1) / kMaskRows, B * N);
  const size_t lds = (size_t)((NB + 3) & ~3) * (12 + 4 * kMaskRows);  // at most 56 KiB (NB <= kMaxBlocks)
  if (dtype == MSD_DTYPE_BF16)
    hipLaunchKernelGGL(rf_block_mask_kernel<MSD_DTYPE_BF16>, grid, dim3(256), lds, stream, p);
  else
    hipLaunchKernelGGL(rf_block_mask_kernel<MSD_DTYPE_F16>, grid, dim3(256), lds, stream, p);
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

int mindiesd_mask_to_index(const signed char* mask, int BN, int QB, int KB, int* blk_idx, int* blk_cnt,
                           int kb_stride, hipStream_t stream) {
  if (!mask || !blk_idx || !blk_cnt || BN <= 0 || QB <= 0 || KB <= 0 || kb_stride < KB) return MSD_ERR_BAD_ARG;
  hipLaunchKernelGGL(mask_to_index_kernel, dim3(QB, BN), dim3(256), 0, stream, mask, blk_idx, blk_cnt, QB, KB,
                     kb_stride);
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

}  // extern "C"
