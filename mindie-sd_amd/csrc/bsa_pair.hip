// Pairing of query blocks for block-sparse attention on gfx950 (MI355X).
//
// The block-sparse kernel of one 128-row query block streams 64 KiB of K/V per selected key block for 8.4 MFLOP of
// work - twice the bytes per flop of the dense kernel, whose workgroup shares every K/V tile between 256 query rows -
// and at DiT sizes that stream (L2 -> LDS, and HBM -> L2 for the tiles the XCD's L2 no longer holds) is what bounds
// it.  Query blocks that select mostly the same key blocks (in video latents: the same spatial region one frame
// apart) can share their tiles: they are paired here, and the attention kernel (the PAIR instantiation of
// fa_fwd16_kernel, flash_attn_fwd.hip) gives every pair one 256-row workgroup: the key blocks both partners selected
// at the dense kernel's rate, then each partner's own key blocks with its four waves, the running softmax going on.
//
// No counterpart in the reference (its sparse kernels are closed vendor binaries behind
// csrc/plugin/block_sparse_attention.cpp:31-121); the result of the attention does not depend on the pairing
// except for the order of the floating-point accumulation.
//
// bsa_bits_kernel:       int8 mask rows -> bit rows + their popcounts.
// bsa_candidates_kernel: per query block the kCand blocks of the same head with the largest similarity
//                        4095 * |row_i AND row_j| / max(|row_i|, |row_j|)  (ties: smaller j).  Normalised, because by
//                        plain overlap an all-ones row would be everybody's first choice.
// bsa_pair_kernel:       one workgroup per head.  Greedy matching on the candidate edges by descending similarity,
//                        computed in parallel rounds: an edge is taken when it is the best remaining edge of both its
//                        ends (the edge a sequential greedy pass would take first among their edges); what is left
//                        after kRounds is paired in ascending order.  Pairs are numbered by descending length of
//                        their shared list (the dispatch order of the first pass); then the three lists of every
//                        pair (shared, only A, only B) by bit operations.
#include "common.hpp"

namespace msd {

constexpr int kCand = 4;      // candidates kept per query block
constexpr int kRounds = 24;   // matching rounds
constexpr int kMaxQB = 1024;  // query blocks per head the edge keys can name (10 bits each)

// similarity of two mask rows, 0 .. 4095
__device__ __forceinline__ int pair_score(int common, int cnt_a, int cnt_b) {
  const int big = max(max(cnt_a, cnt_b), 1);
  return common * 4095 / big;
}
// key of the undirected edge {i, j}: larger = better; unique per edge, the same seen from both ends
__device__ __forceinline__ unsigned edge_key(int score, int i, int j) {
  const int lo = min(i, j), hi = max(i, j);
  return ((unsigned)score << 20) | ((unsigned)(kMaxQB - 1 - lo) << 10) | (unsigned)(kMaxQB - 1 - hi);
}
__device__ __forceinline__ int edge_other_end(unsigned key, int x) {
  const int lo = kMaxQB - 1 - (int)((key >> 10) & 1023), hi = kMaxQB - 1 - (int)(key & 1023);
  return lo == x ? hi : lo;
}

// one wave per mask row: bits[row][w] = mask[row][32 w .. 32 w + 31] != 0, cnt[row] = number of set bits
__global__ __launch_bounds__(256) void bsa_bits_kernel(const signed char* mask, long long rows, int KB, int W,
                                                       unsigned* bits, int* cnt) {
#if defined(__HIP_DEVICE_COMPILE__)
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const signed char* src = mask + row * KB;
  int total = 0;
  for (int k0 = 0; k0 < KB; k0 += 64) {
    const int k = k0 + lane;
    const bool on = k < KB && src[k] != 0;
    const unsigned long long b = __ballot(on);
    total += __popcll(b);
    if (lane == 0) bits[row * W + (k0 >> 5)] = (unsigned)b;
    if (lane == 32 && (k0 >> 5) + 1 < W) bits[row * W + (k0 >> 5) + 1] = (unsigned)(b >> 32);
  }
  if (lane == 0) cnt[row] = total;
#endif
}

// 16 waves = 16 query blocks per workgroup; the head's bit rows are staged in LDS, the lanes of a wave split the
// other blocks between them, keep their own best kCand and merge them by kCand wave-wide maxima.
// cand [BN][QB][kCand] edge keys (0 = none).
__global__ __launch_bounds__(1024) void bsa_candidates_kernel(const unsigned* bits_g, const int* cnt_g, int QB, int W,
                                                              unsigned* cand) {
#if defined(__HIP_DEVICE_COMPILE__)
  extern __shared__ unsigned smem_u[];
  unsigned* bits = smem_u;             // [QB][W]
  int* cnt = (int*)(smem_u + QB * W);  // [QB]
  const int bn = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const unsigned* bg = bits_g + (long long)bn * QB * W;
  for (int e = tid; e < QB * W; e += 1024) bits[e] = bg[e];
  for (int e = tid; e < QB; e += 1024) cnt[e] = cnt_g[(long long)bn * QB + e];
  __syncthreads();
  const int i = blockIdx.x * 16 + wave;
  if (i >= QB) return;
  unsigned best[kCand];
#pragma unroll
  for (int c = 0; c < kCand; ++c) best[c] = 0;
  const unsigned* mine = bits + i * W;
  const int cnt_i = cnt[i];
  for (int j = lane; j < QB; j += 64) {
    if (j == i) continue;
    const unsigned* other = bits + j * W;
    int common = 0;
    for (int w = 0; w < W; ++w) common += __popc(mine[w] & other[w]);
    if (common == 0) continue;
    unsigned key = edge_key(pair_score(common, cnt_i, cnt[j]), i, j);
    // insertion into the lane's descending list
#pragma unroll
    for (int c = 0; c < kCand; ++c) {
      const unsigned hi = max(best[c], key);
      key = min(best[c], key);
      best[c] = hi;
    }
  }
  // merge: kCand times the largest head of all lanes; the lane that owned it moves its list up
  unsigned* out = cand + ((long long)bn * QB + i) * kCand;
#pragma unroll
  for (int c = 0; c < kCand; ++c) {
    unsigned top = best[0];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) top = max(top, (unsigned)__shfl_xor((int)top, o, 64));
    if (best[0] == top && top != 0) {  // keys are unique, so exactly one lane
#pragma unroll
      for (int k = 0; k + 1 < kCand; ++k) best[k] = best[k + 1];
      best[kCand - 1] = 0;
    }
    if (lane == 0) out[c] = top;
  }
#endif
}

// exclusive prefix sum of one value per thread over the 1024 threads of the workgroup (tmp: 16 ints of LDS)
__device__ __forceinline__ int block_scan_1024(int v, int* tmp, int* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int incl = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int up = __shfl_up(incl, o, 64);
    if (lane >= o) incl += up;
  }
  __syncthreads();
  if (lane == 63) tmp[wave] = incl;
  __syncthreads();
  int before = 0, all = 0;
#pragma unroll
  for (int w = 0; w < 16; ++w) {
    const int t = tmp[w];
    before += w < wave ? t : 0;
    all += t;
  }
  *total = all;
  return before + incl - v;
}

// cand nullptr: no matching, blocks are paired in ascending order (2p, 2p + 1).
// pairs [BN][NP][2] (second entry -1 for a block without partner), NP = (QB + 1) / 2
// sh_idx [BN][NP][KB], sh_cnt [BN][NP]: key blocks both partners selected (a single block: all of its list)
// ex_idx [BN][QB][KB], ex_cnt [BN][QB]: key blocks only this query block selected
// init_cnt [BN][QB]: sh_cnt of the block's pair (> 0: the second pass continues the first one's softmax)
__global__ __launch_bounds__(1024) void bsa_pair_kernel(const unsigned* bits_g, const unsigned* cand, int QB, int KB,
                                                        int W, int* pairs, int* sh_idx, int* sh_cnt, int* ex_idx,
                                                        int* ex_cnt, int* init_cnt) {
#if defined(__HIP_DEVICE_COMPILE__)
  extern __shared__ unsigned smem_u[];
  unsigned* bits = smem_u;                       // [QB][W]
  int* partner = (int*)(smem_u + QB * W);        // [QB]
  unsigned* choice = (unsigned*)(partner + QB);  // [QB] best remaining edge of the block
  unsigned* incoming = choice + QB;              // [QB] best remaining edge that names the block as a candidate
  int* pair_no = (int*)(incoming + QB);          // [QB]
  __shared__ int scan_tmp[16];
  const int bn = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int NP = (QB + 1) / 2;
  const unsigned* bg = bits_g + (long long)bn * QB * W;
  for (int e = tid; e < QB * W; e += 1024) bits[e] = bg[e];
  const int x = tid;  // the block this thread speaks for (QB <= 1024)
  unsigned my_edges[kCand];
#pragma unroll
  for (int c = 0; c < kCand; ++c) my_edges[c] = (cand && x < QB) ? cand[((long long)bn * QB + x) * kCand + c] : 0u;
  if (x < QB) partner[x] = -1;
  __syncthreads();
  if (cand) {
    for (int round = 0; round < kRounds; ++round) {
      if (x < QB) incoming[x] = 0;
      __syncthreads();
      unsigned own = 0;
      if (x < QB && partner[x] < 0) {
#pragma unroll
        for (int c = 0; c < kCand; ++c) {
          const unsigned key = my_edges[c];
          if (key == 0) continue;
          const int y = edge_other_end(key, x);
          if (partner[y] >= 0) continue;
          own = max(own, key);
          atomicMax(&incoming[y], key);
        }
      }
      __syncthreads();
      if (x < QB) choice[x] = partner[x] < 0 ? max(own, incoming[x]) : 0u;
      __syncthreads();
      int taken = 0;
      if (x < QB && choice[x] != 0) {
        const int y = edge_other_end(choice[x], x);
        if (choice[y] == choice[x]) {  // the same edge is the best one at both ends
          partner[x] = y;
          taken = 1;
        }
      }
      if (__syncthreads_or(taken) == 0) break;
    }
  }
  // the rest in ascending order: free blocks of rank 2r and 2r + 1 form a pair
  {
    const int is_free = (x < QB && partner[x] < 0) ? 1 : 0;
    int n_free;
    const int rank = block_scan_1024(is_free, scan_tmp, &n_free);
    __syncthreads();
    int* by_rank = (int*)choice;  // reused: block of free rank r
    if (is_free) by_rank[rank] = x;
    __syncthreads();
    if (is_free) {
      const int mate_rank = rank ^ 1;
      partner[x] = mate_rank < n_free ? by_rank[mate_rank] : x;  // the last of an odd number stays alone
    }
    __syncthreads();
  }
  // Pair numbers = dispatch order of the first pass: longest shared list first (measured at the 14B 720p RainFusion
  // workload: 35.0 ms for both passes against 36.0 ms in block order; grouping the pairs of one spatial region
  // over the frames, whose lists are the most alike, was slower than either: 39.0 ms).
  {
    unsigned* okey = choice;  // order key of a pair's first block, ~0 for the other blocks
    const int first = (x < QB && partner[x] >= x) ? 1 : 0;
    if (x < QB) {
      unsigned kk = 0xffffffffu;
      if (first) {
        const int y = partner[x];
        int common = 0;
        for (int w = 0; w < W; ++w) common += __popc(bits[x * W + w] & bits[y * W + w]);
        kk = (unsigned)((4095 - min(common, 4095)) * kMaxQB + x);
      }
      okey[x] = kk;
    }
    __syncthreads();
    int n_pairs = 0, p = 0;
    if (x < QB) {
      const unsigned mine = okey[x];
      for (int y = 0; y < QB; ++y) {
        const unsigned other = okey[y];
        n_pairs += other != 0xffffffffu ? 1 : 0;
        p += other < mine ? 1 : 0;
      }
    }
    if (first) {
      pair_no[x] = p;
      int* pr = pairs + ((long long)bn * NP + p) * 2;
      pr[0] = x;
      pr[1] = partner[x] == x ? -1 : partner[x];
    }
    if (x == 0) {
      for (int q = n_pairs; q < NP; ++q) {  // fewer pairs than slots cannot happen; kept defined
        pairs[((long long)bn * NP + q) * 2] = -1;
        pairs[((long long)bn * NP + q) * 2 + 1] = -1;
        sh_cnt[(long long)bn * NP + q] = 0;
      }
    }
    __syncthreads();
  }
  // lists: one wave per pair, lane w owns word w of the rows (W <= 64 checked on the host)
  for (int i = wave; i < QB; i += 16) {
    const int j = partner[i];
    if (j < i) continue;
    const int p = pair_no[i];
    const bool single = j == i;
    const unsigned a = lane < W ? bits[i * W + lane] : 0u;
    const unsigned b = single ? a : (lane < W ? bits[j * W + lane] : 0u);
    unsigned words[3] = {a & b, single ? 0u : a & ~b, single ? 0u : b & ~a};
    int* dst[3] = {sh_idx + ((long long)bn * NP + p) * KB, ex_idx + ((long long)bn * QB + i) * KB,
                   ex_idx + ((long long)bn * QB + j) * KB};
    int total[3];
#pragma unroll
    for (int l = 0; l < 3; ++l) {
      unsigned word = words[l];
      const int mine = __popc(word);
      int before = mine;  // inclusive scan over the lanes
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int up = __shfl_up(before, o, 64);
        if (lane >= o) before += up;
      }
      total[l] = __shfl(before, 63, 64);
      int pos = before - mine;
      if (!(l == 2 && single)) {
        while (word) {
          const int bit = __ffs(word) - 1;
          word &= word - 1;
          dst[l][pos++] = 32 * lane + bit;
        }
      }
    }
    if (lane == 0) {
      sh_cnt[(long long)bn * NP + p] = total[0];
      ex_cnt[(long long)bn * QB + i] = total[1];
      init_cnt[(long long)bn * QB + i] = total[0];
      if (!single) {
        ex_cnt[(long long)bn * QB + j] = total[2];
        init_cnt[(long long)bn * QB + j] = total[0];
      }
    }
  }
#endif
}

// Workspace of the pairing (ints): bit rows + counts, candidates, pairs, shared lists + counts, exclusive lists +
// counts, init counts.
size_t bsa_pair_ints(long long BN, int QB, int KB) {
  const long long NP = (QB + 1) / 2, W = (KB + 31) / 32;
  return (size_t)(BN * ((long long)QB * W + QB + (long long)QB * kCand + NP * 2 + NP * KB + NP + (long long)QB * KB + QB +
                        QB));
}

bool bsa_pair_supported(int QB, int KB) {
  const int W = (KB + 31) / 32;
  return QB <= kMaxQB && W <= 64 && ((long long)QB * W + 4ll * QB) * 4 <= 150 * 1024;
}

// mask int8 [BN][QB][KB] -> pair tables inside `ws` (bsa_pair_ints(BN, QB, KB) ints); returns pointers into it.
int bsa_build_pairs(const signed char* mask, long long BN, int QB, int KB, int* ws, BsaPairTables* t, hipStream_t stream) {
  if (BN <= 0 || BN > 65535 || !bsa_pair_supported(QB, KB)) return MSD_ERR_UNSUPPORTED;
  const int W = (KB + 31) / 32;
  const long long NP = (QB + 1) / 2;
  unsigned* bits = (unsigned*)ws;
  int* cnt = ws + BN * QB * W;
  unsigned* cand = (unsigned*)(cnt + BN * QB);
  t->pairs = (int*)cand + BN * QB * kCand;
  t->sh_idx = t->pairs + BN * NP * 2;
  t->sh_cnt = t->sh_idx + BN * NP * KB;
  t->ex_idx = t->sh_cnt + BN * NP;
  t->ex_cnt = t->ex_idx + BN * QB * KB;
  t->init_cnt = t->ex_cnt + BN * QB;
  t->NP = (int)NP;
  const int lds1 = (QB * W + QB) * 4, lds2 = (QB * W + 4 * QB) * 4;
  if (hipFuncSetAttribute((const void*)bsa_candidates_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds1) != hipSuccess ||
      hipFuncSetAttribute((const void*)bsa_pair_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds2) != hipSuccess)
    return MSD_ERR_LAUNCH;
  const long long rows = BN * QB;
  if ((rows + 3) / 4 > 0x7fffffffll) return MSD_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(bsa_bits_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, mask, rows, KB, W, bits, cnt);
  hipLaunchKernelGGL(bsa_candidates_kernel, dim3((QB + 15) / 16, (unsigned)BN), dim3(1024), lds1, stream,
                     (const unsigned*)bits, (const int*)cnt, QB, W, cand);
  hipLaunchKernelGGL(bsa_pair_kernel, dim3((unsigned)BN), dim3(1024), lds2, stream, (const unsigned*)bits,
                     (const unsigned*)cand, QB, KB, W, t->pairs, t->sh_idx, t->sh_cnt, t->ex_idx, t->ex_cnt, t->init_cnt);
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

}  // namespace msd
