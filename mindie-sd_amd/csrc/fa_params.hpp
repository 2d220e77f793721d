// Argument block shared by the attention kernels of flash_attn_fwd.hip (head_dim 128) and flash_attn_hd.hip
// (other head dims).
#pragma once
#include "common.hpp"
#include "fa16_work.hpp"

namespace msd {

struct FaParams {
  const void* q;
  const void* k;
  const void* v;
  void* o;
  float* lse;  // optional [B, N, Sq] natural-log sum-exp of the scaled scores
  // element strides of the batch, head and token dimensions (head_dim is contiguous)
  long long q_sb, q_sn, q_ss;
  long long k_sb, k_sn, k_ss;
  long long v_sb, v_sn, v_ss;
  long long o_sb, o_sn, o_ss;
  int B, N, Nkv, Sq, Skv;
  float scale;       // softmax scale
  float scale_log2;  // scale * log2(e)
  // block-sparse selection (nullptr => dense): ascending key-block ids per 128-row query block
  const int* blk_idx;  // [B, N, QB, kb_stride]
  const int* blk_cnt;  // [B, N, QB]
  int kb_stride;
  int QB;
  const int* order;  // optional [B*N*QB] work order (heaviest query blocks first)
  const int* tok;    // GATHER instantiations: [Sq] row of q/out that holds the token at query position i
  // block-sparse attention over paired query blocks (see bsa_pair.hip)
  const int* pairs;     // PAIR kernel: [B * N][NP][2] query blocks of a pair (second -1: none); lists are per pair
  int NP;
  float* state;         // [B * N][Sq] log2-domain log-sum-exp after the first pass (written by it, read by the second)
  const int* init_cnt;  // second pass: [B * N][QB] key blocks the first pass covered for this query block (0: none)
  const int* ex_idx;    // PAIR kernel, optional: [B * N][QB][kb_stride] key blocks only this query block selected, walked by
  const int* ex_cnt;    //   its own four waves after the pair's shared list ([B * N][QB] counts); then no second pass follows
  // general mode (MODE = 1 instantiations only)
  const int* seq_meta;        // optional [B][4]: first query token, query count, first key token, key count of
                              // sequence b inside packed (token, head, dim) tensors; Sq is then the longest count
  int packed_tiles;           // > 0 (with seq_meta): the grid holds this many 128-row query tiles per head, numbered
                              // through the sequences (tile i belongs to the sequence the running sum of
                              // ceil(query count / 128) reaches it in); 0: B x ceil(Sq / 128) tiles per head
  int lse_token_major;        // with seq_meta: lse is [tokens][N] (index (first query token + row) * N + head)
  int causal;                 // key j is visible to query i iff j <= i + (Skv - Sq) (mask aligned bottom-right)
  const unsigned char* mask;  // optional boolean mask, non-zero = attend; keys contiguous
  long long m_sb, m_sn, m_sq; // its element strides over batch, head (0 = broadcast) and query
  int head_dim;               // DPAD instantiations of fa_fwd16_kernel: the tensors' head_dim (a multiple of 8 below 128)
};

#if defined(__HIP_DEVICE_COMPILE__)
// Packed numbering of the query tiles (FaParams::packed_tiles): which sequence tile i of a head belongs to and which
// of that sequence's tiles of `rows` query rows it is.  Every lane of the wave takes one sequence of a group of 64, the running
// sum of the tile counts is a wave scan; the result is wave-uniform.  False: i lies past the last tile.
__device__ __forceinline__ bool packed_find_tile(const int* seq_meta, int nseq, int i, int& seq, int& tile,
                                                 int rows = 128) {
  const int lane = threadIdx.x & 63;
  int base = 0;
  for (int c0 = 0; c0 < nseq; c0 += 64) {
    const int s = c0 + lane;
    const int t = s < nseq ? (seq_meta[4 * s + 1] + rows - 1) / rows : 0;
    int incl = t;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int u = __shfl_up(incl, d, 64);
      if (lane >= d) incl += u;
    }
    const int total = __builtin_amdgcn_readfirstlane(__shfl(incl, 63, 64));  // (scalar: the branch below is uniform)
    if (i < base + total) {
      const int first = base + incl - t;
      const unsigned long long hit = __ballot(t > 0 && i >= first && i < first + t);
      const int l = __ffsll((long long)hit) - 1;  // exactly one lane holds tile i
      // (handed back in scalar registers: everything the caller derives from them - pointers, sequence lengths, loop
      // bounds - stays wave-uniform for the compiler as it is without the table)
      seq = __builtin_amdgcn_readfirstlane(c0 + l);
      tile = __builtin_amdgcn_readfirstlane(i - __shfl(first, l, 64));
      return true;
    }
    base += total;
  }
  return false;
}

// True when the query counts of the table differ enough (the longest more than 1.25 times the mean of the non-empty
// ones) that equal numbers of consecutive tiles per XCD would be unequal work; wave-uniform, the same in every wave.
// `tiles`: the number of query tiles of `rows` rows that the sequences have together.
__device__ __forceinline__ bool seqs_uneven(const int* seq_meta, int nseq, int rows, int& tiles) {
  const int lane = threadIdx.x & 63;
  long long sum = 0;
  int longest = 0, filled = 0;
  tiles = 0;
  for (int c0 = 0; c0 < nseq; c0 += 64) {
    const int s = c0 + lane;
    const int len = s < nseq ? seq_meta[4 * s + 1] : 0;
    int acc = len, mx = len, tl = (len + rows - 1) / rows;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
      acc += __shfl_xor(acc, d, 64);
      mx = max(mx, __shfl_xor(mx, d, 64));
      tl += __shfl_xor(tl, d, 64);
    }
    sum += __builtin_amdgcn_readfirstlane(acc);
    longest = max(longest, __builtin_amdgcn_readfirstlane(mx));
    tiles += __builtin_amdgcn_readfirstlane(tl);
    filled += __popcll(__ballot(len > 0));
  }
  return filled > 1 && 4ll * longest * filled > 5ll * sum;
}

// Which tile a workgroup of the 16x16x32 kernels (fa_fwd16_kernel, fa_fwd16_d64_kernel; tiles of `rows` query rows)
// computes: batch entry b, head n, tile qt of the sequence, bn = b * N + n, the sequence's lengths and first tokens.
// False: nothing to do.  GEN 0: one sequence per batch entry, consecutive tiles of a head on one XCD (workgroups are
// dealt round-robin to the 8 XCDs).  GEN 1: p.seq_meta and / or causal.  GEN 2: GEN 1 with the packed numbering of
// p.packed_tiles.  GEN 3: as GEN 0 (the key mask plays no part here).  PAIR: tiles are the p.NP pairs of a head.
template <int GEN, bool PAIR>
__device__ __forceinline__ bool fa16_find_work(const FaParams& p, int rows, int& bn, int& qt, int& b, int& n, int& Sq,
                                               int& Skv, long long& q_tok0, long long& k_tok0) {
  constexpr bool packed = GEN == 2;
  int q_tiles = PAIR ? p.NP : packed ? p.packed_tiles : (p.Sq + rows - 1) / rows;
  // Sequences of unequal length (general mode with a table): workgroups are dealt to the XCDs one by one instead of in
  // runs - tiles in descending order, the (batch, head) index fastest - so every XCD gets its share of the long ones.
  bool spread = false;
  if constexpr (GEN == 1 || GEN == 2) {
    if (p.seq_meta) {
      int real_tiles;
      spread = seqs_uneven(p.seq_meta, p.B, rows, real_tiles);
      // packed numbering: the grid is sized for an upper bound; the tiles that exist are what is dealt out
      if (packed) q_tiles = min(q_tiles, real_tiles);
    }
  }
  // (fa16_work.hpp: runs of consecutive tiles per XCD; units of a heavy and a light tile - causal: tile t of a head has
  // t + 1 tiles' worth of keys, PAIR: the pairs of a head are numbered by descending length of their lists - so that
  // 12 heads on 8 XCDs are not 1.75 against 1.25 heads' worth of work; or one by one)
  const int groups = (packed ? 1 : p.B) * p.N;
  const fa16::Work w = spread ? fa16::spread(blockIdx.x, groups, q_tiles, packed)
                       : (PAIR || (GEN == 1 && p.causal)) ? fa16::units(blockIdx.x, groups, q_tiles, PAIR)
                                                           : fa16::runs(blockIdx.x, groups, q_tiles);
  if (w.group < 0) return false;
  bn = w.group;
  qt = w.tile;
  if constexpr (packed) {  // bn is the head; the tile's sequence comes from the table
    n = bn;
    if (!packed_find_tile(p.seq_meta, p.B, qt, b, qt, rows)) return false;
    if (p.causal) qt = (p.seq_meta[4 * b + 1] + rows - 1) / rows - 1 - qt;
    bn = b * p.N + n;
  } else {
    b = bn / p.N;
    n = bn - b * p.N;
  }
  Sq = p.Sq;
  Skv = p.Skv;
  q_tok0 = 0;
  k_tok0 = 0;
  if constexpr (GEN == 1 || GEN == 2) {
    if (p.seq_meta) {
      const int* meta = p.seq_meta + 4 * b;
      Sq = meta[1];
      Skv = meta[3];
      if (qt * rows >= Sq) return false;  // the grid is sized for the longest sequence
      q_tok0 = meta[0];
      k_tok0 = meta[2];
    }
  }
  return true;
}

#endif

// Grid of the 16x16x32 kernels (fa16_find_work above) for p, tiles of `rows` query rows.
template <int GEN, bool PAIR>
inline long long fa16_grid(const FaParams& p, int rows) {
  const long long tiles = PAIR ? p.NP : GEN == 2 ? p.packed_tiles : (p.Sq + rows - 1) / rows;
  const long long groups = (GEN == 2 ? 1ll : (long long)p.B) * p.N;
  if (PAIR || (GEN == 1 && p.causal)) return fa16::units_grid(groups, tiles);
  return fa16::runs_grid(groups, tiles);
}

// Dense attention for head dims other than 128 (flash_attn_hd.hip): D a multiple of 8, at most 256; all options of
// the general mode (packed sequences, causal, boolean mask, lse).
int launch_fa_hd(const FaParams& p, int dtype, int D, hipStream_t stream);

// Attention at head_dim 64 exactly (flash_attn_d64.hip); `gen` as the GEN of fa_fwd16_kernel: 0 dense, 1 p.seq_meta
// and / or causal, 2 the same with p.packed_tiles (256-row tiles), 3 a mask row shared by all queries.  `rows`: query
// rows per workgroup, 256 (8 waves) or - gen 0 only - 128 (4 waves, two workgroups per CU).  `supported` is false
// when a K or V (batch, head) slice does not fit the kernel's 32-bit buffer offsets (the general kernel takes those).
bool fa16_d64_supported(const FaParams& p);
int launch_fa16_d64(const FaParams& p, int dtype, hipStream_t stream, int gen = 0, int rows = 256);
// head dims below 64 (multiples of 8), computed as 64
int launch_fa16_d64_padded(const FaParams& p, int dtype, int D, hipStream_t stream, int gen = 0, int rows = 256);

// Attention at head dims above 128 up to 256 (flash_attn_d256.hip; multiples of 8, computed as 256); `gen` as for
// launch_fa16_d64 (its packed tiles are 128 rows); `supported` as above.
bool fa16_d256_supported(const FaParams& p);
int launch_fa16_d256(const FaParams& p, int dtype, int D, hipStream_t stream, int gen = 0);

}  // namespace msd
