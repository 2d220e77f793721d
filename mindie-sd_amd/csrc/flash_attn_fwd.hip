// Flash-attention forward for gfx950 (MI355X): dense and block-sparse, head_dim 128, bf16/fp16.
//
// Replaces the device side of the reference's fused attention ops: the dense vendor kernels
// behind attention_forward (mindiesd/layers/flash_attn/attention_forward.py:24-89) and the
// block-sparse kernels behind torch.ops.mindiesd.block_sparse_attention /
// rainfusionattention (csrc/plugin/block_sparse_attention.cpp:31-121,
// csrc/plugin/rainfusionattention.cpp:27-64).
//
// Two kernels share the algorithm: fa_fwd16_kernel (16x16x32 matrix instruction: plain dense attention, and causal
// and packed variable-length attention without a boolean mask from 256 query rows on) and fa_fwd_kernel (32x32x16
// instruction: block-sparse and masked attention, the short causal / variable-length cases and the tuning variants
// of the dense case).  What follows describes fa_fwd_kernel; fa_fwd16_kernel states its differences.
//
// Algorithm: single pass, online softmax.  One workgroup owns BM = NWAVES*QPW query rows of one
// (batch, head); it walks the key/value sequence in tiles of BN keys staged in LDS (double
// buffered, one barrier per tile).  The kernel works on the TRANSPOSED problem so that every
// softmax row lives in one lane pair:
//     S^T[key, q] = K Q^T      (MFMA 32x32x16, A = K tile from LDS, B = Q^T resident in VGPRs)
//     O^T[d,   q] += V^T P^T   (A = V^T read from the row-major V tile with the transposing
//                               LDS read ds_read_b64_tr_b16, B = P^T straight from the S^T
//                               accumulator registers, no data movement)
// In the 32x32 accumulator a lane holds column q = lane%32 and rows 8*(r/4) + 4*(lane/32) + r%4,
// so a row max / row sum is 16 in-lane operations per 32 keys plus one exchange with lane^32.
//
// LDS layouts (bank-conflict free for their readers, no padding):
//     K tile [key][128]: 16-byte chunk c of row key is stored at chunk c ^ (key & 15)
//     V tile [key][128]: 64-byte chunk c of row key is stored at chunk c ^ (key & 3)
#include <cstdlib>
#include <type_traits>
#include <utility>

#include "common.hpp"
#include "fa_params.hpp"

#ifndef FA16_AHEAD
#define FA16_AHEAD 3  // K operand groups requested ahead of their use in fa_fwd16_kernel
#endif

namespace msd {

// An entry of a device table read through the scalar unit (pointer and index wave-uniform): the value arrives in a
// scalar register and is waited for where it is first used, not where it is requested - a vector load followed by a
// readfirstlane stalls the wave for the whole memory latency at the request.
__device__ __forceinline__ int scalar_load(const int* p, int i) {
  return ((const __attribute__((address_space(4))) int*)p)[i];
}

template <int DT, int NWAVES, int QPW, int BN, bool SPARSE>
struct FaCfg {
  static constexpr int kD = 128;
  static constexpr int kNT = NWAVES * 64;
  static constexpr int kBM = NWAVES * QPW;
  static constexpr int kNQB = QPW / 32;    // 32-query column blocks per wave
  static constexpr int kNKB = BN / 32;     // 32-key row blocks per tile
  static constexpr int kRowBytes = kD * 2;
  static constexpr int kTileBytes = BN * kRowBytes;
  static constexpr int kStageBytes = 2 * kTileBytes;  // K + V
  // epilogue staging of 32 output rows per wave: [32][128] 16-bit with a padded row
  static constexpr int kORowBytes = kRowBytes + 8;
  static constexpr int kOutStageBytes = NWAVES * 32 * kORowBytes;
  // K/V double buffered; the output staging reuses the same memory after the last tile
  static constexpr int kLdsBytes = 2 * kStageBytes > kOutStageBytes ? 2 * kStageBytes : kOutStageBytes;
  static constexpr int kGroupsPerWave = BN / 4 / NWAVES;  // 4-row (1 KiB) LDS-DMA groups per wave and tile
  static_assert(BN % (4 * NWAVES) == 0, "tile must split evenly over the wavefronts");
};

#if defined(__HIP_DEVICE_COMPILE__)
template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>)
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

// LDS-DMA of one K tile and one V tile: every wave issues G pairs of 1 KiB transfers.
// Group i of a wave lies 4 * NWAVES rows below group 0 (a multiple of 16, so the swizzles are the same): one
// per-lane offset per operand serves all groups, the rest goes into the scalar offset.
template <int G, int NWAVES>
__device__ __forceinline__ void tile_dma(__amdgpu_buffer_rsrc_t k_rsrc, __amdgpu_buffer_rsrc_t v_rsrc,
                                         MSD_LDS char* kb, MSD_LDS char* vb, int k_voff, int v_voff, int wave,
                                         int k_soff, int v_soff, int k_row_bytes, int v_row_bytes) {
#pragma unroll
  for (int i = 0; i < G; ++i) {
    const int g = i * NWAVES + wave;  // 4-row group of the tile
    __builtin_amdgcn_raw_ptr_buffer_load_lds(k_rsrc, (MSD_LDS void*)(kb + g * 1024), 16, k_voff,
                                             k_soff + i * 4 * NWAVES * k_row_bytes, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(v_rsrc, (MSD_LDS void*)(vb + g * 1024), 16, v_voff,
                                             v_soff + i * 4 * NWAVES * v_row_bytes, 0, 0);
  }
}
#endif

// Register budget: 8 wavefronts per CU (two per SIMD) in every configuration, i.e. at most 256
// registers per lane; the 4-wave configurations run two workgroups per CU.
// GATHER: the query sequence the kernel works on is a permutation of the rows of q and out (p.tok): query rows
// are fetched and output rows stored through the table.  K and V stay contiguous in the permuted order: tiles
// gathered row by row through the same table measured 8 % slower (the block-sparse walk is bound by the L2-miss
// path, and 2 KiB runs use it worse than 32 KiB tiles), more than the permuted copies of K and V cost.
// INIT (block-sparse only): second pass of the paired scheme - the output rows and p.state already hold the
// normalised result and the log-sum-exp of the key blocks covered by the first pass; the running softmax starts
// from them (maximum = that log-sum-exp, sum = 1) instead of from nothing, and a query block without further key
// blocks is left as it is.  The first pass stores its rows in the 16-bit output type, so a row with key blocks in
// both passes is rounded to 16 bits once more than a one-pass walk would round it (a relative 2^-9 for bf16 on
// the first pass's share of the row).
template <int DT, int NWAVES, int QPW, int BN, bool SPARSE, int SCHED, int MODE = 0, bool GATHER = false,
          bool INIT = false, bool PACKED = false>
__global__ __launch_bounds__(NWAVES * 64, (QPW == 32 ? 2 : 1)) void fa_fwd_kernel(const FaParams p) {
#if defined(__HIP_DEVICE_COMPILE__)  // the host pass only needs the launch stub
  using C = FaCfg<DT, NWAVES, QPW, BN, SPARSE>;
  using E = Elem<DT>;
  using T = typename E::type;
  using X8 = typename E::x8;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  MSD_LDS char* smem = (MSD_LDS char*)smem_raw;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int h = lane >> 5;

  // ---- which (batch, head, query tile): consecutive tiles of one head stay on one XCD -------
  // PACKED (an instantiation of its own, so that the table lookup does not touch the code of the others): the grid
  // holds p.packed_tiles query tiles per head, numbered through the sequences of p.seq_meta
  static_assert(!PACKED || (MODE && !SPARSE && C::kBM == 128), "packed numbering: general dense mode, 128-row tiles");
  constexpr bool packed = PACKED;
  const int q_tiles = packed ? p.packed_tiles : (p.Sq + C::kBM - 1) / C::kBM;
  const int total = (packed ? 1 : p.B) * p.N * q_tiles;
  const int per_xcd = (total + 7) / 8;
  int work = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (SPARSE && p.order) {  // caller's work order: workgroup i takes entry i of the table
    if ((int)blockIdx.x >= total) return;
    work = p.order[blockIdx.x];
  }
  if (work < 0 || work >= total) return;
  int bn = work / q_tiles;
  int qt = work - bn * q_tiles;
  int b, n;
  if constexpr (packed) {  // bn is the head; the tile's sequence comes from the table
    n = bn;
    if (!packed_find_tile(p.seq_meta, p.B, qt, b, qt)) return;
    if (p.causal) qt = (p.seq_meta[4 * b + 1] + C::kBM - 1) / C::kBM - 1 - qt;
    bn = b * p.N + n;
  } else {
    if (MODE && p.causal) qt = q_tiles - 1 - qt;  // the tiles with the most visible keys start first
    b = bn / p.N;
    n = bn - b * p.N;
  }
  const int nkv = n / (p.N / p.Nkv);
  const int q0 = qt * C::kBM;

  const T* qg = (const T*)p.q + b * p.q_sb + n * p.q_sn;
  const T* kg = (const T*)p.k + b * p.k_sb + nkv * p.k_sn;
  const T* vg = (const T*)p.v + b * p.v_sb + nkv * p.v_sn;
  T* og = (T*)p.o + b * p.o_sb + n * p.o_sn;
  // sequence lengths of this (batch) problem; packed sequences bring their own and their token offsets
  int Sq = p.Sq, Skv = p.Skv;
  if (MODE && p.seq_meta) {
    const int* meta = p.seq_meta + 4 * b;
    Sq = meta[1];
    Skv = meta[3];
    if (q0 >= Sq) return;  // the grid is sized for the longest sequence
    qg += (long long)meta[0] * p.q_ss;
    og += (long long)meta[0] * p.o_ss;
    kg += (long long)meta[2] * p.k_ss;
    vg += (long long)meta[2] * p.v_ss;
  }
  const int causal_shift = Skv - Sq;

  // ---- tile stream ----------------------------------------------------------------------------
  // Dense: key tiles 0, BN, 2*BN, ...  Sparse: a workgroup owns kBM/128 query blocks (one per group
  // of 4 waves); it walks the ascending MERGE of their block lists, every key block is staged in
  // LDS once, and a wave computes on it only if its own query block selected it.
  constexpr int kSub = 128 / BN;          // tiles per 128-key block (sparse granularity)
  constexpr int kQBlocks = C::kBM / 128;  // query blocks per workgroup (sparse)
  static_assert(!SPARSE || kQBlocks == 1 || kQBlocks == 2, "sparse kernel handles 1 or 2 query blocks");
  const int grp = SPARSE ? wave / 4 : 0;  // which of the workgroup's query blocks this wave belongs to

  // ---- Q^T operand, resident in registers: lane (q = l32, h) holds d = 16*ks + 8*h .. +8 -----
  X8 qf[C::kNQB][8];
#pragma unroll
  for (int qb = 0; qb < C::kNQB; ++qb) {
    const int qrow = q0 + wave * QPW + qb * 32 + l32;
    const bool ok = qrow < Sq;
    const int qsrc = GATHER ? p.tok[ok ? qrow : 0] : (ok ? qrow : 0);
    const T* src = qg + (long long)qsrc * p.q_ss + 8 * h;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      X8 v = *(const X8*)(src + 16 * ks);
      if (!ok) v = X8{0};
      // fold softmax scale * log2(e) into Q once (the reference rounds q * scale to the input
      // type as well, attention_func.py:40), so the scores come out of the MFMA in log2 units
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = E::from_float((float)v[j] * p.scale_log2);
      qf[qb][ks] = v;
    }
  }

  f32x16_t oacc[4][C::kNQB];
  // m_run: reference maximum (log2 units) that l_run and oacc are expressed in; negm holds -m_run
  // in all 16 accumulator slots of a lane and seeds the score accumulators, so the MFMA chain
  // delivers s - m directly and the softmax needs no subtraction.
  float m_run[C::kNQB], l_run[C::kNQB];
  f32x16_t negm[C::kNQB];
#pragma unroll
  for (int qb = 0; qb < C::kNQB; ++qb) {
    m_run[qb] = 0.f;
    l_run[qb] = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) negm[qb][r] = 0.f;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[db][qb][r] = 0.f;
  }
  bool resumed = false;  // INIT: the running softmax continues the first pass (wave-uniform)
  if constexpr (INIT) {
    static_assert(SPARSE && C::kBM == 128 && C::kNQB == 1, "second pass: one 128-row query block per workgroup");
    const long long qb_lin = (long long)bn * p.QB + qt;
    const int covered = p.init_cnt[qb_lin];
    if (covered > 0) {
      if (p.blk_cnt[qb_lin] == 0) return;  // nothing left to add: the first pass wrote the final rows
      resumed = true;
      const int qrow = q0 + wave * QPW + l32;
      const bool ok = qrow < Sq;
      const int orow = GATHER ? p.tok[ok ? qrow : 0] : (ok ? qrow : 0);
      // A first pass that saw only non-finite scores leaves -inf: such a row starts from nothing at reference 0
      // (a seed of +inf would turn every score into NaN).
      const float lse_in = ok ? p.state[(long long)bn * p.Sq + qrow] : 0.f;
      const bool have = lse_in > -INFINITY;
      const float lse2 = have ? lse_in : 0.f;
      m_run[0] = lse2;
      l_run[0] = (h == 0 && have) ? 1.f : 0.f;  // the two halves of a row add up their sums at the end
#pragma unroll
      for (int r = 0; r < 16; ++r) negm[0][r] = -lse2;
      const T* orow_p = og + (long long)orow * p.o_ss;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const typename E::x4 pk = *(const typename E::x4*)(orow_p + db * 32 + 8 * g + 4 * h);
#pragma unroll
          for (int j = 0; j < 4; ++j) oacc[db][0][4 * g + j] = (ok && have) ? (float)pk[j] : 0.f;
        }
    }
  }

  // ---- global -> LDS staging of one K/V tile (LDS-DMA, no registers) ------------------------------
  // One buffer_load_dwordx4 ... lds moves 64 x 16 bytes: lane L's 16 bytes land at lds_base + 16*L,
  // i.e. one instruction fills 4 consecutive 256-byte rows.  The swizzles are applied on the
  // global side: the lane that fills physical chunk pc of a row fetches the logical chunk
  // pc ^ swizzle(row).  The per-lane byte offset inside a tile never changes; the tile position
  // is a scalar offset.  Rows past the end of the sequence are out of the buffer's range and read
  // as zeros (their scores are masked to -inf below).
  const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void*)kg, 0, Skv > 0 ? (int)(((long long)(Skv - 1) * p.k_ss + C::kD) * 2) : 0, 0x00020000);
  const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void*)vg, 0, Skv > 0 ? (int)(((long long)(Skv - 1) * p.v_ss + C::kD) * 2) : 0, 0x00020000);
  const int k_row_bytes = (int)p.k_ss * 2, v_row_bytes = (int)p.v_ss * 2;
  static_assert((4 * NWAVES) % 16 == 0, "groups of one wave must share their swizzle");
  int k_voff, v_voff;
  {
    const int row = 4 * wave + (lane >> 4);
    const int pc = lane & 15;
    k_voff = row * k_row_bytes + ((pc ^ (row & 15)) << 4);
    v_voff = row * v_row_bytes + ((pc ^ ((row & 3) << 2)) << 4);
  }
  auto load_tile = [&](int key0, int stage) {
    MSD_LDS char* kb = smem + stage * C::kStageBytes;
    tile_dma<C::kGroupsPerWave, NWAVES>(k_rsrc, v_rsrc, kb, kb + C::kTileBytes, k_voff, v_voff, wave,
                                        key0 * k_row_bytes, key0 * v_row_bytes, k_row_bytes, v_row_bytes);
  };

  // per-lane constant parts of the LDS read addresses
  // K operand: row = kb*32 + l32, 16-byte chunk (2*ks + h) ^ (row & 15); (kb*32) & 15 == 0
  const int k_row_off = l32 * C::kRowBytes;
  const int k_swz = l32 & 15;
  // V^T operand (transposing read): this lane addresses key 4*h + (lane%16)/4 (+16*t, +8),
  // bytes 32*((lane/16)&1) + 8*(lane%4) of the 64-byte chunk db ^ (key & 3)
  const int v_key = 4 * h + ((lane & 15) >> 2);  // key & 3 == ((lane&15)>>2) for every base key (multiples of 4)
  const int v_row_off = v_key * C::kRowBytes + 32 * ((lane >> 4) & 1) + 8 * (lane & 3);
  const int v_swz = (lane & 15) >> 2;
  // LDS byte address of this lane's V^T read for head_dim block db of the tile in stage 0, key step 0
  unsigned v_lds[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
    v_lds[db] = (unsigned)(uintptr_t)smem + C::kTileBytes + v_row_off + ((db ^ v_swz) << 6);

  // ---- stream state (all wave-uniform) -----------------------------------------------------------
  // Block lists live in registers, 64 ids per batch (one per lane); the next batch is requested when
  // the current one comes into use and ids are handed out with v_readlane, so no memory access sits
  // between two tiles.
  constexpr int kEnd = 0x7fffffff;
  int l_cur[2] = {0, 0}, l_nxt[2] = {0, 0}, l_pos[2] = {0, 0}, l_n[2] = {0, 0};
  const int* l_ptr[2] = {nullptr, nullptr};
  if (SPARSE) {
#pragma unroll
    for (int i = 0; i < kQBlocks; ++i) {
      const int qblk = qt * kQBlocks + i;
      if (qblk < p.QB) {
        const long long qb_lin = (long long)bn * p.QB + qblk;
        l_ptr[i] = p.blk_idx + qb_lin * p.kb_stride;
        l_n[i] = p.blk_cnt[qb_lin];
        l_cur[i] = lane < l_n[i] ? l_ptr[i][lane] : 0;
        l_nxt[i] = 64 + lane < l_n[i] ? l_ptr[i][64 + lane] : 0;
      }
    }
  }
  auto list_head = [&](int i) -> int {
    return l_pos[i] < l_n[i] ? __builtin_amdgcn_readlane(l_cur[i], l_pos[i] & 63) : kEnd;
  };
  auto list_pop = [&](int i) {
    ++l_pos[i];
    if ((l_pos[i] & 63) == 0) {
      l_cur[i] = l_nxt[i];
      const int j = l_pos[i] + 64 + lane;
      l_nxt[i] = j < l_n[i] ? l_ptr[i][j] : 0;
    }
  };
  // cur_*: the tile being computed; nxt_*: the tile being fetched.  key0 < 0 marks the end.
  int cur_key0 = -1, nxt_key0 = -1, cur_fl = 0, nxt_fl = 0, sub = 0;
  // causal: the last row of this workgroup sees keys <= q0 + kBM - 1 + shift; later tiles are skipped
  int kv_lim = Skv;
  if (MODE && p.causal) kv_lim = max(0, min(Skv, q0 + C::kBM + causal_shift));
  const int dense_tiles = (kv_lim + BN - 1) / BN;
  const unsigned char* mask_g = nullptr;
  // MODE 2 = general mode with a boolean mask: an instantiation of its own, because as a run-time test the mask words
  // cost the causal and variable-length calls registers they do not use.
  constexpr bool masked = MODE == 2;
  if (masked) mask_g = p.mask + b * p.m_sb + n * p.m_sn;
  // Boolean mask of a tile that lies wholly inside the sequence: the lane fetches the BN bytes of its own query row as
  // 16-byte words (any alignment: global loads take unaligned addresses) one tile ahead, into the set that belongs to
  // the tile's LDS stage, so they arrive with the tile's own data and cost no wait of their own.  The tile that runs
  // past the end of the row is tested byte by byte instead (a 16-byte read could leave the mask there).
  i32x4_t mask_w[2][C::kNQB][C::kNKB][2];
  auto mask_fetch = [&](int key0, auto stage_c) __attribute__((always_inline)) {
    constexpr int st = decltype(stage_c)::value;
#pragma unroll
    for (int qb = 0; qb < C::kNQB; ++qb) {
      const int qrow = min(q0 + wave * QPW + qb * 32 + l32, Sq - 1);
      const unsigned char* mrow = mask_g + (long long)qrow * p.m_sq + key0;
#pragma unroll
      for (int kb = 0; kb < C::kNKB; ++kb)
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) __builtin_memcpy(&mask_w[st][qb][kb][hf], mrow + kb * 32 + 16 * hf, 16);
    }
  };
  auto stream_next = [&](int& key0, int& fl) {  // sparse: produce the tile after the one produced last
    if (sub > 0) {  // remaining sub-tiles of the current 128-key block
      key0 = key0 + BN;
      sub = (sub + 1) % kSub;
      return;
    }
    const int ka = list_head(0), kb = kQBlocks > 1 ? list_head(1) : kEnd;
    const int k = ka < kb ? ka : kb;
    if (k == kEnd) {
      key0 = -1;
      fl = 0;
      return;
    }
    fl = (ka == k ? 1 : 0) | (kb == k ? 2 : 0);
    if (ka == k) list_pop(0);
    if (kQBlocks > 1 && kb == k) list_pop(1);
    key0 = k * 128;
    sub = kSub > 1 ? 1 : 0;
  };
  if (SPARSE) {
    stream_next(cur_key0, cur_fl);
    nxt_key0 = cur_key0;
    nxt_fl = cur_fl;
    if (cur_key0 >= 0) {
      load_tile(cur_key0, 0);
      stream_next(nxt_key0, nxt_fl);
    }
  } else {
    load_tile(0, 0);
    if (masked && BN <= Skv) mask_fetch(0, std::integral_constant<int, 0>{});
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the LDS-DMA of this wave has landed
  __syncthreads();
  bool first = !resumed;  // no tile has been folded into this wave's running softmax yet
  bool unseen[C::kNQB];   // general mode: this lane's row has not met a visible key yet
#pragma unroll
  for (int qb = 0; qb < C::kNQB; ++qb) unseen[qb] = true;

  // One tile step: fetch the tile at next_key0 (< 0: none) into the other stage, compute on the tile
  // at key0 if this wave takes part in it.  The LDS stage is a compile-time constant (the loops
  // below are unrolled by two), so every operand read is `lane-constant register + immediate offset`.
  auto tile_step = [&](auto stage_c, const int key0, const int next_key0, const bool active) {
    constexpr int stage = decltype(stage_c)::value;
    if (next_key0 >= 0) load_tile(next_key0, stage ^ 1);
    if (masked && !SPARSE && next_key0 >= 0 && next_key0 + BN <= Skv)
      mask_fetch(next_key0, std::integral_constant<int, stage ^ 1>{});
    if (active) {
    MSD_LDS const char* kb_base = smem + stage * C::kStageBytes;
    MSD_LDS const char* vb_base = kb_base + C::kTileBytes;

    // ---- S^T = K Q^T: kNKB independent accumulation chains per 16-wide step of head_dim -------
    f32x16_t sacc[C::kNKB][C::kNQB];
    X8 afrag[2][C::kNKB];
#pragma unroll
    for (int kb = 0; kb < C::kNKB; ++kb)
      afrag[0][kb] = *(MSD_LDS const X8*)(kb_base + kb * 32 * C::kRowBytes + k_row_off + ((h ^ k_swz) << 4));
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      if (ks + 1 < 8) {
#pragma unroll
        for (int kb = 0; kb < C::kNKB; ++kb)
          afrag[(ks + 1) & 1][kb] = *(MSD_LDS const X8*)(kb_base + kb * 32 * C::kRowBytes + k_row_off +
                                                         (((2 * (ks + 1) + h) ^ k_swz) << 4));
      }
#pragma unroll
      for (int kb = 0; kb < C::kNKB; ++kb)
#pragma unroll
        for (int qb = 0; qb < C::kNQB; ++qb)
          sacc[kb][qb] = E::mfma32(afrag[ks & 1][kb], qf[qb][ks], ks == 0 ? negm[qb] : sacc[kb][qb]);
    }
    if (SCHED == 1) {
      // operand reads run one head_dim step ahead of the matrix instructions that consume them
      __builtin_amdgcn_sched_group_barrier(0x100, C::kNKB, 0);
#pragma unroll
      for (int ks = 0; ks < 7; ++ks) {
        __builtin_amdgcn_sched_group_barrier(0x100, C::kNKB, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, C::kNKB * C::kNQB, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, C::kNKB * C::kNQB, 0);
      __builtin_amdgcn_sched_barrier(0);
    }

    // ---- mask keys past the end of the sequence (last tile only) --------------------------------
    if (key0 + BN > Skv) {
#pragma unroll
      for (int kb = 0; kb < C::kNKB; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = key0 + kb * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
          if (key >= Skv) {
#pragma unroll
            for (int qb = 0; qb < C::kNQB; ++qb) sacc[kb][qb][r] = -INFINITY;
          }
        }
    }
    if (MODE) {
      // causal: only tiles that reach past the diagonal of this wave's first row need element tests
      if (p.causal && key0 + BN - 1 > q0 + wave * QPW + causal_shift) {
#pragma unroll
        for (int qb = 0; qb < C::kNQB; ++qb) {
          const int last_visible = q0 + wave * QPW + qb * 32 + l32 + causal_shift;
#pragma unroll
          for (int kb = 0; kb < C::kNKB; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int key = key0 + kb * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
              if (key > last_visible) sacc[kb][qb][r] = -INFINITY;
            }
        }
      }
      // boolean mask: one byte per (query, key); a lane tests the 16 x kNKB keys of its own query row
      if (masked && !SPARSE && key0 + BN <= Skv) {
        // register r of block kb is key 32 kb + 8 (r / 4) + 4 h + r % 4: dword 2 (r / 4) + h of the block's 32 bytes
#pragma unroll
        for (int qb = 0; qb < C::kNQB; ++qb)
#pragma unroll
          for (int kb = 0; kb < C::kNKB; ++kb)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
              const i32x4_t w4 = mask_w[stage][qb][kb][g4 >> 1];
              const unsigned w = (unsigned)(h ? w4[2 * (g4 & 1) + 1] : w4[2 * (g4 & 1)]);
#pragma unroll
              for (int j = 0; j < 4; ++j)
                if (((w >> (8 * j)) & 0xffu) == 0) sacc[kb][qb][4 * g4 + j] = -INFINITY;
            }
      } else if (masked) {
#pragma unroll
        for (int qb = 0; qb < C::kNQB; ++qb) {
          const int qrow = min(q0 + wave * QPW + qb * 32 + l32, Sq - 1);
          const unsigned char* mrow = mask_g + (long long)qrow * p.m_sq;
#pragma unroll
          for (int kb = 0; kb < C::kNKB; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int key = key0 + kb * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
              if (key < Skv && mrow[key] == 0) sacc[kb][qb][r] = -INFINITY;
            }
        }
      }
    }

    // ---- online softmax in the exp2 domain with a lazily moved reference maximum ------------------
    // sacc already holds s - m_run.  The reference only moves when some row of this tile exceeds
    // it by more than kTau (or on the first tile), so the exponentials need no per-element
    // subtraction and the accumulator rescale is skipped for almost every tile; probabilities stay
    // <= 2^kTau.  Row sums are taken from the rounded probabilities (the values the second product
    // uses) with a packed dot product against ones.
    X8 pf[C::kNQB][C::kNKB][2];
#pragma unroll
    for (int qb = 0; qb < C::kNQB; ++qb) {
      float mx = sacc[0][qb][0];
#pragma unroll
      for (int kb = 0; kb < C::kNKB; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sacc[kb][qb][r]);
      // (the test needs no row maximum: some lane's part exceeds the threshold iff some row's maximum does)
      // General mode: a mask can hide a whole tile from a row, so "nothing folded in yet" is kept per row - a row
      // takes its exact maximum as reference with the first tile that shows it a key, whichever tile that is.
      const bool lane_wants = MODE ? (mx > kTau || (unseen[qb] && mx > -INFINITY)) : mx > kTau;
      if ((!MODE && first) || __builtin_amdgcn_ballot_w64(lane_wants) != 0) {
        mx = half_max(mx);
        const bool fresh = MODE ? unseen[qb] : first;
        // first visible tile: move to the exact row maximum (delta may be negative); later: only upwards
        float delta = fresh ? mx : fmaxf(mx, 0.f);
        delta = (delta == -INFINITY) ? 0.f : delta;
        // (first tile: sums and outputs are still zero; 2^-delta would overflow for rows far below zero and 0 * inf is NaN)
        const float alpha = fresh ? 1.f : fast_exp2(-delta);
        if (MODE) unseen[qb] = unseen[qb] && mx == -INFINITY;
        m_run[qb] += delta;
        l_run[qb] *= alpha;
#pragma unroll
        for (int r = 0; r < 16; ++r) negm[qb][r] = -m_run[qb];
#pragma unroll
        for (int kb = 0; kb < C::kNKB; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) sacc[kb][qb][r] -= delta;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) oacc[db][qb][r] *= alpha;
      }
      float ls = 0.f;
#pragma unroll
      for (int kb = 0; kb < C::kNKB; ++kb) {
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
          X8 pk;
#pragma unroll
          for (int j = 0; j < 8; ++j) pk[j] = E::from_float(fast_exp2(sacc[kb][qb][8 * t2 + j]));
          pf[qb][kb][t2] = pk;
          ls = E::sum8(pk, ls);
        }
      }
      l_run[qb] += ls;
    }

    // ---- O^T += V^T P^T ------------------------------------------------------------------------
    // 128-key tiles: V^T fragments are read one 16-key step ahead of the matrix instructions that use them
    // with asm reads and explicit waits (see lds_read_tr16_async), so that the next tile's LDS-DMA stays in
    // flight until the end of the tile.  With 64-key tiles (two workgroups per CU cover each other's stalls)
    // the builtin and the compiler's own schedule measured faster.
    if constexpr (BN == 128) {
      constexpr int kSteps = C::kNKB * 2;
      s16x4_t vf[2][8];
      auto issue = [&](auto step_c, s16x4_t(&dst)[8]) __attribute__((always_inline)) {
        constexpr int s = decltype(step_c)::value;
        constexpr int off = ((s >> 1) * 32 + (s & 1) * 16) * C::kRowBytes;
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          const unsigned a = v_lds[db] + stage * C::kStageBytes;
          dst[2 * db] = lds_read_tr16_async<off>(a);
          dst[2 * db + 1] = lds_read_tr16_async<off + 8 * C::kRowBytes>(a);
        }
      };
      issue(std::integral_constant<int, 0>{}, vf[0]);
      static_for<kSteps>([&](auto step_c) __attribute__((always_inline)) {
        constexpr int s = decltype(step_c)::value;
        if constexpr (s + 1 < kSteps) {
          issue(std::integral_constant<int, s + 1>{}, vf[(s + 1) & 1]);
          lds_wait_tr<8>(vf[s & 1]);
        } else {
          lds_wait_tr<0>(vf[s & 1]);
        }
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          union { s16x4_t s2[2]; X8 x; } u;
          u.s2[0] = vf[s & 1][2 * db];
          u.s2[1] = vf[s & 1][2 * db + 1];
#pragma unroll
          for (int qb = 0; qb < C::kNQB; ++qb)
            oacc[db][qb] = E::mfma32(u.x, pf[qb][s >> 1][s & 1], oacc[db][qb]);
        }
      });
    } else {
#pragma unroll
    for (int kb = 0; kb < C::kNKB; ++kb) {
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) {
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          MSD_LDS const char* src =
              vb_base + (kb * 32 + 16 * t2) * C::kRowBytes + v_row_off + ((db ^ v_swz) << 6);
          const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((MSD_LDS s16x4_t*)src);
          const s16x4_t hi =
              __builtin_amdgcn_ds_read_tr16_b64_v4i16((MSD_LDS s16x4_t*)(src + 8 * C::kRowBytes));
          union { s16x4_t s[2]; X8 x; } u;
          u.s[0] = lo;
          u.s[1] = hi;
#pragma unroll
          for (int qb = 0; qb < C::kNQB; ++qb) oacc[db][qb] = E::mfma32(u.x, pf[qb][kb][t2], oacc[db][qb]);
        }
      }
    }
    }

      first = false;
    }  // active
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): next tile's LDS-DMA issued by this wave is complete
    __syncthreads();
  };
  if (SPARSE) {
    // the fetched tile becomes current, the one after it is fetched next
    auto sparse_step = [&](auto stage_c) {
      tile_step(stage_c, cur_key0, nxt_key0, ((cur_fl >> grp) & 1) != 0);
      cur_key0 = nxt_key0;
      cur_fl = nxt_fl;
      if (nxt_key0 >= 0) stream_next(nxt_key0, nxt_fl);
    };
    while (cur_key0 >= 0) {
      sparse_step(std::integral_constant<int, 0>{});
      if (cur_key0 < 0) break;
      sparse_step(std::integral_constant<int, 1>{});
    }
  } else {
    for (int t = 0; t < dense_tiles; t += 2) {
      tile_step(std::integral_constant<int, 0>{}, t * BN, t + 1 < dense_tiles ? (t + 1) * BN : -1, true);
      if (t + 1 < dense_tiles)
        tile_step(std::integral_constant<int, 1>{}, (t + 1) * BN, t + 2 < dense_tiles ? (t + 2) * BN : -1, true);
    }
  }

  // ---- epilogue: normalise, transpose 32 query rows at a time through LDS, coalesced store -------
  // Each wave stages only its own rows, and a wave's LDS operations execute in order, so no
  // workgroup barrier is needed here (the loop above ended with one).
  MSD_LDS char* ost = smem + wave * 32 * C::kORowBytes;
#pragma unroll
  for (int qb = 0; qb < C::kNQB; ++qb) {
    const float l_tot = half_sum(l_run[qb]);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const int qrow_l = q0 + wave * QPW + qb * 32 + l32;
    if (p.lse && h == 0 && qrow_l < Sq) {
      long long li = ((long long)b * p.N + n) * p.Sq + (GATHER ? p.tok[qrow_l] : qrow_l);
      if (MODE && p.seq_meta && p.lse_token_major) li = ((long long)p.seq_meta[4 * b] + qrow_l) * p.N + n;
      p.lse[li] = l_tot > 0.f ? m_run[qb] * 0.6931471805599453f + __logf(l_tot) : -INFINITY;
    }
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        typename E::x4 pk;
#pragma unroll
        for (int j = 0; j < 4; ++j) pk[j] = E::from_float(oacc[db][qb][4 * g + j] * inv);
        const int d = db * 32 + 8 * g + 4 * h;
        *(MSD_LDS typename E::x4*)(ost + l32 * C::kORowBytes + d * 2) = pk;
      }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < 32 * 16 / 64; ++i) {
      const int c = i * 64 + lane;
      const int row = c >> 4, c16 = c & 15;
      const int qrow = q0 + wave * QPW + qb * 32 + row;
      // rows are padded by 8 bytes, so a 16-byte chunk is read as two 8-byte halves
      const i32x2_t lo = *(MSD_LDS const i32x2_t*)(ost + row * C::kORowBytes + c16 * 16);
      const i32x2_t hi = *(MSD_LDS const i32x2_t*)(ost + row * C::kORowBytes + c16 * 16 + 8);
      if (qrow < Sq) {
        i32x4_t v = {lo[0], lo[1], hi[0], hi[1]};
        const int orow = GATHER ? p.tok[qrow] : qrow;
        *(i32x4_t*)(og + (long long)orow * p.o_ss + c16 * 8) = v;
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
#endif  // __HIP_DEVICE_COMPILE__
}

// Dense attention on the 16x16x32 matrix instruction (8 waves x 32 query rows, 128-key tiles).  The same
// transposed formulation as fa_fwd_kernel; what changes is the shape of the register tiles.  With c = lane % 16
// and g = lane / 16:
//     S^T block (16 keys x 16 queries):  A = K rows 16*kb + c, head_dim 32*ks + 8*g .. +8 (one 16-byte LDS read),
//                                        B = Q^T resident (query 16*nq + c, same head_dim slice);
//                                        the lane receives keys 16*kb + 4*g + i (i < 4) of query 16*nq + c
//     O^T block (16 dims x 16 queries):  B = P^T of 32 keys straight from two S^T blocks (slot 8*g + t holds key
//                                        32*j + 4*g + t for t < 4 and key 32*j + 16 + 4*g + t - 4 for t >= 4),
//                                        A = V^T in the same slot order from two transposing LDS reads
// A row maximum is 32 in-lane operations per tile and query column plus two lane exchanges (rows of 16 lanes, then
// halves).  The instruction sustains 2.4 PFLOP/s where the 32x32x16 form stops at 2.1-2.2.
// LDS: K stages at 0 and 32 KiB, V stages at 64 and 96 KiB, so that stage and row offsets of every read fit the
// 16-bit offset field.  K rows are swizzled as in fa_fwd_kernel; V: 32-byte chunk c32 of row key is stored at chunk
// c32 ^ (key & 7) - a half-wave of the transposing read covers 8 rows x 32 bytes.
// PAIR: first pass of the paired block-sparse scheme (bsa_pair.hip).  The workgroup's 256 rows are two 128-row query
// blocks that need not be neighbours (waves 0-3: p.pairs[..][0], waves 4-7: p.pairs[..][1]; -1 = no second block,
// those waves compute on zeros and store nothing); the key tiles are the 128-key blocks of the pair's list
// (p.blk_idx / p.blk_cnt indexed by pair) instead of the whole sequence.  Besides the normalised rows it writes
// p.state, the log2-domain log-sum-exp the second pass resumes from.  GATHER as in fa_fwd_kernel.
//
// GEN 1: the general mode without a boolean mask: per-sequence lengths and token offsets from p.seq_meta and / or a
// causal mask aligned to the bottom-right corner.  No per-row flags are needed for it: a row either sees key 0, which
// lies in its first tile, or (causal with more queries than keys) no key at all, and the first tile's rule for the
// reference maximum covers both.  GEN 2: the same with the packed tile numbering of p.packed_tiles (256-row tiles).
// GEN 3: a boolean mask over the keys that all queries of a (batch, head) share (p.mask with m_sq = 0, a key-padding
// mask; neither causal nor per-sequence lengths).  The 128 bytes of the next tile are fetched during the second product and reduced to four
// 32-bit words of visible keys in scalar registers; a tile with all of its keys visible runs the plain code, the
// others test their scores against the words.  The rule of the first tile stays in force until a tile has shown the
// wave a key: that tile holds the first visible key, which every row sees, so once more no row needs a state of
// its own.
//
// DPAD: tensors whose head_dim lies between 64 and 128 (p.head_dim, a multiple of 8), computed as head_dim 128: the
// query operand is zero from p.head_dim on, and the lanes that would stage the 16-byte chunks of K and V past it
// request an offset beyond the buffers' range instead, for which the DMA writes zeros without touching memory.  The
// output columns past p.head_dim are not stored.
template <int DT, int NWAVES = 8, bool PAIR = false, bool GATHER = false, int GEN = 0, bool DPAD = false>
__global__ __launch_bounds__(NWAVES * 64, 1) void fa_fwd16_kernel(const FaParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  using E = Elem<DT>;
  using T = typename E::type;
  using X8 = typename E::x8;
  constexpr int BN = 128, kBM = NWAVES * 32, kRowBytes = 256, kTileBytes = BN * kRowBytes;
  constexpr int kORowBytes = kRowBytes + 8;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  MSD_LDS char* smem = (MSD_LDS char*)smem_raw;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 15;
  const int g = lane >> 4;

  static_assert(!PAIR || NWAVES == 8, "a pair is two groups of four waves");
  constexpr bool gen = GEN != 0, packed = GEN == 2, keymask = GEN == 3;
  static_assert(!gen || (!PAIR && !GATHER), "general mode: dense tensors in their own order");
  int bn, qt, b, n, Sq, Skv;
  long long q_tok0, k_tok0;  // general mode: first token of the sequence in packed tensors
  if (!fa16_find_work<GEN, PAIR>(p, kBM, bn, qt, b, n, Sq, Skv, q_tok0, k_tok0)) return;
  const int nkv = n / (p.N / p.Nkv);
  // first query row of this wave; rows at or beyond row_end do not exist (tail of the sequence / of the block)
  int row0 = qt * kBM + wave * 32, row_end = Sq;
  if constexpr (PAIR) {
    const int qblk = p.pairs[((long long)bn * p.NP + qt) * 2 + (wave >> 2)];
    row0 = qblk * 128 + (wave & 3) * 32;
    row_end = qblk < 0 ? 0 : min(Sq, qblk * 128 + 128);
    if (qblk < 0) row0 = 0;
  }

  const T* qg = (const T*)p.q + b * p.q_sb + n * p.q_sn + q_tok0 * p.q_ss;
  const T* kg = (const T*)p.k + b * p.k_sb + nkv * p.k_sn + k_tok0 * p.k_ss;
  const T* vg = (const T*)p.v + b * p.v_sb + nkv * p.v_sn + k_tok0 * p.v_ss;
  T* og = (T*)p.o + b * p.o_sb + n * p.o_sn + q_tok0 * p.o_ss;

  // ---- Q^T operand, resident: lane (c, g) holds query 16*nq + c, head_dim 32*ks + 8*g .. +8 --------------
  X8 qf[2][4];
#pragma unroll
  for (int nq = 0; nq < 2; ++nq) {
    const int qrow = row0 + nq * 16 + c;
    const bool ok = qrow < row_end;
    const int qsrc = GATHER ? p.tok[ok ? qrow : 0] : (ok ? qrow : 0);
    const T* src = qg + (long long)qsrc * p.q_ss + 8 * g;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      X8 v;
      if constexpr (DPAD) {
        const bool in = ok && 32 * ks + 8 * g < p.head_dim;  // (a chunk of 8 lies wholly inside or outside)
        v = in ? *(const X8*)(src + 32 * ks) : X8{0};
      } else {
        v = *(const X8*)(src + 32 * ks);
        if (!ok) v = X8{0};
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = E::from_float((float)v[j] * p.scale_log2);
      qf[nq][ks] = v;
    }
  }

  f32x4_t oacc[8][2];
  float l_run[2];
  // Row sums come off the matrix pipe: ones x P^T gives every lane the sum of its query column over the 128 keys of a
  // tile (8 more matrix instructions per tile in place of 32 v_dot2).  lt holds the sums of the tile before; they are
  // added to l_run at the start of the next softmax, before a rescale, when the matrix results have long landed.
  f32x4_t lt[2] = {f32x4_t{0.f, 0.f, 0.f, 0.f}, f32x4_t{0.f, 0.f, 0.f, 0.f}};
  X8 ones;
#pragma unroll
  for (int j = 0; j < 8; ++j) ones[j] = E::from_float(1.f);
  f32x4_t negm[2];  // minus the reference maximum (log2 units), in the four slots that seed an accumulator
#pragma unroll
  for (int nq = 0; nq < 2; ++nq) {
    l_run[nq] = 0.f;
    negm[nq] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int db = 0; db < 8; ++db) oacc[db][nq] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  // ---- global -> LDS staging (LDS-DMA; swizzles applied on the global side) -------------------------------
  // (a sequence without keys exposes nothing: every row reads as zeros and no tile is computed)
  const int row_elems = DPAD ? p.head_dim : 128;
  const int k_range = gen && Skv <= 0 ? 0 : (int)(((long long)(Skv - 1) * p.k_ss + row_elems) * 2);
  const int v_range = gen && Skv <= 0 ? 0 : (int)(((long long)(Skv - 1) * p.v_ss + row_elems) * 2);
  const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)kg, 0, k_range, 0x00020000);
  const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)vg, 0, v_range, 0x00020000);
  const int k_row_bytes = (int)p.k_ss * 2, v_row_bytes = (int)p.v_ss * 2;
  int k_voff, v_voff;
  {
    const int row = 4 * wave + (lane >> 4);  // groups of one wave lie 4 * NWAVES rows apart: same swizzles
    const int pc = lane & 15;                // physical 16-byte chunk this lane fills
    const int kc = pc ^ (row & 15), vc = (((pc >> 1) ^ (row & 7)) << 1) | (pc & 1);  // logical chunks of the row
    k_voff = row * k_row_bytes + (kc << 4);
    v_voff = row * v_row_bytes + (vc << 4);
    if constexpr (DPAD) {  // chunks past the head_dim: an offset beyond every range, the DMA writes zeros for them
      if (kc * 8 >= p.head_dim) k_voff = 0x7ffffff0;
      if (vc * 8 >= p.head_dim) v_voff = 0x7ffffff0;
    }
  }
  auto load_tile = [&](int key0, int stage) {
    tile_dma<BN / 4 / NWAVES, NWAVES>(k_rsrc, v_rsrc, smem + stage * kTileBytes, smem + (2 + stage) * kTileBytes, k_voff,
                                      v_voff, wave, key0 * k_row_bytes, key0 * v_row_bytes, k_row_bytes, v_row_bytes);
  };

  // per-lane parts of the LDS read addresses
  // K operand: row 16*kb + c, 16-byte chunk (4*ks + g) ^ c
  unsigned k_lds[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) k_lds[ks] = (unsigned)(uintptr_t)smem + c * kRowBytes + (((4 * ks + g) ^ c) << 4);
  // V^T operand: the lane points at key 4*g + c/4 (+32*j, +16), 8 bytes at 8*(c%4) of 32-byte chunk db ^ (key & 7)
  // (blocks db and db + 4 differ in bit 7 of the address only: four registers, the other four by one XOR)
  unsigned v_lds[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
    v_lds[db] = (unsigned)(uintptr_t)smem + 2 * kTileBytes + (4 * g + (c >> 2)) * kRowBytes +
                ((db ^ (4 * (g & 1) + (c >> 2))) << 5) + 8 * (c & 3);

  // causal: query i sees keys <= i + causal_shift; the last row of this workgroup bounds the tiles it walks
  const int causal_shift = Skv - Sq;
  const bool causal = gen && !keymask && p.causal;  // (with a key mask: neither causal nor per-sequence lengths)
  const int kv_lim = causal ? max(0, min(Skv, qt * kBM + kBM + causal_shift)) : Skv;
  const int tiles = (kv_lim + BN - 1) / BN;
  // PAIR: the ids of the list are fetched with scalar loads two tiles ahead of their use
  int l_n = 0, id_a = -1, id_b = -1;  // id_a: the tile being computed (already requested), id_b: the one after it
  const int* l_ptr = nullptr;
  if constexpr (PAIR) {
    const long long pair_lin = (long long)bn * p.NP + qt;
    l_ptr = p.blk_idx + pair_lin * p.kb_stride;
    l_n = __builtin_amdgcn_readfirstlane(p.blk_cnt[pair_lin]);
    if (l_n > 0) id_a = scalar_load(l_ptr, 0);
    if (l_n > 1) id_b = scalar_load(l_ptr, 1);
    if (l_n > 0) load_tile(id_a * BN, 0);
  } else {
    load_tile(0, 0);
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  __syncthreads();
  bool first = true;

  // ---- key mask (GEN 3): words of visible keys of the current tile; bit l of word j = key 4 * l + j ------------
  unsigned kvis[4] = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};
  unsigned kraw = 0;  // the lane's four mask bytes of the tile that comes next (lanes 0 .. 31)
  const unsigned char* mask_g = nullptr;
  if constexpr (keymask) mask_g = p.mask + b * p.m_sb + n * p.m_sn;
  auto mask_request = [&](int key0) __attribute__((always_inline)) {  // the load only
    if constexpr (keymask) {
      kraw = 0;
      const int k4 = key0 + 4 * (lane & 31);
      if (key0 + BN <= Skv) {
        __builtin_memcpy(&kraw, mask_g + k4, 4);  // (any alignment)
      } else {                                    // the tile that runs past the row: byte by byte, inside the row
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const unsigned byte = mask_g[min(k4 + j, Skv - 1)];
          kraw |= (k4 + j < Skv ? byte : 0u) << (8 * j);
        }
      }
    }
  };
  auto mask_reduce = [&]() __attribute__((always_inline)) {  // bytes -> words in scalar registers
    if constexpr (keymask) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        kvis[j] = (unsigned)__builtin_amdgcn_ballot_w64(lane < 32 && ((kraw >> (8 * j)) & 0xffu) != 0);
    }
  };
  if constexpr (keymask) {
    if (tiles > 0) mask_request(0);
    mask_reduce();
  }

  auto tile_step = [&](auto stage_c, const int key0, const int next_key0) {
    constexpr int stage = decltype(stage_c)::value;
    if (next_key0 >= 0) load_tile(next_key0, stage ^ 1);
    const unsigned kv_all = kvis[0] & kvis[1] & kvis[2] & kvis[3];

    // ---- S^T = K Q^T: 16 accumulation chains; operand reads in groups of 2 key blocks of one 32-wide head_dim
    // step, kAhead groups ahead of the matrix instructions that use them (ring of kAhead + 1) -----------------
    f32x4_t sacc[8][2];
    constexpr int kAhead = FA16_AHEAD;
    X8 afrag[kAhead + 1][2];
    auto k_read = [&](auto gi_c, X8(&dst)[2]) __attribute__((always_inline)) {
      constexpr int gi = decltype(gi_c)::value;
      constexpr int ks = gi >> 2, qu = gi & 3;
#pragma unroll
      for (int i = 0; i < 2; ++i)
        dst[i] = *(MSD_LDS const X8*)(uintptr_t)(k_lds[ks] + stage * kTileBytes + (2 * qu + i) * 16 * kRowBytes);
    };
    static_for<kAhead>([&](auto gi_c) __attribute__((always_inline)) { k_read(gi_c, afrag[decltype(gi_c)::value]); });
    static_for<16>([&](auto gi_c) __attribute__((always_inline)) {
      constexpr int gi = decltype(gi_c)::value;
      constexpr int ks = gi >> 2, qu = gi & 3;
      if constexpr (gi + kAhead < 16) k_read(std::integral_constant<int, gi + kAhead>{}, afrag[(gi + kAhead) % (kAhead + 1)]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int nq = 0; nq < 2; ++nq)
          sacc[2 * qu + i][nq] =
              E::mfma16(afrag[gi % (kAhead + 1)][i], qf[nq][ks], ks == 0 ? negm[nq] : sacc[2 * qu + i][nq]);
    });
    __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0);
#pragma unroll
    for (int gi = 0; gi < 16 - kAhead; ++gi) {
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 4 * kAhead, 0);
    __builtin_amdgcn_sched_barrier(0);

    // ---- keys past the end of the sequence (last tile only) ---------------------------------------------------
    if (key0 + BN > Skv) {
#pragma unroll
      for (int kb = 0; kb < 8; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (key0 + 16 * kb + 4 * g + i >= Skv) {
            sacc[kb][0][i] = -INFINITY;
            sacc[kb][1][i] = -INFINITY;
          }
    }

    // ---- causal: keys beyond the diagonal (the tiles that cross it for some row of this wave) ------------------
    if constexpr (gen) {
      if (causal && key0 + BN - 1 > row0 + causal_shift) {
        const int lim = row0 + c + causal_shift - key0 - 4 * g;  // visible: 16 * kb + i <= lim (+16 for nq = 1)
#pragma unroll
        for (int kb = 0; kb < 8; ++kb)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            if (16 * kb + i > lim) sacc[kb][0][i] = -INFINITY;
            if (16 * kb + i > lim + 16) sacc[kb][1][i] = -INFINITY;
          }
      }
    }

    // ---- key mask: tiles that hide some of their keys ----------------------------------------------------------
    if constexpr (keymask) {
      if (kv_all != 0xffffffffu) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const unsigned w = kvis[i] >> g;  // key 16 * kb + 4 * g + i is bit 4 * kb + g of word i
#pragma unroll
          for (int kb = 0; kb < 8; ++kb)
            if (!((w >> (4 * kb)) & 1u)) {
              sacc[kb][0][i] = -INFINITY;
              sacc[kb][1][i] = -INFINITY;
            }
        }
      }
    }

    // ---- online softmax (exp2 domain, lazily moved reference maximum; see fa_fwd_kernel) ---------------------
    X8 pf[2][4];
    bool seen = !keymask;  // key mask: this tile showed some row of the wave a key (all rows share the mask)
#pragma unroll
    for (int nq = 0; nq < 2; ++nq) {
      float mx = sacc[0][nq][0];
#pragma unroll
      for (int kb = 0; kb < 8; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) mx = fmaxf(mx, sacc[kb][nq][i]);
      if constexpr (keymask) seen = seen || __builtin_amdgcn_ballot_w64(mx > -INFINITY) != 0;
      // (the test needs no row maximum: some lane's part exceeds the threshold iff some row's maximum does)
      float delta = 0.f, alpha = 1.f;
      int moved = 0;
      if (first || __builtin_amdgcn_ballot_w64(mx > kTau) != 0) {
        mx = quarter_max(mx);
        delta = first ? mx : fmaxf(mx, 0.f);
        delta = (delta == -INFINITY) ? 0.f : delta;
        // (first tile: sums and outputs are still zero; 2^-delta would overflow for rows far below zero and 0 * inf is NaN)
        alpha = first ? 1.f : fast_exp2(-delta);
        moved = 1;
      }
      l_run[nq] += lt[nq][0];
      // the rescale itself: in place, skipped when the reference did not move (see cond_rescale_fa16)
      cond_rescale_fa16(__builtin_amdgcn_readfirstlane(moved), delta, alpha, l_run[nq], negm[nq], sacc[0][nq], sacc[1][nq],
                        sacc[2][nq], sacc[3][nq], sacc[4][nq], sacc[5][nq], sacc[6][nq], sacc[7][nq], oacc[0][nq],
                        oacc[1][nq], oacc[2][nq], oacc[3][nq], oacc[4][nq], oacc[5][nq], oacc[6][nq], oacc[7][nq]);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        X8 pk;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          pk[t] = E::from_float(fast_exp2(sacc[2 * j][nq][t]));
          pk[4 + t] = E::from_float(fast_exp2(sacc[2 * j + 1][nq][t]));
        }
        pf[nq][j] = pk;
      }
    }

    // ---- O^T += V^T P^T: 8 steps of (32 keys) x (4 head_dim blocks); V^T fragments requested one step ahead
    // with asm reads and explicit waits, so that the next tile's LDS-DMA stays in flight (see lds_read_tr16_async)
    s16x4_t vf[2][8];
    auto issue = [&](auto step_c, s16x4_t(&dst)[8]) __attribute__((always_inline)) {
      constexpr int s = decltype(step_c)::value;
      constexpr int j = s >> 1, dbh = s & 1;
      constexpr int off = stage * kTileBytes + 32 * j * kRowBytes;
#pragma unroll
      for (int d4 = 0; d4 < 4; ++d4) {
        const unsigned a = v_lds[d4] ^ (dbh << 7);
        dst[2 * d4] = lds_read_tr16_async<off>(a);
        dst[2 * d4 + 1] = lds_read_tr16_async<off + 16 * kRowBytes>(a);
      }
    };
    if constexpr (keymask) {
      if (next_key0 >= 0) mask_request(next_key0);  // lands during the second product
    }
    issue(std::integral_constant<int, 0>{}, vf[0]);
    static_for<8>([&](auto step_c) __attribute__((always_inline)) {
      constexpr int s = decltype(step_c)::value;
      constexpr int j = s >> 1, dbh = s & 1;
      if constexpr (s + 1 < 8) {
        issue(std::integral_constant<int, s + 1>{}, vf[(s + 1) & 1]);
        lds_wait_tr<8>(vf[s & 1]);
      } else {
        lds_wait_tr<0>(vf[s & 1]);
      }
#pragma unroll
      for (int d4 = 0; d4 < 4; ++d4) {
        union { s16x4_t s2[2]; X8 x; } u;
        u.s2[0] = vf[s & 1][2 * d4];
        u.s2[1] = vf[s & 1][2 * d4 + 1];
#pragma unroll
        for (int nq = 0; nq < 2; ++nq) oacc[4 * dbh + d4][nq] = E::mfma16(u.x, pf[nq][j], oacc[4 * dbh + d4][nq]);
      }
      if constexpr (dbh == 0) {  // the row sums of these 32 keys
#pragma unroll
        for (int nq = 0; nq < 2; ++nq)
          lt[nq] = E::mfma16(ones, pf[nq][j], j == 0 ? f32x4_t{0.f, 0.f, 0.f, 0.f} : lt[nq]);
      }
    });

    first = first && !seen;  // (without a key mask: false from the first tile on)
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's part of the next tile has landed
    mask_reduce();
    __syncthreads();
  };
  if constexpr (PAIR) {
    for (int pos = 0; pos < l_n; pos += 2) {
      const int id_c = scalar_load(l_ptr, pos + 2 < l_n ? pos + 2 : 0);
      const int id_d = scalar_load(l_ptr, pos + 3 < l_n ? pos + 3 : 0);
      tile_step(std::integral_constant<int, 0>{}, id_a * BN, pos + 1 < l_n ? id_b * BN : -1);
      if (pos + 1 < l_n) tile_step(std::integral_constant<int, 1>{}, id_b * BN, pos + 2 < l_n ? id_c * BN : -1);
      id_a = id_c;
      id_b = id_d;
    }
    // ---- second phase (p.ex_idx given): the key blocks that only one partner selected ----------------------------
    // Each group of four waves walks the list of its own query block in sub-tiles of 64 keys, staged into its own half
    // of the four LDS buffers by its own waves; the eight waves still meet at one barrier per sub-tile, and the
    // running softmax simply goes on.  The traffic of these blocks (64 KiB for 128 rows, twice the bytes per flop of
    // the shared tiles) runs beside other workgroups' shared phases instead of in a launch of its own.
    if (p.ex_idx) {
      const int grp = wave >> 2, w4 = wave & 3;
      constexpr int kHalf = kTileBytes / 2;
      const long long pair_lin = (long long)bn * p.NP + qt;
      const int qb_mine = __builtin_amdgcn_readfirstlane(p.pairs[pair_lin * 2 + grp]);
      const int qb_other = __builtin_amdgcn_readfirstlane(p.pairs[pair_lin * 2 + (grp ^ 1)]);
      const int* e_ptr = p.ex_idx + ((long long)bn * p.QB + max(qb_mine, 0)) * p.kb_stride;
      const int e_n = qb_mine >= 0 ? __builtin_amdgcn_readfirstlane(p.ex_cnt[(long long)bn * p.QB + qb_mine]) : 0;
      const int e_o = qb_other >= 0 ? __builtin_amdgcn_readfirstlane(p.ex_cnt[(long long)bn * p.QB + qb_other]) : 0;
      const int my_steps = 2 * e_n, steps = 2 * max(e_n, e_o);
      // this group's halves of the stages; its waves stage rows 4 * w4 + 16 * i of a sub-tile
      auto load_half = [&](int key0, int stage) {
        MSD_LDS char* kb = smem + stage * kTileBytes + grp * kHalf;
        MSD_LDS char* vb = smem + (2 + stage) * kTileBytes + grp * kHalf;
        const int g16 = 16 * grp;
        const int kvo = k_voff - g16 * k_row_bytes, vvo = v_voff - g16 * v_row_bytes;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int g4 = i * 4 + w4;  // 4-row group of the sub-tile
          __builtin_amdgcn_raw_ptr_buffer_load_lds(k_rsrc, (MSD_LDS void*)(kb + g4 * 1024), 16, kvo,
                                                   (key0 + 16 * i) * k_row_bytes, 0, 0);
          __builtin_amdgcn_raw_ptr_buffer_load_lds(v_rsrc, (MSD_LDS void*)(vb + g4 * 1024), 16, vvo,
                                                   (key0 + 16 * i) * v_row_bytes, 0, 0);
        }
      };
      auto half_step = [&](auto stage_c, const int key0, const int next_key0) {
        constexpr int stage = decltype(stage_c)::value;
        if (next_key0 >= 0) load_half(next_key0, stage ^ 1);
        if (key0 >= 0) {
          // S^T = K Q^T over 4 key blocks (see tile_step), read from this group's half of the stage
          unsigned kl[4];
#pragma unroll
          for (int ks = 0; ks < 4; ++ks) kl[ks] = k_lds[ks] + grp * kHalf;
          f32x4_t sacc[4][2];
          constexpr int kAhead = FA16_AHEAD;
          X8 afrag[kAhead + 1][2];
          auto k_read = [&](auto gi_c, X8(&dst)[2]) __attribute__((always_inline)) {
            constexpr int gi = decltype(gi_c)::value;
            constexpr int ks = gi >> 1, qu = gi & 1;
#pragma unroll
            for (int i = 0; i < 2; ++i)
              dst[i] = *(MSD_LDS const X8*)(uintptr_t)(kl[ks] + stage * kTileBytes + (2 * qu + i) * 16 * kRowBytes);
          };
          static_for<kAhead>([&](auto gi_c) __attribute__((always_inline)) { k_read(gi_c, afrag[decltype(gi_c)::value]); });
          static_for<8>([&](auto gi_c) __attribute__((always_inline)) {
            constexpr int gi = decltype(gi_c)::value;
            constexpr int ks = gi >> 1, qu = gi & 1;
            if constexpr (gi + kAhead < 8) k_read(std::integral_constant<int, gi + kAhead>{}, afrag[(gi + kAhead) % (kAhead + 1)]);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
              for (int nq = 0; nq < 2; ++nq)
                sacc[2 * qu + i][nq] =
                    E::mfma16(afrag[gi % (kAhead + 1)][i], qf[nq][ks], ks == 0 ? negm[nq] : sacc[2 * qu + i][nq]);
          });
          __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0);
#pragma unroll
          for (int gi = 0; gi < 8 - kAhead; ++gi) {
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
          }
          __builtin_amdgcn_sched_group_barrier(0x008, 4 * kAhead, 0);
          __builtin_amdgcn_sched_barrier(0);
          if (key0 + 64 > Skv) {
#pragma unroll
            for (int kb = 0; kb < 4; ++kb)
#pragma unroll
              for (int i = 0; i < 4; ++i)
                if (key0 + 16 * kb + 4 * g + i >= Skv) {
                  sacc[kb][0][i] = -INFINITY;
                  sacc[kb][1][i] = -INFINITY;
                }
          }
          X8 pf[2][2];
#pragma unroll
          for (int nq = 0; nq < 2; ++nq) {
            float mx = sacc[0][nq][0];
#pragma unroll
            for (int kb = 0; kb < 4; ++kb)
#pragma unroll
              for (int i = 0; i < 4; ++i) mx = fmaxf(mx, sacc[kb][nq][i]);
            l_run[nq] += lt[nq][0];
            // (the rare path as plain code: this phase is bound by its memory traffic)
            if (first || __builtin_amdgcn_ballot_w64(mx > kTau) != 0) {
              mx = quarter_max(mx);
              float delta = first ? mx : fmaxf(mx, 0.f);
              delta = (delta == -INFINITY) ? 0.f : delta;
              const float alpha = first ? 1.f : fast_exp2(-delta);
              l_run[nq] *= alpha;
#pragma unroll
              for (int i = 0; i < 4; ++i) negm[nq][i] -= delta;
#pragma unroll
              for (int kb = 0; kb < 4; ++kb)
#pragma unroll
                for (int i = 0; i < 4; ++i) sacc[kb][nq][i] -= delta;
#pragma unroll
              for (int db = 0; db < 8; ++db)
#pragma unroll
                for (int i = 0; i < 4; ++i) oacc[db][nq][i] *= alpha;
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              X8 pk;
#pragma unroll
              for (int t = 0; t < 4; ++t) {
                pk[t] = E::from_float(fast_exp2(sacc[2 * j][nq][t]));
                pk[4 + t] = E::from_float(fast_exp2(sacc[2 * j + 1][nq][t]));
              }
              pf[nq][j] = pk;
            }
          }
          s16x4_t vf[2][8];
          unsigned vl[4];
#pragma unroll
          for (int d4 = 0; d4 < 4; ++d4) vl[d4] = v_lds[d4] + grp * kHalf;
          auto issue = [&](auto step_c, s16x4_t(&dst)[8]) __attribute__((always_inline)) {
            constexpr int s = decltype(step_c)::value;
            constexpr int j = s >> 1, dbh = s & 1;
            constexpr int off = stage * kTileBytes + 32 * j * kRowBytes;
#pragma unroll
            for (int d4 = 0; d4 < 4; ++d4) {
              const unsigned a = vl[d4] ^ (dbh << 7);
              dst[2 * d4] = lds_read_tr16_async<off>(a);
              dst[2 * d4 + 1] = lds_read_tr16_async<off + 16 * kRowBytes>(a);
            }
          };
          issue(std::integral_constant<int, 0>{}, vf[0]);
          static_for<4>([&](auto step_c) __attribute__((always_inline)) {
            constexpr int s = decltype(step_c)::value;
            constexpr int j = s >> 1, dbh = s & 1;
            if constexpr (s + 1 < 4) {
              issue(std::integral_constant<int, s + 1>{}, vf[(s + 1) & 1]);
              lds_wait_tr<8>(vf[s & 1]);
            } else {
              lds_wait_tr<0>(vf[s & 1]);
            }
#pragma unroll
            for (int d4 = 0; d4 < 4; ++d4) {
              union { s16x4_t s2[2]; X8 x; } u;
              u.s2[0] = vf[s & 1][2 * d4];
              u.s2[1] = vf[s & 1][2 * d4 + 1];
#pragma unroll
              for (int nq = 0; nq < 2; ++nq) oacc[4 * dbh + d4][nq] = E::mfma16(u.x, pf[nq][j], oacc[4 * dbh + d4][nq]);
            }
            if constexpr (dbh == 0) {
#pragma unroll
              for (int nq = 0; nq < 2; ++nq)
                lt[nq] = E::mfma16(ones, pf[nq][j], j == 0 ? f32x4_t{0.f, 0.f, 0.f, 0.f} : lt[nq]);
            }
          });
          first = false;
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's part of the next sub-tile has landed
        __syncthreads();
      };
      // key of sub-tile st of this group (-1: past its list); the block ids come by scalar loads one block ahead
      int e_cur = my_steps > 0 ? scalar_load(e_ptr, 0) : 0;
      if (my_steps > 0) load_half(e_cur * 128, 0);
      __builtin_amdgcn_s_waitcnt(0x0f70);
      __syncthreads();
      for (int st = 0; st < steps; st += 2) {  // one 128-key block per iteration: its two halves
        const int e_next = st + 2 < my_steps ? scalar_load(e_ptr, (st >> 1) + 1) : 0;
        const bool mine = st < my_steps;
        half_step(std::integral_constant<int, 0>{}, mine ? e_cur * 128 : -1, mine ? e_cur * 128 + 64 : -1);
        half_step(std::integral_constant<int, 1>{}, mine ? e_cur * 128 + 64 : -1, st + 2 < my_steps ? e_next * 128 : -1);
        e_cur = e_next;
      }
    }
  } else {
    for (int t = 0; t < tiles; t += 2) {
      tile_step(std::integral_constant<int, 0>{}, t * BN, t + 1 < tiles ? (t + 1) * BN : -1);
      if (t + 1 < tiles) tile_step(std::integral_constant<int, 1>{}, (t + 1) * BN, t + 2 < tiles ? (t + 2) * BN : -1);
    }
  }

  // ---- epilogue: normalise, transpose the wave's 32 query rows through LDS, coalesced store --------------------
  MSD_LDS char* ost = smem + wave * 32 * kORowBytes;
#pragma unroll
  for (int nq = 0; nq < 2; ++nq) {
    const float l_tot = l_run[nq] + lt[nq][0];  // complete sums: the matrix product runs over all keys of a tile
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const int qrow_l = row0 + nq * 16 + c;
    if (p.lse && g == 0 && qrow_l < row_end)
      p.lse[((long long)b * p.N + n) * p.Sq + (GATHER ? p.tok[qrow_l] : qrow_l)] =
          l_tot > 0.f ? -negm[nq][0] * 0.6931471805599453f + __logf(l_tot) : -INFINITY;
    if constexpr (PAIR) {  // (only a second launch would read it)
      if (!p.ex_idx && g == 0 && qrow_l < row_end)
        p.state[((long long)b * p.N + n) * p.Sq + qrow_l] = l_tot > 0.f ? -negm[nq][0] + __log2f(l_tot) : -INFINITY;
    }
#pragma unroll
    for (int db = 0; db < 8; ++db) {
      typename E::x4 pk;
#pragma unroll
      for (int i = 0; i < 4; ++i) pk[i] = E::from_float(oacc[db][nq][i] * inv);
      *(MSD_LDS typename E::x4*)(ost + (nq * 16 + c) * kORowBytes + (16 * db + 4 * g) * 2) = pk;
    }
  }
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int i = 0; i < 32 * 16 / 64; ++i) {
    const int ch = i * 64 + lane;
    const int row = ch >> 4, c16 = ch & 15;
    const int qrow = row0 + row;
    const i32x2_t lo = *(MSD_LDS const i32x2_t*)(ost + row * kORowBytes + c16 * 16);
    const i32x2_t hi = *(MSD_LDS const i32x2_t*)(ost + row * kORowBytes + c16 * 16 + 8);
    if (qrow < row_end && (!DPAD || c16 * 8 < p.head_dim)) {
      i32x4_t v = {lo[0], lo[1], hi[0], hi[1]};
      const int orow = GATHER ? p.tok[qrow] : qrow;
      *(i32x4_t*)(og + (long long)orow * p.o_ss + c16 * 8) = v;
    }
  }
#endif  // __HIP_DEVICE_COMPILE__
}

template <int DT, int NWAVES = 8, bool PAIR = false, bool GATHER = false, int GEN = 0, bool DPAD = false>
static int launch_fa16(const FaParams& p, hipStream_t stream) {
  constexpr int kLds = 4 * 128 * 256;  // two K and two V stages of 128 keys
  auto kern = fa_fwd16_kernel<DT, NWAVES, PAIR, GATHER, GEN, DPAD>;
  if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kLds) != hipSuccess)
    return MSD_ERR_LAUNCH;
  const long long grid = fa16_grid<GEN, PAIR>(p, NWAVES * 32);
  if (grid > 0x7ffffff0ll) return MSD_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NWAVES * 64), kLds, stream, p);
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

template <int DT, int NWAVES, int QPW, int BN, bool SPARSE, int SCHED, int MODE = 0, bool GATHER = false,
          bool INIT = false, bool PACKED = false>
static int launch_fa(const FaParams& p, hipStream_t stream) {
  using C = FaCfg<DT, NWAVES, QPW, BN, SPARSE>;
  auto kern = fa_fwd_kernel<DT, NWAVES, QPW, BN, SPARSE, SCHED, MODE, GATHER, INIT, PACKED>;
  // per device and idempotent, so it is simply repeated on every launch
  if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, C::kLdsBytes) != hipSuccess)
    return MSD_ERR_LAUNCH;
  const int q_tiles = (p.Sq + C::kBM - 1) / C::kBM;
  const int total = PACKED ? p.N * p.packed_tiles : p.B * p.N * q_tiles;
  const int grid = ((total + 7) / 8) * 8;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(C::kNT), C::kLdsBytes, stream, p);
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

// cumulative lengths (device) -> the [B][4] table of the packed / general entry points, clamped to the tensors
__global__ void varlen_meta_kernel(const int* cu_q, const int* cu_k, int B, int total_q, int total_k, int max_q,
                                   int max_k, int* meta) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= B) return;
  const int q0 = min(max(cu_q[b], 0), total_q), k0 = min(max(cu_k[b], 0), total_k);
  const int lq = min(min(max(cu_q[b + 1] - cu_q[b], 0), total_q - q0), max_q);
  const int lk = min(min(max(cu_k[b + 1] - cu_k[b], 0), total_k - k0), max_k);
  *(i32x4_t*)(meta + 4 * b) = i32x4_t{q0, lq, k0, lk};
}

}  // namespace msd

using namespace msd;

extern "C" {

#ifndef MSD_SHORT_KV
#define MSD_SHORT_KV 384
#endif
constexpr int kCus = 256;  // compute units of the MI355X
constexpr int kShortKv = MSD_SHORT_KV;  // dense calls with at most this many keys run on the 4-wave kernel (see below)
// general mode: query rows (of the longest sequence; packed: of the average one) from which the 8-wave kernel is used
#ifndef MSD_GEN16_MIN_ROWS
#define MSD_GEN16_MIN_ROWS 256
#endif
constexpr int kGen16MinRows = MSD_GEN16_MIN_ROWS;

static int check_common(const void* q, const void* k, const void* v, const void* out, int dtype, int B, int N,
                        int Nkv, int Sq, int Skv, int D, const long long* st, float scale, bool any_head_dim = false) {
  if (!q || !k || !v || !out) return MSD_ERR_BAD_ARG;
  if (B <= 0 || N <= 0 || Nkv <= 0 || Sq <= 0 || Skv <= 0 || N % Nkv != 0) return MSD_ERR_BAD_ARG;
  // the dense entry points take head dims 8, 16, ... 256 (flash_attn_hd.hip); everything else is head_dim 128 only
  if (D != 128 && !(any_head_dim && D > 0 && D <= 256 && (D & 7) == 0)) return MSD_ERR_UNSUPPORTED;
  if (!(scale > 0.f)) return MSD_ERR_UNSUPPORTED;
  if (dtype != MSD_DTYPE_BF16 && dtype != MSD_DTYPE_F16) return MSD_ERR_BAD_ARG;
  // 16-byte vector accesses: every row start must be 16-byte aligned
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) return MSD_ERR_BAD_ARG;
  long long any = 0;
  for (int i = 0; i < 12; ++i) any |= st[i];
  if (any & 7) return MSD_ERR_BAD_ARG;
  // K/V tiles are fetched with 32-bit buffer offsets relative to the (batch, head) base
  if (D == 128 && ((long long)Skv * st[5] * 2 >= (1ll << 31) || (long long)Skv * st[8] * 2 >= (1ll << 31)))
    return MSD_ERR_UNSUPPORTED;
  return MSD_OK;
}

static FaParams make_params(const void* q, const void* k, const void* v, void* out, float* lse, int B, int N, int Nkv,
                            int Sq, int Skv, const long long* st, float scale) {
  FaParams p{};
  p.q = q; p.k = k; p.v = v; p.o = out; p.lse = lse;
  p.q_sb = st[0]; p.q_sn = st[1]; p.q_ss = st[2];
  p.k_sb = st[3]; p.k_sn = st[4]; p.k_ss = st[5];
  p.v_sb = st[6]; p.v_sn = st[7]; p.v_ss = st[8];
  p.o_sb = st[9]; p.o_sn = st[10]; p.o_ss = st[11];
  p.B = B; p.N = N; p.Nkv = Nkv; p.Sq = Sq; p.Skv = Skv;
  p.scale = scale;
  p.scale_log2 = scale * 1.4426950408889634f;
  return p;
}

int mindiesd_block_sparse_attention_fwd(const void* q, const void* k, const void* v, void* out, float* lse, int dtype,
                                        int B, int N, int Nkv, int Sq, int Skv, int D, long long q_sb, long long q_sn,
                                        long long q_ss, long long k_sb, long long k_sn, long long k_ss,
                                        long long v_sb, long long v_sn, long long v_ss, long long o_sb,
                                        long long o_sn, long long o_ss, float scale, const int* blk_idx,
                                        const int* blk_cnt, int kb_stride, const int* order, hipStream_t stream) {
  const long long st[12] = {q_sb, q_sn, q_ss, k_sb, k_sn, k_ss, v_sb, v_sn, v_ss, o_sb, o_sn, o_ss};
  const int rc = check_common(q, k, v, out, dtype, B, N, Nkv, Sq, Skv, D, st, scale);
  if (rc != MSD_OK) return rc;
  if (!blk_idx || !blk_cnt || kb_stride <= 0) return MSD_ERR_BAD_ARG;
  FaParams p = make_params(q, k, v, out, lse, B, N, Nkv, Sq, Skv, st, scale);
  p.blk_idx = blk_idx; p.blk_cnt = blk_cnt; p.kb_stride = kb_stride; p.order = order;
  p.QB = (Sq + 127) / 128;
  // one query block per workgroup, 64-key sub-tiles, two workgroups per CU
  if (dtype == MSD_DTYPE_BF16) return launch_fa<MSD_DTYPE_BF16, 4, 32, 64, true, 1>(p, stream);
  return launch_fa<MSD_DTYPE_F16, 4, 32, 64, true, 1>(p, stream);
}

// The same with the query side addressed through a table: query position i (the position the block lists and the
// rows of k and v refer to) is row token_order[i] of q and of out (S entries, every row exactly once).  With k and
// v permuted and q, out left in their original order this saves the permuted copy of q and the inverse
// permutation of the output.
int mindiesd_block_sparse_attention_gather_fwd(const void* q, const void* k, const void* v, void* out, float* lse,
                                               int dtype, int B, int N, int Nkv, int S, int D, long long q_sb,
                                               long long q_sn, long long q_ss, long long k_sb, long long k_sn,
                                               long long k_ss, long long v_sb, long long v_sn, long long v_ss,
                                               long long o_sb, long long o_sn, long long o_ss, float scale,
                                               const int* blk_idx, const int* blk_cnt, int kb_stride,
                                               const int* token_order, hipStream_t stream) {
  const long long st[12] = {q_sb, q_sn, q_ss, k_sb, k_sn, k_ss, v_sb, v_sn, v_ss, o_sb, o_sn, o_ss};
  const int rc = check_common(q, k, v, out, dtype, B, N, Nkv, S, S, D, st, scale);
  if (rc != MSD_OK) return rc;
  if (!blk_idx || !blk_cnt || kb_stride <= 0 || !token_order) return MSD_ERR_BAD_ARG;
  FaParams p = make_params(q, k, v, out, lse, B, N, Nkv, S, S, st, scale);
  p.blk_idx = blk_idx; p.blk_cnt = blk_cnt; p.kb_stride = kb_stride; p.tok = token_order;
  p.QB = (S + 127) / 128;
  if (dtype == MSD_DTYPE_BF16) return launch_fa<MSD_DTYPE_BF16, 4, 32, 64, true, 1, 0, true>(p, stream);
  return launch_fa<MSD_DTYPE_F16, 4, 32, 64, true, 1, 0, true>(p, stream);
}

// Block-sparse attention driven by the int8 mask itself, over paired query blocks (bsa_pair.hip): pairing + lists,
// then one 256-row workgroup per pair: the key blocks both partners selected (the dense kernel's inner loop), then
// what only one of them selected, with that partner's four waves, the running softmax going on.  Same result as
// mindiesd_block_sparse_attention_fwd on the lists of the mask up to the order of accumulation.
size_t mindiesd_block_sparse_attention_paired_workspace_size(int B, int N, int Sq, int Skv) {
  if (B <= 0 || N <= 0 || Sq <= 0 || Skv <= 0) return 0;
  const long long BN = (long long)B * N;
  const int QB = (Sq + 127) / 128, KB = (Skv + 127) / 128;
  return bsa_pair_ints(BN, QB, KB) * sizeof(int) + (size_t)BN * Sq * sizeof(float);
}

int mindiesd_block_sparse_attention_paired_fwd(const void* q, const void* k, const void* v, void* out, float* lse,
                                               int dtype, int B, int N, int Nkv, int Sq, int Skv, int D,
                                               long long q_sb, long long q_sn, long long q_ss, long long k_sb,
                                               long long k_sn, long long k_ss, long long v_sb, long long v_sn,
                                               long long v_ss, long long o_sb, long long o_sn, long long o_ss,
                                               float scale, const signed char* mask, const int* token_order,
                                               void* workspace, size_t ws_bytes, hipStream_t stream) {
  const long long st[12] = {q_sb, q_sn, q_ss, k_sb, k_sn, k_ss, v_sb, v_sn, v_ss, o_sb, o_sn, o_ss};
  int rc = check_common(q, k, v, out, dtype, B, N, Nkv, Sq, Skv, D, st, scale);
  if (rc != MSD_OK) return rc;
  if (!mask || !workspace || ((uintptr_t)workspace & 15)) return MSD_ERR_BAD_ARG;
  if (token_order && Sq != Skv) return MSD_ERR_BAD_ARG;
  const int QB = (Sq + 127) / 128, KB = (Skv + 127) / 128;
  if (!bsa_pair_supported(QB, KB)) return MSD_ERR_UNSUPPORTED;
  if (ws_bytes < mindiesd_block_sparse_attention_paired_workspace_size(B, N, Sq, Skv)) return MSD_ERR_WORKSPACE;
  const long long BN = (long long)B * N;
  BsaPairTables t;
  float* state = (float*)workspace;  // first, so that it stays 16-byte aligned
  rc = bsa_build_pairs(mask, BN, QB, KB, (int*)(state + BN * Sq), &t, stream);
  if (rc != MSD_OK) return rc;
  FaParams p = make_params(q, k, v, out, lse, B, N, Nkv, Sq, Skv, st, scale);
  p.tok = token_order;
  p.QB = QB;
  p.state = state;
  // one workgroup per pair: the shared list with all eight waves, then each partner's own list with its four
  p.pairs = t.pairs; p.NP = t.NP;
  p.blk_idx = t.sh_idx; p.blk_cnt = t.sh_cnt; p.kb_stride = KB;
#if !defined(MSD_BSA_TWO_PASS)
  p.ex_idx = t.ex_idx; p.ex_cnt = t.ex_cnt;
#endif
  if (dtype == MSD_DTYPE_BF16)
    rc = token_order ? launch_fa16<MSD_DTYPE_BF16, 8, true, true>(p, stream) : launch_fa16<MSD_DTYPE_BF16, 8, true, false>(p, stream);
  else
    rc = token_order ? launch_fa16<MSD_DTYPE_F16, 8, true, true>(p, stream) : launch_fa16<MSD_DTYPE_F16, 8, true, false>(p, stream);
  if (rc != MSD_OK) return rc;
#if !defined(MSD_BSA_TWO_PASS)
  return MSD_OK;
#endif
  // (two launches: pass 2, one workgroup per query block over its exclusive list, resuming from pass 1)
  p.ex_idx = nullptr; p.ex_cnt = nullptr;
  p.blk_idx = t.ex_idx; p.blk_cnt = t.ex_cnt; p.init_cnt = t.init_cnt;
  if (dtype == MSD_DTYPE_BF16)
    return token_order ? launch_fa<MSD_DTYPE_BF16, 4, 32, 64, true, 1, 0, true, true>(p, stream)
                       : launch_fa<MSD_DTYPE_BF16, 4, 32, 64, true, 1, 0, false, true>(p, stream);
  return token_order ? launch_fa<MSD_DTYPE_F16, 4, 32, 64, true, 1, 0, true, true>(p, stream)
                     : launch_fa<MSD_DTYPE_F16, 4, 32, 64, true, 1, 0, false, true>(p, stream);
}

// True when B x N x ceil(Sq / 256) workgroups of 256 rows would fill the chip badly (see mindiesd_flash_attention_fwd).
static bool prefers_half_tiles(int B, int N, int Sq) {
  const long long tiles256 = (long long)B * N * ((Sq + 255) / 256);
  bool half_tiles = 2 * tiles256 <= kCus || (tiles256 > kCus && 2 * tiles256 <= 3 * kCus);
  if (const char* rows = getenv("MINDIESD_DENSE_TILE_ROWS")) {
    if (atoi(rows) == 256) half_tiles = false;
    if (atoi(rows) == 128) half_tiles = true;
  }
  return half_tiles;
}

int mindiesd_flash_attention_fwd(const void* q, const void* k, const void* v, void* out, float* lse, int dtype,
                                 int B, int N, int Nkv, int Sq, int Skv, int D, long long q_sb, long long q_sn,
                                 long long q_ss, long long k_sb, long long k_sn, long long k_ss, long long v_sb,
                                 long long v_sn, long long v_ss, long long o_sb, long long o_sn, long long o_ss,
                                 float scale, hipStream_t stream) {
  const long long st[12] = {q_sb, q_sn, q_ss, k_sb, k_sn, k_ss, v_sb, v_sn, v_ss, o_sb, o_sn, o_ss};
  const int rc = check_common(q, k, v, out, dtype, B, N, Nkv, Sq, Skv, D, st, scale, true);
  if (rc != MSD_OK) return rc;
  FaParams p = make_params(q, k, v, out, lse, B, N, Nkv, Sq, Skv, st, scale);
  // Grids of 256-row workgroups that fill the 256 CUs badly - at most half of them busy, or a second round for at
  // most half of them - run as 128-row workgroups of four waves, two to a CU (head dims 128 and up to 64).
  // MINDIESD_DENSE_TILE_ROWS = 256 or 128 in the environment overrides the choice (the tests reach both kinds of
  // kernel at every size that way).
  const bool half_tiles = prefers_half_tiles(B, N, Sq);
  if (D == 64 && fa16_d64_supported(p)) return launch_fa16_d64(p, dtype, stream, 0, half_tiles ? 128 : 256);
  // Head dims between 64 and 128 run as head_dim 128 on the 16x16x32 kernel (the part of the matrix work spent on
  // the padding costs less than the general kernel's staging through registers: 72 -> 580 vs 730 TFLOP/s of real
  // work, 112 -> 800 vs 1130), when the 256-byte rows the DMA fetches stay inside the kernel's 32-bit offsets.
  if (D > 64 && D < 128 && (long long)Skv * k_ss * 2 < 0x7fffff00ll &&
      (long long)Skv * v_ss * 2 < 0x7fffff00ll) {  // (below the offset that stands for "no data" in the kernel)
    p.head_dim = D;
    if (dtype == MSD_DTYPE_BF16) return launch_fa16<MSD_DTYPE_BF16, 8, false, false, 0, true>(p, stream);
    return launch_fa16<MSD_DTYPE_F16, 8, false, false, 0, true>(p, stream);
  }
  // (the rule for short key sequences below is head_dim 128's alone: at the other widths the alternative is the
  // general kernel, which these beat at 77 keys already)
  if (D > 128 && fa16_d256_supported(p)) return launch_fa16_d256(p, dtype, D, stream);
  if (D < 64 && fa16_d64_supported(p)) return launch_fa16_d64_padded(p, dtype, D, stream, 0, half_tiles ? 128 : 256);
  if (D != 128) return launch_fa_hd(p, dtype, D, stream);
  // A few key tiles per query tile (cross attention over a short text): the launch is mostly reading Q and writing O,
  // and two 4-wave workgroups per CU overlap one's memory phases with the other's tiles better than one 8-wave
  // workgroup does (75600 queries x 40 heads: 0.42 vs 0.53 ms at 77 keys, 0.62 vs 0.70 at 226, equal at 512).
  // The same 4-wave kernel takes the grids that fill the chip badly (half_tiles above): it reaches 86 % of the 8-wave
  // kernel's rate on a full chip, and B x N = 16: S 1024 / 1536 / 2048 31 -> 25, 43 -> 35, 56 -> 46 us, S 4608 (288
  // workgroups of 256 rows) 218 -> 206 us; 24 heads at S 3072: 152 -> 139 us.  (In between - 129 .. 256 workgroups -
  // and from 385 on the 8-wave kernel is faster.)
  if (Skv <= kShortKv || half_tiles) {
    if (dtype == MSD_DTYPE_BF16) return launch_fa<MSD_DTYPE_BF16, 4, 32, 64, false, 1, 1>(p, stream);
    return launch_fa<MSD_DTYPE_F16, 4, 32, 64, false, 1, 1>(p, stream);
  }
  if (dtype == MSD_DTYPE_BF16) return launch_fa16<MSD_DTYPE_BF16>(p, stream);
  return launch_fa16<MSD_DTYPE_F16>(p, stream);
}

// Block-sparse attention with an optional causal mask inside the selected blocks (queries and keys of equal
// length: key j is visible to query i iff j <= i).
int mindiesd_ada_block_sparse_attention_fwd(const void* q, const void* k, const void* v, void* out, int dtype, int B,
                                            int N, int Nkv, int S, int D, long long q_sb, long long q_sn,
                                            long long q_ss, long long k_sb, long long k_sn, long long k_ss,
                                            long long v_sb, long long v_sn, long long v_ss, long long o_sb,
                                            long long o_sn, long long o_ss, float scale, const int* blk_idx,
                                            const int* blk_cnt, int kb_stride, int causal, hipStream_t stream) {
  const long long st[12] = {q_sb, q_sn, q_ss, k_sb, k_sn, k_ss, v_sb, v_sn, v_ss, o_sb, o_sn, o_ss};
  const int rc = check_common(q, k, v, out, dtype, B, N, Nkv, S, S, D, st, scale);
  if (rc != MSD_OK) return rc;
  if (!blk_idx || !blk_cnt || kb_stride <= 0) return MSD_ERR_BAD_ARG;
  FaParams p = make_params(q, k, v, out, nullptr, B, N, Nkv, S, S, st, scale);
  p.blk_idx = blk_idx; p.blk_cnt = blk_cnt; p.kb_stride = kb_stride;
  p.QB = (S + 127) / 128;
  p.causal = causal ? 1 : 0;
  if (!causal) {
    if (dtype == MSD_DTYPE_BF16) return launch_fa<MSD_DTYPE_BF16, 4, 32, 64, true, 1>(p, stream);
    return launch_fa<MSD_DTYPE_F16, 4, 32, 64, true, 1>(p, stream);
  }
  if (dtype == MSD_DTYPE_BF16) return launch_fa<MSD_DTYPE_BF16, 4, 32, 64, true, 1, 1>(p, stream);
  return launch_fa<MSD_DTYPE_F16, 4, 32, 64, true, 1, 1>(p, stream);
}

// Block-sparse attention with per-sequence lengths: seq_meta [B][4] = {first query token, query count, first key
// token, key count} as in mindiesd_flash_attention_general_fwd.  With batch strides 0 the tensors are packed
// (token, head, dim) arrays; with ordinary batch strides and first tokens 0 it gives every batch entry its own
// length inside [B][N][S][128] tensors.  Sq / Skv are the longest counts; the lists are per (batch, head, query
// block of that length).  Query rows past a sequence's count are not written.
int mindiesd_block_sparse_attention_general_fwd(const void* q, const void* k, const void* v, void* out, float* lse,
                                                int dtype, int B, int N, int Nkv, int Sq, int Skv, int D,
                                                long long q_sb, long long q_sn, long long q_ss, long long k_sb,
                                                long long k_sn, long long k_ss, long long v_sb, long long v_sn,
                                                long long v_ss, long long o_sb, long long o_sn, long long o_ss,
                                                float scale, const int* blk_idx, const int* blk_cnt, int kb_stride,
                                                const int* seq_meta, int lse_token_major, int causal,
                                                hipStream_t stream) {
  const long long st[12] = {q_sb, q_sn, q_ss, k_sb, k_sn, k_ss, v_sb, v_sn, v_ss, o_sb, o_sn, o_ss};
  const int rc = check_common(q, k, v, out, dtype, B, N, Nkv, Sq, Skv, D, st, scale);
  if (rc != MSD_OK) return rc;
  if (!blk_idx || !blk_cnt || kb_stride <= 0) return MSD_ERR_BAD_ARG;
  FaParams p = make_params(q, k, v, out, lse, B, N, Nkv, Sq, Skv, st, scale);
  p.blk_idx = blk_idx; p.blk_cnt = blk_cnt; p.kb_stride = kb_stride;
  p.QB = (Sq + 127) / 128;
  p.seq_meta = seq_meta; p.lse_token_major = lse_token_major ? 1 : 0;
  p.causal = causal ? 1 : 0;
  if (dtype == MSD_DTYPE_BF16) return launch_fa<MSD_DTYPE_BF16, 4, 32, 64, true, 1, 1>(p, stream);
  return launch_fa<MSD_DTYPE_F16, 4, 32, 64, true, 1, 1>(p, stream);
}

// Dense attention with the options the plain entry point leaves out: packed variable-length sequences,
// a causal mask aligned to the bottom-right corner, a boolean attention mask.  Rows whose keys are all
// masked give zeros.
int mindiesd_flash_attention_general_fwd(const void* q, const void* k, const void* v, void* out, float* lse, int dtype,
                                         int B, int N, int Nkv, int Sq, int Skv, int D, long long q_sb, long long q_sn,
                                         long long q_ss, long long k_sb, long long k_sn, long long k_ss,
                                         long long v_sb, long long v_sn, long long v_ss, long long o_sb,
                                         long long o_sn, long long o_ss, float scale, const int* seq_meta, int causal,
                                         const unsigned char* mask, long long m_sb, long long m_sn, long long m_sq,
                                         hipStream_t stream) {
  const long long st[12] = {q_sb, q_sn, q_ss, k_sb, k_sn, k_ss, v_sb, v_sn, v_ss, o_sb, o_sn, o_ss};
  const int rc = check_common(q, k, v, out, dtype, B, N, Nkv, Sq, Skv, D, st, scale, true);
  if (rc != MSD_OK) return rc;
  if (seq_meta && (mask || lse)) return MSD_ERR_UNSUPPORTED;  // packed sequences: neither mask nor lse layout defined
  // m_sq == 0: one mask row shared by all queries (a key-padding mask expanded over the query dimension)
  if (mask && (m_sb < 0 || m_sn < 0 || (m_sq != 0 && m_sq < Skv))) return MSD_ERR_BAD_ARG;
  FaParams p = make_params(q, k, v, out, lse, B, N, Nkv, Sq, Skv, st, scale);
  p.seq_meta = seq_meta; p.causal = causal ? 1 : 0;
  p.mask = mask; p.m_sb = m_sb; p.m_sn = m_sn; p.m_sq = m_sq;
  // one mask row for all queries, no other option: the key-mask instantiations of the 16x16x32 kernels
  const bool key_mask = mask && m_sq == 0 && !causal && !seq_meta;
  const bool long_rows = Sq >= kGen16MinRows && (D != 128 || Skv > kShortKv);
  if (long_rows && (!mask || key_mask)) {  // head dims up to 128 on the 16x16x32 kernels, padded where need be
    const int gen = key_mask ? 3 : 1;
    if (D == 64 && fa16_d64_supported(p)) return launch_fa16_d64(p, dtype, stream, gen);
    if (D < 64 && fa16_d64_supported(p)) return launch_fa16_d64_padded(p, dtype, D, stream, gen);
    if (D > 64 && D < 128 && (long long)Skv * k_ss * 2 < 0x7fffff00ll && (long long)Skv * v_ss * 2 < 0x7fffff00ll) {
      p.head_dim = D;
      if (dtype == MSD_DTYPE_BF16)
        return key_mask ? launch_fa16<MSD_DTYPE_BF16, 8, false, false, 3, true>(p, stream)
                        : launch_fa16<MSD_DTYPE_BF16, 8, false, false, 1, true>(p, stream);
      return key_mask ? launch_fa16<MSD_DTYPE_F16, 8, false, false, 3, true>(p, stream)
                      : launch_fa16<MSD_DTYPE_F16, 8, false, false, 1, true>(p, stream);
    }
    if (D > 128 && fa16_d256_supported(p)) return launch_fa16_d256(p, dtype, D, stream, gen);
  }
  if (D != 128) return launch_fa_hd(p, dtype, D, stream);
  if (key_mask && long_rows) {
    if (dtype == MSD_DTYPE_BF16) return launch_fa16<MSD_DTYPE_BF16, 8, false, false, 3>(p, stream);
    return launch_fa16<MSD_DTYPE_F16, 8, false, false, 3>(p, stream);
  }
  if (mask) {
    if (dtype == MSD_DTYPE_BF16) return launch_fa<MSD_DTYPE_BF16, 4, 32, 64, false, 1, 2>(p, stream);
    return launch_fa<MSD_DTYPE_F16, 4, 32, 64, false, 1, 2>(p, stream);
  }
  // Without a mask, long sequences run on the 16x16x32 kernel's general instantiation (256-row tiles); short ones
  // fill the chip better with the 128-row tiles of the 4-wave kernel, and so do causal calls whose grid of 256-row
  // workgroups would fill it badly (the rule of mindiesd_flash_attention_fwd; B x N 16: S 1024 / 2048 32 -> 25,
  // 54 -> 42 us, 48 heads at S 2048 82 -> 75 us).
  if (long_rows && !(causal && !seq_meta && prefers_half_tiles(B, N, Sq))) {
    if (dtype == MSD_DTYPE_BF16) return launch_fa16<MSD_DTYPE_BF16, 8, false, false, 1>(p, stream);
    return launch_fa16<MSD_DTYPE_F16, 8, false, false, 1>(p, stream);
  }
  if (dtype == MSD_DTYPE_BF16) return launch_fa<MSD_DTYPE_BF16, 4, 32, 64, false, 1, 1>(p, stream);
  return launch_fa<MSD_DTYPE_F16, 4, 32, 64, false, 1, 1>(p, stream);
}

// cu_seqlens_q / cu_seqlens_k (device, int32, B + 1 entries each) -> seq_meta [B][4] for the two entry points that
// take it, without a host read-back: first tokens clamped to the tensors, counts to what is left behind them and to
// max_q / max_k (pass the token totals when the longest sequence is not known).
int mindiesd_varlen_meta(const int* cu_seqlens_q, const int* cu_seqlens_k, int B, int total_q, int total_k, int max_q,
                         int max_k, int* seq_meta, hipStream_t stream) {
  if (!cu_seqlens_q || !cu_seqlens_k || !seq_meta || B <= 0 || total_q < 0 || total_k < 0 || max_q < 0 || max_k < 0)
    return MSD_ERR_BAD_ARG;
  if ((uintptr_t)seq_meta & 15) return MSD_ERR_BAD_ARG;
  hipLaunchKernelGGL(varlen_meta_kernel, dim3((B + 255) / 256), dim3(256), 0, stream, cu_seqlens_q, cu_seqlens_k, B,
                     total_q, total_k, max_q, max_k, seq_meta);
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

// Packed sequences whose lengths only the device knows: q, out [total_q][N][D], k, v [total_k][Nkv][D] (token, head
// strides), seq_meta as above with B sequences.  The grid is sized from the token total - at most
// ceil(total_q / 128) + B query tiles per head exist whatever the lengths are - and every workgroup looks its
// sequence up in the table, where mindiesd_flash_attention_general_fwd with Sq = total_q as the only known bound
// launches B x ceil(total_q / 128) workgroups per head, nearly all of which return at once.  The query counts of the
// table must not add up to more than total_q (tiles beyond the bound are not computed).
int mindiesd_flash_attention_packed_fwd(const void* q, const void* k, const void* v, void* out, int dtype, int B, int N,
                                        int Nkv, int total_q, int total_k, int D, long long q_sn, long long q_ss,
                                        long long k_sn, long long k_ss, long long v_sn, long long v_ss, long long o_sn,
                                        long long o_ss, float scale, const int* seq_meta, int causal,
                                        hipStream_t stream) {
  const long long st[12] = {0, q_sn, q_ss, 0, k_sn, k_ss, 0, v_sn, v_ss, 0, o_sn, o_ss};
  const int rc = check_common(q, k, v, out, dtype, B, N, Nkv, total_q, total_k, D, st, scale, true);
  if (rc != MSD_OK) return rc;
  if (!seq_meta) return MSD_ERR_BAD_ARG;
  FaParams p = make_params(q, k, v, out, nullptr, B, N, Nkv, total_q, total_k, st, scale);
  p.seq_meta = seq_meta; p.causal = causal ? 1 : 0;
  const long long tiles = ((long long)total_q + 127) / 128 + B;
  if (tiles * N > 0x7ffffff0ll) return MSD_ERR_UNSUPPORTED;
  p.packed_tiles = (int)tiles;
  // long sequences on average: the 8-wave kernels, whose tiles are 256 rows
  const bool long_rows = total_q / B >= kGen16MinRows && (D != 128 || total_k / B > kShortKv);
  if (D <= 64 && long_rows && fa16_d64_supported(p)) {
    p.packed_tiles = (int)(((long long)total_q + 255) / 256 + B);
    return D == 64 ? launch_fa16_d64(p, dtype, stream, 2) : launch_fa16_d64_padded(p, dtype, D, stream, 2);
  }
  if (D > 64 && D < 128 && long_rows && (long long)total_k * k_ss * 2 < 0x7fffff00ll &&
      (long long)total_k * v_ss * 2 < 0x7fffff00ll) {
    p.packed_tiles = (int)(((long long)total_q + 255) / 256 + B);
    p.head_dim = D;
    if (dtype == MSD_DTYPE_BF16) return launch_fa16<MSD_DTYPE_BF16, 8, false, false, 2, true>(p, stream);
    return launch_fa16<MSD_DTYPE_F16, 8, false, false, 2, true>(p, stream);
  }
  if (D > 128 && long_rows && (long long)total_k * k_ss * 2 < 0x7fffff00ll && (long long)total_k * v_ss * 2 < 0x7fffff00ll) {
    p.packed_tiles = (int)(((long long)total_q + 127) / 128 + B);  // (this kernel's tiles are 128 rows)
    return launch_fa16_d256(p, dtype, D, stream, 2);
  }
  if (D != 128) return launch_fa_hd(p, dtype, D, stream);
  if (long_rows) {
    p.packed_tiles = (int)(((long long)total_q + 255) / 256 + B);
    if (dtype == MSD_DTYPE_BF16) return launch_fa16<MSD_DTYPE_BF16, 8, false, false, 2>(p, stream);
    return launch_fa16<MSD_DTYPE_F16, 8, false, false, 2>(p, stream);
  }
  if (dtype == MSD_DTYPE_BF16) return launch_fa<MSD_DTYPE_BF16, 4, 32, 64, false, 1, 1, false, false, true>(p, stream);
  return launch_fa<MSD_DTYPE_F16, 4, 32, 64, false, 1, 1, false, false, true>(p, stream);
}

}  // extern "C"
