// Flash-attention forward for gfx950 (MI355X) at head dims above 128, up to 256: bf16/fp16; dense, and (from 256
// query rows on) causal, packed variable-length sequences and key-padding masks.
//
// The reference's fused dense ops (mindiesd/layers/flash_attn/prompt_flash_attn.py:48, fused_attn_score.py:48,
// csrc/plugin/la.cpp:27-58) take whatever head_dim the model has; the general kernel of flash_attn_hd.hip covers these
// widths with a plain data path (tiles through registers).  This file carries the design of fa_fwd16_kernel
// (flash_attn_fwd.hip, head_dim 128) over to rows of 512 bytes:
//   * 8 waves x 16 query rows per workgroup (one 16-query column block per wave: the output accumulators of a wider
//     block would not leave room for two waves per SIMD), 64-key tiles, K and V tiles staged by LDS-DMA (two stages each);
//   * the transposed problem S^T = K Q^T, O^T += V^T P^T on the 16x16x32 matrix instruction, Q^T resident with
//     scale * log2(e) folded in, P^T straight from the score accumulators, V^T by the transposing LDS read;
//   * lazily moved reference maximum seeded into the score accumulators, row sums on the matrix pipe (ones x P^T).
// Head dims between 128 and 256 are computed as 256: the query operand is zero from the real head_dim on, and the
// lanes that would stage the 16-byte chunks of K and V past it request an offset beyond the buffers' range, for which
// the DMA writes zeros without touching memory; output columns past the head_dim are not stored.
//
// Register tiles, with c = lane % 16 and g = lane / 16:
//     S^T block (16 keys x 16 queries):  A = K rows 16*kb + c, head_dim 32*ks + 8*g .. +8 (one 16-byte LDS read),
//                                        B = Q^T resident (query c, same head_dim slice);
//                                        the lane receives keys 16*kb + 4*g + i (i < 4) of query c
//     O^T block (16 dims x 16 queries):  B = P^T of 32 keys straight from two S^T blocks (slot 8*g + t holds key
//                                        32*j + 4*g + t for t < 4 and key 32*j + 16 + 4*g + t - 4 for t >= 4),
//                                        A = V^T in the same slot order from two transposing LDS reads
// LDS: rows of 512 bytes.  K stages at 0 and 32 KiB: 16-byte chunk p of row r sits at chunk p ^ (r & 15) (the XOR
// stays inside a 256-byte half), so the 16 rows one quarter-wave reads cover all banks.  V stages at 64 and 96 KiB:
// 32-byte chunk p of row r sits at chunk p ^ (r & 7).
#include <type_traits>
#include <utility>

#include "common.hpp"
#include "fa_params.hpp"

namespace msd {

#if defined(__HIP_DEVICE_COMPILE__)
namespace d256 {
template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>)
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}
}  // namespace d256
#endif

constexpr int kD256Waves = 8, kD256BN = 64, kD256RowBytes = 512;
constexpr int kD256TileBytes = kD256BN * kD256RowBytes;  // 32 KiB
constexpr int kD256Lds = 4 * kD256TileBytes;              // two K and two V stages
#ifndef FA16_D256_AHEAD
#define FA16_D256_AHEAD 3
#endif
constexpr int kD256Ahead = FA16_D256_AHEAD;               // K operand groups requested ahead of their use

// GEN as in fa_fwd16_kernel (flash_attn_fwd.hip): 0 dense; 1 per-sequence lengths (p.seq_meta) and / or causal;
// 2 the same with the packed tile numbering (128-row tiles here); 3 a boolean mask row shared by all queries.
template <int DT, bool DPAD, int GEN = 0>
__global__ __launch_bounds__(kD256Waves * 64, 1) void fa_fwd16_d256_kernel(const FaParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  using namespace d256;
  using E = Elem<DT>;
  using T = typename E::type;
  using X8 = typename E::x8;
  constexpr int NWAVES = kD256Waves, BN = kD256BN, kBM = NWAVES * 16, kRowBytes = kD256RowBytes;
  constexpr int kTileBytes = kD256TileBytes, kORowBytes = kRowBytes + 8;
  static_assert(NWAVES * 16 * kORowBytes <= kD256Lds, "the output staging reuses the tile stages");
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  MSD_LDS char* smem = (MSD_LDS char*)smem_raw;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 15;
  const int g = lane >> 4;

  constexpr bool gen = GEN != 0, keymask = GEN == 3;
  int bn, qt, b, n, Sq, Skv;
  long long q_tok0, k_tok0;  // general mode: first token of the sequence in packed tensors
  if (!fa16_find_work<GEN, false>(p, kBM, bn, qt, b, n, Sq, Skv, q_tok0, k_tok0)) return;
  const int nkv = n / (p.N / p.Nkv);
  const int row0 = qt * kBM + wave * 16;  // first query row of this wave
  const int hd = DPAD ? p.head_dim : 256;

  const T* qg = (const T*)p.q + b * p.q_sb + n * p.q_sn + q_tok0 * p.q_ss;
  const T* kg = (const T*)p.k + b * p.k_sb + nkv * p.k_sn + k_tok0 * p.k_ss;
  const T* vg = (const T*)p.v + b * p.v_sb + nkv * p.v_sn + k_tok0 * p.v_ss;
  T* og = (T*)p.o + b * p.o_sb + n * p.o_sn + q_tok0 * p.o_ss;

  // ---- Q^T operand, resident: lane (c, g) holds query c, head_dim 32*ks + 8*g .. +8 --------------------------
  X8 qf[8];
  {
    const int qrow = row0 + c;
    const bool ok = qrow < Sq;
    const T* src = qg + (long long)(ok ? qrow : 0) * p.q_ss + 8 * g;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      const bool in = ok && 32 * ks + 8 * g < hd;  // (a chunk of 8 lies wholly inside or outside)
      X8 v = in ? *(const X8*)(src + 32 * ks) : X8{0};
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = E::from_float((float)v[j] * p.scale_log2);
      qf[ks] = v;
    }
  }

  f32x4_t oacc[16];
  float l_run = 0.f;
  // Row sums come off the matrix pipe: ones x P^T gives every lane the sum of its query column over the 64 keys of a
  // tile.  lt holds the sums of the tile before; they are added to l_run at the start of the next softmax, before a
  // rescale, when the matrix results have long landed.
  f32x4_t lt = f32x4_t{0.f, 0.f, 0.f, 0.f};
  X8 ones;
#pragma unroll
  for (int j = 0; j < 8; ++j) ones[j] = E::from_float(1.f);
  f32x4_t negm = f32x4_t{0.f, 0.f, 0.f, 0.f};  // minus the reference maximum (log2 units), seeds an accumulator
#pragma unroll
  for (int db = 0; db < 16; ++db) oacc[db] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // ---- global -> LDS staging (LDS-DMA; swizzles applied on the global side) -------------------------------
  // One instruction moves 2 rows of 512 bytes; a wave issues four per operand and tile (rows 2*wave.. and 16, 32, 48
  // below: the same swizzles, so one per-lane offset per operand serves all four).  Keys past the end of the
  // sequence lie outside the descriptors' range and read as zeros.
  // (a sequence without keys exposes nothing: every row reads as zeros and no tile is computed)
  const int k_range = gen && Skv <= 0 ? 0 : (int)(((long long)(Skv - 1) * p.k_ss + hd) * 2);
  const int v_range = gen && Skv <= 0 ? 0 : (int)(((long long)(Skv - 1) * p.v_ss + hd) * 2);
  const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)kg, 0, k_range, 0x00020000);
  const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)vg, 0, v_range, 0x00020000);
  const int k_row_bytes = (int)p.k_ss * 2, v_row_bytes = (int)p.v_ss * 2;
  int k_voff, v_voff;
  {
    const int row = 2 * wave + (lane >> 5);
    const int pc = lane & 31;  // physical 16-byte chunk this lane fills
    const int kc = pc ^ (row & 15), vc = (((pc >> 1) ^ (row & 7)) << 1) | (pc & 1);  // logical chunks of the row
    k_voff = row * k_row_bytes + (kc << 4);
    v_voff = row * v_row_bytes + (vc << 4);
    if constexpr (DPAD) {  // chunks past the head_dim: an offset beyond every range, the DMA writes zeros for them
      if (kc * 8 >= hd) k_voff = 0x7ffffff0;
      if (vc * 8 >= hd) v_voff = 0x7ffffff0;
    }
  }
  auto load_tile = [&](int key0, int stage) {
    MSD_LDS char* kb = smem + stage * kTileBytes;
    MSD_LDS char* vb = smem + (2 + stage) * kTileBytes;
#pragma unroll
    for (int i = 0; i < 32 / NWAVES; ++i) {
      const int grp = i * NWAVES + wave;  // 2-row group of the tile
      __builtin_amdgcn_raw_ptr_buffer_load_lds(k_rsrc, (MSD_LDS void*)(kb + grp * 1024), 16, k_voff,
                                               (key0 + i * 2 * NWAVES) * k_row_bytes, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(v_rsrc, (MSD_LDS void*)(vb + grp * 1024), 16, v_voff,
                                               (key0 + i * 2 * NWAVES) * v_row_bytes, 0, 0);
    }
  };

  // per-lane parts of the LDS read addresses
  // K operand: row 16*kb + c, 16-byte chunk (4*ks + g) ^ c (ks >= 4: the second 256-byte half of the row)
  unsigned k_lds[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) k_lds[ks] = (unsigned)(uintptr_t)smem + c * kRowBytes + (((4 * ks + g) ^ c) << 4);
  // V^T operand: the lane points at key 4*g + c/4 (+32*j, +16), 8 bytes at 8*(c%4) of 32-byte chunk db ^ (key & 7)
  // (db >= 8: the second 256-byte half of the row)
  unsigned v_lds[8];
  {
    const int key = 4 * g + (c >> 2);
#pragma unroll
    for (int db = 0; db < 8; ++db)
      v_lds[db] = (unsigned)(uintptr_t)smem + 2 * kTileBytes + key * kRowBytes + ((db ^ (key & 7)) << 5) + 8 * (c & 3);
  }

  // causal: query i sees keys <= i + causal_shift; the last row of this workgroup bounds the tiles it walks
  const int causal_shift = Skv - Sq;
  const bool causal = gen && !keymask && p.causal;  // (with a key mask: neither causal nor per-sequence lengths)
  const int kv_lim = causal ? max(0, min(Skv, qt * kBM + kBM + causal_shift)) : Skv;
  const int tiles = (kv_lim + BN - 1) / BN;
  load_tile(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  __syncthreads();
  bool first = true;

  // ---- key mask (GEN 3): words of visible keys of the current 64-key tile; bit l of word j = key 4 * l + j (l < 16) --
  // (see fa_fwd16_kernel: the bytes of the next tile are fetched during the second product and reduced to scalar words)
  unsigned kvis[4] = {0xffffu, 0xffffu, 0xffffu, 0xffffu};
  unsigned kraw = 0;  // the lane's four mask bytes of the tile that comes next (lanes 0 .. 15)
  const unsigned char* mask_g = nullptr;
  if constexpr (keymask) mask_g = p.mask + b * p.m_sb + n * p.m_sn;
  auto mask_request = [&](int key0) __attribute__((always_inline)) {  // the load only
    if constexpr (keymask) {
      kraw = 0;
      const int k4 = key0 + 4 * (lane & 15);
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
        kvis[j] = (unsigned)__builtin_amdgcn_ballot_w64(lane < 16 && ((kraw >> (8 * j)) & 0xffu) != 0);
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

    // ---- S^T = K Q^T: 4 accumulation chains of eight; operand reads in groups of 2 key blocks of one 32-wide
    // head_dim step, kAhead groups ahead of the matrix instructions that use them (ring of kAhead + 1) ----------
    f32x4_t sacc[4];
    constexpr int kAhead = kD256Ahead;
    X8 afrag[kAhead + 1][2];
    auto k_read = [&](auto gi_c, X8(&dst)[2]) __attribute__((always_inline)) {
      constexpr int gi = decltype(gi_c)::value;
      constexpr int ks = gi >> 1, qu = gi & 1;
#pragma unroll
      for (int i = 0; i < 2; ++i)
        dst[i] = *(MSD_LDS const X8*)(uintptr_t)(k_lds[ks & 3] + stage * kTileBytes + (ks >> 2) * 256 +
                                                 (2 * qu + i) * 16 * kRowBytes);
    };
    static_for<kAhead>([&](auto gi_c) __attribute__((always_inline)) { k_read(gi_c, afrag[decltype(gi_c)::value]); });
    static_for<16>([&](auto gi_c) __attribute__((always_inline)) {
      constexpr int gi = decltype(gi_c)::value;
      constexpr int ks = gi >> 1, qu = gi & 1;
      if constexpr (gi + kAhead < 16) k_read(std::integral_constant<int, gi + kAhead>{}, afrag[(gi + kAhead) % (kAhead + 1)]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
        sacc[2 * qu + i] = E::mfma16(afrag[gi % (kAhead + 1)][i], qf[ks], ks == 0 ? negm : sacc[2 * qu + i]);
    });
    __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0);
#pragma unroll
    for (int gi = 0; gi < 16 - kAhead; ++gi) {
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 2 * kAhead, 0);
    __builtin_amdgcn_sched_barrier(0);

    // ---- keys past the end of the sequence (last tile only) ---------------------------------------------------
    if (key0 + BN > Skv) {
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (key0 + 16 * kb + 4 * g + i >= Skv) sacc[kb][i] = -INFINITY;
    }

    // ---- causal: keys beyond the diagonal (the tiles that cross it for some row of this wave) ------------------
    if constexpr (gen) {
      if (causal && key0 + BN - 1 > row0 + causal_shift) {
        const int lim = row0 + c + causal_shift - key0 - 4 * g;  // visible: 16 * kb + i <= lim
#pragma unroll
        for (int kb = 0; kb < 4; ++kb)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (16 * kb + i > lim) sacc[kb][i] = -INFINITY;
      }
    }

    // ---- key mask: tiles that hide some of their keys ----------------------------------------------------------
    if constexpr (keymask) {
      if (kv_all != 0xffffu) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const unsigned w = kvis[i] >> g;  // key 16 * kb + 4 * g + i is bit 4 * kb + g of word i
#pragma unroll
          for (int kb = 0; kb < 4; ++kb)
            if (!((w >> (4 * kb)) & 1u)) sacc[kb][i] = -INFINITY;
        }
      }
    }

    // ---- online softmax (exp2 domain): the reference maximum moves only when some row of the wave exceeds it by
    // more than 2^kTau (or on the first tile), so most tiles rescale nothing -------------------------------------
    X8 pf[2];
    bool seen = !keymask;  // key mask: this tile showed some row of the wave a key (all rows share the mask)
    {
      float mx = sacc[0][0];
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) mx = fmaxf(mx, sacc[kb][i]);
      if constexpr (keymask) seen = __builtin_amdgcn_ballot_w64(mx > -INFINITY) != 0;
      // (the test needs no row maximum: some lane's part exceeds the threshold iff some row's maximum does)
      l_run += lt[0];
      if (first || __builtin_amdgcn_ballot_w64(mx > kTau) != 0) {
        mx = quarter_max(mx);
        float delta = first ? mx : fmaxf(mx, 0.f);
        delta = (delta == -INFINITY) ? 0.f : delta;
        // (first tile: sums and outputs are still zero; 2^-delta would overflow for rows far below zero and 0 * inf is NaN)
        const float alpha = first ? 1.f : fast_exp2(-delta);
        l_run *= alpha;
#pragma unroll
        for (int i = 0; i < 4; ++i) negm[i] -= delta;
#pragma unroll
        for (int kb = 0; kb < 4; ++kb)
#pragma unroll
          for (int i = 0; i < 4; ++i) sacc[kb][i] -= delta;
#pragma unroll
        for (int db = 0; db < 16; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) oacc[db][i] *= alpha;
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        X8 pk;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          pk[t] = E::from_float(fast_exp2(sacc[2 * j][t]));
          pk[4 + t] = E::from_float(fast_exp2(sacc[2 * j + 1][t]));
        }
        pf[j] = pk;
      }
    }

    // ---- O^T += V^T P^T: 8 steps of (32 keys) x (4 head_dim blocks); V^T fragments requested one step ahead
    // with asm reads and explicit waits, so that the next tile's LDS-DMA stays in flight (see lds_read_tr16_async)
    s16x4_t vf[2][8];
    auto issue = [&](auto step_c, s16x4_t(&dst)[8]) __attribute__((always_inline)) {
      constexpr int s = decltype(step_c)::value;
      constexpr int j = s >> 2, dq = s & 3;
      static_for<4>([&](auto d4_c) __attribute__((always_inline)) {
        constexpr int d4 = decltype(d4_c)::value;
        constexpr int db = 4 * dq + d4;
        constexpr int off = stage * kTileBytes + 32 * j * kRowBytes + (db >> 3) * 256;
        dst[2 * d4] = lds_read_tr16_async<off>(v_lds[db & 7]);
        dst[2 * d4 + 1] = lds_read_tr16_async<off + 16 * kRowBytes>(v_lds[db & 7]);
      });
    };
    if constexpr (keymask) {
      if (next_key0 >= 0) mask_request(next_key0);  // lands during the second product
    }
    issue(std::integral_constant<int, 0>{}, vf[0]);
    static_for<8>([&](auto step_c) __attribute__((always_inline)) {
      constexpr int s = decltype(step_c)::value;
      constexpr int j = s >> 2, dq = s & 3;
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
        oacc[4 * dq + d4] = E::mfma16(u.x, pf[j], oacc[4 * dq + d4]);
      }
      if constexpr (dq == 0)  // the row sums of these 32 keys
        lt = E::mfma16(ones, pf[j], j == 0 ? f32x4_t{0.f, 0.f, 0.f, 0.f} : lt);
    });

    first = first && !seen;  // (without a key mask: false from the first tile on)
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's part of the next tile has landed
    mask_reduce();
    __syncthreads();
  };
  for (int t = 0; t < tiles; t += 2) {
    tile_step(std::integral_constant<int, 0>{}, t * BN, t + 1 < tiles ? (t + 1) * BN : -1);
    if (t + 1 < tiles) tile_step(std::integral_constant<int, 1>{}, (t + 1) * BN, t + 2 < tiles ? (t + 2) * BN : -1);
  }

  // ---- epilogue: normalise, transpose the wave's 16 query rows through LDS, coalesced store --------------------
  MSD_LDS char* ost = smem + wave * 16 * kORowBytes;
  {
    const float l_tot = l_run + lt[0];  // complete sums: the matrix product runs over all keys of a tile
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const int qrow_l = row0 + c;
    if (p.lse && g == 0 && qrow_l < Sq)
      p.lse[((long long)b * p.N + n) * p.Sq + qrow_l] =
          l_tot > 0.f ? -negm[0] * 0.6931471805599453f + __logf(l_tot) : -INFINITY;
#pragma unroll
    for (int db = 0; db < 16; ++db) {
      typename E::x4 pk;
#pragma unroll
      for (int i = 0; i < 4; ++i) pk[i] = E::from_float(oacc[db][i] * inv);
      *(MSD_LDS typename E::x4*)(ost + c * kORowBytes + (16 * db + 4 * g) * 2) = pk;
    }
  }
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int i = 0; i < 16 * 32 / 64; ++i) {
    const int ch = i * 64 + lane;
    const int row = ch >> 5, c32 = ch & 31;
    const int qrow = row0 + row;
    // rows are padded by 8 bytes, so a 16-byte chunk is read as two 8-byte halves
    const i32x2_t lo = *(MSD_LDS const i32x2_t*)(ost + row * kORowBytes + c32 * 16);
    const i32x2_t hi = *(MSD_LDS const i32x2_t*)(ost + row * kORowBytes + c32 * 16 + 8);
    if (qrow < Sq && c32 * 8 < hd) {
      i32x4_t v = {lo[0], lo[1], hi[0], hi[1]};
      *(i32x4_t*)(og + (long long)qrow * p.o_ss + c32 * 8) = v;
    }
  }
#endif  // __HIP_DEVICE_COMPILE__
}

template <int DT, bool DPAD, int GEN>
static int launch_d256(const FaParams& p, hipStream_t stream) {
  auto kern = fa_fwd16_d256_kernel<DT, DPAD, GEN>;
  if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kD256Lds) != hipSuccess)
    return MSD_ERR_LAUNCH;
  const long long grid = fa16_grid<GEN, false>(p, kD256Waves * 16);
  if (grid > 0x7ffffff0ll) return MSD_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(kD256Waves * 64), kD256Lds, stream, p);
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

bool fa16_d256_supported(const FaParams& p) {
  // K/V tiles are fetched with 32-bit buffer offsets relative to the (batch, head) base, below the offset that stands
  // for "no data"
  return (long long)p.Skv * p.k_ss * 2 < 0x7fffff00ll && (long long)p.Skv * p.v_ss * 2 < 0x7fffff00ll;
}

template <int DT, bool DPAD>
static int launch_d256_gen(const FaParams& p, int gen, hipStream_t stream) {
  switch (gen) {
    case 1: return launch_d256<DT, DPAD, 1>(p, stream);
    case 2: return launch_d256<DT, DPAD, 2>(p, stream);
    case 3: return launch_d256<DT, DPAD, 3>(p, stream);
    default: return launch_d256<DT, DPAD, 0>(p, stream);
  }
}

int launch_fa16_d256(const FaParams& p, int dtype, int D, hipStream_t stream, int gen) {
  if (!fa16_d256_supported(p) || D <= 128 || D > 256 || (D & 7) || gen < 0 || gen > 3) return MSD_ERR_UNSUPPORTED;
  const bool bf = dtype == MSD_DTYPE_BF16;
  if (D == 256)
    return bf ? launch_d256_gen<MSD_DTYPE_BF16, false>(p, gen, stream) : launch_d256_gen<MSD_DTYPE_F16, false>(p, gen, stream);
  FaParams pp = p;
  pp.head_dim = D;
  return bf ? launch_d256_gen<MSD_DTYPE_BF16, true>(pp, gen, stream) : launch_d256_gen<MSD_DTYPE_F16, true>(pp, gen, stream);
}

}  // namespace msd
