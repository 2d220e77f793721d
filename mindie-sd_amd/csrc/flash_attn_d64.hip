// Flash-attention forward for gfx950 (MI355X) at head_dim 64: bf16/fp16; dense, and (from 256 query rows on) causal,
// packed variable-length sequences and key-padding masks.
//
// head_dim 64 is what the reference's own tests of attention_forward run
// (tests/layers/flash_attn/test_attn_forward.py:31-169) and what its fused dense ops
// (mindiesd/layers/flash_attn/prompt_flash_attn.py:48, fused_attn_score.py:48, csrc/plugin/la.cpp:27-58) see from
// models with 64-wide heads.  The general kernel of flash_attn_hd.hip covers every head_dim with a plain data path;
// this file carries the design of fa_fwd16_kernel (flash_attn_fwd.hip, head_dim 128) over to 64:
//   * 8 waves x 32 query rows per workgroup, 128-key tiles, K and V tiles staged by LDS-DMA (two stages each);
//   * the transposed problem S^T = K Q^T, O^T += V^T P^T on the 16x16x32 matrix instruction, Q^T resident with
//     scale * log2(e) folded in, P^T straight from the score accumulators, V^T by the transposing LDS read;
//   * lazily moved reference maximum seeded into the score accumulators, row sums on the matrix pipe (ones x P^T).
// At this head_dim a score costs half the matrix work of head_dim 128 and the same vector work, so the vector ALU is
// the busier pipe; what the design saves over the general kernel is the vector work of the row sums and of the
// register staging, and the waits of the latter.
//
// Register tiles, with c = lane % 16 and g = lane / 16:
//     S^T block (16 keys x 16 queries):  A = K rows 16*kb + c, head_dim 32*ks + 8*g .. +8 (one 16-byte LDS read),
//                                        B = Q^T resident (query 16*nq + c, same head_dim slice);
//                                        the lane receives keys 16*kb + 4*g + i (i < 4) of query 16*nq + c
//     O^T block (16 dims x 16 queries):  B = P^T of 32 keys straight from two S^T blocks (slot 8*g + t holds key
//                                        32*j + 4*g + t for t < 4 and key 32*j + 16 + 4*g + t - 4 for t >= 4),
//                                        A = V^T in the same slot order from two transposing LDS reads
// LDS: rows of 128 bytes.  K stages at 0 and 16 KiB: 16-byte chunk p of row r sits at chunk p ^ ((r >> 1) & 7), so
// the 16 rows one quarter-wave reads cover all banks.  V stages at 32 and 48 KiB: 32-byte chunk p of row r sits at
// chunk p ^ ((r >> 1) & 3) - a half-wave of the transposing read covers 8 rows x 32 bytes.
#include <type_traits>
#include <utility>

#include "common.hpp"
#include "fa_params.hpp"

namespace msd {

#if defined(__HIP_DEVICE_COMPILE__)
namespace d64 {
template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>)
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

// Rescale of one 16-query column block when its reference maximum moves: l *= alpha, the seed and the 8 score blocks
// -= delta, the 4 output blocks *= alpha - 53 registers updated in place by asm blocks that skip themselves when the
// wave-uniform flag is zero (the same construction as cond_rescale_fa16 in common.hpp, which explains why the test
// sits inside the asm).  None of the values may be the result of a matrix instruction still in flight.
__device__ __forceinline__ void cond_rescale(int flag, float delta, float alpha, float& l, f32x4_t& negm, f32x4_t& s0,
                                             f32x4_t& s1, f32x4_t& s2, f32x4_t& s3, f32x4_t& s4, f32x4_t& s5,
                                             f32x4_t& s6, f32x4_t& s7, f32x4_t& o0, f32x4_t& o1, f32x4_t& o2,
                                             f32x4_t& o3) {
  float negm_0 = negm[0], negm_1 = negm[1], negm_2 = negm[2], negm_3 = negm[3];
  float s0_0 = s0[0], s0_1 = s0[1], s0_2 = s0[2], s0_3 = s0[3];
  float s1_0 = s1[0], s1_1 = s1[1], s1_2 = s1[2], s1_3 = s1[3];
  float s2_0 = s2[0], s2_1 = s2[1], s2_2 = s2[2], s2_3 = s2[3];
  float s3_0 = s3[0], s3_1 = s3[1], s3_2 = s3[2], s3_3 = s3[3];
  float s4_0 = s4[0], s4_1 = s4[1], s4_2 = s4[2], s4_3 = s4[3];
  float s5_0 = s5[0], s5_1 = s5[1], s5_2 = s5[2], s5_3 = s5[3];
  float s6_0 = s6[0], s6_1 = s6[1], s6_2 = s6[2], s6_3 = s6[3];
  float s7_0 = s7[0], s7_1 = s7[1], s7_2 = s7[2], s7_3 = s7[3];
  float o0_0 = o0[0], o0_1 = o0[1], o0_2 = o0[2], o0_3 = o0[3];
  float o1_0 = o1[0], o1_1 = o1[1], o1_2 = o1[2], o1_3 = o1[3];
  float o2_0 = o2[0], o2_1 = o2[1], o2_2 = o2[2], o2_3 = o2[3];
  float o3_0 = o3[0], o3_1 = o3[1], o3_2 = o3[2], o3_3 = o3[3];
  asm volatile("s_cmp_eq_u32 %25, 0\n\t" "s_cbranch_scc1 .Lmsd_skip%=\n\t" "v_mul_f32 %0, %0, %27\n\t"
               "v_sub_f32 %1, %1, %26\n\t" "v_sub_f32 %2, %2, %26\n\t" "v_sub_f32 %3, %3, %26\n\t"
               "v_sub_f32 %4, %4, %26\n\t" "v_sub_f32 %5, %5, %26\n\t" "v_sub_f32 %6, %6, %26\n\t"
               "v_sub_f32 %7, %7, %26\n\t" "v_sub_f32 %8, %8, %26\n\t" "v_sub_f32 %9, %9, %26\n\t"
               "v_sub_f32 %10, %10, %26\n\t" "v_sub_f32 %11, %11, %26\n\t" "v_sub_f32 %12, %12, %26\n\t"
               "v_sub_f32 %13, %13, %26\n\t" "v_sub_f32 %14, %14, %26\n\t" "v_sub_f32 %15, %15, %26\n\t"
               "v_sub_f32 %16, %16, %26\n\t" "v_sub_f32 %17, %17, %26\n\t" "v_sub_f32 %18, %18, %26\n\t"
               "v_sub_f32 %19, %19, %26\n\t" "v_sub_f32 %20, %20, %26\n\t" "v_sub_f32 %21, %21, %26\n\t"
               "v_sub_f32 %22, %22, %26\n\t" "v_sub_f32 %23, %23, %26\n\t" "v_sub_f32 %24, %24, %26\n\t"
               "s_nop 7\n\t" ".Lmsd_skip%=:"
               : "+v"(l), "+v"(negm_0), "+v"(negm_1), "+v"(negm_2), "+v"(negm_3), "+v"(s0_0), "+v"(s0_1), "+v"(s0_2),
                 "+v"(s0_3), "+v"(s1_0), "+v"(s1_1), "+v"(s1_2), "+v"(s1_3), "+v"(s2_0), "+v"(s2_1), "+v"(s2_2),
                 "+v"(s2_3), "+v"(s3_0), "+v"(s3_1), "+v"(s3_2), "+v"(s3_3), "+v"(s4_0), "+v"(s4_1), "+v"(s4_2),
                 "+v"(s4_3)
               : "s"(flag), "v"(delta), "v"(alpha)
               : "scc");
  asm volatile("s_cmp_eq_u32 %28, 0\n\t" "s_cbranch_scc1 .Lmsd_skip%=\n\t" "v_sub_f32 %0, %0, %29\n\t"
               "v_sub_f32 %1, %1, %29\n\t" "v_sub_f32 %2, %2, %29\n\t" "v_sub_f32 %3, %3, %29\n\t"
               "v_sub_f32 %4, %4, %29\n\t" "v_sub_f32 %5, %5, %29\n\t" "v_sub_f32 %6, %6, %29\n\t"
               "v_sub_f32 %7, %7, %29\n\t" "v_sub_f32 %8, %8, %29\n\t" "v_sub_f32 %9, %9, %29\n\t"
               "v_sub_f32 %10, %10, %29\n\t" "v_sub_f32 %11, %11, %29\n\t" "v_mul_f32 %12, %12, %30\n\t"
               "v_mul_f32 %13, %13, %30\n\t" "v_mul_f32 %14, %14, %30\n\t" "v_mul_f32 %15, %15, %30\n\t"
               "v_mul_f32 %16, %16, %30\n\t" "v_mul_f32 %17, %17, %30\n\t" "v_mul_f32 %18, %18, %30\n\t"
               "v_mul_f32 %19, %19, %30\n\t" "v_mul_f32 %20, %20, %30\n\t" "v_mul_f32 %21, %21, %30\n\t"
               "v_mul_f32 %22, %22, %30\n\t" "v_mul_f32 %23, %23, %30\n\t" "v_mul_f32 %24, %24, %30\n\t"
               "v_mul_f32 %25, %25, %30\n\t" "v_mul_f32 %26, %26, %30\n\t" "v_mul_f32 %27, %27, %30\n\t"
               "s_nop 7\n\t" ".Lmsd_skip%=:"
               : "+v"(s5_0), "+v"(s5_1), "+v"(s5_2), "+v"(s5_3), "+v"(s6_0), "+v"(s6_1), "+v"(s6_2), "+v"(s6_3),
                 "+v"(s7_0), "+v"(s7_1), "+v"(s7_2), "+v"(s7_3), "+v"(o0_0), "+v"(o0_1), "+v"(o0_2), "+v"(o0_3),
                 "+v"(o1_0), "+v"(o1_1), "+v"(o1_2), "+v"(o1_3), "+v"(o2_0), "+v"(o2_1), "+v"(o2_2), "+v"(o2_3),
                 "+v"(o3_0), "+v"(o3_1), "+v"(o3_2), "+v"(o3_3)
               : "s"(flag), "v"(delta), "v"(alpha)
               : "scc");
  negm = f32x4_t{negm_0, negm_1, negm_2, negm_3};
  s0 = f32x4_t{s0_0, s0_1, s0_2, s0_3};
  s1 = f32x4_t{s1_0, s1_1, s1_2, s1_3};
  s2 = f32x4_t{s2_0, s2_1, s2_2, s2_3};
  s3 = f32x4_t{s3_0, s3_1, s3_2, s3_3};
  s4 = f32x4_t{s4_0, s4_1, s4_2, s4_3};
  s5 = f32x4_t{s5_0, s5_1, s5_2, s5_3};
  s6 = f32x4_t{s6_0, s6_1, s6_2, s6_3};
  s7 = f32x4_t{s7_0, s7_1, s7_2, s7_3};
  o0 = f32x4_t{o0_0, o0_1, o0_2, o0_3};
  o1 = f32x4_t{o1_0, o1_1, o1_2, o1_3};
  o2 = f32x4_t{o2_0, o2_1, o2_2, o2_3};
  o3 = f32x4_t{o3_0, o3_1, o3_2, o3_3};
}
}  // namespace d64
#endif

constexpr int kD64Waves = 8, kD64BN = 128, kD64RowBytes = 128;
constexpr int kD64TileBytes = kD64BN * kD64RowBytes;  // 16 KiB
constexpr int kD64Lds = 4 * kD64TileBytes;            // two K and two V stages
constexpr int kD64Ahead = 3;                          // K operand groups requested ahead of their use

// GEN as in fa_fwd16_kernel (flash_attn_fwd.hip): 0 dense; 1 per-sequence lengths (p.seq_meta) and / or causal;
// 2 the same with the packed tile numbering; 3 a boolean mask row shared by all queries of a (batch, head).
// DPAD: head dims below 64 (p.head_dim, a multiple of 8) computed as 64: the query operand is zero from
// the real head_dim on, the lanes that would stage the 16-byte chunks of K and V past it request an offset beyond
// the buffers' range (the DMA writes zeros for them without touching memory), output columns past it are not stored.
// NW: waves per workgroup, 32 query rows each - 8 (one workgroup per CU), or 4 (two per CU: for grids that fill the
// chip badly as 256-row workgroups).
template <int DT, int GEN = 0, bool DPAD = false, int NW = kD64Waves>
__global__ __launch_bounds__(NW * 64, NW == 8 ? 1 : 2) void fa_fwd16_d64_kernel(const FaParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  using namespace d64;
  using E = Elem<DT>;
  using T = typename E::type;
  using X8 = typename E::x8;
  constexpr int NWAVES = NW, BN = kD64BN, kBM = NWAVES * 32, kRowBytes = kD64RowBytes;
  constexpr int kTileBytes = kD64TileBytes, kORowBytes = kRowBytes + 8;
  static_assert(NWAVES * 32 * kORowBytes <= kD64Lds, "the output staging reuses the tile stages");
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  MSD_LDS char* smem = (MSD_LDS char*)smem_raw;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 15;
  const int g = lane >> 4;

  constexpr bool gen = GEN != 0, keymask = GEN == 3;
  const int hd = DPAD ? p.head_dim : 64;
  int bn, qt, b, n, Sq, Skv;
  long long q_tok0, k_tok0;  // general mode: first token of the sequence in packed tensors
  if (!fa16_find_work<GEN, false>(p, kBM, bn, qt, b, n, Sq, Skv, q_tok0, k_tok0)) return;
  const int nkv = n / (p.N / p.Nkv);
  const int row0 = qt * kBM + wave * 32;  // first query row of this wave

  const T* qg = (const T*)p.q + b * p.q_sb + n * p.q_sn + q_tok0 * p.q_ss;
  const T* kg = (const T*)p.k + b * p.k_sb + nkv * p.k_sn + k_tok0 * p.k_ss;
  const T* vg = (const T*)p.v + b * p.v_sb + nkv * p.v_sn + k_tok0 * p.v_ss;
  T* og = (T*)p.o + b * p.o_sb + n * p.o_sn + q_tok0 * p.o_ss;

  // ---- Q^T operand, resident: lane (c, g) holds query 16*nq + c, head_dim 32*ks + 8*g .. +8 --------------
  X8 qf[2][2];
#pragma unroll
  for (int nq = 0; nq < 2; ++nq) {
    const int qrow = row0 + nq * 16 + c;
    const bool ok = qrow < Sq;
    const T* src = qg + (long long)(ok ? qrow : 0) * p.q_ss + 8 * g;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const bool in = ok && (!DPAD || 32 * ks + 8 * g < hd);  // (a chunk of 8 lies wholly inside or outside)
      X8 v = in ? *(const X8*)(src + 32 * ks) : X8{0};
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = E::from_float((float)v[j] * p.scale_log2);
      qf[nq][ks] = v;
    }
  }

  f32x4_t oacc[4][2];
  float l_run[2];
  // Row sums come off the matrix pipe: ones x P^T gives every lane the sum of its query column over the 128 keys of a
  // tile.  lt holds the sums of the tile before; they are added to l_run at the start of the next softmax, before a
  // rescale, when the matrix results have long landed.
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
    for (int db = 0; db < 4; ++db) oacc[db][nq] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  // ---- global -> LDS staging (LDS-DMA; swizzles applied on the global side) -------------------------------
  // One instruction moves 8 rows of 128 bytes; a wave issues two per operand and tile (rows 8*wave.. and 64 below:
  // the same swizzles, so one per-lane offset per operand serves both).  Keys past the end of the sequence lie
  // outside the descriptors' range and read as zeros.
  // (a sequence without keys exposes nothing: every row reads as zeros and no tile is computed)
  const int k_range = gen && Skv <= 0 ? 0 : (int)(((long long)(Skv - 1) * p.k_ss + hd) * 2);
  const int v_range = gen && Skv <= 0 ? 0 : (int)(((long long)(Skv - 1) * p.v_ss + hd) * 2);
  const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)kg, 0, k_range, 0x00020000);
  const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)vg, 0, v_range, 0x00020000);
  const int k_row_bytes = (int)p.k_ss * 2, v_row_bytes = (int)p.v_ss * 2;
  int k_voff, v_voff;
  {
    const int row = 8 * wave + (lane >> 3);
    const int pc = lane & 7;  // physical 16-byte chunk this lane fills
    const int kc = pc ^ ((row >> 1) & 7), vc = (((pc >> 1) ^ ((row >> 1) & 3)) << 1) | (pc & 1);  // logical chunks
    k_voff = row * k_row_bytes + (kc << 4);
    v_voff = row * v_row_bytes + (vc << 4);
    if constexpr (DPAD) {  // chunks past the head_dim: an offset beyond every range
      if (kc * 8 >= hd) k_voff = 0x7ffffff0;
      if (vc * 8 >= hd) v_voff = 0x7ffffff0;
    }
  }
  auto load_tile = [&](int key0, int stage) {
    MSD_LDS char* kb = smem + stage * kTileBytes;
    MSD_LDS char* vb = smem + (2 + stage) * kTileBytes;
#pragma unroll
    for (int i = 0; i < 16 / NWAVES; ++i) {
      const int grp = i * NWAVES + wave;  // 8-row group of the tile
      __builtin_amdgcn_raw_ptr_buffer_load_lds(k_rsrc, (MSD_LDS void*)(kb + grp * 1024), 16, k_voff,
                                               (key0 + i * 8 * NWAVES) * k_row_bytes, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(v_rsrc, (MSD_LDS void*)(vb + grp * 1024), 16, v_voff,
                                               (key0 + i * 8 * NWAVES) * v_row_bytes, 0, 0);
    }
  };

  // per-lane parts of the LDS read addresses
  // K operand: row 16*kb + c, 16-byte chunk (4*ks + g) ^ ((c >> 1) & 7)
  unsigned k_lds[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
    k_lds[ks] = (unsigned)(uintptr_t)smem + c * kRowBytes + (((4 * ks + g) ^ ((c >> 1) & 7)) << 4);
  // V^T operand: the lane points at key 4*g + c/4 (+32*j, +16), 8 bytes at 8*(c%4) of 32-byte chunk db ^ ((key >> 1) & 3)
  unsigned v_lds[4];
  {
    const int key = 4 * g + (c >> 2);
#pragma unroll
    for (int db = 0; db < 4; ++db)
      v_lds[db] = (unsigned)(uintptr_t)smem + 2 * kTileBytes + key * kRowBytes + ((db ^ ((key >> 1) & 3)) << 5) +
                  8 * (c & 3);
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

  // ---- key mask (GEN 3): words of visible keys of the current tile; bit l of word j = key 4 * l + j ------------
  // (see fa_fwd16_kernel: the bytes of the next tile are fetched during the second product and reduced to scalar words)
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

    // ---- S^T = K Q^T: 16 accumulation chains of two; operand reads in groups of 2 key blocks of one 32-wide head_dim
    // step, kAhead groups ahead of the matrix instructions that use them (ring of kAhead + 1) -----------------
    f32x4_t sacc[8][2];
    constexpr int kAhead = kD64Ahead;
    X8 afrag[kAhead + 1][2];
    auto k_read = [&](auto gi_c, X8(&dst)[2]) __attribute__((always_inline)) {
      constexpr int gi = decltype(gi_c)::value;
      constexpr int ks = gi >> 2, qu = gi & 3;
#pragma unroll
      for (int i = 0; i < 2; ++i)
        dst[i] = *(MSD_LDS const X8*)(uintptr_t)(k_lds[ks] + stage * kTileBytes + (2 * qu + i) * 16 * kRowBytes);
    };
    static_for<kAhead>([&](auto gi_c) __attribute__((always_inline)) { k_read(gi_c, afrag[decltype(gi_c)::value]); });
    static_for<8>([&](auto gi_c) __attribute__((always_inline)) {
      constexpr int gi = decltype(gi_c)::value;
      constexpr int ks = gi >> 2, qu = gi & 3;
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

    // ---- online softmax (exp2 domain): the reference maximum moves only when some row of the wave exceeds it by
    // more than 2^kTau (or on the first tile), so most tiles rescale nothing -------------------------------------
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
      cond_rescale(__builtin_amdgcn_readfirstlane(moved), delta, alpha, l_run[nq], negm[nq], sacc[0][nq], sacc[1][nq],
                   sacc[2][nq], sacc[3][nq], sacc[4][nq], sacc[5][nq], sacc[6][nq], sacc[7][nq], oacc[0][nq],
                   oacc[1][nq], oacc[2][nq], oacc[3][nq]);
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

    // ---- O^T += V^T P^T: 4 steps of (32 keys) x (4 head_dim blocks); V^T fragments requested one step ahead
    // with asm reads and explicit waits, so that the next tile's LDS-DMA stays in flight (see lds_read_tr16_async)
    s16x4_t vf[2][8];
    auto issue = [&](auto step_c, s16x4_t(&dst)[8]) __attribute__((always_inline)) {
      constexpr int j = decltype(step_c)::value;
      constexpr int off = stage * kTileBytes + 32 * j * kRowBytes;
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        dst[2 * db] = lds_read_tr16_async<off>(v_lds[db]);
        dst[2 * db + 1] = lds_read_tr16_async<off + 16 * kRowBytes>(v_lds[db]);
      }
    };
    if constexpr (keymask) {
      if (next_key0 >= 0) mask_request(next_key0);  // lands during the second product
    }
    issue(std::integral_constant<int, 0>{}, vf[0]);
    static_for<4>([&](auto step_c) __attribute__((always_inline)) {
      constexpr int j = decltype(step_c)::value;
      if constexpr (j + 1 < 4) {
        issue(std::integral_constant<int, j + 1>{}, vf[(j + 1) & 1]);
        lds_wait_tr<8>(vf[j & 1]);
      } else {
        lds_wait_tr<0>(vf[j & 1]);
      }
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        union { s16x4_t s2[2]; X8 x; } u;
        u.s2[0] = vf[j & 1][2 * db];
        u.s2[1] = vf[j & 1][2 * db + 1];
#pragma unroll
        for (int nq = 0; nq < 2; ++nq) oacc[db][nq] = E::mfma16(u.x, pf[nq][j], oacc[db][nq]);
      }
      // the row sums of these 32 keys
#pragma unroll
      for (int nq = 0; nq < 2; ++nq)
        lt[nq] = E::mfma16(ones, pf[nq][j], j == 0 ? f32x4_t{0.f, 0.f, 0.f, 0.f} : lt[nq]);
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

  // ---- epilogue: normalise, transpose the wave's 32 query rows through LDS, coalesced store --------------------
  MSD_LDS char* ost = smem + wave * 32 * kORowBytes;
#pragma unroll
  for (int nq = 0; nq < 2; ++nq) {
    const float l_tot = l_run[nq] + lt[nq][0];  // complete sums: the matrix product runs over all keys of a tile
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const int qrow_l = row0 + nq * 16 + c;
    if (p.lse && g == 0 && qrow_l < Sq)
      p.lse[((long long)b * p.N + n) * p.Sq + qrow_l] =
          l_tot > 0.f ? -negm[nq][0] * 0.6931471805599453f + __logf(l_tot) : -INFINITY;
#pragma unroll
    for (int db = 0; db < 4; ++db) {
      typename E::x4 pk;
#pragma unroll
      for (int i = 0; i < 4; ++i) pk[i] = E::from_float(oacc[db][nq][i] * inv);
      *(MSD_LDS typename E::x4*)(ost + (nq * 16 + c) * kORowBytes + (16 * db + 4 * g) * 2) = pk;
    }
  }
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int i = 0; i < 32 * 8 / 64; ++i) {
    const int ch = i * 64 + lane;
    const int row = ch >> 3, c8 = ch & 7;
    const int qrow = row0 + row;
    // rows are padded by 8 bytes, so a 16-byte chunk is read as two 8-byte halves
    const i32x2_t lo = *(MSD_LDS const i32x2_t*)(ost + row * kORowBytes + c8 * 16);
    const i32x2_t hi = *(MSD_LDS const i32x2_t*)(ost + row * kORowBytes + c8 * 16 + 8);
    if (qrow < Sq && (!DPAD || c8 * 8 < hd)) {
      i32x4_t v = {lo[0], lo[1], hi[0], hi[1]};
      *(i32x4_t*)(og + (long long)qrow * p.o_ss + c8 * 8) = v;
    }
  }
#endif  // __HIP_DEVICE_COMPILE__
}


template <int DT, int GEN, bool DPAD = false, int NW = kD64Waves>
static int launch_d64(const FaParams& p, hipStream_t stream) {
  auto kern = fa_fwd16_d64_kernel<DT, GEN, DPAD, NW>;
  if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kD64Lds) != hipSuccess)
    return MSD_ERR_LAUNCH;
  const long long grid = fa16_grid<GEN, false>(p, NW * 32);
  if (grid > 0x7ffffff0ll) return MSD_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NW * 64), kD64Lds, stream, p);
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

bool fa16_d64_supported(const FaParams& p) {
  // K/V tiles are fetched with 32-bit buffer offsets relative to the (batch, head) base, below the offset that stands
  // for "no data"
  return (long long)p.Skv * p.k_ss * 2 < 0x7fffff00ll && (long long)p.Skv * p.v_ss * 2 < 0x7fffff00ll;
}

int launch_fa16_d64_padded(const FaParams& p, int dtype, int D, hipStream_t stream, int gen, int rows) {
  if (!fa16_d64_supported(p) || D <= 0 || D >= 64 || (D & 7) || gen < 0 || gen > 3) return MSD_ERR_UNSUPPORTED;
  if (rows != 256 && !(rows == 128 && gen == 0)) return MSD_ERR_UNSUPPORTED;
  FaParams pp = p;
  pp.head_dim = D;
  const bool bf = dtype == MSD_DTYPE_BF16;
  if (rows == 128)
    return bf ? launch_d64<MSD_DTYPE_BF16, 0, true, 4>(pp, stream) : launch_d64<MSD_DTYPE_F16, 0, true, 4>(pp, stream);
  switch (gen) {
    case 1: return bf ? launch_d64<MSD_DTYPE_BF16, 1, true>(pp, stream) : launch_d64<MSD_DTYPE_F16, 1, true>(pp, stream);
    case 2: return bf ? launch_d64<MSD_DTYPE_BF16, 2, true>(pp, stream) : launch_d64<MSD_DTYPE_F16, 2, true>(pp, stream);
    case 3: return bf ? launch_d64<MSD_DTYPE_BF16, 3, true>(pp, stream) : launch_d64<MSD_DTYPE_F16, 3, true>(pp, stream);
    default: return bf ? launch_d64<MSD_DTYPE_BF16, 0, true>(pp, stream) : launch_d64<MSD_DTYPE_F16, 0, true>(pp, stream);
  }
}

int launch_fa16_d64(const FaParams& p, int dtype, hipStream_t stream, int gen, int rows) {
  if (!fa16_d64_supported(p) || gen < 0 || gen > 3) return MSD_ERR_UNSUPPORTED;
  if (rows != 256 && !(rows == 128 && gen == 0)) return MSD_ERR_UNSUPPORTED;
  const bool bf = dtype == MSD_DTYPE_BF16;
  if (rows == 128)
    return bf ? launch_d64<MSD_DTYPE_BF16, 0, false, 4>(p, stream) : launch_d64<MSD_DTYPE_F16, 0, false, 4>(p, stream);
  switch (gen) {
    case 1: return bf ? launch_d64<MSD_DTYPE_BF16, 1>(p, stream) : launch_d64<MSD_DTYPE_F16, 1>(p, stream);
    case 2: return bf ? launch_d64<MSD_DTYPE_BF16, 2>(p, stream) : launch_d64<MSD_DTYPE_F16, 2>(p, stream);
    case 3: return bf ? launch_d64<MSD_DTYPE_BF16, 3>(p, stream) : launch_d64<MSD_DTYPE_F16, 3>(p, stream);
    default: return bf ? launch_d64<MSD_DTYPE_BF16, 0>(p, stream) : launch_d64<MSD_DTYPE_F16, 0>(p, stream);
  }
}

}  // namespace msd
