// Flash-attention forward for gfx950 (MI355X): dense and block-sparse, head_dim 128, bf16/fp16.
//
// Replaces the device side of the reference's fused attention ops: the dense vendor kernels
// behind attention_forward (mindiesd/layers/flash_attn/attention_forward.py:24-89) and the
// block-sparse kernels behind torch.ops.mindiesd.block_sparse_attention /
// rainfusionattention (csrc/plugin/block_sparse_attention.cpp:31-121,
// csrc/plugin/rainfusionattention.cpp:27-64).
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
#include "common.hpp"

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
};

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
  static constexpr int kChunksPerThread = BN * 16 / kNT;  // 16-byte chunks of one tile per thread
  static_assert(BN * 16 % kNT == 0, "tile must split evenly over the threads");
};

// Register budget: 8 wavefronts per CU (two per SIMD) in every configuration, i.e. at most 256
// registers per lane; the 4-wave configurations run two workgroups per CU.
template <int DT, int NWAVES, int QPW, int BN, bool SPARSE>
__global__ __launch_bounds__(NWAVES * 64, (QPW == 32 ? 2 : 1)) void fa_fwd_kernel(const FaParams p) {
  using C = FaCfg<DT, NWAVES, QPW, BN, SPARSE>;
  using E = Elem<DT>;
  using T = typename E::type;
  using X8 = typename E::x8;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  MSD_LDS char* smem = (MSD_LDS char*)smem_raw;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int h = lane >> 5;

  // ---- which (batch, head, query tile): consecutive tiles of one head stay on one XCD -------
  const int q_tiles = (p.Sq + C::kBM - 1) / C::kBM;
  const int total = p.B * p.N * q_tiles;
  const int per_xcd = (total + 7) / 8;
  int work = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (work >= total) return;
  if (SPARSE && p.order) work = p.order[work];
  const int bn = work / q_tiles;
  const int qt = work - bn * q_tiles;
  const int b = bn / p.N;
  const int n = bn - b * p.N;
  const int nkv = n / (p.N / p.Nkv);
  const int q0 = qt * C::kBM;

  const T* qg = (const T*)p.q + b * p.q_sb + n * p.q_sn;
  const T* kg = (const T*)p.k + b * p.k_sb + nkv * p.k_sn;
  const T* vg = (const T*)p.v + b * p.v_sb + nkv * p.v_sn;

  // ---- tile list ----------------------------------------------------------------------------
  int n_tiles;
  const int* sel = nullptr;
  constexpr int kSub = 128 / BN;  // tiles per 128-key block (sparse granularity)
  if (SPARSE) {
    const long long qb_lin = (long long)bn * p.QB + qt;  // BM == 128 for the sparse kernel
    sel = p.blk_idx + qb_lin * p.kb_stride;
    n_tiles = p.blk_cnt[qb_lin] * kSub;
  } else {
    n_tiles = (p.Skv + BN - 1) / BN;
  }

  // ---- Q^T operand, resident in registers: lane (q = l32, h) holds d = 16*ks + 8*h .. +8 -----
  X8 qf[C::kNQB][8];
#pragma unroll
  for (int qb = 0; qb < C::kNQB; ++qb) {
    const int qrow = q0 + wave * QPW + qb * 32 + l32;
    const bool ok = qrow < p.Sq;
    const T* src = qg + (long long)(ok ? qrow : 0) * p.q_ss + 8 * h;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      X8 v = *(const X8*)(src + 16 * ks);
      if (!ok) v = X8{0};
      qf[qb][ks] = v;
    }
  }

  f32x16_t oacc[4][C::kNQB];
  float m_run[C::kNQB], l_run[C::kNQB];
#pragma unroll
  for (int qb = 0; qb < C::kNQB; ++qb) {
    m_run[qb] = -INFINITY;
    l_run[qb] = 0.f;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[db][qb][r] = 0.f;
  }

  // ---- global -> register -> LDS staging of one K/V tile ----------------------------------------
  i32x4_t kreg[C::kChunksPerThread], vreg[C::kChunksPerThread];
  auto tile_key0 = [&](int t) -> int {
    if (SPARSE) return sel[t / kSub] * 128 + (t % kSub) * BN;
    return t * BN;
  };
  auto load_tile = [&](int t) {
    const int key0 = tile_key0(t);
#pragma unroll
    for (int i = 0; i < C::kChunksPerThread; ++i) {
      const int c = i * C::kNT + tid;
      const int row = c >> 4, c16 = c & 15;
      const int key = key0 + row;
      const bool ok = key < p.Skv;
      const long long kr = (long long)(ok ? key : 0);
      i32x4_t kk = *(const i32x4_t*)(kg + kr * p.k_ss + c16 * 8);
      i32x4_t vv = *(const i32x4_t*)(vg + kr * p.v_ss + c16 * 8);
      if (!ok) { kk = i32x4_t{0, 0, 0, 0}; vv = i32x4_t{0, 0, 0, 0}; }
      kreg[i] = kk;
      vreg[i] = vv;
    }
  };
  auto store_tile = [&](int stage) {
    MSD_LDS char* kb = smem + stage * C::kStageBytes;
    MSD_LDS char* vb = kb + C::kTileBytes;
#pragma unroll
    for (int i = 0; i < C::kChunksPerThread; ++i) {
      const int c = i * C::kNT + tid;
      const int row = c >> 4, c16 = c & 15;
      *(MSD_LDS i32x4_t*)(kb + row * C::kRowBytes + ((c16 ^ (row & 15)) << 4)) = kreg[i];
      *(MSD_LDS i32x4_t*)(vb + row * C::kRowBytes + ((c16 ^ ((row & 3) << 2)) << 4)) = vreg[i];
    }
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

  if (n_tiles > 0) {
    load_tile(0);
    store_tile(0);
  }
  __syncthreads();

  for (int t = 0; t < n_tiles; ++t) {
    const int stage = t & 1;
    if (t + 1 < n_tiles) load_tile(t + 1);

    MSD_LDS const char* kb_base = smem + stage * C::kStageBytes;
    MSD_LDS const char* vb_base = kb_base + C::kTileBytes;

    // ---- S^T = K Q^T -------------------------------------------------------------------------
    f32x16_t sacc[C::kNKB][C::kNQB];
#pragma unroll
    for (int kb = 0; kb < C::kNKB; ++kb)
#pragma unroll
      for (int qb = 0; qb < C::kNQB; ++qb)
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[kb][qb][r] = 0.f;
#pragma unroll
    for (int kb = 0; kb < C::kNKB; ++kb) {
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        const X8 a = *(MSD_LDS const X8*)(kb_base + kb * 32 * C::kRowBytes + k_row_off +
                                          (((2 * ks + h) ^ k_swz) << 4));
#pragma unroll
        for (int qb = 0; qb < C::kNQB; ++qb) sacc[kb][qb] = E::mfma32(a, qf[qb][ks], sacc[kb][qb]);
      }
    }

    // ---- mask keys past the end of the sequence (last tile only) --------------------------------
    const int key0 = tile_key0(t);
    if (key0 + BN > p.Skv) {
#pragma unroll
      for (int kb = 0; kb < C::kNKB; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = key0 + kb * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
          if (key >= p.Skv) {
#pragma unroll
            for (int qb = 0; qb < C::kNQB; ++qb) sacc[kb][qb][r] = -INFINITY;
          }
        }
    }

    // ---- online softmax; P^T is packed in place as the B operand of the second product ----------
    X8 pf[C::kNQB][C::kNKB][2];
#pragma unroll
    for (int qb = 0; qb < C::kNQB; ++qb) {
      float mx = sacc[0][qb][0];
#pragma unroll
      for (int kb = 0; kb < C::kNKB; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sacc[kb][qb][r]);
      mx = fmaxf(mx, xor32(mx));
      const float m_new = fmaxf(m_run[qb], mx);
      const float mc = (m_new == -INFINITY) ? 0.f : m_new * p.scale_log2;
      const float alpha = fast_exp2(m_run[qb] * p.scale_log2 - mc);
      m_run[qb] = m_new;
      float ls = 0.f;
#pragma unroll
      for (int kb = 0; kb < C::kNKB; ++kb) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float e = fast_exp2(__builtin_fmaf(sacc[kb][qb][r], p.scale_log2, -mc));
          ls += e;
          sacc[kb][qb][r] = e;
        }
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
          X8 pk;
#pragma unroll
          for (int j = 0; j < 8; ++j) pk[j] = E::from_float(sacc[kb][qb][8 * t2 + j]);
          pf[qb][kb][t2] = pk;
        }
      }
      l_run[qb] = l_run[qb] * alpha + ls;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][qb][r] *= alpha;
    }

    // ---- O^T += V^T P^T ------------------------------------------------------------------------
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

    if (t + 1 < n_tiles) store_tile(stage ^ 1);
    __syncthreads();
  }

  // ---- epilogue: normalise, transpose 32 query rows at a time through LDS, coalesced store -------
  // Each wave stages only its own rows, and a wave's LDS operations execute in order, so no
  // workgroup barrier is needed here (the loop above ended with one).
  MSD_LDS char* ost = smem + wave * 32 * C::kORowBytes;
  T* og = (T*)p.o + b * p.o_sb + n * p.o_sn;
#pragma unroll
  for (int qb = 0; qb < C::kNQB; ++qb) {
    const float l_tot = l_run[qb] + xor32(l_run[qb]);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const int qrow_l = q0 + wave * QPW + qb * 32 + l32;
    if (p.lse && h == 0 && qrow_l < p.Sq) {
      const long long li = ((long long)b * p.N + n) * p.Sq + qrow_l;
      p.lse[li] = l_tot > 0.f ? m_run[qb] * p.scale + __logf(l_tot) : -INFINITY;
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
      if (qrow < p.Sq) {
        i32x4_t v = {lo[0], lo[1], hi[0], hi[1]};
        *(i32x4_t*)(og + (long long)qrow * p.o_ss + c16 * 8) = v;
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
}

template <int DT, int NWAVES, int QPW, int BN, bool SPARSE>
static int launch_fa(const FaParams& p, hipStream_t stream) {
  using C = FaCfg<DT, NWAVES, QPW, BN, SPARSE>;
  auto kern = fa_fwd_kernel<DT, NWAVES, QPW, BN, SPARSE>;
  static bool configured = false;  // raising the dynamic LDS limit is idempotent
  if (!configured) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, C::kLdsBytes) !=
        hipSuccess)
      return MSD_ERR_LAUNCH;
    configured = true;
  }
  const int q_tiles = (p.Sq + C::kBM - 1) / C::kBM;
  const int total = p.B * p.N * q_tiles;
  const int grid = ((total + 7) / 8) * 8;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(C::kNT), C::kLdsBytes, stream, p);
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

}  // namespace msd

using namespace msd;

extern "C" {

// Tuning hook used by the benchmark sweep: selects the dense kernel variant
// (0: 8 waves x 32 rows, 128-key tiles; 1: 4 waves x 32 rows, 64-key tiles;
//  2: 4 waves x 64 rows, 64-key tiles; 3: 8 waves x 32 rows, 64-key tiles).
static int g_dense_variant = 0;
void mindiesd_set_dense_variant(int v) { g_dense_variant = v; }

int mindiesd_flash_attention_fwd(const void* q, const void* k, const void* v, void* out, float* lse, int dtype,
                                 int B, int N, int Nkv, int Sq, int Skv, int D, long long q_sb, long long q_sn,
                                 long long q_ss, long long k_sb, long long k_sn, long long k_ss, long long v_sb,
                                 long long v_sn, long long v_ss, long long o_sb, long long o_sn, long long o_ss,
                                 float scale, hipStream_t stream) {
  if (!q || !k || !v || !out) return MSD_ERR_BAD_ARG;
  if (B <= 0 || N <= 0 || Nkv <= 0 || Sq <= 0 || Skv <= 0 || N % Nkv != 0) return MSD_ERR_BAD_ARG;
  if (D != 128) return MSD_ERR_UNSUPPORTED;
  if (dtype != MSD_DTYPE_BF16 && dtype != MSD_DTYPE_F16) return MSD_ERR_BAD_ARG;
  // 16-byte vector accesses: every row start must be 16-byte aligned
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) return MSD_ERR_BAD_ARG;
  if ((q_sb | q_sn | q_ss | k_sb | k_sn | k_ss | v_sb | v_sn | v_ss | o_sb | o_sn | o_ss) & 7) return MSD_ERR_BAD_ARG;
  FaParams p{};
  p.q = q; p.k = k; p.v = v; p.o = out; p.lse = lse;
  p.q_sb = q_sb; p.q_sn = q_sn; p.q_ss = q_ss;
  p.k_sb = k_sb; p.k_sn = k_sn; p.k_ss = k_ss;
  p.v_sb = v_sb; p.v_sn = v_sn; p.v_ss = v_ss;
  p.o_sb = o_sb; p.o_sn = o_sn; p.o_ss = o_ss;
  p.B = B; p.N = N; p.Nkv = Nkv; p.Sq = Sq; p.Skv = Skv;
  p.scale = scale;
  p.scale_log2 = scale * 1.4426950408889634f;
  if (dtype == MSD_DTYPE_BF16) {
    switch (g_dense_variant) {
      case 1: return launch_fa<MSD_DTYPE_BF16, 4, 32, 64, false>(p, stream);
      case 2: return launch_fa<MSD_DTYPE_BF16, 4, 64, 64, false>(p, stream);
      case 3: return launch_fa<MSD_DTYPE_BF16, 8, 32, 64, false>(p, stream);
      default: return launch_fa<MSD_DTYPE_BF16, 8, 32, 128, false>(p, stream);
    }
  }
  return launch_fa<MSD_DTYPE_F16, 8, 32, 128, false>(p, stream);
}

}  // extern "C"
