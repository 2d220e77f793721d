// Flash-attention forward for gfx950 (MI355X) at head dims other than 128: bf16/fp16, head_dim a multiple of 8
// up to 256, dense, with the options of the general mode (packed variable-length sequences, bottom-right causal
// mask, boolean attention mask, log-sum-exp output).
//
// The reference's fused dense ops (mindiesd/layers/flash_attn/prompt_flash_attn.py:48,
// fused_attn_score.py:48, csrc/plugin/la.cpp:27-58) take any head_dim the vendor kernels accept; its own tests
// of attention_forward run head_dim 64 (tests/layers/flash_attn/test_attn_forward.py:31-169).  The DiT shapes this
// library is tuned for all have head_dim 128 and run on flash_attn_fwd.hip; this file covers the rest with one
// kernel per padded head_dim DP in {64, 128, 256}.
//
// Same algorithm as flash_attn_fwd.hip (single pass, online softmax, transposed problem S^T = K Q^T,
// O^T += V^T P^T on the 32x32x16 matrix instruction, P^T straight from the score accumulators, V^T by the
// transposing LDS read), with a plain data path instead of the tuned one: K/V tiles of BN keys go through registers
// into LDS (requested one tile ahead, zero-filled beyond head_dim and beyond the sequence, rows padded by 16 bytes
// against bank conflicts), two LDS stages, one barrier per tile.  The reference maximum of the running softmax is
// moved lazily, as in flash_attn_fwd.hip: only when some row of the wave exceeds it by more than 2^kTauHd (or sees
// its first visible key); the score accumulators are seeded with minus the reference, so the exponential applies
// to the matrix result directly and a tile without a move costs no rescaling of the output accumulators.
#include "common.hpp"
#include "fa_params.hpp"

namespace msd {

template <int DP>
struct HdCfg {
  static constexpr int kNW = 4;                      // waves per workgroup, 32 query rows each
  static constexpr int kBM = kNW * 32;
  static constexpr int kBN = DP <= 64 ? 128 : (DP <= 128 ? 64 : 32);  // keys per tile
  static constexpr int kNKB = kBN / 32;
  static constexpr int kCols = DP / 8;               // 16-byte chunks per row
  static constexpr int kRowBytes = DP * 2 + 16;
  static constexpr int kTileBytes = kBN * kRowBytes;
  static constexpr int kStageBytes = 2 * kTileBytes;  // K + V
  static constexpr int kORowBytes = DP * 2 + 8;
  static constexpr int kOutBytes = kNW * 32 * kORowBytes;
  static constexpr int kLds = 2 * kStageBytes > kOutBytes ? 2 * kStageBytes : kOutBytes;
  static constexpr int kChunksPerThread = kBN * kCols / (kNW * 64);
  static_assert(kBN * kCols % (kNW * 64) == 0, "tile chunks must split evenly over the threads");
};

constexpr float kTauHd = 8.0f;  // probabilities stay below 2^8: exact in fp32, representable in bf16 and fp16

// VAR selects what would otherwise be run-time branches around the tile loop (as such they cost the calls that do not
// use them 2 % with the mask and 13 % with the table lookup): 0 = plain (causal and host-sized packed sequences are
// run-time options), 1 = packed numbering - the grid holds p.packed_tiles query tiles per head, numbered through the
// sequences of p.seq_meta -, 2 = boolean mask.
template <int DT, int DP, int VAR = 0>
__global__ __launch_bounds__(256, (DP <= 128 ? 2 : 1)) void fa_hd_kernel(const FaParams p, const int D) {
#if defined(__HIP_DEVICE_COMPILE__)
  using C = HdCfg<DP>;
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

  // consecutive query tiles of one head stay on one XCD (workgroups are dealt round-robin to the 8 XCDs)
  constexpr bool packed = VAR == 1;
  constexpr bool masked = VAR == 2;
  const int q_tiles = packed ? p.packed_tiles : (p.Sq + C::kBM - 1) / C::kBM;
  const int total = (packed ? 1 : p.B) * p.N * q_tiles;
  const int per_xcd = (total + 7) / 8;
  const int work = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (work >= total) return;
  const int bn = work / q_tiles;
  int qt = work - bn * q_tiles;
  int b, n;
  if constexpr (packed) {
    static_assert(C::kBM == 128, "packed numbering counts 128-row tiles");
    n = bn;
    if (!packed_find_tile(p.seq_meta, p.B, qt, b, qt)) return;
    if (p.causal) qt = (p.seq_meta[4 * b + 1] + C::kBM - 1) / C::kBM - 1 - qt;
  } else {
    if (p.causal) qt = q_tiles - 1 - qt;
    b = bn / p.N;
    n = bn - b * p.N;
  }
  const int nkv = n / (p.N / p.Nkv);
  const int q0 = qt * C::kBM;

  const T* qg = (const T*)p.q + b * p.q_sb + n * p.q_sn;
  const T* kg = (const T*)p.k + b * p.k_sb + nkv * p.k_sn;
  const T* vg = (const T*)p.v + b * p.v_sb + nkv * p.v_sn;
  T* og = (T*)p.o + b * p.o_sb + n * p.o_sn;
  int Sq = p.Sq, Skv = p.Skv;
  if (p.seq_meta) {
    const int* meta = p.seq_meta + 4 * b;
    Sq = meta[1];
    Skv = meta[3];
    if (q0 >= Sq) return;
    qg += (long long)meta[0] * p.q_ss;
    og += (long long)meta[0] * p.o_ss;
    kg += (long long)meta[2] * p.k_ss;
    vg += (long long)meta[2] * p.v_ss;
  }
  const int causal_shift = Skv - Sq;

  // ---- Q^T operand, resident: lane (q = l32, h) holds head_dim 16*ks + 8*h .. +8, scale * log2(e) folded in -------
  constexpr int kKS = DP / 16;
  X8 qf[kKS];
  {
    const int qrow = q0 + wave * 32 + l32;
    const bool ok = qrow < Sq;
    const T* src = qg + (long long)(ok ? qrow : 0) * p.q_ss + 8 * h;
#pragma unroll
    for (int ks = 0; ks < kKS; ++ks) {
      X8 v = X8{0};
      if (ok && 16 * ks + 8 * h < D) v = *(const X8*)(src + 16 * ks);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = E::from_float((float)v[j] * p.scale_log2);
      qf[ks] = v;
    }
  }

  constexpr int kDB = DP / 32;
  f32x16_t oacc[kDB];
#pragma unroll
  for (int db = 0; db < kDB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
  // m_run: reference maximum (log2 units) the sums and outputs are expressed in, -inf until the row has seen a
  // visible key; negm: minus that reference (0 while it is -inf) in the 16 slots that seed a score accumulator
  float m_run = -INFINITY, l_run = 0.f;
  f32x16_t negm;
#pragma unroll
  for (int r = 0; r < 16; ++r) negm[r] = 0.f;

  // ---- tile staging: thread t owns chunks t, t + 256, ... of the K tile and of the V tile ---------------------------
  i32x4_t kreg[C::kChunksPerThread], vreg[C::kChunksPerThread];
  auto fetch = [&](int key0) {
#pragma unroll
    for (int i = 0; i < C::kChunksPerThread; ++i) {
      const int ch = tid + i * 256;
      const int row = ch / C::kCols, col = ch - row * C::kCols;
      const int key = key0 + row;
      const bool ok = key < Skv && col * 8 < D;
      kreg[i] = ok ? *(const i32x4_t*)(kg + (long long)key * p.k_ss + col * 8) : i32x4_t{0, 0, 0, 0};
      vreg[i] = ok ? *(const i32x4_t*)(vg + (long long)key * p.v_ss + col * 8) : i32x4_t{0, 0, 0, 0};
    }
  };
  auto stash = [&](int stage) {
    MSD_LDS char* kb = smem + stage * C::kStageBytes;
#pragma unroll
    for (int i = 0; i < C::kChunksPerThread; ++i) {
      const int ch = tid + i * 256;
      const int row = ch / C::kCols, col = ch - row * C::kCols;
      *(MSD_LDS i32x4_t*)(kb + row * C::kRowBytes + col * 16) = kreg[i];
      *(MSD_LDS i32x4_t*)(kb + C::kTileBytes + row * C::kRowBytes + col * 16) = vreg[i];
    }
  };

  int kv_lim = Skv;
  if (p.causal) kv_lim = max(0, min(Skv, q0 + C::kBM + causal_shift));
  const int tiles = (kv_lim + C::kBN - 1) / C::kBN;
  const unsigned char* mask_g = masked ? p.mask + b * p.m_sb + n * p.m_sn : nullptr;

  // V^T operand: the lane addresses key 4*h + (lane%16)/4 (+8 for the second read), head_dim 16*((lane/16)&1) +
  // 4*(lane%4) of a 32-wide block
  const int v_off = (4 * h + ((lane & 15) >> 2)) * C::kRowBytes + 32 * ((lane >> 4) & 1) + 8 * (lane & 3);

  // Boolean mask of a tile that lies wholly inside the sequence: the lane fetches the bytes of its own query row that
  // belong to its score registers as 4-byte words (register r of block kb is key 32 kb + 8 (r / 4) + 4 h + r % 4: one
  // word per r / 4; any alignment - global loads take unaligned addresses), one tile ahead.  With a mask the K/V
  // chunks of the next tile are requested after the mask test instead of at the top of the step, so that the words
  // are never waited for with younger requests in flight.  The tile that runs past the end of the row is tested byte
  // by byte instead (a 4-byte read could leave the mask there).
  unsigned mask_w[C::kNKB][4];
  auto mask_fetch = [&](int key0) __attribute__((always_inline)) {
    const int qrow = min(q0 + wave * 32 + l32, Sq - 1);
    const unsigned char* mrow = mask_g + (long long)qrow * p.m_sq + key0 + 4 * h;
#pragma unroll
    for (int kb = 0; kb < C::kNKB; ++kb)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) __builtin_memcpy(&mask_w[kb][g4], mrow + kb * 32 + 8 * g4, 4);
  };

  if (tiles > 0) {
    if (masked && C::kBN <= Skv) mask_fetch(0);
    fetch(0);
    stash(0);
  }
  __syncthreads();

  for (int t = 0; t < tiles; ++t) {
    const int stage = t & 1;
    const int key0 = t * C::kBN;
    if (!masked && t + 1 < tiles) fetch(key0 + C::kBN);
    MSD_LDS const char* kb_base = smem + stage * C::kStageBytes;
    MSD_LDS const char* vb_base = kb_base + C::kTileBytes;

    // ---- S^T = K Q^T --------------------------------------------------------------------------------------------
    f32x16_t sacc[C::kNKB];
#pragma unroll
    for (int ks = 0; ks < kKS; ++ks)
#pragma unroll
      for (int kb = 0; kb < C::kNKB; ++kb) {
        const X8 a = *(MSD_LDS const X8*)(kb_base + (kb * 32 + l32) * C::kRowBytes + (2 * ks + h) * 16);
        sacc[kb] = E::mfma32(a, qf[ks], ks == 0 ? negm : sacc[kb]);   // = score - reference
      }

    // ---- visibility: end of the sequence, causal diagonal, boolean mask -----------------------------------------
    const int qrow = q0 + wave * 32 + l32;
    const bool edge = key0 + C::kBN > Skv;
    const bool diag = p.causal && key0 + C::kBN - 1 > q0 + wave * 32 + causal_shift;
    if (masked && !edge) {
#pragma unroll
      for (int kb = 0; kb < C::kNKB; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (((mask_w[kb][r >> 2] >> (8 * (r & 3))) & 0xffu) == 0) sacc[kb][r] = -INFINITY;
    }
    if (masked && t + 1 < tiles) {
      if (key0 + 2 * C::kBN <= Skv) mask_fetch(key0 + C::kBN);
      fetch(key0 + C::kBN);
    }
    if (edge || diag) {
      const int last_visible = p.causal ? qrow + causal_shift : 0x7fffffff;
      const unsigned char* mrow = (masked && edge) ? mask_g + (long long)min(qrow, Sq - 1) * p.m_sq : nullptr;
#pragma unroll
      for (int kb = 0; kb < C::kNKB; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = key0 + kb * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
          bool vis = key < Skv && key <= last_visible;
          if (vis && mrow) vis = mrow[key] != 0;
          if (!vis) sacc[kb][r] = -INFINITY;
        }
    }

    // ---- online softmax (exp2 domain) -----------------------------------------------------------------------------
    float mx = sacc[0][0];
#pragma unroll
    for (int kb = 0; kb < C::kNKB; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sacc[kb][r]);
    // mx = the lane's largest score minus the reference (minus 0 while the row has no reference yet).  A lane asks
    // for a move when its part exceeds the threshold or shows the row its first visible key; some lane of a row
    // does so iff the row's maximum does.
    const bool unseen = m_run == -INFINITY;
    if (__builtin_amdgcn_ballot_w64(unseen ? mx > -INFINITY : mx > kTauHd) != 0) {
      mx = half_max(mx);
      // first visible key: the exact row maximum becomes the reference (whatever its sign); later: only upwards
      float delta = unseen ? mx : fmaxf(mx, 0.f);
      delta = (delta == -INFINITY) ? 0.f : delta;
      // (a row without a reference has zero sums and outputs: factor 1, not 2^-delta, which may overflow)
      const float alpha = unseen ? 1.f : fast_exp2(-delta);
      if (!unseen || mx > -INFINITY) m_run = (unseen ? 0.f : m_run) + delta;
      l_run *= alpha;
#pragma unroll
      for (int r = 0; r < 16; ++r) negm[r] = m_run == -INFINITY ? 0.f : -m_run;
#pragma unroll
      for (int kb = 0; kb < C::kNKB; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[kb][r] -= delta;
#pragma unroll
      for (int db = 0; db < kDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
    }
    X8 pf[C::kNKB][2];
    float ls = 0.f;
#pragma unroll
    for (int kb = 0; kb < C::kNKB; ++kb)
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) {
        X8 pk;
#pragma unroll
        for (int j = 0; j < 8; ++j) pk[j] = E::from_float(fast_exp2(sacc[kb][8 * t2 + j]));
        pf[kb][t2] = pk;
        ls = E::sum8(pk, ls);  // the sum of the rounded probabilities, the values the second product uses
      }
    l_run += ls;

    // ---- O^T += V^T P^T ---------------------------------------------------------------------------------------------
#pragma unroll
    for (int kb = 0; kb < C::kNKB; ++kb)
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
        for (int db = 0; db < kDB; ++db) {
          MSD_LDS const char* src = vb_base + (kb * 32 + 16 * t2) * C::kRowBytes + v_off + db * 64;
          union { s16x4_t s[2]; X8 x; } u;
          u.s[0] = lds_read_tr16((const void*)src);
          u.s[1] = lds_read_tr16((const void*)(src + 8 * C::kRowBytes));
          oacc[db] = E::mfma32(u.x, pf[kb][t2], oacc[db]);
        }

    if (t + 1 < tiles) stash(stage ^ 1);
    __syncthreads();
  }

  // ---- epilogue: normalise, transpose the wave's 32 rows through LDS, 16-byte stores --------------------------------
  MSD_LDS char* ost = smem + wave * 32 * C::kORowBytes;
  const float l_tot = half_sum(l_run);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  {
    const int qrow = q0 + wave * 32 + l32;
    if (p.lse && h == 0 && qrow < Sq) {
      long long li = ((long long)b * p.N + n) * p.Sq + qrow;
      if (p.seq_meta && p.lse_token_major) li = ((long long)p.seq_meta[4 * b] + qrow) * p.N + n;
      p.lse[li] = l_tot > 0.f ? m_run * 0.6931471805599453f + __logf(l_tot) : -INFINITY;
    }
  }
#pragma unroll
  for (int db = 0; db < kDB; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      typename E::x4 pk;
#pragma unroll
      for (int j = 0; j < 4; ++j) pk[j] = E::from_float(oacc[db][4 * g + j] * inv);
      *(MSD_LDS typename E::x4*)(ost + l32 * C::kORowBytes + (db * 32 + 8 * g + 4 * h) * 2) = pk;
    }
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int i = 0; i < 32 * C::kCols / 64; ++i) {
    const int ch = i * 64 + lane;
    const int row = ch / C::kCols, col = ch - row * C::kCols;
    const int qrow = q0 + wave * 32 + row;
    const i32x2_t lo = *(MSD_LDS const i32x2_t*)(ost + row * C::kORowBytes + col * 16);
    const i32x2_t hi = *(MSD_LDS const i32x2_t*)(ost + row * C::kORowBytes + col * 16 + 8);
    if (qrow < Sq && col * 8 < D) {
      const i32x4_t v = {lo[0], lo[1], hi[0], hi[1]};
      *(i32x4_t*)(og + (long long)qrow * p.o_ss + col * 8) = v;
    }
  }
#endif  // __HIP_DEVICE_COMPILE__
}

template <int DT, int DP, int VAR>
static int launch_hd_p(const FaParams& p, int D, hipStream_t stream) {
  using C = HdCfg<DP>;
  constexpr bool PACKED = VAR == 1;
  auto kern = fa_hd_kernel<DT, DP, VAR>;
  if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, C::kLds) != hipSuccess)
    return MSD_ERR_LAUNCH;
  const long long total = PACKED ? (long long)p.N * p.packed_tiles
                                 : (long long)p.B * p.N * ((p.Sq + C::kBM - 1) / C::kBM);
  if (total > 0x7ffffff0ll) return MSD_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(kern, dim3((unsigned)((total + 7) / 8 * 8)), dim3(256), C::kLds, stream, p, D);
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

template <int DT, int DP>
static int launch_hd(const FaParams& p, int D, hipStream_t stream) {
  if (p.packed_tiles > 0) return launch_hd_p<DT, DP, 1>(p, D, stream);  // (never together with a mask)
  return p.mask ? launch_hd_p<DT, DP, 2>(p, D, stream) : launch_hd_p<DT, DP, 0>(p, D, stream);
}

int launch_fa_hd(const FaParams& p, int dtype, int D, hipStream_t stream) {
  if (D <= 0 || D > 256 || (D & 7)) return MSD_ERR_UNSUPPORTED;
  const bool bf = dtype == MSD_DTYPE_BF16;
  if (D <= 64) return bf ? launch_hd<MSD_DTYPE_BF16, 64>(p, D, stream) : launch_hd<MSD_DTYPE_F16, 64>(p, D, stream);
  if (D <= 128) return bf ? launch_hd<MSD_DTYPE_BF16, 128>(p, D, stream) : launch_hd<MSD_DTYPE_F16, 128>(p, D, stream);
  return bf ? launch_hd<MSD_DTYPE_BF16, 256>(p, D, stream) : launch_hd<MSD_DTYPE_F16, 256>(p, D, stream);
}

}  // namespace msd
