// FP8 (OCP E4M3) attention for gfx950 (MI355X): quantisation passes + flash-attention forward on
// the fp8 matrix cores (v_mfma_f32_32x32x64_f8f6f4, twice the bf16 rate).
//
// Takes the place of the vendor ops behind the reference's FP8 attention path:
//   fa_block_quant_preprocess / npu_dynamic_block_quant   mindiesd/layers/quant/block_quant.py:19-48
//   FP8RotateQuantFA -> npu_fused_infer_attention_score_v2 mindiesd/quantization/layer.py:283-324
//
// Recipe (Wan2.1-14B 480p workload): Q and K as E4M3 with one fp32 scale per (head, 128-token block)
// over all 128 channels, V as E4M3 with one fp32 scale per (head, channel), P re-quantised to E4M3
// per tile, fp32 accumulation, 16-bit output.
//
// Layouts produced by the quantisation pass and consumed by the attention kernel:
//   Q8, K8 : [B][N][S][128] bytes, row major.
//   V8T    : [B][N][128][S128] bytes (S rounded up to 128, zero padded), i.e. V transposed so that
//            a lane of the second product reads its 32 keys as 32 contiguous bytes.  Inside every
//            group of 64 keys the keys are stored in the order in which the S^T accumulator of the
//            first product hands them to the second one: position 32*h + j holds key
//            32*(j/16) + 8*((j%16)/4) + 4*h + j%4   (h = 0,1 the wave half, j = 0..31).
#include <mutex>
#include <type_traits>

#include "common.hpp"

// (batch x head) pairs that mindiesd_fp8_v_quant_static accepts: its scratch is a fixed device array
#define MINDIESD_FP8_V_QUANT_STATIC_MAX_HEADS 4096

namespace msd {

constexpr float kE4M3Max = 448.0f;
constexpr int kMaxDevices = 64;  // device ordinals the per-device scratch table covers

__device__ __forceinline__ float clamp448(float x) { return __builtin_amdgcn_fmed3f(x, -kE4M3Max, kE4M3Max); }

// four floats -> four E4M3 bytes (RNE, saturating), first value in the lowest byte
__device__ __forceinline__ int pack4_e4m3(float a, float b, float c, float d) {
  int w = 0;
  w = __builtin_amdgcn_cvt_pk_fp8_f32(clamp448(a), clamp448(b), w, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(clamp448(c), clamp448(d), w, true);
  return w;
}
// probabilities are already inside the range: no clamp
__device__ __forceinline__ int pack4_e4m3_noclamp(float a, float b, float c, float d) {
  int w;
  asm volatile("" : "=v"(w));  // any register content: both halves are overwritten (saves the move zero would cost)
  w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, w, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
  return w;
}

// Quantisation scale of a block with maximum magnitude amax: amax / 448, or (pow2) the smallest power of two
// that is not below it, so that the scale can later be applied by the matrix instruction's exponent operand.
__device__ __forceinline__ float block_scale(float amax, int pow2) {
  if (!(amax > 0.f)) return 1.0f;
  const float sc = __fdiv_rn(amax, kE4M3Max);
  if (!pow2) return sc;
  const unsigned bits = __builtin_bit_cast(unsigned, sc);
  const unsigned e = max((bits >> 23) + ((bits & 0x7fffffu) ? 1u : 0u), 1u);  // at least 2^-126
  return __builtin_bit_cast(float, e << 23);
}

template <int DT>
__device__ __forceinline__ void load8(const typename Elem<DT>::type* p, float (&f)[8]) {
  union { i32x4_t v; typename Elem<DT>::type e[8]; } u;
  u.v = *(const i32x4_t*)p;
#pragma unroll
  for (int j = 0; j < 8; ++j) f[j] = (float)u.e[j];
}

__device__ __forceinline__ float block_max_256(float v, float* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  v = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  return v;
}

// ---- block quantisation: one scale per (batch, head, `bs` tokens) over all 128 channels --------------
// x [B][N][S][128] (strided) -> q [B][N][S][128] bytes (contiguous), scale [B][N][ceil(S/bs)].
template <int DT>
__global__ __launch_bounds__(256) void block_quant_kernel(const void* x_, unsigned char* q, float* scale,
                                                          long long sb, long long sn, long long ss, int N, int S,
                                                          int bs, float prescale, int pow2) {
#if defined(__HIP_DEVICE_COMPILE__)
  using T = typename Elem<DT>::type;
  __shared__ float red[4];
  const int blk = blockIdx.x, bn = blockIdx.y;
  const int b = bn / N, n = bn - b * N;
  const int nblk = gridDim.x;
  const T* x = (const T*)x_ + b * sb + n * sn;
  const int row0 = blk * bs, rows = min(bs, S - row0);
  const int c16 = threadIdx.x & 15, rgrp = threadIdx.x >> 4;
  float amax = 0.f;
  for (int r = rgrp; r < rows; r += 16) {
    float f[8];
    load8<DT>(x + (long long)(row0 + r) * ss + c16 * 8, f);
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(__fmul_rn(f[j], prescale)));
  }
  amax = block_max_256(amax, red);
  const float sc = block_scale(amax, pow2);
  if (threadIdx.x == 0) scale[(long long)bn * nblk + blk] = sc;
  unsigned char* qo = q + ((long long)bn * S + row0) * 128 + c16 * 8;
  for (int r = rgrp; r < rows; r += 16) {
    float f[8];
    load8<DT>(x + (long long)(row0 + r) * ss + c16 * 8, f);   // second read hits L2
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = __fdiv_rn(__fmul_rn(f[j], prescale), sc);
    i32x2_t w = {pack4_e4m3(f[0], f[1], f[2], f[3]), pack4_e4m3(f[4], f[5], f[6], f[7])};
    *(i32x2_t*)(qo + (long long)r * 128) = w;
  }
#endif
}

// The same for blocks of BS = 128 or 256 tokens with the block held in registers: a thread requests its
// BS / 16 rows x 8 channels at once (more requests in flight than the row loop above) and quantises them without a
// second read.
template <int DT, int BS>
__global__ __launch_bounds__(256) void block_quant_reg_kernel(const void* x_, unsigned char* q, float* scale,
                                                             long long sb, long long sn, long long ss, int N, int S,
                                                             float prescale, int pow2) {
#if defined(__HIP_DEVICE_COMPILE__)
  using T = typename Elem<DT>::type;
  constexpr int kRows = BS / 16;  // rows per thread
  __shared__ float red[4];
  const int blk = blockIdx.x, bn = blockIdx.y;
  const int b = bn / N, n = bn - b * N;
  const int nblk = gridDim.x;
  const T* x = (const T*)x_ + b * sb + n * sn;
  const int row0 = blk * BS, rows = min(BS, S - row0);
  const int c16 = threadIdx.x & 15, rgrp = threadIdx.x >> 4;
  union { i32x4_t v; T e[8]; } u[kRows];
#pragma unroll
  for (int i = 0; i < kRows; ++i) {
    const int r = rgrp + 16 * i;
    u[i].v = i32x4_t{0, 0, 0, 0};
    if (r < rows) u[i].v = *(const i32x4_t*)(x + (long long)(row0 + r) * ss + c16 * 8);
  }
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < kRows; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(__fmul_rn((float)u[i].e[j], prescale)));
  amax = block_max_256(amax, red);
  const float sc = block_scale(amax, pow2);
  if (threadIdx.x == 0) scale[(long long)bn * nblk + blk] = sc;
  unsigned char* qo = q + ((long long)bn * S + row0) * 128 + c16 * 8;
#pragma unroll
  for (int i = 0; i < kRows; ++i) {
    const int r = rgrp + 16 * i;
    float f[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = __fdiv_rn(__fmul_rn((float)u[i].e[j], prescale), sc);
    const i32x2_t w = {pack4_e4m3(f[0], f[1], f[2], f[3]), pack4_e4m3(f[4], f[5], f[6], f[7])};
    if (r < rows) *(i32x2_t*)(qo + (long long)r * 128) = w;
  }
#endif
}

// ---- rotation + block quantisation in one pass ------------------------------------------------------------------
// y = x @ R (R a fixed [128][128] matrix, e.g. a Hadamard rotation that spreads outliers over the channels),
// y rounded to the 16-bit input type as a separate matmul would leave it, then quantised like
// block_quant_kernel with 128-token blocks.  x is read once and only the E4M3 codes are written: 3 bytes
// per element instead of the 7 of matmul + quantisation.
// One workgroup = one 128-token block; R^T sits in LDS (16-byte chunk c of row n at chunk c ^ (n & 15)); wave w
// owns tokens 32w..32w+31.  R^T is the first matrix operand, so a lane holds one token and, per register
// quad, four consecutive output channels = one dword of codes.
// (launch bounds: at least 4 waves per SIMD = 128 registers per lane, so that the four workgroups whose LDS fits a CU
// are resident together - the pass is bound by memory latency)
template <int DT>
__global__ __launch_bounds__(256, 4) void rot_block_quant_kernel(const void* x_, const void* rot_t_, unsigned char* q,
                                                              float* scale, long long sb, long long sn, long long ss,
                                                              int N, int S, float prescale, int pow2) {
#if defined(__HIP_DEVICE_COMPILE__)
  using E = Elem<DT>;
  using T = typename E::type;
  using X8 = typename E::x8;
  __shared__ __attribute__((aligned(16))) char rt_lds[128 * 256];
  __shared__ float red[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, h = lane >> 5;
  const int blk = blockIdx.x, bn = blockIdx.y;
  const int b = bn / N, n = bn - b * N;
  const int nblk = gridDim.x;
  const T* x = (const T*)x_ + b * sb + n * sn;
  const int row0 = blk * 128;
  // R^T [out channel][in channel] -> LDS
  const char* rt = (const char*)rot_t_;
#pragma unroll
  for (int pass = 0; pass < 8; ++pass) {
    const int row = pass * 16 + (tid >> 4), c = tid & 15;
    *(i32x4_t*)(rt_lds + row * 256 + ((c ^ (row & 15)) << 4)) = *(const i32x4_t*)(rt + row * 256 + c * 16);
  }
  // this lane's token: in channels 16ks + 8h .. +7 for ks = 0..7
  const int tok = row0 + wave * 32 + l32;
  const bool ok = tok < S;
  X8 xf[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    xf[ks] = *(const X8*)(x + (long long)(ok ? tok : 0) * ss + 16 * ks + 8 * h);
    if (!ok) xf[ks] = X8{0};
  }
  __syncthreads();
  f32x16_t acc[4];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb) {
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[nb][r] = 0.f;
    const int row = nb * 32 + l32;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      const X8 rf = *(const X8*)(rt_lds + row * 256 + (((2 * ks + h) ^ (row & 15)) << 4));
      acc[nb] = E::mfma32(rf, xf[ks], acc[nb]);
    }
  }
  // round to the 16-bit type (what a separate matmul would have stored), block maximum
  float amax = 0.f;
#pragma unroll
  for (int nb = 0; nb < 4; ++nb)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      acc[nb][r] = __fmul_rn((float)E::from_float(acc[nb][r]), prescale);
      amax = fmaxf(amax, fabsf(acc[nb][r]));
    }
  amax = block_max_256(amax, red);
  const float sc = block_scale(amax, pow2);
  if (tid == 0) scale[(long long)bn * nblk + blk] = sc;
  // The codes of a token (128 bytes) are spread over the lanes in dwords; they go through LDS (R^T is no longer
  // needed: block_max_256 has synchronised the workgroup after the last matrix instruction) so that the stores to
  // global memory are whole 16-byte chunks of consecutive rows.  16-byte chunk c of token row r sits at chunk
  // c ^ (r & 7).
  {
    const int r = wave * 32 + l32;
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int w = pack4_e4m3(__fdiv_rn(acc[nb][4 * g], sc), __fdiv_rn(acc[nb][4 * g + 1], sc),
                                 __fdiv_rn(acc[nb][4 * g + 2], sc), __fdiv_rn(acc[nb][4 * g + 3], sc));
        const int byte = nb * 32 + 8 * g + 4 * h;
        *(int*)(rt_lds + r * 128 + (((byte >> 4) ^ (r & 7)) << 4) + (byte & 15)) = w;
      }
  }
  __syncthreads();
  unsigned char* qo = q + ((long long)bn * S + row0) * 128;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = (tid >> 3) + 32 * i, c = tid & 7;
    const i32x4_t w = *(const i32x4_t*)(rt_lds + r * 128 + ((c ^ (r & 7)) << 4));
    if (row0 + r < S) *(i32x4_t*)(qo + (long long)r * 128 + c * 16) = w;
  }
#endif
}

// ---- V: per-channel maximum over the sequence ------------------------------------------------------------
__global__ void fill_u32_kernel(unsigned* p, unsigned v, long long n) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

// amax_bits [B][N][128] must be zero-filled; non-negative floats order like their bit patterns.
template <int DT>
__global__ __launch_bounds__(256) void channel_amax_kernel(const void* v_, unsigned* amax_bits, long long sb,
                                                           long long sn, long long ss, int N, int S) {
#if defined(__HIP_DEVICE_COMPILE__)
  using T = typename Elem<DT>::type;
  __shared__ float part[16][128];
  const int bn = blockIdx.y, b = bn / N, n = bn - b * N;
  const T* v = (const T*)v_ + b * sb + n * sn;
  const int c16 = threadIdx.x & 15, rgrp = threadIdx.x >> 4;
  const int row0 = blockIdx.x * 1024, rows = min(1024, S - row0);
  float m[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) m[j] = 0.f;
  // 8 rows of a thread are requested before the first one is used (rows past the end read row 0 again)
  for (int r0 = rgrp; r0 < rows; r0 += 128) {
    union { i32x4_t v; T e[8]; } u[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int r = r0 + 16 * i;
      u[i].v = *(const i32x4_t*)(v + (long long)(row0 + (r < rows ? r : 0)) * ss + c16 * 8);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) m[j] = fmaxf(m[j], fabsf((float)u[i].e[j]));
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) part[rgrp][c16 * 8 + j] = m[j];
  __syncthreads();
  if (threadIdx.x < 128) {
    float a = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) a = fmaxf(a, part[r][threadIdx.x]);
    atomicMax(amax_bits + (long long)bn * 128 + threadIdx.x, __builtin_bit_cast(unsigned, a));
  }
#endif
}

// position of key kk (0..63) inside its 64-key group of V8T
__host__ __device__ __forceinline__ int v8t_pos(int kk) {
  const int blk32 = kk >> 5, r = kk & 31;
  const int g8 = r >> 3, within = r & 7;
  const int h = within >> 2, e = within & 3;
  return 32 * h + 16 * blk32 + 4 * g8 + e;
}

// V [B][N][S][128] -> V8T [B][N][128][S128] bytes + per-channel scale [B][N][128] = amax/448.
// One workgroup = 128 keys of one (batch, head): every channel row it writes is one full 128-byte line.
// A thread takes 8 channels of two groups of 4 consecutive keys: 4 consecutive keys are 4 consecutive positions of
// V8T (v8t_pos), so their codes of one channel leave as one dword.  LDS tile [channel][128 positions], 16-byte chunk
// c of a row stored at chunk c ^ ((channel >> 3) & 7): the 16 threads of a key group, 8 channels apart, then write
// to 8 different bank groups.
template <int DT>
__global__ __launch_bounds__(256) void v_quant_transpose_kernel(const void* v_, const unsigned* amax_bits,
                                                                unsigned char* v8t, float* vscale, long long sb,
                                                                long long sn, long long ss, int N, int S, int S128) {
#if defined(__HIP_DEVICE_COMPILE__)
  using T = typename Elem<DT>::type;
  __shared__ __attribute__((aligned(16))) unsigned char tile[128 * 128];
  const int grp = blockIdx.x, bn = blockIdx.y, b = bn / N, n = bn - b * N;
  const T* v = (const T*)v_ + b * sb + n * sn;
  const int c16 = threadIdx.x & 15, qd = threadIdx.x >> 4;
  float sc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float a = __builtin_bit_cast(float, amax_bits[(long long)bn * 128 + c16 * 8 + j]);
    sc[j] = a > 0.f ? __fdiv_rn(a, kE4M3Max) : 1.0f;
  }
  if (grp == 0 && qd == 0) {
#pragma unroll
    for (int j = 0; j < 8; ++j) vscale[(long long)bn * 128 + c16 * 8 + j] = sc[j];
  }
  // keys 4 * qd + j and 64 + 4 * qd + j (j < 4): all 8 rows are requested before the first one is used
  union { i32x4_t v; T e[8]; } u[2][4];
#pragma unroll
  for (int half = 0; half < 2; ++half)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int key = grp * 128 + half * 64 + 4 * qd + j;
      u[half][j].v = i32x4_t{0, 0, 0, 0};
      if (key < S) u[half][j].v = *(const i32x4_t*)(v + (long long)key * ss + c16 * 8);
    }
  const int swz = c16 & 7;  // (channel >> 3) & 7 of this thread's channels
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int pos = half * 64 + v8t_pos(4 * qd);  // multiple of 4
    const int off = (((pos >> 4) ^ swz) << 4) + (pos & 15);
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const int w = pack4_e4m3(__fdiv_rn((float)u[half][0].e[c], sc[c]), __fdiv_rn((float)u[half][1].e[c], sc[c]),
                               __fdiv_rn((float)u[half][2].e[c], sc[c]), __fdiv_rn((float)u[half][3].e[c], sc[c]));
      *(int*)&tile[(c16 * 8 + c) * 128 + off] = w;
    }
  }
  __syncthreads();
  // 128 channel rows x 128 bytes: 8 lanes write one row
  for (int i = threadIdx.x; i < 128 * 8; i += 256) {
    const int ch = i >> 3, part = i & 7;
    const i32x4_t w = *(const i32x4_t*)&tile[ch * 128 + ((part ^ ((ch >> 3) & 7)) << 4)];
    *(i32x4_t*)(v8t + ((long long)bn * 128 + ch) * S128 + grp * 128 + part * 16) = w;
  }
#endif
}

// ---- attention ------------------------------------------------------------------------------------------------
struct Fp8Params {
  const unsigned char* q8;
  const unsigned char* k8;
  const unsigned char* v8t;
  const float* q_scale;  // [B][N][ceil(Sq/128)]
  const float* k_scale;  // [B][N][ceil(Skv/128)], or [B][N][ceil(Skv/256)] with k_shift = 1
  const float* v_scale;  // [B][N][128]
  void* o;
  long long o_sb, o_sn, o_ss;
  int B, N, Sq, Skv, S128;
  float scale_log2;  // softmax scale * log2(e)
  int k_shift;       // a K scale covers 128 << k_shift keys
};

// Two rules for the E4M3 probabilities of a tile (x = score - reference maximum, in log2 units):
//  * PL = false ("exp2"): P = 2^(x + kPShift) by v_exp_f32, rounded by v_cvt_pk_fp8_f32.  With the lazy-maximum
//    threshold kTau8 the largest value is 2^(kTau8 + kPShift) = 256 <= 448 and values down to 2^-13 survive as
//    subnormals.
//  * PL = true ("linear", the default): the E4M3 CODE itself is computed, code = rne(8 * (x + kShiftL + 7)) saturated
//    to [0, 255] by v_cvt_pk_u8_f32.  An E4M3 code read as an integer is 8 * (exponent + 7) + mantissa eighths, so
//    this is 2^floor(x') * (1 + frac(x')) with frac rounded to eighths (x' = x + kShiftL): the exponential with its
//    mantissa interpolated linearly between powers of two, at most 6 % above 2^x'.  The denominator is summed from
//    the same codes, so the common factor cancels; what is left is a relative error of 3 % rms per probability, the
//    size of the E4M3 rounding itself.  One multiply-add and one conversion per score replace multiply-add,
//    exponential and half an E4M3 pack (the two quarter-rate instructions of the other rule).  Codes below 8
//    (x' < -6) are the format's subnormals, where the linear rule falls off faster than 2^x'; the shift is therefore
//    as large as E4M3 allows (2^(kTauL + kShiftL) = 2^8.75 = 431 <= 448, code 126) so that only probabilities below
//    2^-13.75 of the reference maximum are affected, and the threshold for moving the reference is 2^kTauL.
constexpr float kTau8 = 4.0f;
constexpr float kPShift = 4.0f;
constexpr float kTauL = 1.0f;
constexpr float kShiftL = 7.75f;
constexpr float kSeedL = 8.0f * (kShiftL + 7.0f);  // the code of x = 0

// 8 waves x 32 query rows, 128-key tiles, K tile [key][128 B] and V^T tile [channel][128 B] in LDS
// (16 KiB each, double buffered); 16-byte chunk c of row r is stored at chunk c ^ ((r >> 1) & 7).
// P2 (log2 domain): q_scale and k_scale are powers of two and the query codes already carry the softmax scale
// times log2(e).  The two scales then go into the exponent operands of the scaled matrix instruction and the
// score accumulators are seeded with kPShift - m, so the matrix core delivers s - m + kPShift and the softmax is
// exp2 and rounding alone (no multiply-add per score).
// (launch bounds: 8 waves per workgroup, at least 2 waves per SIMD = the one workgroup a CU holds with 96 KiB of LDS;
// the register budget is 256 per lane)
template <int DT, bool P2, bool PL>
__global__ __launch_bounds__(512, 2) void fp8_fa_fwd_kernel(const Fp8Params p) {
#if defined(__HIP_DEVICE_COMPILE__)
  using E = Elem<DT>;
  using T = typename E::type;
  constexpr int NW = 8, BM = 256, BN = 128;
  constexpr int kTile = BN * 128;        // bytes of one K (or V^T) tile
  constexpr int kStage = 2 * kTile;
  constexpr int kORow = 256 + 8;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  MSD_LDS char* smem = (MSD_LDS char*)smem_raw;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, h = lane >> 5;

  const int q_tiles = (p.Sq + BM - 1) / BM;
  const int total = p.B * p.N * q_tiles;
  const int per_xcd = (total + 7) / 8;
  const int work = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (work >= total) return;
  const int bn = work / q_tiles, qt = work - bn * q_tiles;
  const int b = bn / p.N, n = bn - b * p.N;
  const int q0 = qt * BM;
  const int qblocks = (p.Sq + 127) / 128, kblocks = (p.Skv + 127) / 128;
  const int n_tiles = kblocks;

  // Q^T operand: lane (q = l32, h) holds bytes 64*ks + 32*h .. +32 of its row
  const int qrow = q0 + wave * 32 + l32;
  const bool q_ok = qrow < p.Sq;
  const unsigned char* qsrc = p.q8 + ((long long)bn * p.Sq + (q_ok ? qrow : 0)) * 128 + 32 * h;
  i32x8_t qf[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    const i32x4_t lo = *(const i32x4_t*)(qsrc + 64 * ks), hi = *(const i32x4_t*)(qsrc + 64 * ks + 16);
    qf[ks] = q_ok ? i32x8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]} : i32x8_t{0, 0, 0, 0, 0, 0, 0, 0};
  }
  // all 32 rows of a wave lie in one 128-row scale block
  const int qblk = min((q0 + wave * 32) >> 7, qblocks - 1);
  const float q_sc_raw = p.q_scale[(long long)bn * qblocks + qblk];
  const float q_sc = q_sc_raw * p.scale_log2;
  // E8M0 code of a power of two; the factor 8 of the linear code rule rides on it
  const int q_exp = (int)((__builtin_bit_cast(unsigned, q_sc_raw) >> 23) & 0xffu) + (PL ? 3 : 0);
  // seed of the score accumulators at reference 0, lazy threshold and units per log2 step in the accumulator's domain
  constexpr float kSeed = PL ? kSeedL : kPShift;
  constexpr float kUnit = PL ? 8.0f : 1.0f;
  constexpr float kTau = PL ? kTauL : kTau8;
  // read through the constant address space: a scalar load, which does not queue behind the tile requests
  typedef const __attribute__((address_space(4))) float* ConstF;
  const int k_shift = p.k_shift;
  const ConstF k_sc = (ConstF)(uintptr_t)(p.k_scale + (long long)bn * ((kblocks + (1 << k_shift) - 1) >> k_shift));

  f32x16_t oacc[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
  float m_run = P2 ? 0.f : -INFINITY;
  f32x16_t negm;  // P2: kSeed - kUnit * m_run in every slot, the seed of the score accumulators
#pragma unroll
  for (int r = 0; r < 16; ++r) negm[r] = kSeed;
  bool first = true;

  // ---- LDS-DMA staging: one instruction = 8 rows x 128 bytes ----------------------------------------------------
  const unsigned char* kg = p.k8 + (long long)bn * p.Skv * 128;
  const unsigned char* vg = p.v8t + (long long)bn * 128 * p.S128;
  const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)kg, 0, p.Skv * 128, 0x00020000);
  const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)vg, 0, 128 * p.S128, 0x00020000);
  int k_voff[2], v_voff[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = 8 * (i * NW + wave) + (lane >> 3);
    const int c = (lane & 7) ^ ((row >> 1) & 7);
    k_voff[i] = row * 128 + c * 16;          // + key0 * 128 (scalar)
    v_voff[i] = row * p.S128 + c * 16;       // + key0 (scalar); row = channel
  }
  auto load_tile = [&](int t, int stage) {
    MSD_LDS char* kb = smem + stage * kStage;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int g = i * NW + wave;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(k_rsrc, (MSD_LDS void*)(kb + g * 1024), 16, k_voff[i], t * BN * 128, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(v_rsrc, (MSD_LDS void*)(kb + kTile + g * 1024), 16, v_voff[i], t * BN, 0,
                                               0);
    }
  };

  // operand read addresses: row = blk*32 + l32, bytes 64*ks + 32*h .. +32 = chunks 4*ks + 2*h, +1 of the row.  The
  // four per-lane addresses (k step x half of the 32 bytes) are kept in registers; stage, operand and 32-row block
  // are compile-time constants that go into the offset field of the reads.
  const int row_off = l32 * 128;
  const int swz = (l32 >> 1) & 7;
  unsigned rd[2][2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
#pragma unroll
    for (int j = 0; j < 2; ++j)
      rd[ks][j] = (unsigned)(uintptr_t)smem + row_off + (((4 * ks + 2 * h + j) ^ swz) << 4);

  // Row sums come from the matrix core: one extra MFMA per 64 keys with an all-ones A operand
  // leaves sum_k P8[k][q] in every row of lacc, so the softmax needs no per-element additions and
  // the denominator is built from exactly the quantised probabilities the numerator uses.
  f32x16_t lacc;
#pragma unroll
  for (int r = 0; r < 16; ++r) lacc[r] = 0.f;
  const i32x8_t ones8 = {0x38383838, 0x38383838, 0x38383838, 0x38383838,
                         0x38383838, 0x38383838, 0x38383838, 0x38383838};  // E4M3 1.0

  // three stages: tile t + 2 is requested when tile t starts, so a request has two tile times to land
  if (n_tiles > 0) load_tile(0, 0);
  if (n_tiles > 1) load_tile(1, 1);
  __builtin_amdgcn_s_waitcnt(0x0f74);  // all but the four requests of tile 1
  __syncthreads();

  // The K scale of a tile is fetched one tile ahead.
  float k_sc_cur = n_tiles > 0 ? k_sc[0] : 0.f;
  auto tile_step = [&](const int t, auto stage_c) {
    constexpr int stage = decltype(stage_c)::value;
    const float k_sc_next = k_sc[(t + 1 < n_tiles ? t + 1 : t) >> k_shift];
    // issued after the last tile as well (past the end of the buffers: nobody uses it), so that the number of
    // requests in flight is the same on every path
    load_tile(t + 2, (stage + 2) % 3);

    // ---- S^T = K Q^T (fp8, unscaled form of the scaled MFMA) ---------------------------------------------------
    f32x16_t sacc[4];
    const int k_exp = (int)((__builtin_bit_cast(unsigned, k_sc_cur) >> 23) & 0xffu);
    // the first product of a chain takes its seed as the C operand: kPShift - m (P2) or the constant zero (no
    // accumulator is cleared by moves)
    const f32x16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        constexpr int kOff = stage * kStage;
        const i32x4_t lo = *(MSD_LDS const i32x4_t*)(uintptr_t)(rd[ks][0] + kOff + kb * 32 * 128);
        const i32x4_t hi = *(MSD_LDS const i32x4_t*)(uintptr_t)(rd[ks][1] + kOff + kb * 32 * 128);
        const i32x8_t a = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        if (P2)
          sacc[kb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, qf[ks], ks == 0 ? negm : sacc[kb], 0, 0, 0,
                                                                     k_exp, 0, q_exp);
        else
          sacc[kb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, qf[ks], ks == 0 ? zero16 : sacc[kb], 0, 0, 0, 0,
                                                                     0, 0);
      }
    }

    const int key0 = t * BN;
    if (key0 + BN > p.Skv) {
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (key0 + kb * 32 + 8 * (r >> 2) + 4 * h + (r & 3) >= p.Skv) sacc[kb][r] = -INFINITY;
    }

    // ---- online softmax (exp2 domain, lazily moved reference maximum), P -> E4M3 -------------------------------
    const float c = q_sc * k_sc_cur;  // dequantisation scales of this tile folded into the softmax scale
    k_sc_cur = k_sc_next;
    float mx = sacc[0][0];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sacc[kb][r]);
    i32x8_t pf[2];
    if (P2) {
      // sacc = kUnit * (s - m_run) + kSeed; the reference maximum moves when a row exceeds it by more than kTau
      // (tested on the lanes' own parts: one of them exceeds the threshold iff a row maximum does)
      mx = (mx - kSeed) * (1.0f / kUnit);
      if (first || __builtin_amdgcn_ballot_w64(mx > kTau) != 0) {
        mx = half_max(mx);
        float delta = first ? mx : fmaxf(mx, 0.f);
        delta = (delta == -INFINITY) ? 0.f : delta;
        // (first tile: sums and outputs are still zero; 2^-delta would overflow for rows far below zero and 0 * inf is NaN)
        const float alpha = first ? 1.f : fast_exp2(-delta);
        m_run += delta;
#pragma unroll
        for (int r = 0; r < 16; ++r) negm[r] = kSeed - kUnit * m_run;
#pragma unroll
        for (int kb = 0; kb < 4; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) sacc[kb][r] -= kUnit * delta;
#pragma unroll
        for (int r = 0; r < 16; ++r) lacc[r] *= alpha;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
      }
      first = false;
    } else {
    mx *= c;
    if (__builtin_amdgcn_ballot_w64(mx > m_run + kTau) != 0) {
      mx = half_max(mx);
      const float m_new = fmaxf(m_run, mx);
      const float alpha = fast_exp2(m_run - (m_new == -INFINITY ? 0.f : m_new));
      m_run = m_new;
#pragma unroll
      for (int r = 0; r < 16; ++r) lacc[r] *= alpha;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
    }
    }  // !P2
    const float mc = P2 ? 0.f : (m_run == -INFINITY ? 0.f : m_run) - kPShift;
    // linear rule: code = c8 * raw score + off8 with off8 = kSeedL - 8 * reference
    const float c8 = c * 8.0f;
    const float off8 = __builtin_fmaf(-8.0f, m_run == -INFINITY ? 0.f : m_run, kSeedL);
    // probabilities of keys 64 * kk .. + 64 of the tile, rounded to E4M3 and packed as the B operand
    auto exp_pack = [&](const int kk) {
#pragma unroll
      for (int kb = 2 * kk; kb < 2 * kk + 2; ++kb) {
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          if (PL) {
            unsigned w;
            asm volatile("" : "=v"(w));  // any register content: all four bytes are overwritten
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const float y = P2 ? sacc[kb][4 * g4 + j] : __builtin_fmaf(sacc[kb][4 * g4 + j], c8, off8);
              w = __builtin_amdgcn_cvt_pk_u8_f32(y, j, w);
            }
            pf[kk][(kb & 1) * 4 + g4] = (int)w;
          } else if (P2)
            pf[kk][(kb & 1) * 4 + g4] =
                pack4_e4m3_noclamp(fast_exp2(sacc[kb][4 * g4]), fast_exp2(sacc[kb][4 * g4 + 1]),
                                   fast_exp2(sacc[kb][4 * g4 + 2]), fast_exp2(sacc[kb][4 * g4 + 3]));
          else
            pf[kk][(kb & 1) * 4 + g4] = pack4_e4m3_noclamp(fast_exp2(__builtin_fmaf(sacc[kb][4 * g4], c, -mc)),
                                                           fast_exp2(__builtin_fmaf(sacc[kb][4 * g4 + 1], c, -mc)),
                                                           fast_exp2(__builtin_fmaf(sacc[kb][4 * g4 + 2], c, -mc)),
                                                           fast_exp2(__builtin_fmaf(sacc[kb][4 * g4 + 3], c, -mc)));
        }
      }
    };
    // ---- O^T += V^T P^T (fp8), row sums ---------------------------------------------------------------------------
    auto pv = [&](const int kk) {
      lacc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ones8, pf[kk], lacc, 0, 0, 0, 0, 0, 0);
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        constexpr int kOff = stage * kStage + kTile;
        const i32x4_t lo = *(MSD_LDS const i32x4_t*)(uintptr_t)(rd[kk][0] + kOff + db * 32 * 128);
        const i32x4_t hi = *(MSD_LDS const i32x4_t*)(uintptr_t)(rd[kk][1] + kOff + db * 32 * 128);
        const i32x8_t a = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        oacc[db] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, pf[kk], oacc[db], 0, 0, 0, 0, 0, 0);
      }
    };
    // The products of the first 64 keys run on the matrix core while the vector unit rounds the probabilities of
    // the other 64: the scheduler is told to put one product in front of every kValuPerMfma vector instructions.
    exp_pack(0);
    __builtin_amdgcn_sched_barrier(0);
    pv(0);
    exp_pack(1);
    constexpr int kValuPerMfma = PL ? (P2 ? 8 : 14) : (P2 ? 10 : 16);
    __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
    for (int i = 0; i < 5; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x402, kValuPerMfma, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    pv(1);

    // tile t + 1 has to be there: everything but the four requests issued in this step
    __builtin_amdgcn_s_waitcnt(0x0f74);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };
  for (int t = 0; t < n_tiles; t += 3) {
    tile_step(t, std::integral_constant<int, 0>{});
    if (t + 1 < n_tiles) tile_step(t + 1, std::integral_constant<int, 1>{});
    if (t + 2 < n_tiles) tile_step(t + 2, std::integral_constant<int, 2>{});
  }
  // the requests past the last tile still write into the stages, which the output staging reuses
  __builtin_amdgcn_s_waitcnt(0x0f70);
  __syncthreads();

  // ---- epilogue: 1/l, per-channel V scale, transpose through LDS, coalesced store -----------------------------------
  // (the 2^kPShift factor is in both the accumulator and the running sum, so it cancels)
  const float l_tot = lacc[0];  // every row of lacc holds the full sum over all keys
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  const float* vs = p.v_scale + (long long)bn * 128;
  MSD_LDS char* ost = smem + wave * 32 * kORow;
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int d = db * 32 + 8 * g + 4 * h;
      const f32x4_t sv = *(const f32x4_t*)(vs + d);
      typename E::x4 pk;
#pragma unroll
      for (int j = 0; j < 4; ++j) pk[j] = E::from_float(oacc[db][4 * g + j] * inv * sv[j]);
      *(MSD_LDS typename E::x4*)(ost + l32 * kORow + d * 2) = pk;
    }
  __builtin_amdgcn_wave_barrier();
  T* og = (T*)p.o + b * p.o_sb + n * p.o_sn;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int cidx = i * 64 + lane;
    const int row = cidx >> 4, c16 = cidx & 15;
    const int qr = q0 + wave * 32 + row;
    const i32x2_t lo = *(MSD_LDS const i32x2_t*)(ost + row * kORow + c16 * 16);
    const i32x2_t hi = *(MSD_LDS const i32x2_t*)(ost + row * kORow + c16 * 16 + 8);
    if (qr < p.Sq) *(i32x4_t*)(og + (long long)qr * p.o_ss + c16 * 8) = i32x4_t{lo[0], lo[1], hi[0], hi[1]};
  }
#endif
}

// grid = one workgroup per 256 query rows of a (batch, head), rounded up to a multiple of 8
template <int DT, bool P2, bool PL>
int fp8_fa_launch(const Fp8Params& p, int grid, hipStream_t stream) {
  constexpr int kLds = 3 * 32768;  // 3 stages x 32 KiB; the output staging (66 KiB) reuses them
  auto kern = fp8_fa_fwd_kernel<DT, P2, PL>;
  if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kLds) != hipSuccess)
    return MSD_ERR_LAUNCH;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(512), kLds, stream, p);
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

}  // namespace msd

using namespace msd;

extern "C" {

int mindiesd_fa_block_quant(const void* x, void* q, float* scale, int dtype, int B, int N, int S, int D,
                            long long x_sb, long long x_sn, long long x_ss, int block_size, float prescale,
                            int pow2_scale, hipStream_t stream) {
  if (!x || !q || !scale || B <= 0 || N <= 0 || S <= 0 || !(prescale > 0.f)) return MSD_ERR_BAD_ARG;
  if (D != 128) return MSD_ERR_UNSUPPORTED;
  if (block_size != 128 && block_size != 256 && block_size != 512) return MSD_ERR_BAD_ARG;
  if (dtype != MSD_DTYPE_BF16 && dtype != MSD_DTYPE_F16) return MSD_ERR_BAD_ARG;
  if (((uintptr_t)x & 15) || ((uintptr_t)q & 7) || ((x_sb | x_sn | x_ss) & 7)) return MSD_ERR_BAD_ARG;
  if ((long long)B * N > 65535) return MSD_ERR_UNSUPPORTED;  // grid.y
  dim3 grid((S + block_size - 1) / block_size, B * N);
  auto launch = [&](auto kern) {
    hipLaunchKernelGGL(kern, grid, dim3(256), 0, stream, x, (unsigned char*)q, scale, x_sb, x_sn, x_ss, N, S, prescale,
                       pow2_scale ? 1 : 0);
    return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
  };
  const bool bf = dtype == MSD_DTYPE_BF16;
  if (block_size == 128)
    return bf ? launch(block_quant_reg_kernel<MSD_DTYPE_BF16, 128>) : launch(block_quant_reg_kernel<MSD_DTYPE_F16, 128>);
  if (block_size == 256)
    return bf ? launch(block_quant_reg_kernel<MSD_DTYPE_BF16, 256>) : launch(block_quant_reg_kernel<MSD_DTYPE_F16, 256>);
  // 512 tokens: 32 rows per thread would take the whole register file (one workgroup per SIMD: 0.190 vs 0.176 ms)
  if (bf)
    hipLaunchKernelGGL(block_quant_kernel<MSD_DTYPE_BF16>, grid, dim3(256), 0, stream, x, (unsigned char*)q, scale, x_sb,
                       x_sn, x_ss, N, S, block_size, prescale, pow2_scale ? 1 : 0);
  else
    hipLaunchKernelGGL(block_quant_kernel<MSD_DTYPE_F16>, grid, dim3(256), 0, stream, x, (unsigned char*)q, scale, x_sb,
                       x_sn, x_ss, N, S, block_size, prescale, pow2_scale ? 1 : 0);
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

// y = x @ rot (rot_t = rot transposed, [128][128] contiguous, same 16-bit type as x), rounded to the
// 16-bit type, then quantised per (head, 128 tokens): codes [B][N][S][128], scale [B][N][ceil(S/128)].
int mindiesd_fa_rot_block_quant(const void* x, const void* rot_t, void* q, float* scale, int dtype, int B, int N, int S,
                                int D, long long x_sb, long long x_sn, long long x_ss, float prescale, int pow2_scale,
                                hipStream_t stream) {
  if (!x || !rot_t || !q || !scale || B <= 0 || N <= 0 || S <= 0 || !(prescale > 0.f)) return MSD_ERR_BAD_ARG;
  if (D != 128) return MSD_ERR_UNSUPPORTED;
  if (dtype != MSD_DTYPE_BF16 && dtype != MSD_DTYPE_F16) return MSD_ERR_BAD_ARG;
  if ((((uintptr_t)x | (uintptr_t)rot_t) & 15) || ((uintptr_t)q & 15) || ((x_sb | x_sn | x_ss) & 7)) return MSD_ERR_BAD_ARG;
  const dim3 grid((S + 127) / 128, B * N);
  if (grid.y > 65535) return MSD_ERR_UNSUPPORTED;
  if (dtype == MSD_DTYPE_BF16)
    hipLaunchKernelGGL(rot_block_quant_kernel<MSD_DTYPE_BF16>, grid, dim3(256), 0, stream, x, rot_t, (unsigned char*)q,
                       scale, x_sb, x_sn, x_ss, N, S, prescale, pow2_scale ? 1 : 0);
  else
    hipLaunchKernelGGL(rot_block_quant_kernel<MSD_DTYPE_F16>, grid, dim3(256), 0, stream, x, rot_t, (unsigned char*)q,
                       scale, x_sb, x_sn, x_ss, N, S, prescale, pow2_scale ? 1 : 0);
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

// bytes of the caller-provided scratch for mindiesd_fp8_v_quant (per-channel maxima)
size_t mindiesd_fp8_v_quant_workspace_size(int B, int N) { return (size_t)B * N * 128 * sizeof(unsigned); }

// The three launches of the V quantisation; amax is scratch of B * N * 128 words that the first launch clears.
static int v_quant_launch(const void* v, void* v8t, float* v_scale, int dtype, int B, int N, int S, long long v_sb,
                          long long v_sn, long long v_ss, unsigned* amax, hipStream_t stream) {
  const long long nbits = (long long)B * N * 128;
  const int S128 = (S + 127) / 128 * 128;
  hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)((nbits + 255) / 256)), dim3(256), 0, stream, amax, 0u, nbits);
  dim3 g1((S + 1023) / 1024, B * N), g2(S128 / 128, B * N);
  if (dtype == MSD_DTYPE_BF16) {
    hipLaunchKernelGGL(channel_amax_kernel<MSD_DTYPE_BF16>, g1, dim3(256), 0, stream, v, amax, v_sb, v_sn, v_ss, N, S);
    hipLaunchKernelGGL(v_quant_transpose_kernel<MSD_DTYPE_BF16>, g2, dim3(256), 0, stream, v, (const unsigned*)amax,
                       (unsigned char*)v8t, v_scale, v_sb, v_sn, v_ss, N, S, S128);
  } else {
    hipLaunchKernelGGL(channel_amax_kernel<MSD_DTYPE_F16>, g1, dim3(256), 0, stream, v, amax, v_sb, v_sn, v_ss, N, S);
    hipLaunchKernelGGL(v_quant_transpose_kernel<MSD_DTYPE_F16>, g2, dim3(256), 0, stream, v, (const unsigned*)amax,
                       (unsigned char*)v8t, v_scale, v_sb, v_sn, v_ss, N, S, S128);
  }
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

static int v_quant_check(const void* v, const void* v8t, const float* v_scale, int dtype, int B, int N, int S, int D,
                         long long v_sb, long long v_sn, long long v_ss) {
  if (!v || !v8t || !v_scale || B <= 0 || N <= 0 || S <= 0) return MSD_ERR_BAD_ARG;
  if (D != 128) return MSD_ERR_UNSUPPORTED;
  if (dtype != MSD_DTYPE_BF16 && dtype != MSD_DTYPE_F16) return MSD_ERR_BAD_ARG;
  if (((uintptr_t)v & 15) || ((uintptr_t)v8t & 15) || ((v_sb | v_sn | v_ss) & 7)) return MSD_ERR_BAD_ARG;
  if ((long long)B * N > 65535) return MSD_ERR_UNSUPPORTED;  // grid.y
  return MSD_OK;
}

int mindiesd_fp8_v_quant(const void* v, void* v8t, float* v_scale, int dtype, int B, int N, int S, int D,
                         long long v_sb, long long v_sn, long long v_ss, void* workspace, size_t ws_bytes,
                         hipStream_t stream) {
  const int rc = v_quant_check(v, v8t, v_scale, dtype, B, N, S, D, v_sb, v_sn, v_ss);
  if (rc != MSD_OK) return rc;
  if (!workspace) return MSD_ERR_BAD_ARG;
  if (ws_bytes < mindiesd_fp8_v_quant_workspace_size(B, N)) return MSD_ERR_WORKSPACE;
  return v_quant_launch(v, v8t, v_scale, dtype, B, N, S, v_sb, v_sn, v_ss, (unsigned*)workspace, stream);
}

// ---- the same without any allocation on the caller's or the library's side ------------------------------------
// The per-channel maxima live in a device array that is part of the library's code object: every GPU the library
// runs on holds its own copy (2 MiB) at its own address until the process ends.  `g_v_quant_scratch` names the
// array for the device compiler only; host code must use the address hipGetSymbolAddress returns for the current
// device, looked up once per device and kept in g_v_quant_scratch_ptr.
static __device__ __align__(256) unsigned g_v_quant_scratch[MINDIESD_FP8_V_QUANT_STATIC_MAX_HEADS * 128];
static unsigned* g_v_quant_scratch_ptr[kMaxDevices];
static std::mutex g_v_quant_scratch_mutex;

int mindiesd_fp8_v_quant_static_max_heads(void) { return MINDIESD_FP8_V_QUANT_STATIC_MAX_HEADS; }

int mindiesd_fp8_v_quant_static(const void* v, void* v8t, float* v_scale, int dtype, int B, int N, int S, int D,
                                long long v_sb, long long v_sn, long long v_ss, hipStream_t stream) {
  const int rc = v_quant_check(v, v8t, v_scale, dtype, B, N, S, D, v_sb, v_sn, v_ss);
  if (rc != MSD_OK) return rc;
  if ((long long)B * N > MINDIESD_FP8_V_QUANT_STATIC_MAX_HEADS) return MSD_ERR_WORKSPACE;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return MSD_ERR_LAUNCH;
  unsigned* scratch;
  {
    std::lock_guard<std::mutex> guard(g_v_quant_scratch_mutex);
    if (!g_v_quant_scratch_ptr[dev]) {
      void* ptr = nullptr;
      if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_v_quant_scratch)) != hipSuccess || !ptr) return MSD_ERR_LAUNCH;
      g_v_quant_scratch_ptr[dev] = (unsigned*)ptr;
    }
    scratch = g_v_quant_scratch_ptr[dev];
  }
  return v_quant_launch(v, v8t, v_scale, dtype, B, N, S, v_sb, v_sn, v_ss, scratch, stream);
}

int mindiesd_fp8_attention_fwd(const void* q8, const void* k8, const void* v8t, const float* q_scale,
                               const float* k_scale, const float* v_scale, void* out, int out_dtype, int B, int N,
                               int Sq, int Skv, int D, long long o_sb, long long o_sn, long long o_ss, float scale,
                               int flags, hipStream_t stream) {
  if (!q8 || !k8 || !v8t || !q_scale || !k_scale || !v_scale || !out) return MSD_ERR_BAD_ARG;
  if (B <= 0 || N <= 0 || Sq <= 0 || Skv <= 0) return MSD_ERR_BAD_ARG;
  if (D != 128 || !(scale > 0.f)) return MSD_ERR_UNSUPPORTED;
  if (out_dtype != MSD_DTYPE_BF16 && out_dtype != MSD_DTYPE_F16) return MSD_ERR_BAD_ARG;
  if (flags & ~(MSD_FP8_LOG2_DOMAIN | MSD_FP8_P_EXP2 | MSD_FP8_K_BLOCK_256)) return MSD_ERR_BAD_ARG;
  if (((uintptr_t)q8 | (uintptr_t)k8 | (uintptr_t)v8t | (uintptr_t)out) & 15) return MSD_ERR_BAD_ARG;
  if ((o_sb | o_sn | o_ss) & 7) return MSD_ERR_BAD_ARG;
  const int S128 = (Skv + 127) / 128 * 128;
  if ((long long)Skv * 128 >= (1ll << 31) || 128ll * S128 >= (1ll << 31)) return MSD_ERR_UNSUPPORTED;
  Fp8Params p{};
  p.q8 = (const unsigned char*)q8; p.k8 = (const unsigned char*)k8; p.v8t = (const unsigned char*)v8t;
  p.q_scale = q_scale; p.k_scale = k_scale; p.v_scale = v_scale;
  p.o = out; p.o_sb = o_sb; p.o_sn = o_sn; p.o_ss = o_ss;
  p.B = B; p.N = N; p.Sq = Sq; p.Skv = Skv; p.S128 = S128;
  p.scale_log2 = scale * 1.4426950408889634f;
  p.k_shift = (flags & MSD_FP8_K_BLOCK_256) ? 1 : 0;
  const int q_tiles = (Sq + 255) / 256;
  const int total = B * N * q_tiles;
  const int grid = (total + 7) / 8 * 8;
  const bool bf = out_dtype == MSD_DTYPE_BF16;
  const bool p2 = (flags & MSD_FP8_LOG2_DOMAIN) != 0, pl = (flags & MSD_FP8_P_EXP2) == 0;
  if (p2 && pl) return bf ? fp8_fa_launch<MSD_DTYPE_BF16, true, true>(p, grid, stream)
                          : fp8_fa_launch<MSD_DTYPE_F16, true, true>(p, grid, stream);
  if (p2) return bf ? fp8_fa_launch<MSD_DTYPE_BF16, true, false>(p, grid, stream)
                    : fp8_fa_launch<MSD_DTYPE_F16, true, false>(p, grid, stream);
  if (pl) return bf ? fp8_fa_launch<MSD_DTYPE_BF16, false, true>(p, grid, stream)
                    : fp8_fa_launch<MSD_DTYPE_F16, false, true>(p, grid, stream);
  return bf ? fp8_fa_launch<MSD_DTYPE_BF16, false, false>(p, grid, stream)
            : fp8_fa_launch<MSD_DTYPE_F16, false, false>(p, grid, stream);
}

}  // extern "C"
