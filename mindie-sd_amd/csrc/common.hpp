// Shared device/host helpers for the gfx950 (MI355X, CDNA4) kernels of this library.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace msd {

// ---- vector types -------------------------------------------------------------------
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x8_t __attribute__((ext_vector_type(8)));
typedef int i32x2_t __attribute__((ext_vector_type(2)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));

// ---- error codes returned by every extern "C" entry point ----------------------------
enum : int {
  MSD_OK = 0,
  MSD_ERR_BAD_ARG = 1,      // null pointer, non-positive size, unsupported head_dim/dtype
  MSD_ERR_UNSUPPORTED = 2,  // shape or option outside what the kernels implement
  MSD_ERR_WORKSPACE = 3,    // workspace too small
  MSD_ERR_LAUNCH = 4,       // hipLaunch / runtime error (hipGetLastError != hipSuccess)
};

enum : int { MSD_DTYPE_BF16 = 0, MSD_DTYPE_F16 = 1 };
// flag bits of mindiesd_fp8_attention_fwd (the same values as in include/mindiesd_hip.h)
enum : int { MSD_FP8_LOG2_DOMAIN = 1, MSD_FP8_P_EXP2 = 2, MSD_FP8_K_BLOCK_256 = 4 };

// ---- element traits: 16-bit storage type -> MFMA operand type + builtins -------------
template <int DT>
struct Elem;
template <>
struct Elem<MSD_DTYPE_BF16> {
  typedef __bf16 type;
  typedef bf16x8_t x8;
  typedef bf16x4_t x4;
  static __device__ __forceinline__ f32x16_t mfma32(x8 a, x8 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4_t mfma16(x8 a, x8 b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ type from_float(float f) { return (__bf16)f; }
  // acc + sum of the 8 elements (v_dot2_f32_bf16 against ones)
  static __device__ __forceinline__ float sum8(x8 v, float acc) {
    typedef __bf16 x2 __attribute__((ext_vector_type(2)));
    const x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
    union { x8 v; x2 p[4]; } u;
    u.v = v;
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_fdot2_f32_bf16(u.p[i], ones, acc, false);
    return acc;
  }
};
template <>
struct Elem<MSD_DTYPE_F16> {
  typedef _Float16 type;
  typedef f16x8_t x8;
  typedef f16x4_t x4;
  static __device__ __forceinline__ f32x16_t mfma32(x8 a, x8 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4_t mfma16(x8 a, x8 b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ type from_float(float f) { return (_Float16)f; }
  static __device__ __forceinline__ float sum8(x8 v, float acc) {
    typedef _Float16 x2 __attribute__((ext_vector_type(2)));
    const x2 ones = {(_Float16)1.0f, (_Float16)1.0f};
    union { x8 v; x2 p[4]; } u;
    u.v = v;
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_fdot2(u.p[i], ones, acc, false);
    return acc;
  }
};

// LDS pointer in address space 3 (needed by the transposing LDS read builtin).
#define MSD_LDS __attribute__((address_space(3)))

// One ds_read_b64_tr_b16: the 16 lanes of a quarter-wave each point at 4 consecutive
// 16-bit elements; viewing those 64 elements as a 4 x 16 matrix (row j = lanes 4j..4j+3),
// lane i receives column i (4 elements, one from each row).
__device__ __forceinline__ s16x4_t lds_read_tr16(const void* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((MSD_LDS s16x4_t*)(uintptr_t)(p));
}

// The same read written as inline asm, for loops that keep LDS-DMA requests in flight: the compiler orders
// the builtin after every LDS-DMA still outstanding (it waits for vmcnt(0)), which would make each tile wait
// for the whole next tile before its first V read.  The asm form carries no such dependence; in exchange the
// compiler does not know that the result arrives later, so the caller must pass the registers through
// lds_wait_tr<N>() (s_waitcnt lgkmcnt(N), N = number of LDS reads issued after them that may stay in
// flight) before using them.
template <int OFFSET>
__device__ __forceinline__ s16x4_t lds_read_tr16_async(unsigned lds_addr) {
  static_assert(OFFSET >= 0 && OFFSET < 65536, "ds offset field is 16 bits");
  s16x4_t r;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r) : "v"(lds_addr), "n"(OFFSET));
  return r;
}
template <int N>
__device__ __forceinline__ void lds_wait_tr(s16x4_t (&r)[8]) {
  static_assert(N >= 0 && N <= 15, "lgkmcnt is a 4-bit counter");
  asm volatile("s_waitcnt lgkmcnt(%8)"
               : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7])
               : "n"(N));
}

// Combine a value with the one held by the lane 32 positions away (the other half of the
// wavefront) using v_permlane32_swap: after the swap one result register holds lanes 0..31 of
// the input in both halves and the other holds lanes 32..63 in both halves.
// (Written as inline asm: with the builtin the optimiser of this toolchain folds the second
// result into the first when both inputs hold the same value.  The leading s_nop covers the
// VALU-write -> permlane-swap hazard that the compiler cannot see inside an asm block.)
__device__ __forceinline__ void half_swap(float v, float& lo, float& hi) {
  float a = v, b = v;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  lo = a;
  hi = b;
}
__device__ __forceinline__ float half_max(float v) {
  float lo, hi;
  half_swap(v, lo, hi);
  return fmaxf(lo, hi);
}
__device__ __forceinline__ float half_sum(float v) {
  float lo, hi;
  half_swap(v, lo, hi);
  return lo + hi;
}

// Sums over the two wave halves of two values at once: lanes 0..31 receive the total of x, lanes 32..63 the total
// of y (the swap leaves x's lower and y's lower half in one register, their upper halves in the other).
__device__ __forceinline__ float half_pair_sum(float x, float y) {
  float a = x, b = y;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  return a + b;
}

// The same across the four 16-lane rows of a wavefront: v_permlane16_swap exchanges the odd rows of its first
// operand with the even rows of its second, so with both holding v one result has rows (0, 0, 2, 2) of v and
// the other rows (1, 1, 3, 3); combining them and then the two halves leaves the result of all four rows in
// every lane.
__device__ __forceinline__ void row_swap(float v, float& even, float& odd) {
  float a = v, b = v;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  even = a;
  odd = b;
}
__device__ __forceinline__ float quarter_max(float v) {
  float e, o;
  row_swap(v, e, o);
  return half_max(fmaxf(e, o));
}

// Rescale of one 16-query column block of fa_fwd16_kernel when its reference maximum moves: l *= alpha, the seed and
// the 8 score blocks -= delta, the 8 output blocks *= alpha - 69 registers updated in place by three asm blocks, each
// skipped by its own branch when the wave-uniform flag is zero.  The test and the branches sit inside the asm, so the
// compiler sees straight-line code that leaves every value in its register.  Written as an if/else in C++, the rarely
// taken update lands in other registers and the path that skips it pays some 100 register moves per tile to meet it
// at the join.  (None of the values may be the result of a matrix instruction still in flight: the compiler cannot
// place the wait states such a read needs inside an asm block.  Here the scores have been read by the maximum and
// the outputs were written a whole phase earlier.)
__device__ __forceinline__ void cond_rescale_fa16(int flag, float delta, float alpha, float& l, f32x4_t& negm, f32x4_t& s0,
                                                  f32x4_t& s1, f32x4_t& s2, f32x4_t& s3, f32x4_t& s4, f32x4_t& s5,
                                                  f32x4_t& s6, f32x4_t& s7, f32x4_t& o0, f32x4_t& o1, f32x4_t& o2,
                                                  f32x4_t& o3, f32x4_t& o4, f32x4_t& o5, f32x4_t& o6, f32x4_t& o7) {
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
  float o4_0 = o4[0], o4_1 = o4[1], o4_2 = o4[2], o4_3 = o4[3];
  float o5_0 = o5[0], o5_1 = o5[1], o5_2 = o5[2], o5_3 = o5[3];
  float o6_0 = o6[0], o6_1 = o6[1], o6_2 = o6[2], o6_3 = o6[3];
  float o7_0 = o7[0], o7_1 = o7[1], o7_2 = o7[2], o7_3 = o7[3];
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
  asm volatile("s_cmp_eq_u32 %24, 0\n\t" "s_cbranch_scc1 .Lmsd_skip%=\n\t" "v_sub_f32 %0, %0, %25\n\t"
               "v_sub_f32 %1, %1, %25\n\t" "v_sub_f32 %2, %2, %25\n\t" "v_sub_f32 %3, %3, %25\n\t"
               "v_sub_f32 %4, %4, %25\n\t" "v_sub_f32 %5, %5, %25\n\t" "v_sub_f32 %6, %6, %25\n\t"
               "v_sub_f32 %7, %7, %25\n\t" "v_sub_f32 %8, %8, %25\n\t" "v_sub_f32 %9, %9, %25\n\t"
               "v_sub_f32 %10, %10, %25\n\t" "v_sub_f32 %11, %11, %25\n\t" "v_mul_f32 %12, %12, %26\n\t"
               "v_mul_f32 %13, %13, %26\n\t" "v_mul_f32 %14, %14, %26\n\t" "v_mul_f32 %15, %15, %26\n\t"
               "v_mul_f32 %16, %16, %26\n\t" "v_mul_f32 %17, %17, %26\n\t" "v_mul_f32 %18, %18, %26\n\t"
               "v_mul_f32 %19, %19, %26\n\t" "v_mul_f32 %20, %20, %26\n\t" "v_mul_f32 %21, %21, %26\n\t"
               "v_mul_f32 %22, %22, %26\n\t" "v_mul_f32 %23, %23, %26\n\t" "s_nop 7\n\t"
               ".Lmsd_skip%=:"
               : "+v"(s5_0), "+v"(s5_1), "+v"(s5_2), "+v"(s5_3), "+v"(s6_0), "+v"(s6_1), "+v"(s6_2), "+v"(s6_3),
                 "+v"(s7_0), "+v"(s7_1), "+v"(s7_2), "+v"(s7_3), "+v"(o0_0), "+v"(o0_1), "+v"(o0_2), "+v"(o0_3),
                 "+v"(o1_0), "+v"(o1_1), "+v"(o1_2), "+v"(o1_3), "+v"(o2_0), "+v"(o2_1), "+v"(o2_2), "+v"(o2_3)
               : "s"(flag), "v"(delta), "v"(alpha)
               : "scc");
  asm volatile("s_cmp_eq_u32 %20, 0\n\t" "s_cbranch_scc1 .Lmsd_skip%=\n\t" "v_mul_f32 %0, %0, %21\n\t"
               "v_mul_f32 %1, %1, %21\n\t" "v_mul_f32 %2, %2, %21\n\t" "v_mul_f32 %3, %3, %21\n\t"
               "v_mul_f32 %4, %4, %21\n\t" "v_mul_f32 %5, %5, %21\n\t" "v_mul_f32 %6, %6, %21\n\t"
               "v_mul_f32 %7, %7, %21\n\t" "v_mul_f32 %8, %8, %21\n\t" "v_mul_f32 %9, %9, %21\n\t"
               "v_mul_f32 %10, %10, %21\n\t" "v_mul_f32 %11, %11, %21\n\t" "v_mul_f32 %12, %12, %21\n\t"
               "v_mul_f32 %13, %13, %21\n\t" "v_mul_f32 %14, %14, %21\n\t" "v_mul_f32 %15, %15, %21\n\t"
               "v_mul_f32 %16, %16, %21\n\t" "v_mul_f32 %17, %17, %21\n\t" "v_mul_f32 %18, %18, %21\n\t"
               "v_mul_f32 %19, %19, %21\n\t" "s_nop 7\n\t" ".Lmsd_skip%=:"
               : "+v"(o3_0), "+v"(o3_1), "+v"(o3_2), "+v"(o3_3), "+v"(o4_0), "+v"(o4_1), "+v"(o4_2), "+v"(o4_3),
                 "+v"(o5_0), "+v"(o5_1), "+v"(o5_2), "+v"(o5_3), "+v"(o6_0), "+v"(o6_1), "+v"(o6_2), "+v"(o6_3),
                 "+v"(o7_0), "+v"(o7_1), "+v"(o7_2), "+v"(o7_3)
               : "s"(flag), "v"(alpha)
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
  o4 = f32x4_t{o4_0, o4_1, o4_2, o4_3};
  o5 = f32x4_t{o5_0, o5_1, o5_2, o5_3};
  o6 = f32x4_t{o6_0, o6_1, o6_2, o6_3};
  o7 = f32x4_t{o7_0, o7_1, o7_2, o7_3};
}

// Pair tables of the block-sparse attention over paired query blocks (built by bsa_pair.hip, consumed by flash_attn_fwd.hip).
struct BsaPairTables {
  int* pairs;     // [BN][NP][2]
  int* sh_idx;    // [BN][NP][KB]
  int* sh_cnt;    // [BN][NP]
  int* ex_idx;    // [BN][QB][KB]
  int* ex_cnt;    // [BN][QB]
  int* init_cnt;  // [BN][QB]
  int NP;
};
size_t bsa_pair_ints(long long BN, int QB, int KB);
bool bsa_pair_supported(int QB, int KB);
int bsa_build_pairs(const signed char* mask, long long BN, int QB, int KB, int* ws, BsaPairTables* t, hipStream_t stream);

// Lazy-rescale threshold of the online softmax, in log2 units.
constexpr float kTau = 8.0f;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// round-to-nearest-even fp32 -> bf16 bits, then back to fp32 (used where a rounding point
// of the reference arithmetic has to be reproduced exactly)
__device__ __forceinline__ float round_bf16(float f) { return (float)(__bf16)f; }

}  // namespace msd
