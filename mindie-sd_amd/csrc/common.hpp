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
__device__ __forceinline__ float quarter_sum(float v) {
  float e, o;
  row_swap(v, e, o);
  return half_sum(e + o);
}

// Lazy-rescale threshold of the online softmax, in log2 units.
constexpr float kTau = 8.0f;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// round-to-nearest-even fp32 -> bf16 bits, then back to fp32 (used where a rounding point
// of the reference arithmetic has to be reproduced exactly)
__device__ __forceinline__ float round_bf16(float f) { return (float)(__bf16)f; }

}  // namespace msd
