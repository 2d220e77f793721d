// MXFP8 (OCP MX: E4M3 elements, one E8M0 scale per 32 elements along K) quantisation and GEMM for
// gfx950 (MI355X), with an optional SwiGLU epilogue fused into the output tile.
//
// Takes the place of the vendor ops behind the reference's MXFP8 linear layer:
//   npu_dynamic_mx_quant                 mindiesd/quantization/layer.py:338-341
//   npu_quant_matmul(group_sizes=[1,1,32], e8m0 scales, fp32 bias)   layer.py:351-361
// The reference applies SiLU * up in the model after the matmul (mindiesd/layers/activation.py:34-61);
// here silu(gate) * up is computed on the accumulators before anything is written.
//
// C[m][n] = sum_k X[m][k] * W[n][k]: both operands are K-contiguous.  In one
// v_mfma_scale_f32_32x32x64_f8f6f4 the lane (row = lane%32, half h = lane/32) holds K-values
// 16h..16h+15 (registers 0-3) and 32+16h..32+16h+15 (registers 4-7) of the 64-wide step, i.e. two
// 16-byte chunks, one from each 32-element MX block; the scale byte supplied by lane (row, h) is
// applied to MX block h of that row.  X is the A operand (row m), W the B operand (column n).
//
// Workgroup tile: 256 rows of X x 256 rows of W (for SwiGLU: 128 gate rows f0.. and the 128 up
// rows F+f0.., so both halves of an output element meet in the same lane and register), K step
// 128 bytes, LDS double buffered (2 x 64 KiB) and filled by LDS-DMA; 8 waves as 4 (M) x 2 (N), each
// 64 x 128 = 2 x 4 MFMA blocks.  LDS rows are 128 bytes; 16-byte chunk c of row r sits at
// chunk c ^ ((r >> 1) & 7) (bank-conflict free for the 16-byte operand reads).
#include "common.hpp"

namespace msd {

constexpr float kE4M3MaxMx = 448.0f;

// ---- MX quantisation of a [M][K] 16-bit matrix along K -----------------------------------------------------
// 4 lanes share one 32-element block (8 elements = 16 bytes each).
template <int DT>
__global__ __launch_bounds__(256) void mx_quant_kernel(const void* x_, unsigned char* q, unsigned char* e8m0,
                                                       long long M, int K, long long x_stride) {
#if defined(__HIP_DEVICE_COMPILE__)
  using T = typename Elem<DT>::type;
  const long long chunk = (long long)blockIdx.x * 256 + threadIdx.x;  // 8-element chunk index
  const int chunks_per_row = K >> 3;
  const long long row = chunk / chunks_per_row;
  const int c = (int)(chunk - row * chunks_per_row);
  const bool ok = row < M;
  float f[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) f[j] = 0.f;
  if (ok) {
    union { i32x4_t v; T e[8]; } u;
    u.v = *(const i32x4_t*)((const T*)x_ + row * x_stride + c * 8);
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = (float)u.e[j];
  }
  float amax = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(f[j]));
  amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
  amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
  // floor(log2(amax)) = biased exponent - 127 for normal numbers; shared = that - 8 (E4M3 emax)
  const int be = (int)((__builtin_bit_cast(unsigned, amax) >> 23) & 0xff);
  int sbyte = be - 8;  // = shared + 127
  sbyte = sbyte < 0 ? 0 : (sbyte > 254 ? 254 : sbyte);
  if (amax == 0.f) sbyte = 0;
  const float inv = __builtin_bit_cast(float, (unsigned)(254 - sbyte) << 23);  // 2^-(sbyte-127), exact
  if (ok) {
    int w[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      int t = 0;
      t = __builtin_amdgcn_cvt_pk_fp8_f32(__builtin_amdgcn_fmed3f(f[4 * j] * inv, -kE4M3MaxMx, kE4M3MaxMx),
                                          __builtin_amdgcn_fmed3f(f[4 * j + 1] * inv, -kE4M3MaxMx, kE4M3MaxMx), t, false);
      t = __builtin_amdgcn_cvt_pk_fp8_f32(__builtin_amdgcn_fmed3f(f[4 * j + 2] * inv, -kE4M3MaxMx, kE4M3MaxMx),
                                          __builtin_amdgcn_fmed3f(f[4 * j + 3] * inv, -kE4M3MaxMx, kE4M3MaxMx), t, true);
      w[j] = t;
    }
    *(i32x2_t*)(q + row * K + c * 8) = i32x2_t{w[0], w[1]};
    if ((c & 3) == 0) e8m0[row * (K >> 5) + (c >> 2)] = (unsigned char)sbyte;
  }
#endif
}

// ---- GEMM -------------------------------------------------------------------------------------------------------
struct GemmParams {
  const unsigned char* a;    // X codes [M][K]
  const unsigned char* as;   // X scales [M][K/32]
  const unsigned char* w;    // W codes [Nw][K]
  const unsigned char* ws;   // W scales [Nw][K/32]
  const float* bias;         // optional [Nw]
  void* out;                 // [M][Nout] 16-bit
  int M, K, Nw, Nout;        // Nout = Nw (plain) or Nw/2 (SwiGLU)
  int tiles_m, tiles_n;
};

// Work decomposition: one workgroup of 4 waves owns a 256 x 256 tile of (X rows) x (W rows); every wave owns
// 128 x 128 of it as 4 x 4 accumulator blocks (256 accumulator registers, one wave per SIMD), so each
// 64-wide K step costs 16 KiB of LDS reads per wave for 16 matrix instructions.  K is walked in stages of
// 64 codes (32 KiB of LDS: X 256 x 64 B, W 256 x 64 B) through a ring of four buffers filled by LDS-DMA:
// while stage kt is multiplied from registers, stage kt+1 is read from LDS into the other register set,
// stage kt+2 has just landed and stages kt+3 and kt+4 are in flight.
template <int DT, bool SWIGLU>
__global__ __launch_bounds__(256, 1) void mxfp8_gemm_kernel(const GemmParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  using E = Elem<DT>;
  using T = typename E::type;
  constexpr int BM = 256, BNW = 256, BK = 64, NW = 4, NS = 4;
  constexpr int kATile = BM * BK, kWTile = BNW * BK, kStage = kATile + kWTile;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  MSD_LDS char* smem = (MSD_LDS char*)smem_raw;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, h = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;

  // ---- tile order: groups of 8 M-tiles walk the N-tiles together (X and W panels stay in L2) ------------
  const int per_xcd = (p.tiles_m * p.tiles_n + 7) / 8;
  const int lin = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (lin >= p.tiles_m * p.tiles_n) return;
  constexpr int GM = 8;
  const int grp = lin / (GM * p.tiles_n);
  const int gm0 = grp * GM;
  const int gsz = min(GM, p.tiles_m - gm0);
  const int in_grp = lin - grp * GM * p.tiles_n;
  const int tm = gm0 + in_grp % gsz;
  const int tn = in_grp / gsz;
  const int m0 = tm * BM;
  // W rows of this tile: plain: 256 consecutive rows; SwiGLU: 128 gate rows + the matching 128 up rows
  const int half = p.Nw >> 1;
  const int f0 = SWIGLU ? tn * 128 : tn * 256;

  // ---- LDS-DMA: one instruction = 16 rows x 64 bytes; 16 + 16 instructions per stage, 4 + 4 per wave ----------
  // A row keeps its four 16-byte chunks at positions chunk ^ ((row >> 2) & 3), which makes the 16-byte
  // operand reads of 16 consecutive rows hit 16 different bank groups.
  const __amdgpu_buffer_rsrc_t a_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.a, 0, (int)min((long long)p.M * p.K, 0x7fffffffll), 0x00020000);
  const __amdgpu_buffer_rsrc_t w_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.w, 0, (int)min((long long)p.Nw * p.K, 0x7fffffffll), 0x00020000);
  constexpr int kOutOfRange = 0x7ffffff0;  // lane offset beyond any buffer: the access reads zeros
  const int k_tiles = p.K / BK;
  const __amdgpu_buffer_rsrc_t none_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)p.a, 0, 0, 0x00020000);
  int a_voff[4], w_voff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = 16 * (i * NW + wave) + (lane >> 2);  // row inside the 256-row tile
    const int c = (lane & 3) ^ ((row >> 2) & 3);
    a_voff[i] = (m0 + row) * p.K + c * 16;  // rows past M are out of range and read as zeros
    int wrow;
    if (SWIGLU) wrow = row < 128 ? f0 + row : half + f0 + (row - 128);
    else wrow = f0 + row;
    // rows past the matrix (or past the gate half) must not alias other rows: push them out of range
    const bool w_ok = SWIGLU ? (f0 + (row & 127) < half) : (wrow < p.Nw);
    w_voff[i] = w_ok ? wrow * p.K + c * 16 : kOutOfRange;
  }
  // Stages past the end of K are requested through an empty descriptor: the DMA then writes zeros and
  // costs no memory traffic, which keeps the number of outstanding operations the same in every iteration.
  auto load_stage = [&](int kt, int buf) {
    MSD_LDS char* ab = smem + buf * kStage;
    const bool valid = kt < k_tiles;
    const __amdgpu_buffer_rsrc_t ar = valid ? a_rsrc : none_rsrc;
    const __amdgpu_buffer_rsrc_t wr = valid ? w_rsrc : none_rsrc;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int g = i * NW + wave;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ar, (MSD_LDS void*)(ab + g * 1024), 16, a_voff[i], kt * BK, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(wr, (MSD_LDS void*)(ab + kATile + g * 1024), 16, w_voff[i], kt * BK, 0,
                                               0);
    }
  };

  // ---- scales: staged through LDS in chunks of 8 stages (16 scale bytes = 512 K-values per row) -------------------
  // One 16-byte DMA per row and chunk instead of one dword per row and stage pair: a scale row is a
  // 128-byte line per 4096 K-values, so short reads of it cost a full L2 request each.  Rows past the
  // matrices read zeros (scale 2^-127) against all-zero data, which contributes exactly 0.
  const int kblk_row = p.K >> 5;  // scale bytes per row
  const __amdgpu_buffer_rsrc_t as_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.as, 0, (int)((long long)p.M * kblk_row), 0x00020000);
  const __amdgpu_buffer_rsrc_t ws_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.ws, 0, (int)((long long)p.Nw * kblk_row), 0x00020000);
  constexpr int kScBase = NS * kStage, kScBuf = 2 * 256 * 16;  // two chunk buffers: [X rows | W rows] x 16 B
  int as_voff, ws_voff;
  {
    const int row = 64 * wave + lane;  // wave w stages rows 64w .. 64w+63 of both operands
    as_voff = (m0 + row) * kblk_row;
    int wrow;
    if (SWIGLU) wrow = row < 128 ? f0 + row : half + f0 + (row - 128);
    else wrow = f0 + row;
    const bool w_ok = SWIGLU ? (f0 + (row & 127) < half) : (wrow < p.Nw);
    ws_voff = w_ok ? wrow * kblk_row : kOutOfRange;
  }
  // Requested at the end of every fourth stage so that the number of outstanding operations repeats with
  // the ring; the request that falls in the middle of a chunk (or past the end of K) goes through the
  // empty descriptor into a scrap area and costs nothing.
  auto load_scale_chunk = [&](int kt_next) {  // kt_next: multiple of 4; the chunk starts at stage kt_next + 4
    const int chunk = __builtin_amdgcn_readfirstlane((kt_next + 4) >> 3);
    const bool real = ((kt_next + 4) & 7) == 0 && kt_next + 4 < k_tiles;
    const __amdgpu_buffer_rsrc_t ar = real ? as_rsrc : none_rsrc;
    const __amdgpu_buffer_rsrc_t wr = real ? ws_rsrc : none_rsrc;
    const int dst = __builtin_amdgcn_readfirstlane(real ? kScBase + (chunk & 1) * kScBuf + wave * 1024
                                                        : kScBase + 2 * kScBuf);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(ar, (MSD_LDS void*)(smem + dst), 16, as_voff, chunk * 16, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(wr, (MSD_LDS void*)(smem + dst + (real ? 4096 : 0)), 16, ws_voff,
                                             chunk * 16, 0, 0);
  };
  bool w_okk[4];
  int as_lds[4], ws_lds[4];  // LDS offsets of the lane's scale rows inside a chunk buffer
#pragma unroll
  for (int mb = 0; mb < 4; ++mb) as_lds[mb] = kScBase + (wm * 128 + mb * 32 + l32) * 16;
#pragma unroll
  for (int nb = 0; nb < 4; ++nb) {
    // wave column range: SwiGLU: gate cols wn*64 + {0,32}, up cols the same; plain: wn*128 + nb*32
    int wrow;
    if (SWIGLU) wrow = (nb < 2 ? 0 : half) + f0 + wn * 64 + (nb & 1) * 32 + l32;
    else wrow = f0 + wn * 128 + nb * 32 + l32;
    w_okk[nb] = SWIGLU ? (f0 + wn * 64 + (nb & 1) * 32 + l32 < half) : (wrow < p.Nw);
    const int lrow = SWIGLU ? ((nb < 2 ? 0 : 128) + wn * 64 + (nb & 1) * 32 + l32) : (wn * 128 + nb * 32 + l32);
    ws_lds[nb] = kScBase + 4096 + lrow * 16;
  }
  struct Scales {
    int a[4], w[4];
  };
  // dword of stage pair `pair` (two stages = 128 K-values = 4 MX blocks)
  auto read_scales = [&](int pair, Scales& s) {
    const int off = ((pair >> 2) & 1) * kScBuf + (pair & 3) * 4;
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) s.a[mb] = *(MSD_LDS const int*)(smem + as_lds[mb] + off);
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) s.w[nb] = *(MSD_LDS const int*)(smem + ws_lds[nb] + off);
  };

  f32x16_t acc[4][4];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mb][nb][r] = 0.f;

  const int swz = (l32 >> 2) & 3;
  const int sh = 8 * h;  // the lane's MX block inside a 64-wide K step is block h
  // LDS offsets of this lane's two operand chunks (MX block 0: chunk h, MX block 1: chunk 2 + h)
  const int c_lo = (h ^ swz) << 4, c_hi = ((2 + h) ^ swz) << 4;
  int a_row_off[4], w_row_off[4];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb) a_row_off[mb] = (wm * 128 + mb * 32 + l32) * BK;
#pragma unroll
  for (int nb = 0; nb < 4; ++nb) {
    const int lrow = SWIGLU ? ((nb < 2 ? 0 : 128) + wn * 64 + (nb & 1) * 32 + l32) : (wn * 128 + nb * 32 + l32);
    w_row_off[nb] = kATile + lrow * BK;
  }
  struct Frags {
    i32x8_t a[4], w[4];
  };
  auto read_frags = [&](int buf, Frags& f) {
    MSD_LDS const char* base = smem + buf * kStage;
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
      const i32x4_t lo = *(MSD_LDS const i32x4_t*)(base + a_row_off[mb] + c_lo);
      const i32x4_t hi = *(MSD_LDS const i32x4_t*)(base + a_row_off[mb] + c_hi);
      f.a[mb] = i32x8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
      const i32x4_t lo = *(MSD_LDS const i32x4_t*)(base + w_row_off[nb] + c_lo);
      const i32x4_t hi = *(MSD_LDS const i32x4_t*)(base + w_row_off[nb] + c_hi);
      f.w[nb] = i32x8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
  };

  // Workgroup barrier without the memory fence of __syncthreads(): the fence would wait for every DMA in
  // flight, the explicit counts below wait only for the stage that is needed.  The empty asm statements
  // keep the compiler from moving LDS accesses across the barrier.
  auto wg_barrier = [] {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  // s_waitcnt immediates: vmcnt in bits 3:0 (+ 15:14), lgkmcnt(0) unless noted
  constexpr int kWaitVm16 = 0x4070, kWaitVm18 = 0x4072;
  constexpr int kWaitVm24Only = 0x4f78;  // vmcnt(24), LDS reads not waited for

  // ---- prologue: the same issue order the main loop produces, so its wait counts apply from stage 0 -----------
  // Per wave a stage is 8 DMA instructions and a scale chunk is 2.
  Scales sc, sn;
  load_scale_chunk(-4);
  load_stage(0, 0);
  load_stage(1, 1);
  load_stage(2, 2);
  load_stage(3, 3);
  __builtin_amdgcn_s_waitcnt(kWaitVm24Only);  // scale chunk 0 and stage 0 landed
  wg_barrier();
  Frags fr[2];
  read_frags(0, fr[0]);
  read_scales(0, sn);
  __builtin_amdgcn_s_waitcnt(kWaitVm16);  // stage 1 landed, stage 0 is in registers
  wg_barrier();
  load_stage(4, 0);

  // ---- main loop, unrolled over the ring so buffers, register sets, scale selectors and wait counts are
  // static.  The stage count is rounded up to a multiple of four; the extra stages multiply zeros.
  auto stage_step = [&](int kt, auto j_c) {
    constexpr int J = decltype(j_c)::value;   // kt % 4
    constexpr int CUR = J & 1, NXT = CUR ^ 1;
    constexpr int OPSEL = (J & 1) ? 2 : 0;    // odd stages use scale bytes 2 and 3 of the pair's dword
    // nothing moves across a stage boundary
    __builtin_amdgcn_sched_barrier(0);
    if ((J & 1) == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        sc.a[i] = (int)((unsigned)sn.a[i] >> sh);
        sc.w[i] = (int)((unsigned)sn.w[i] >> sh);
      }
    }
    read_frags((J + 1) % NS, fr[NXT]);
    if (J & 1) read_scales((kt + 1) >> 1, sn);
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
      for (int mb = 0; mb < 4; ++mb)
        acc[mb][nb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fr[CUR].a[mb], fr[CUR].w[nb], acc[mb][nb], 0, 0,
                                                                      OPSEL, sc.a[mb], OPSEL, sc.w[nb]);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one matrix instruction
    }
    // stage kt+2 must have landed (mine: the wait; everybody's: the barrier), and every wave must be done
    // reading the buffer of stage kt+1 before it is refilled with stage kt+5.  Outstanding after stage
    // kt+2: stages kt+3 and kt+4, plus the two scale requests made at the end of every fourth stage.
    __builtin_amdgcn_s_waitcnt((J == 1 || J == 2) ? kWaitVm18 : kWaitVm16);
    wg_barrier();
    if (J == 0) load_scale_chunk(kt);
    load_stage(kt + 5, (J + 1) % NS);
  };
  for (int kt = 0; kt < k_tiles; kt += 4) {
    stage_step(kt, std::integral_constant<int, 0>{});
    stage_step(kt + 1, std::integral_constant<int, 1>{});
    stage_step(kt + 2, std::integral_constant<int, 2>{});
    stage_step(kt + 3, std::integral_constant<int, 3>{});
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);  // the trailing (empty) DMA requests
  __syncthreads();  // the staging below reuses the ring

  // ---- epilogue: bias, SwiGLU, 16-bit, transpose through LDS, coalesced rows -------------------------------------
  // accumulator (mb, nb): row m = wm*128 + mb*32 + 8*(r/4) + 4*h + r%4, column = l32 of block nb
  constexpr int kOutCols = SWIGLU ? 64 : 128;          // output columns per wave
  constexpr int kORow = kOutCols * 2 + 8;              // padded staging row (bytes)
  MSD_LDS char* ost = smem + wave * 32 * kORow;       // 32 rows per wave at a time
  float bias_v[4];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb) {
    int wrow;
    if (SWIGLU) wrow = (nb < 2 ? 0 : half) + f0 + wn * 64 + (nb & 1) * 32 + l32;
    else wrow = f0 + wn * 128 + nb * 32 + l32;
    bias_v[nb] = (p.bias && w_okk[nb]) ? p.bias[wrow] : 0.f;
  }
  T* og = (T*)p.out;
  const int col0 = SWIGLU ? f0 + wn * 64 : f0 + wn * 128;
  constexpr int kChunks = kOutCols / 8;  // 16-byte chunks per row
#pragma unroll
  for (int mb = 0; mb < 4; ++mb) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = 8 * (r >> 2) + 4 * h + (r & 3);
      if (SWIGLU) {
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
          const float g = acc[mb][nb][r] + bias_v[nb];
          const float u = acc[mb][nb + 2][r] + bias_v[nb + 2];
          const float sg = g * __builtin_amdgcn_rcpf(1.0f + fast_exp2(-1.4426950408889634f * g));
          *(MSD_LDS T*)(ost + row * kORow + (nb * 32 + l32) * 2) = E::from_float(sg * u);
        }
      } else {
#pragma unroll
        for (int nb = 0; nb < 4; ++nb)
          *(MSD_LDS T*)(ost + row * kORow + (nb * 32 + l32) * 2) = E::from_float(acc[mb][nb][r] + bias_v[nb]);
      }
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < 32 * kChunks / 64; ++i) {
      const int cidx = i * 64 + lane;
      const int row = cidx / kChunks, c16 = cidx % kChunks;
      const int m = m0 + wm * 128 + mb * 32 + row;
      const int col = col0 + c16 * 8;
      const i32x2_t lo = *(MSD_LDS const i32x2_t*)(ost + row * kORow + c16 * 16);
      const i32x2_t hi = *(MSD_LDS const i32x2_t*)(ost + row * kORow + c16 * 16 + 8);
      if (m < p.M && col < p.Nout) *(i32x4_t*)(og + (long long)m * p.Nout + col) = i32x4_t{lo[0], lo[1], hi[0], hi[1]};
    }
    __builtin_amdgcn_wave_barrier();
  }
#endif
}

}  // namespace msd

using namespace msd;

extern "C" {

int mindiesd_mx_quant(const void* x, void* q, void* e8m0, int dtype, long long M, int K, long long x_stride,
                      hipStream_t stream) {
  if (!x || !q || !e8m0 || M <= 0 || K <= 0) return MSD_ERR_BAD_ARG;
  if (K % 32 != 0 || x_stride % 8 != 0 || ((uintptr_t)x & 15) || ((uintptr_t)q & 7)) return MSD_ERR_BAD_ARG;
  if (dtype != MSD_DTYPE_BF16 && dtype != MSD_DTYPE_F16) return MSD_ERR_BAD_ARG;
  const long long chunks = M * (K / 8);
  const unsigned grid = (unsigned)((chunks + 255) / 256);
  if (dtype == MSD_DTYPE_BF16)
    hipLaunchKernelGGL(mx_quant_kernel<MSD_DTYPE_BF16>, dim3(grid), dim3(256), 0, stream, x, (unsigned char*)q,
                       (unsigned char*)e8m0, M, K, x_stride);
  else
    hipLaunchKernelGGL(mx_quant_kernel<MSD_DTYPE_F16>, dim3(grid), dim3(256), 0, stream, x, (unsigned char*)q,
                       (unsigned char*)e8m0, M, K, x_stride);
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

// out[M][Nout] = act(X W^T + bias); swiglu != 0: W = [gate rows | up rows], Nout = Nw/2,
// out = silu(gate) * up; otherwise Nout = Nw.
int mindiesd_mxfp8_gemm(const void* a, const void* a_scale, const void* w, const void* w_scale, const float* bias,
                        void* out, int out_dtype, int M, int K, int Nw, int swiglu, hipStream_t stream) {
  if (!a || !a_scale || !w || !w_scale || !out || M <= 0 || K <= 0 || Nw <= 0) return MSD_ERR_BAD_ARG;
  if (K % 128 != 0) return MSD_ERR_UNSUPPORTED;
  if (swiglu && (Nw % 16 != 0)) return MSD_ERR_UNSUPPORTED;
  if (!swiglu && (Nw % 8 != 0)) return MSD_ERR_UNSUPPORTED;
  if (out_dtype != MSD_DTYPE_BF16 && out_dtype != MSD_DTYPE_F16) return MSD_ERR_BAD_ARG;
  if (((uintptr_t)a | (uintptr_t)w | (uintptr_t)out) & 15) return MSD_ERR_BAD_ARG;
  if (((uintptr_t)a_scale | (uintptr_t)w_scale) & 3) return MSD_ERR_BAD_ARG;
  // 32-bit buffer offsets
  if ((long long)M * K >= (1ll << 31) - 1024 || (long long)Nw * K >= (1ll << 31) - 1024) return MSD_ERR_UNSUPPORTED;
  GemmParams p{};
  p.a = (const unsigned char*)a; p.as = (const unsigned char*)a_scale;
  p.w = (const unsigned char*)w; p.ws = (const unsigned char*)w_scale;
  p.bias = bias; p.out = out;
  p.M = M; p.K = K; p.Nw = Nw; p.Nout = swiglu ? Nw / 2 : Nw;
  p.tiles_m = (M + 255) / 256;
  p.tiles_n = swiglu ? (Nw / 2 + 127) / 128 : (Nw + 255) / 256;
  constexpr int kLds = 4 * (256 * 64 + 256 * 64) + 2 * 8192 + 1024;  // ring of four 32 KiB stages + two scale chunk buffers + scrap;
                                                             // the output staging (4 x 32 rows x 264 B) reuses the ring
  const int total = p.tiles_m * p.tiles_n;
  const int grid = (total + 7) / 8 * 8;
#define MSD_LAUNCH_GEMM(DTV, SW)                                                                                   \
  {                                                                                                                \
    auto kern = mxfp8_gemm_kernel<DTV, SW>;                                                                        \
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kLds) != hipSuccess)    \
      return MSD_ERR_LAUNCH;                                                                                       \
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), kLds, stream, p);                                              \
  }
  if (out_dtype == MSD_DTYPE_BF16) {
    if (swiglu) MSD_LAUNCH_GEMM(MSD_DTYPE_BF16, true) else MSD_LAUNCH_GEMM(MSD_DTYPE_BF16, false)
  } else {
    if (swiglu) MSD_LAUNCH_GEMM(MSD_DTYPE_F16, true) else MSD_LAUNCH_GEMM(MSD_DTYPE_F16, false)
  }
#undef MSD_LAUNCH_GEMM
  return hipGetLastError() == hipSuccess ? MSD_OK : MSD_ERR_LAUNCH;
}

}  // extern "C"
