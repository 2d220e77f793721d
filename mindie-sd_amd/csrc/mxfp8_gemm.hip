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
// applied to MX block h of that row.  W is the first matrix operand (accumulator rows n), X the second
// (accumulator columns m): a lane then owns four consecutive output columns per register quad.
//
// Workgroup tile: 256 rows of X x 256 rows of W (for SwiGLU: 128 gate rows f0.. and the 128 up rows
// F+f0.., so both halves of an output element meet in the same lane and register); the kernel comment
// below describes how the tile is walked.  LDS rows are 128 bytes; 16-byte chunk c of row r sits at
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

// Work decomposition: one workgroup of 4 waves (one per SIMD, 256 accumulator registers each) owns a
// 256 x 256 tile of (X rows) x (W rows), seen as 2 x 2 quadrants of 128 x 128; inside a quadrant every
// wave owns 64 x 64 (2 x 2 accumulator blocks).  K is walked in blocks of 128 codes.  The unit of LDS
// traffic is one operand half of one K block: 128 rows x 128 bytes = 16 KiB, so that every DMA
// instruction moves full 128-byte lines.  Per K block the quadrants are visited in the order
// (A0,W0) (A1,W0) (A1,W1) (A0,W1): consecutive steps share one operand half, which stays in registers,
// so every step reads exactly one new unit from LDS into the register set that has just become free
// (the roles of the two A sets swap from one K block to the next, hence the unrolling over 8 steps).
// Units are consumed in the order W0 A0 A1 W1 | W0 A0 A1 W1 | ... and travel through a ring of eight LDS
// slots: during step t unit t+2 goes from LDS into registers, unit t+3 has landed, units t+4 .. t+9 are
// in flight.
template <int DT, bool SWIGLU>
__global__ __launch_bounds__(256, 1) void mxfp8_gemm_kernel(const GemmParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  using E = Elem<DT>;
  using T = typename E::type;
  constexpr int BM = 256, BK = 128, NW = 4, NU = 8;
  constexpr int kUnit = 128 * BK;  // 16 KiB
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
  // W rows of this tile: plain: 256 consecutive rows; SwiGLU: 128 gate rows (half W0) + the matching 128
  // up rows (half W1), so both parts of an output element meet in the same lane and register index
  const int half = p.Nw >> 1;
  const int f0 = SWIGLU ? tn * 128 : tn * 256;

  // ---- LDS-DMA: one instruction = 8 rows x 128 bytes; 16 instructions per unit, 4 per wave ---------------------
  // A row keeps its eight 16-byte chunks at positions chunk ^ ((row >> 1) & 7), which makes the 16-byte
  // operand reads of 16 consecutive rows hit 16 different bank groups.  Rows past the end of a matrix are
  // beyond the descriptor's range and read as zeros; gate rows past the gate part read up rows, whose
  // products land in columns that are never stored.
  const __amdgpu_buffer_rsrc_t a_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.a, 0, (int)((long long)p.M * p.K), 0x00020000);
  const __amdgpu_buffer_rsrc_t w_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.w, 0, (int)((long long)p.Nw * p.K), 0x00020000);
  const __amdgpu_buffer_rsrc_t none_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)p.a, 0, 0, 0x00020000);
  const int k_blocks = p.K / BK;
  int a_voff[4], w_voff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = 8 * (i * NW + wave) + (lane >> 3);  // row inside the 128-row unit
    const int c = (lane & 7) ^ ((row >> 1) & 7);
    a_voff[i] = (m0 + row) * p.K + c * 16;
    w_voff[i] = (f0 + row) * p.K + c * 16;
  }
  const int a1_off = 128 * p.K;                          // second half of the X rows
  const int w1_off = (SWIGLU ? half : 128) * p.K;        // second half of the W rows
  // kind: 0 = W0, 1 = A0, 2 = A1, 3 = W1 (the order of consumption).  K blocks past the end are requested
  // through an empty descriptor: the DMA then writes zeros and costs no memory traffic, which keeps the
  // number of outstanding operations the same in every step.
  auto load_unit = [&](int kb, auto kind_c, int slot) {
    constexpr int KIND = decltype(kind_c)::value;
    constexpr bool IS_A = KIND == 1 || KIND == 2, SECOND = KIND >= 2;
    const bool valid = kb < k_blocks;
    const __amdgpu_buffer_rsrc_t rs = valid ? (IS_A ? a_rsrc : w_rsrc) : none_rsrc;
    MSD_LDS char* ub = smem + slot * kUnit;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int vo = (IS_A ? a_voff[i] : w_voff[i]) + (SECOND ? (IS_A ? a1_off : w1_off) : 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (MSD_LDS void*)(ub + (i * NW + wave) * 1024), 16, vo, kb * BK, 0, 0);
    }
  };

  // ---- scales: staged through LDS in chunks of 4 K blocks (16 scale bytes = 512 K-values per row) -------------------
  // One 16-byte DMA per row and chunk: a scale row is a 128-byte line per 4096 K-values, so short reads
  // of it would cost a full L2 request each.
  const int kblk_row = p.K >> 5;  // scale bytes per row
  const __amdgpu_buffer_rsrc_t as_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.as, 0, (int)((long long)p.M * kblk_row), 0x00020000);
  const __amdgpu_buffer_rsrc_t ws_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.ws, 0, (int)((long long)p.Nw * kblk_row), 0x00020000);
  constexpr int kScBase = NU * kUnit, kScBuf = 2 * 256 * 16;  // two chunk buffers: [X rows | W rows] x 16 B
  int as_voff, ws_voff;
  {
    const int row = 64 * wave + lane;  // wave w stages rows 64w .. 64w+63 of both operands
    as_voff = (m0 + row) * kblk_row;
    const int wrow = row < 128 ? f0 + row : (SWIGLU ? half + f0 + (row - 128) : f0 + row);
    ws_voff = wrow * kblk_row;
  }
  // Requested in every eighth step so that the number of outstanding operations repeats with the
  // unrolled loop; the request that falls in the middle of a chunk (or past the end of K) goes through
  // the empty descriptor into a scrap area and costs nothing.
  auto load_scale_chunk = [&](int t) {  // t: multiple of 8; a chunk is requested 16 steps before its first step
    const int chunk = __builtin_amdgcn_readfirstlane((t + 16) >> 4);
    const bool real = (t & 15) == 0 && 4 * chunk < k_blocks;
    const __amdgpu_buffer_rsrc_t ar = real ? as_rsrc : none_rsrc;
    const __amdgpu_buffer_rsrc_t wr = real ? ws_rsrc : none_rsrc;
    const int dst = __builtin_amdgcn_readfirstlane(real ? kScBase + (chunk & 1) * kScBuf + wave * 1024
                                                        : kScBase + 2 * kScBuf);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(ar, (MSD_LDS void*)(smem + dst), 16, as_voff, chunk * 16, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(wr, (MSD_LDS void*)(smem + dst + (real ? 4096 : 0)), 16, ws_voff,
                                             chunk * 16, 0, 0);
  };
  // LDS offsets of the lane's scale rows inside a chunk buffer: X rows a*128 + wm*64 + mb*32 + l32,
  // W rows (tile-local) w*128 + wn*64 + nb*32 + l32
  const int as_lds = kScBase + (wm * 64 + l32) * 16;
  const int ws_lds = kScBase + 4096 + (wn * 64 + l32) * 16;
  struct Scales {
    int a[2][2], w[2][2];  // [half][block]: one dword = the 4 MX blocks of one K block
  };
  auto read_scales = [&](int kb, Scales& s) {
    const int off = ((kb >> 2) & 1) * kScBuf + (kb & 3) * 4;
#pragma unroll
    for (int hf = 0; hf < 2; ++hf)
#pragma unroll
      for (int blk = 0; blk < 2; ++blk) {
        s.a[hf][blk] = *(MSD_LDS const int*)(smem + as_lds + off + (hf * 128 + blk * 32) * 16);
        s.w[hf][blk] = *(MSD_LDS const int*)(smem + ws_lds + off + (hf * 128 + blk * 32) * 16);
      }
  };

  f32x16_t acc[2][2][2][2];  // [A half][W half][mb][nb]
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) (&acc[0][0][0][0])[i][r] = 0.f;

  const int swz = (l32 >> 1) & 7;
  const int sh = 8 * h;  // the lane's MX block inside a 64-wide K step is block h
  // operand fragments of one unit: [block][k step]; k step ks takes chunk 4ks + h (MX block 2ks) and
  // chunk 4ks + 2 + h (MX block 2ks + 1) of the lane's row
  struct Frag {
    i32x8_t v[2][2];
  };
  int c_off[2][2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    c_off[ks][0] = ((4 * ks + h) ^ swz) << 4;
    c_off[ks][1] = ((4 * ks + 2 + h) ^ swz) << 4;
  }
  const int a_row_off = (wm * 64 + l32) * BK, w_row_off = (wn * 64 + l32) * BK;
  auto read_unit = [&](int slot, Frag& f, bool is_a) {
    MSD_LDS const char* base = smem + slot * kUnit + (is_a ? a_row_off : w_row_off);
#pragma unroll
    for (int blk = 0; blk < 2; ++blk)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const i32x4_t lo = *(MSD_LDS const i32x4_t*)(base + blk * 32 * BK + c_off[ks][0]);
        const i32x4_t hi = *(MSD_LDS const i32x4_t*)(base + blk * 32 * BK + c_off[ks][1]);
        f.v[blk][ks] = i32x8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
  };

  // Workgroup barrier without the memory fence of __syncthreads(): the fence would wait for every DMA in
  // flight, the explicit counts below wait only for the unit that is needed.  The empty asm statements
  // keep the compiler from moving LDS accesses across the barrier.
  auto wg_barrier = [] {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  // s_waitcnt immediates: vmcnt in bits 3:0 (+ 15:14), lgkmcnt(0) unless noted
  constexpr int kWaitVm20 = 0x4074, kWaitVm24 = 0x4078, kWaitVm26 = 0x407a;
  constexpr int kWaitVm24Only = 0x4f78;  // vmcnt(24), LDS reads not waited for

  // ---- prologue: the same issue order the main loop produces, so its wait counts apply from step 0 -------------
  // Per wave a unit is 4 DMA instructions and a scale chunk is 2.
  using IC0 = std::integral_constant<int, 0>;
  using IC1 = std::integral_constant<int, 1>;
  using IC2 = std::integral_constant<int, 2>;
  using IC3 = std::integral_constant<int, 3>;
  Scales sc, sn;
  load_scale_chunk(-16);
  load_unit(0, IC0{}, 0);
  load_unit(0, IC1{}, 1);
  load_unit(0, IC2{}, 2);
  load_unit(0, IC3{}, 3);
  load_unit(1, IC0{}, 4);
  load_unit(1, IC1{}, 5);
  load_unit(1, IC2{}, 6);
  load_unit(1, IC3{}, 7);
  __builtin_amdgcn_s_waitcnt(kWaitVm24Only);  // scale chunk 0, units 0 and 1 landed
  wg_barrier();
  Frag fx, fy, fp, fq;  // X rows: fx, fy; W rows: fp, fq
  read_unit(0, fp, false);
  read_unit(1, fx, true);
  read_scales(0, sn);
  __builtin_amdgcn_s_waitcnt(kWaitVm20);  // unit 2 landed, units 0 and 1 are in registers
  wg_barrier();
  load_unit(2, IC0{}, 0);

  // ---- main loop -----------------------------------------------------------------------------------------------------
  // step t = 4 * kb + q computes quadrant q of K block kb from the register sets (fa, fw), loads unit t+2
  // from LDS into fl and requests unit t+9 (into the slot of unit t+1, read during the previous step).
  auto step = [&](int t, auto j_c, const Frag& fa, const Frag& fw, Frag& fl) {
    constexpr int J = decltype(j_c)::value;  // t % 8
    constexpr int Q = J & 3;
    constexpr int AH = (Q == 1 || Q == 2) ? 1 : 0, WH = Q >= 2 ? 1 : 0;
    constexpr int LKIND = (J + 2) & 3;  // kind of the unit that goes into registers
    // nothing moves across a step boundary
    __builtin_amdgcn_sched_barrier(0);
    if (Q == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        (&sc.a[0][0])[i] = (int)((unsigned)(&sn.a[0][0])[i] >> sh);
        (&sc.w[0][0])[i] = (int)((unsigned)(&sn.w[0][0])[i] >> sh);
      }
    }
    // first half: the k step 0 products and the LDS reads of the next unit (early, so that their latency
    // is over long before the end of the step); second half: the k step 1 products, the DMA requests
    // and the scale reads.  The split also keeps the two products of one accumulator apart.
    read_unit((J + 2) & 7, fl, LKIND == 1 || LKIND == 2);
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
        acc[AH][WH][mb][nb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
            fw.v[nb][0], fa.v[mb][0], acc[AH][WH][mb][nb], 0, 0, 0, sc.w[WH][nb], 0, sc.a[AH][mb]);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // two LDS reads
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one matrix instruction
    }
    __builtin_amdgcn_sched_barrier(0);
    if (J == 0) load_scale_chunk(t);
    load_unit((t + 9) >> 2, std::integral_constant<int, (J + 1) & 3>{}, (J + 1) & 7);
    if (Q == 3) read_scales((t >> 2) + 1, sn);
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
        acc[AH][WH][mb][nb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
            fw.v[nb][1], fa.v[mb][1], acc[AH][WH][mb][nb], 0, 0, 2, sc.w[WH][nb], 2, sc.a[AH][mb]);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                  // one matrix instruction
      __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);                  // one DMA request
      if (J == 0 && i < 2) __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
      if (Q == 3) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);      // two scale reads
    }
    // Unit t+3 must have landed (mine: the wait; everybody's: the barrier), and every wave must be done
    // reading the slot of unit t+2 before the next step refills it.  Requested after unit t+3: six
    // units, plus the two scale requests of step 0 unless they came before it.
    __builtin_amdgcn_s_waitcnt(J <= 5 ? kWaitVm26 : kWaitVm24);
    wg_barrier();
  };
  const int n_steps = 4 * ((k_blocks + 1) & ~1);  // whole pairs of K blocks; a padding block multiplies zeros
  for (int t = 0; t < n_steps; t += 8) {
    step(t + 0, std::integral_constant<int, 0>{}, fx, fp, fy);
    step(t + 1, std::integral_constant<int, 1>{}, fy, fp, fq);
    step(t + 2, std::integral_constant<int, 2>{}, fy, fq, fp);
    step(t + 3, std::integral_constant<int, 3>{}, fx, fq, fy);
    step(t + 4, std::integral_constant<int, 4>{}, fy, fp, fx);
    step(t + 5, std::integral_constant<int, 5>{}, fx, fp, fq);
    step(t + 6, std::integral_constant<int, 6>{}, fx, fq, fp);
    step(t + 7, std::integral_constant<int, 7>{}, fy, fq, fx);
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);  // the trailing (empty) DMA requests

  // ---- epilogue: bias, SwiGLU, 16-bit, straight from the accumulators ----------------------------------------------
  // W rows are the first matrix operand, so accumulator [a][w][mb][nb] register r holds
  // X row a*128 + wm*64 + mb*32 + l32 and W row (tile-local) w*128 + wn*64 + nb*32 + 8*(r/4) + 4*h + r%4:
  // four consecutive output columns per register quad, written as one 8-byte store (the two halves of
  // the wave complete 16 bytes, the four quads and two blocks the 128-byte line).  Output columns of the
  // wave: SwiGLU: f0 + wn*64 + [0,64) (gate from w = 0, up from w = 1); plain: f0 + w*128 + wn*64 + [0,64).
  T* og = (T*)p.out;
  auto write_tile = [&](auto bias_c) {
    constexpr bool BIAS = decltype(bias_c)::value;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      // the bias of this block's columns, fetched once for all rows (columns past the end read column 0: never stored)
      f32x4_t bias_r[2][4];  // [w][j]; SwiGLU: w = 0 gate, w = 1 up
      if (BIAS) {
#pragma unroll
        for (int w = 0; w < 2; ++w)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int col = f0 + (SWIGLU ? 0 : w * 128) + wn * 64 + nb * 32 + 8 * j + 4 * h;
            bias_r[w][j] = *(const f32x4_t*)(p.bias + (SWIGLU ? w * half : 0) + (col < p.Nout ? col : 0));
          }
      }
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) {
          const int m = m0 + a * 128 + wm * 64 + mb * 32 + l32;
          T* orow = og + (long long)m * p.Nout;
#pragma unroll
          for (int w = 0; w < (SWIGLU ? 1 : 2); ++w)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int ncol = wn * 64 + nb * 32 + 8 * j + 4 * h;  // first of the four columns, tile-local
              const int col = f0 + (SWIGLU ? 0 : w * 128) + ncol;
              const bool col_ok = col < p.Nout;
              float v[4];
              if (SWIGLU) {
                f32x4_t bg = {0.f, 0.f, 0.f, 0.f}, bu = {0.f, 0.f, 0.f, 0.f};
                if (BIAS) {
                  bg = bias_r[0][j];
                  bu = bias_r[1][j];
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                  const float g = acc[a][0][mb][nb][4 * j + e] + bg[e];
                  const float u = acc[a][1][mb][nb][4 * j + e] + bu[e];
                  v[e] = g * __builtin_amdgcn_rcpf(1.0f + fast_exp2(-1.4426950408889634f * g)) * u;
                }
              } else {
                f32x4_t bv = {0.f, 0.f, 0.f, 0.f};
                if (BIAS) bv = bias_r[w][j];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = acc[a][w][mb][nb][4 * j + e] + bv[e];
              }
              if (m < p.M && col_ok) {
                T t4[4] = {E::from_float(v[0]), E::from_float(v[1]), E::from_float(v[2]), E::from_float(v[3])};
                *(i32x2_t*)(orow + col) = *(const i32x2_t*)t4;
              }
            }
        }
    }
  };
  if (p.bias) write_tile(std::true_type{});
  else write_tile(std::false_type{});
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
  if ((long long)(M + 256) * K >= (1ll << 31) || (long long)(Nw + 256) * K >= (1ll << 31)) return MSD_ERR_UNSUPPORTED;
  GemmParams p{};
  p.a = (const unsigned char*)a; p.as = (const unsigned char*)a_scale;
  p.w = (const unsigned char*)w; p.ws = (const unsigned char*)w_scale;
  p.bias = bias; p.out = out;
  p.M = M; p.K = K; p.Nw = Nw; p.Nout = swiglu ? Nw / 2 : Nw;
  p.tiles_m = (M + 255) / 256;
  p.tiles_n = swiglu ? (Nw / 2 + 127) / 128 : (Nw + 255) / 256;
  constexpr int kLds = 8 * 16384 + 2 * 8192 + 1024;  // ring of eight 16 KiB units + two scale chunk buffers + scrap
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
