// Weight-gradient side of the backward pass, shared by the fused and the alternating backend:
//   * transpose of R for the reverse contraction      (reference: Python-side permute+contiguous,
//     flashrnn/flashrnn/flashrnn.py:746 and :874)
//   * dR[g,n,d,p] = sum_{b,t} dG_g[b,t,n,d] * h_{t-1}[b,n,p]  as one split-K MFMA GEMM over all
//     compute units after the scan                    (reference: cuBLAS gemmsb with k = B*T,
//     flashrnn/flashrnn/fused/flashrnn_fused_backward.cu:1049-1055)
//   * final reduction of the split-K partial sums and of the per-batch-tile bias sums
//     (reference: gradientBiasAggregationKernel, flashrnn_fused_backward.cu:626-665).
// Both GEMM operands are stored with the contraction index (b,t) as the slow index, so tiles are
// transposed on their way into LDS (bf16; the fp32 MFMA takes them as they are).
#include "frnn_grad.h"
#include <cstdlib>
#include <type_traits>

namespace frnn {

// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256) transpose_r_kernel(const T* __restrict__ R, T* __restrict__ Rt, int N, int D, int GR) {
  __shared__ T tile[32][33];
  const int g = blockIdx.z / N, n = blockIdx.z % N;
  const int d0 = blockIdx.y * 32, p0 = blockIdx.x * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const T* src = R + ((size_t)(g * N + n) * D) * D;
  for (int r = ty; r < 32; r += 8) tile[r][tx] = src[(size_t)(d0 + r) * D + p0 + tx];  // [d][p]
  __syncthreads();
  T* dst = Rt + (size_t)n * D * ((size_t)GR * D);
  for (int r = ty; r < 32; r += 8) dst[(size_t)(p0 + r) * ((size_t)GR * D) + (size_t)g * D + d0 + tx] = tile[tx][r];
}

int launch_transpose_r(int dtype, const void* R, void* Rt, int N, int D, int GR, hipStream_t st) {
  const dim3 grid(D / 32, D / 32, GR * N);
  if (dtype != FRNN_F32)
    hipLaunchKernelGGL(transpose_r_kernel<unsigned short>, grid, dim3(256), 0, st, (const unsigned short*)R, (unsigned short*)Rt, N, D, GR);
  else
    hipLaunchKernelGGL(transpose_r_kernel<float>, grid, dim3(256), 0, st, (const float*)R, (float*)Rt, N, D, GR);
  return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------------------------
// dR GEMM.  Workgroup tile TM (units d of one gate) x TM (previous units p), 4 waves in 2 x 2,
// 32 rows (b,t) per LDS stage; grid (tiles, N, splits).
// ---------------------------------------------------------------------------------------------
// Which tile of which (head, split) a workgroup computes.  All tiles of one (head, split) read the same rows of h, and
// the tiles of one gate row the same rows of dG, so they should run at the same time behind the same L2: the device hands
// consecutive workgroups to its 8 XCDs in turn (each with an L2 of its own), so the workgroups of one XCD, every 8th in
// launch order, take the tiles of one (head, split) after another.  Without this each of the 4 gate tiles of LSTM D = 64
// and D = 256 ran on an XCD of its own and h came from HBM four times (3.2 GB per launch instead of 2.0 at B = 256,
// T = 1024).  The last (head, split) pairs, less than 8, keep the plain order.
__device__ __forceinline__ void gemm_tile_of(const GradGemmArgs& a, int TM, int& g, int& dt, int& pt, int& n, int& split) {
  const int tiles = a.D / TM;
  const int per_pair = gridDim.x, pairs = gridDim.y * gridDim.z;
  const int lin = blockIdx.x + per_pair * (blockIdx.y + gridDim.y * blockIdx.z);
  int tile, pair;
  if (lin < (pairs / 8) * 8 * per_pair) {
    const int j = lin / 8;
    tile = j % per_pair;
    pair = (j / per_pair) * 8 + lin % 8;
  } else {
    tile = lin % per_pair;
    pair = lin / per_pair;
  }
  n = pair % a.N; split = pair / a.N;
  pt = tile % tiles; tile /= tiles;
  dt = tile % tiles;
  g = tile / tiles;
}

template <int WT>
__device__ __forceinline__ void gemm_store_partial(const GradGemmArgs& a, int TM, int g, int n, int split, int dt, int pt,
                                                   int wm, int wn, int r16, int q4, const f32x4 (&acc)[WT][WT], int span) {
  const int D = a.D;
  float* out = a.part + ((((size_t)split * a.GR + g) * a.N + n) * D) * D;
#pragma unroll
  for (int i = 0; i < WT; ++i)
#pragma unroll
    for (int j = 0; j < WT; ++j) {
      const int d = dt * TM + wm * span + i * 16 + q4 * 4;  // span: units per wave
      const int p = pt * TM + wn * span + j * 16 + r16;
#pragma unroll
      for (int e = 0; e < 4; ++e) out[(size_t)(d + e) * D + p] = acc[i][j][e];
    }
}

// 16-bit storage types.  Both operands arrive with the contraction index as the slow one.  The stages are brought in
// by direct global-to-LDS loads (global_load_lds_dwordx4: no registers, no LDS store instructions) and transposed on
// their way OUT of LDS by ds_read_b64_tr_b16.  Workgroup tile TM x TM, WD x WD waves of (TM / WD)^2 each.
//   LDS stage of one operand: [32 rows (b,t)][TM units], rows as they lie in memory.  A load instruction of a wave
//   fills 1024 consecutive bytes (lane i writes bytes 16i..16i+15), which lane fetches which 16-byte chunk of the
//   row is free to choose: the chunks of row r are stored at position (chunk ^ f(r)), f even, so that the
//   transposing reads below, which touch 32 bytes of each of 8 rows at the same unit offset per pass, fall on 8
//   different groups of 8 banks.
//   ds_read_b64_tr_b16, as measured: in a group of 16 lanes, lane i receives element i % 4 of the 8-byte pieces
//   that lanes i/4, i/4 + 4, i/4 + 8, i/4 + 12 point at.  Source lane s = a + 4j points at (row k0 + j, units
//   u0 + 4a ..): lane i then holds rows k0 .. k0+3 of unit u0 + i, i.e. 4 consecutive k of its own MFMA row.  Two
//   reads (k0 = 4q and 16 + 4q for lane group q) give the 8 k of a v_mfma_f32_16x16x32 operand; both operands use
//   the same assignment of k to (group, element), which is all the instruction needs.
//   NS stages are in flight: the loads of stage s + NS - 1 are issued right after the barrier that frees its
//   buffer; one barrier per stage.
template <typename T, int TM, int WD, int NS>
__global__ void __launch_bounds__(64 * WD * WD) grad_gemm16_kernel(const GradGemmArgs a) {
  typedef ST<T> X;
  static_assert(sizeof(T) == 2, "16-bit storage types");
  constexpr int NW = WD * WD, NT = 64 * NW;
  constexpr int WT = TM / (16 * WD);    // MFMA tiles per wave per dimension
  constexpr int CPR = TM / 8;           // 16-byte chunks per staged row
  constexpr int KB = 32;                // rows (b,t) per stage
  constexpr int OPB = KB * TM * 2;      // bytes of one operand of one stage
  constexpr int IPW = CPR / NW;         // load instructions per wave and stage (CPR instructions: CPR/2 per operand)
  static_assert(CPR >= NW && CPR % NW == 0 && NS >= 2, "every wave issues the same number of loads");
  extern __shared__ __attribute__((aligned(16))) unsigned char gemm_smem[];  // [NS][operand][KB rows][TM units]
  typedef __attribute__((address_space(3))) unsigned char lds_byte;
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  lds_byte* const sm = (lds_byte*)gemm_smem;

  int g, dt, pt;
  int n, split;
  gemm_tile_of(a, TM, g, dt, pt, n, split);
  const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = w / WD, wn = w % WD;
  const int r16 = lane & 15, q4 = lane >> 4;
  const int N = a.N, Tn = a.T;
  const long rows = (long)a.B * Tn;
  const long r_begin = (long)split * a.rows_per_split;
  const long r_end = min(rows, r_begin + a.rows_per_split);
  const size_t ND = (size_t)N * a.D;
  // (a row of 128 units fills the 64 banks once: 8 rows, 8 groups of 8 banks; shorter rows share them.  Rows of 96 or
  // 160 units, 12 or 20 chunks, start 16 banks apart modulo 64, so rows r, r + 4, r + 8, r + 12 would meet: they are
  // shifted by 0, 2, 4, 6 chunks, with wrap-around instead of the exclusive or, which then puts two of the 16 rows of a
  // read on every bank, as few as there can be)
  constexpr bool POW2 = (CPR & (CPR - 1)) == 0;
  auto fz = [](int row) { return !POW2 ? 2 * ((row / 4) % 4) : TM >= 128 ? 2 * (row % 8) : 2 * ((row / (128 / TM)) % (CPR / 2)); };
  auto swz = [](int chunk, int f) { return POW2 ? (chunk ^ f) : (chunk + f) % CPR; };        // position of a chunk in its row
  auto unswz = [](int pos, int f) { return POW2 ? (pos ^ f) : (pos - f + CPR) % CPR; };      // chunk at a position

  const T* __restrict__ G = static_cast<const T*>(a.gsrc[g]) + (size_t)n * a.D + dt * TM;
  const long gld = a.gld[g];
  const T* __restrict__ H = static_cast<const T*>(a.states_h) + (size_t)n * a.D + pt * TM;
  const T* __restrict__ H0 = static_cast<const T*>(a.s0_h) + (size_t)n * a.D + pt * TM;

  // This wave's load instructions: instruction q = w + NW*i of the stage; the first CPR/2 fill operand A (dG), the
  // others operand B (h of the step before); instruction j of an operand fills chunk positions 64j .. 64j+63.
  // A stage whose 32 rows are all valid and hold no first step of a sequence (t = 0, where h comes from the
  // initial state) is affine in the row: the lane's offset never changes and the stage's base address, uniform,
  // advances in scalar registers, so a load costs no vector instruction besides itself.  The other stages (one in
  // T / 32, and the last of a split) compute their addresses per lane.
  unsigned voff[IPW];  // this lane's byte offset from the stage base of its operand
  int lrow[IPW], lchunk[IPW];
#pragma unroll
  for (int i = 0; i < IPW; ++i) {
    const int q = w + NW * i, j = q % (CPR / 2);
    const bool isb = q >= CPR / 2;  // uniform
    const int P = 64 * j + lane;
    lrow[i] = P / CPR; lchunk[i] = unswz(P % CPR, fz(lrow[i]));
    voff[i] = (unsigned)(((size_t)lrow[i] * (isb ? ND : (size_t)gld) + lchunk[i] * 8) * sizeof(T));
  }
  auto dma = [&](const T* p, lds_byte* dst) __attribute__((always_inline)) {
    // (as asm: the compiler, which cannot tell which stage a later LDS read belongs to, would put a wait for
    // every load in flight in front of the fragment reads; the waits are placed by hand below)
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(p), "s"((unsigned)(size_t)dst) : "memory", "m0");
  };
  auto dma_affine = [&](const T* base, unsigned off, lds_byte* dst) __attribute__((always_inline)) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"((unsigned)(size_t)dst) : "memory", "m0");
  };
  long next_seq = (long)(((unsigned)r_begin + (unsigned)Tn - 1u) / (unsigned)Tn) * Tn;  // (uniform) first row at or behind the stage's first that starts a sequence
  // loads of the stage that begins at row r0 into buffer buf
  auto issue = [&](long r0, int buf) __attribute__((always_inline)) {
    while (next_seq < r0) next_seq += Tn;
    const bool plain = r0 + KB <= r_end && next_seq >= r0 + KB;  // uniform
    const T* const baseA = G + (size_t)r0 * gld;
    const T* const baseB = H + (size_t)(r0 - 1) * ND;  // (before the tensor for r0 = 0, whose stage is never plain)
#pragma unroll
    for (int i = 0; i < IPW; ++i) {
      const int q = w + NW * i, j = q % (CPR / 2);
      const int isb = q >= CPR / 2 ? 1 : 0;  // uniform
      lds_byte* dst = sm + (buf * 2 + isb) * OPB + j * 1024;
      if (plain) {
        dma_affine(isb ? baseB : baseA, voff[i], dst);
      } else {
        // rows beyond the end fetch the last valid row (and are zeroed in LDS afterwards)
        long r = r0 + lrow[i];
        r = r < r_end ? r : r_end - 1;
        const T* p;
        if (isb) {
          const unsigned b = (unsigned)r / (unsigned)Tn;  // (B * T < 2^31, checked on the host)
          p = ((unsigned)r - b * (unsigned)Tn > 0) ? H + (size_t)(r - 1) * ND : H0 + (size_t)b * ND;
        } else {
          p = G + (size_t)r * gld;
        }
        dma(p + lchunk[i] * 8, dst);
      }
    }
  };

  f32x4 acc[WT][WT];
#pragma unroll
  for (int i = 0; i < WT; ++i)
#pragma unroll
    for (int j = 0; j < WT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // fragment reads: lane (group q4, s = r16) points at row 4*q4 + s/4 (+16 for the second read), units 4*(s%4)..
  const int krow = 4 * q4 + (r16 >> 2), sub = r16 & 3;
  const int f1 = fz(krow);  // (= fz(krow + 16): the second read's address is the first's plus 16 rows)
  const int ro1 = krow * (TM * 2) + (sub & 1) * 8;
  const int ga0 = (wm * (TM / WD)) / 8 + (sub >> 1), gb0 = (wn * (TM / WD)) / 8 + (sub >> 1);
  // byte offsets within a stage buffer (operand B: + OPB), the same for every stage
  int oa1[WT], ob1[WT];
#pragma unroll
  for (int i = 0; i < WT; ++i) {
    oa1[i] = ro1 + (swz(ga0 + 2 * i, f1) << 4);
    ob1[i] = OPB + ro1 + (swz(gb0 + 2 * i, f1) << 4);
  }
  constexpr int O2 = 16 * TM * 2;

  const int nst = (int)((r_end - r_begin + KB - 1) / KB);
#pragma unroll
  for (int s = 0; s < NS - 1; ++s)
    if (s < nst) issue(r_begin + (long)s * KB, s);
  // one stage; `buf` is a compile-time constant (the loop below is unrolled over the NS buffers), so that the
  // buffer's position goes into the offset field of the LDS reads
  auto stage = [&](int s, auto BUF) __attribute__((always_inline)) {
    constexpr int buf = decltype(BUF)::value;
    // stage s has landed once at most the loads of the NS-2 stages behind it are in flight
    if (s + NS - 2 < nst) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(IPW * (NS - 2)) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // every wave's part of stage s is there; every wave is done with the buffer of stage s - 1
    // (a barrier that orders LDS only: __syncthreads() would wait for the loads in flight)
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (s + NS - 1 < nst) issue(r_begin + (long)(s + NS - 1) * KB, (buf + NS - 1) % NS);
    const long nvalid = r_end - (r_begin + (long)s * KB);
    if (nvalid < KB) {  // (uniform; the last stage of a split only) rows beyond the end count as zero
      for (int P = (int)nvalid * CPR + tid; P < KB * CPR; P += NT) {
        *(__attribute__((address_space(3))) u32x4*)(sm + (buf * 2) * OPB + P * 16) = u32x4{0u, 0u, 0u, 0u};
        *(__attribute__((address_space(3))) u32x4*)(sm + (buf * 2 + 1) * OPB + P * 16) = u32x4{0u, 0u, 0u, 0u};
      }
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
    lds_byte* const sb = sm + (buf * 2) * OPB;
    typename X::Frag af[WT], bfr[WT];
#pragma unroll
    for (int i = 0; i < WT; ++i) {
      const s16x4 a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(sb + oa1[i]));
      const s16x4 a2 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(sb + oa1[i] + O2));
      const s16x4 b1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(sb + ob1[i]));
      const s16x4 b2 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(sb + ob1[i] + O2));
      af[i] = __builtin_bit_cast(typename X::Frag, __builtin_shufflevector(a1, a2, 0, 1, 2, 3, 4, 5, 6, 7));
      bfr[i] = __builtin_bit_cast(typename X::Frag, __builtin_shufflevector(b1, b2, 0, 1, 2, 3, 4, 5, 6, 7));
    }
    __builtin_amdgcn_sched_barrier(0);  // all reads in front of the first MFMA: their latency is paid once
#pragma unroll
    for (int i = 0; i < WT; ++i)
#pragma unroll
      for (int j = 0; j < WT; ++j) acc[i][j] = X::mfma(af[i], bfr[j], acc[i][j]);
  };
  for (int s = 0; s < nst; s += NS) {
    stage(s, std::integral_constant<int, 0>{});
    if (s + 1 < nst) stage(s + 1, std::integral_constant<int, 1 % NS>{});
    if (NS > 2 && s + 2 < nst) stage(s + 2, std::integral_constant<int, 2 % NS>{});
    static_assert(NS <= 3, "the stage loop is written out for up to 3 buffers");
  }
  gemm_store_partial<WT>(a, TM, g, n, split, dt, pt, wm, wn, r16, q4, acc, TM / WD);
}

// fp32 storage: the MFMA (16x16x4) takes the operands as they are stored, [row][unit]
template <int TM> struct GemmStage32 {
  static constexpr int LD = TM + 4;
  float a[32][LD], b[32][LD];
};

template <int TM>
__global__ void __launch_bounds__(256) grad_gemm32_kernel(const GradGemmArgs a) {
  typedef float T;
  typedef ST<T> X;
  constexpr int EV = TM / 8;           // elements per thread per staged row
  constexpr int WT = TM / 32;          // MFMA tiles per wave per dimension
  constexpr int WD = 2;                // 2 x 2 waves
  __shared__ __attribute__((aligned(16))) GemmStage32<TM> sm;

  int g, dt, pt;
  int n, split;
  gemm_tile_of(a, TM, g, dt, pt, n, split);
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int wm = w >> 1, wn = w & 1;
  const int r16 = lane & 15, q4 = lane >> 4;
  const int D = a.D, N = a.N, Tn = a.T;
  const long rows = (long)a.B * Tn;
  const long r_begin = (long)split * a.rows_per_split;
  const long r_end = min(rows, r_begin + a.rows_per_split);
  const size_t ND = (size_t)N * D;

  const T* __restrict__ G = static_cast<const T*>(a.gsrc[g]) + (size_t)n * D + dt * TM;
  const long gld = a.gld[g];
  const T* __restrict__ H = static_cast<const T*>(a.states_h) + (size_t)n * D + pt * TM;
  const T* __restrict__ H0 = static_cast<const T*>(a.s0_h) + (size_t)n * D + pt * TM;

  f32x4 acc[WT][WT];
#pragma unroll
  for (int i = 0; i < WT; ++i)
#pragma unroll
    for (int j = 0; j < WT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int rr = tid / (TM / EV), cc = (tid % (TM / EV)) * EV;
  T ga[EV], hb[EV];
  auto fetch = [&](long r0) __attribute__((always_inline)) {
    const long r = r0 + rr;
    if (r < r_end) {
      const long b = r / Tn, t = r - b * Tn;
      const T* gp = G + (size_t)r * gld + cc;
      const T* hp = (t > 0) ? H + (size_t)(r - 1) * ND + cc : H0 + (size_t)b * ND + cc;
#pragma unroll
      for (int e = 0; e < EV; ++e) { ga[e] = gp[e]; hb[e] = hp[e]; }
    } else {
#pragma unroll
      for (int e = 0; e < EV; ++e) { ga[e] = 0.0f; hb[e] = 0.0f; }
    }
  };
  fetch(r_begin);
  for (long r0 = r_begin; r0 < r_end; r0 += 32) {
    __syncthreads();  // previous stage fully consumed
#pragma unroll
    for (int e = 0; e < EV; ++e) { sm.a[rr][cc + e] = ga[e]; sm.b[rr][cc + e] = hb[e]; }
    __syncthreads();
    if (r0 + 32 < r_end) fetch(r0 + 32);
#pragma unroll
    for (int k4 = 0; k4 < 8; ++k4) {
      float af[WT], bfr[WT];
#pragma unroll
      for (int i = 0; i < WT; ++i) {
        af[i] = sm.a[k4 * 4 + q4][wm * (TM / 2) + i * 16 + r16];
        bfr[i] = sm.b[k4 * 4 + q4][wn * (TM / 2) + i * 16 + r16];
      }
#pragma unroll
      for (int i = 0; i < WT; ++i)
#pragma unroll
        for (int j = 0; j < WT; ++j) acc[i][j] = X::mfma(af[i], bfr[j], acc[i][j]);
    }
  }
  gemm_store_partial<WT>(a, TM, g, n, split, dt, pt, wm, wn, r16, q4, acc, TM / WD);
}

// side of the square workgroup tile: the largest of 256, 128 (16-bit types only), 64, 32 that divides D; 96 and 160
// (16-bit types) for the head dims that only much smaller powers of two divide: every pair of tiles of a gate streams
// both of its operand slabs, so D = 96 as 9 pairs of 32-unit tiles took 1.30 ms at B256 T1024 N8 against 0.40 for D = 64
static int gemm_tile_side(int dtype, int D) {
  if (dtype != FRNN_F32 && D % 256 == 0) return 256;
  if (dtype != FRNN_F32 && D % 128 == 0) return 128;
  if (dtype != FRNN_F32 && D % 96 == 0 && D / 96 <= 2) return 96;     // 96, 192
  if (dtype != FRNN_F32 && D % 160 == 0 && D / 160 <= 3) return 160;  // 160, 320, 480
  return (D % 64 == 0) ? 64 : 32;
}

// split-K factor.  Tiles of up to 128 units (workgroups of 4 waves): a workgroup waits for its loads once per stage,
// so the kernel lives on many workgroups per compute unit (measured: time falls with the split count until about 8
// per unit).  Tiles of 256 units (16 waves, 96 KB of LDS: one workgroup per compute unit, three stages in flight):
// one workgroup per compute unit, all in one round (measured at D = 256, 768, 1024: best at 190-260 workgroups).
// Bounded by 4 stages per split and by 64 MiB of partial sums.
int grad_gemm_splits(int dtype, int B, int T, int N, int D, int GR) {
  const int TM = gemm_tile_side(dtype, D);
  const long tiles = (long)GR * (D / TM) * (D / TM) * N;
  const long chunks = ((long)B * T + 31) / 32;
  const long out_bytes = (long)GR * N * D * D * 4;
  // (heads of one 64- or 128-unit tile per gate, 16-bit types: three workgroups per compute unit, measured: LSTM N = 12
  // D = 64, 48 tiles, best at 16 splits from B = 16 to B = 256, 0.402 against 0.440 ms with 43 at B = 256)
  const long many = (dtype != FRNN_F32 && TM == D && TM >= 64) ? 768 : 2048;
  long s = TM == 256 ? (256 + tiles / 2) / tiles : (many + tiles - 1) / tiles;
  if (s > 64) s = 64;
  if (s > (64l << 20) / out_bytes) s = (64l << 20) / out_bytes;
  if (s > chunks / 4) s = chunks / 4;
  if (const char* e = getenv("FRNN_GEMM_SPLITS")) s = atoi(e);
  if (s > 64) s = 64;
  if (s < 1) s = 1;
  return (int)s;
}

template <typename T, int TM, int WD>
static int launch_gemm16(const GradGemmArgs& a, dim3 grid, hipStream_t st) {
  constexpr int NS = 3;
  const size_t lds = (size_t)NS * 2 * 32 * TM * 2;
  if (lds > 65536) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&grad_gemm16_kernel<T, TM, WD, NS>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  hipLaunchKernelGGL((grad_gemm16_kernel<T, TM, WD, NS>), grid, dim3(64 * WD * WD), lds, st, a);
  return (int)hipGetLastError();
}
template <typename T>
static int launch_gemm16_any(int TM, const GradGemmArgs& a, dim3 grid, hipStream_t st) {
  if (TM == 256) return launch_gemm16<T, 256, 4>(a, grid, st);
  if (TM == 128) return launch_gemm16<T, 128, 2>(a, grid, st);
  if (TM == 64) return launch_gemm16<T, 64, 2>(a, grid, st);
  if (TM == 96) return launch_gemm16<T, 96, 2>(a, grid, st);
  if (TM == 160) return launch_gemm16<T, 160, 2>(a, grid, st);
  return launch_gemm16<T, 32, 2>(a, grid, st);
}

int launch_grad_gemm(int dtype, GradGemmArgs a, int splits, hipStream_t st) {
  const int TM = gemm_tile_side(dtype, a.D);
  const long chunks = ((long)a.B * a.T + 31) / 32;
  a.rows_per_split = (int)(((chunks + splits - 1) / splits) * 32);
  const dim3 grid(a.GR * (a.D / TM) * (a.D / TM), a.N, splits);
  if (dtype == FRNN_BF16) return launch_gemm16_any<bf16_t>(TM, a, grid, st);
  if (dtype == FRNN_F16) return launch_gemm16_any<half_t>(TM, a, grid, st);
  if (TM == 64) hipLaunchKernelGGL((grad_gemm32_kernel<64>), grid, dim3(256), 0, st, a);
  else hipLaunchKernelGGL((grad_gemm32_kernel<32>), grid, dim3(256), 0, st, a);
  return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------------------------
// out[i] = sum_s part[s][i]: i < n_r for the dR partials (splits_r of them), then i - n_r < n_b
// for the bias partials (splits_b of them).
// ---------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) grad_reduce_kernel(const float* __restrict__ part_r, int splits_r, size_t n_r, float* __restrict__ dR,
                                                          const float* __restrict__ part_b, int splits_b, size_t n_b, float* __restrict__ db) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n_r) {
    float s = 0.f;
#pragma unroll 16
    for (int k = 0; k < splits_r; ++k) s += part_r[(size_t)k * n_r + i];
    dR[i] = s;
  } else if (i - n_r < n_b) {
    const size_t j = i - n_r;
    float s = 0.f;
#pragma unroll 16
    for (int k = 0; k < splits_b; ++k) s += part_b[(size_t)k * n_b + j];
    db[j] = s;
  }
}

int launch_grad_reduce(const float* part_r, int splits_r, size_t n_r, float* dR,
                       const float* part_b, int splits_b, size_t n_b, float* db, hipStream_t st) {
  const size_t total = n_r + n_b;
  hipLaunchKernelGGL(grad_reduce_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                     part_r, splits_r, n_r, dR, part_b, splits_b, n_b, db);
  return (int)hipGetLastError();
}

__global__ void __launch_bounds__(256) fill_zero_kernel(unsigned* p, size_t words) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < words) p[i] = 0u;
}
int launch_fill_zero(void* p, size_t bytes, hipStream_t st) {
  const size_t words = (bytes + 3) / 4;
  if (words == 0) return 0;
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, st, (unsigned*)p, words);
  return (int)hipGetLastError();
}

}  // namespace frnn
