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
__device__ __forceinline__ void gemm_tile_of(const GradGemmArgs& a, int TM, int& g, int& dt, int& pt) {
  const int tiles = a.D / TM;
  int tile = blockIdx.x;
  pt = tile % tiles; tile /= tiles;
  dt = tile % tiles;
  g = tile / tiles;
}

template <int WT>
__device__ __forceinline__ void gemm_store_partial(const GradGemmArgs& a, int TM, int g, int n, int split, int dt, int pt,
                                                   int wm, int wn, int r16, int q4, const f32x4 (&acc)[WT][WT]) {
  const int D = a.D;
  float* out = a.part + ((((size_t)split * a.GR + g) * a.N + n) * D) * D;
#pragma unroll
  for (int i = 0; i < WT; ++i)
#pragma unroll
    for (int j = 0; j < WT; ++j) {
      const int d = dt * TM + wm * (TM / 2) + i * 16 + q4 * 4;
      const int p = pt * TM + wn * (TM / 2) + j * 16 + r16;
#pragma unroll
      for (int e = 0; e < 4; ++e) out[(size_t)(d + e) * D + p] = acc[i][j][e];
    }
}

// 16-bit storage types.  Both operands arrive with the contraction index as the slow one, so a stage
// is transposed on its way into LDS: [unit][row pair], one dword = rows (2k, 2k+1) of a unit, 17 dwords
// per unit (16 + 1 pad).  The odd stride puts the 64 lanes of a transposing store on 32 different banks
// (a thread stores 4 adjacent units of one row pair, 16 threads cover 64 units, a wave 4 row pairs) and
// keeps the fragment reads (4 consecutive dwords per lane) conflict-free; an 8-element row stride would
// be a multiple of the bank count for every choice of padding that keeps 16-byte reads aligned
// (measured: bank conflicts in 83 % of the LDS-active cycles, the kernel was LDS-bound).
// Two stages alternate, so that one barrier per stage is enough: the global loads of stage s+1 are
// issued before the MFMAs of stage s and stored to the other buffer after them.
template <int TM> struct GemmStage16 {
  static constexpr int LD = 17;
  unsigned a[2][TM][LD], b[2][TM][LD];
};

template <typename T, int TM>
__global__ void __launch_bounds__(256) grad_gemm16_kernel(const GradGemmArgs a) {
  typedef ST<T> X;
  static_assert(sizeof(T) == 2, "16-bit storage types");
  constexpr int WT = TM / 32;                     // MFMA tiles per wave per dimension
  constexpr int TPR = TM >= 64 ? 16 : TM / 4;     // threads per row pair
  constexpr int CH = TM / (4 * TPR);              // chunks of 4 units per thread and row
  extern __shared__ __attribute__((aligned(16))) unsigned char gemm_smem[];
  GemmStage16<TM>& sm = *reinterpret_cast<GemmStage16<TM>*>(gemm_smem);

  int g, dt, pt;
  gemm_tile_of(a, TM, g, dt, pt);
  const int n = blockIdx.y, split = blockIdx.z;
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

  const int rp = tid / TPR, uc = (tid % TPR) * 4;
  const bool active = rp < 16;
  uint2 ga[CH][2], hb[CH][2];
  auto fetch = [&](long r0) __attribute__((always_inline)) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const long r = r0 + 2 * rp + h;
      const bool ok = active && r < r_end;
      const long b = r / Tn, t = r - b * Tn;
      const T* gp = G + (size_t)r * gld + uc;
      const T* hp = (t > 0) ? H + (size_t)(r - 1) * ND + uc : H0 + (size_t)b * ND + uc;
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        ga[c][h] = make_uint2(0u, 0u); hb[c][h] = make_uint2(0u, 0u);
        if (ok) {
          ga[c][h] = *reinterpret_cast<const uint2*>(gp + c * 64);
          hb[c][h] = *reinterpret_cast<const uint2*>(hp + c * 64);
        }
      }
    }
  };
  auto stage = [&](int buf) __attribute__((always_inline)) {
    if (!active) return;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      // element e of row 2rp in the low half, of row 2rp+1 in the high half
      unsigned (*sa)[GemmStage16<TM>::LD] = &sm.a[buf][uc + c * 64];
      unsigned (*sb)[GemmStage16<TM>::LD] = &sm.b[buf][uc + c * 64];
      sa[0][rp] = (ga[c][0].x & 0xffffu) | (ga[c][1].x << 16);
      sa[1][rp] = (ga[c][0].x >> 16) | (ga[c][1].x & 0xffff0000u);
      sa[2][rp] = (ga[c][0].y & 0xffffu) | (ga[c][1].y << 16);
      sa[3][rp] = (ga[c][0].y >> 16) | (ga[c][1].y & 0xffff0000u);
      sb[0][rp] = (hb[c][0].x & 0xffffu) | (hb[c][1].x << 16);
      sb[1][rp] = (hb[c][0].x >> 16) | (hb[c][1].x & 0xffff0000u);
      sb[2][rp] = (hb[c][0].y & 0xffffu) | (hb[c][1].y << 16);
      sb[3][rp] = (hb[c][0].y >> 16) | (hb[c][1].y & 0xffff0000u);
    }
  };
  fetch(r_begin);
  stage(0);
  __syncthreads();
  int cur = 0;
  for (long r0 = r_begin; r0 < r_end; r0 += 32) {
    const bool more = r0 + 32 < r_end;
    if (more) fetch(r0 + 32);
    typename X::Frag af[WT], bfr[WT];
#pragma unroll
    for (int i = 0; i < WT; ++i) {
      const unsigned* pa = &sm.a[cur][wm * (TM / 2) + i * 16 + r16][q4 * 4];
      const unsigned* pb = &sm.b[cur][wn * (TM / 2) + i * 16 + r16][q4 * 4];
      const u32x4 va = {pa[0], pa[1], pa[2], pa[3]}, vb = {pb[0], pb[1], pb[2], pb[3]};
      af[i] = __builtin_bit_cast(typename X::Frag, va);
      bfr[i] = __builtin_bit_cast(typename X::Frag, vb);
    }
#pragma unroll
    for (int i = 0; i < WT; ++i)
#pragma unroll
      for (int j = 0; j < WT; ++j) acc[i][j] = X::mfma(af[i], bfr[j], acc[i][j]);
    if (more) stage(cur ^ 1);
    __syncthreads();  // the other buffer is complete, and this one has been read by every wave
    cur ^= 1;
  }
  gemm_store_partial<WT>(a, TM, g, n, split, dt, pt, wm, wn, r16, q4, acc);
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
  __shared__ __attribute__((aligned(16))) GemmStage32<TM> sm;

  int g, dt, pt;
  gemm_tile_of(a, TM, g, dt, pt);
  const int n = blockIdx.y, split = blockIdx.z;
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
  gemm_store_partial<WT>(a, TM, g, n, split, dt, pt, wm, wn, r16, q4, acc);
}

// side of the square workgroup tile: the largest of 128 (16-bit types only), 64, 32 that divides D
static int gemm_tile_side(int dtype, int D) {
  if (dtype != FRNN_F32 && D % 128 == 0) return 128;
  return (D % 64 == 0) ? 64 : 32;
}

// split-K factor.  A workgroup waits for its global loads once per stage, so the kernel lives on many
// workgroups per compute unit (measured: time falls with the split count until about 8 per unit);
// bounded by 4 stages per split and by 64 MiB of partial sums.
int grad_gemm_splits(int dtype, int B, int T, int N, int D, int GR) {
  const int TM = gemm_tile_side(dtype, D);
  const long tiles = (long)GR * (D / TM) * (D / TM) * N;
  const long chunks = ((long)B * T + 31) / 32;
  const long out_bytes = (long)GR * N * D * D * 4;
  long s = (2048 + tiles - 1) / tiles;
  if (s > 64) s = 64;
  if (s > (64l << 20) / out_bytes) s = (64l << 20) / out_bytes;
  if (s > chunks / 4) s = chunks / 4;
  if (const char* e = getenv("FRNN_GEMM_SPLITS")) s = atoi(e);
  if (s > 64) s = 64;
  if (s < 1) s = 1;
  return (int)s;
}

template <typename T, int TM>
static int launch_gemm16(const GradGemmArgs& a, dim3 grid, hipStream_t st) {
  const size_t lds = sizeof(GemmStage16<TM>);
  if (lds > 65536) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&grad_gemm16_kernel<T, TM>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  hipLaunchKernelGGL((grad_gemm16_kernel<T, TM>), grid, dim3(256), lds, st, a);
  return (int)hipGetLastError();
}

int launch_grad_gemm(int dtype, GradGemmArgs a, int splits, hipStream_t st) {
  const int TM = gemm_tile_side(dtype, a.D);
  const long chunks = ((long)a.B * a.T + 31) / 32;
  a.rows_per_split = (int)(((chunks + splits - 1) / splits) * 32);
  const dim3 grid(a.GR * (a.D / TM) * (a.D / TM), a.N, splits);
  if (dtype == FRNN_BF16) {
    if (TM == 128) return launch_gemm16<bf16_t, 128>(a, grid, st);
    if (TM == 64) return launch_gemm16<bf16_t, 64>(a, grid, st);
    return launch_gemm16<bf16_t, 32>(a, grid, st);
  } else if (dtype == FRNN_F16) {
    if (TM == 128) return launch_gemm16<half_t, 128>(a, grid, st);
    if (TM == 64) return launch_gemm16<half_t, 64>(a, grid, st);
    return launch_gemm16<half_t, 32>(a, grid, st);
  }
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
