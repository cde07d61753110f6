// Alternating backend ("hip"): one kernel launch per time step (the recurrent product of a tile
// on MFMA, then its gate math); the recurrent matrix is re-read from L2/HBM every step, so any
// head dimension works.  Replaces flashrnn/flashrnn/alternating/flashrnn_forward.cu:150-267,
// flashrnn_backward.cu:267-431 and the four *_pointwise.cu files.
//
// Differences from the reference: product and gate math of a step share one launch and the
// pre-activations stay in fp32 registers/LDS between them (the reference launches a cuBLAS GEMM and
// a pointwise kernel and rounds the pre-activations to the storage type in between,
// flashrnn_forward.cu:176-181); tensors are read and written in the public layouts; everything
// runs on the caller's stream.
#include "frnn_alt.h"
#include "frnn_pointwise.h"

namespace frnn {

__device__ __forceinline__ float ld(const bf16_t* p) { return (float)*p; }
__device__ __forceinline__ float ld(const half_t* p) { return (float)*p; }
__device__ __forceinline__ float ld(const float* p) { return *p; }
__device__ __forceinline__ void st_(bf16_t* p, float v) { *reinterpret_cast<unsigned short*>(p) = f2bf(v); }
__device__ __forceinline__ void st_(half_t* p, float v) { *p = (half_t)v; }
__device__ __forceinline__ void st_(float* p, float v) { *p = v; }

// ---------------------------------------------------------------------------------------------
// One launch per time step.  A workgroup owns a 16-unit tile of one head (all its gate rows) and
// a 16-row batch tile: its 4 waves split the contraction of the recurrent product, operands go
// from global memory straight into MFMA fragments (both are contiguous in k), the partial sums
// meet in LDS, and the tile's 256 elements get their gate math one per thread.  The product and
// the gate math of a step were two launches at first; at 2-3 us per dependent launch, fusing
// them halved the time of a sequence.
//   MFMA result layout: lane l holds units 4*(l/16)+i (i = 0..3) of batch row l%16.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ int red_index(int u, int bl) { return ((u >> 2) * 16 + bl) * 4 + (u & 3); }

struct AltStepFwdArgs {
  const void* Wx; const void* R; const void* b; const void* s0; void* states; void* cache;
  float* sfp;       // [S][B][N][D] fp32 copy of the running state: the states tensor is the
                    // storage-type output, the recurrence itself is carried unrounded (only the h
                    // that feeds the product is read back in the storage type), as in the fused path
  int B, T, N, D, t, training;
  float h_clip;     // > 0: new h clamped to [-h_clip, h_clip]
  int from_sfp;     // this step takes s_{t-1} from sfp (every step but the first; the first too when the
                    // caller carries the state of an earlier call in sfp)
};

template <int F, typename T>
__global__ void __launch_bounds__(256) alt_step_fwd_kernel(const AltStepFwdArgs a) {
  typedef Cell<F> C;
  typedef ST<T> X;
  typedef typename X::Frag Frag;
  typedef CellMath<F, X::FAST> CM;
  constexpr int GR = C::GR, GW = C::GW, GT = C::GT, S = C::S, NC = C::NC;
  __shared__ __attribute__((aligned(16))) float red[4][GR][256];
  const int d0 = blockIdx.x * 16, n = blockIdx.y, bt = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int r16 = lane & 15, q4 = lane >> 4;
  const int D = a.D, N = a.N, B = a.B, Tn = a.T, t = a.t;
  const size_t ND = (size_t)N * D, BND = (size_t)B * ND;
  const T* Wx = static_cast<const T*>(a.Wx);
  const T* R = static_cast<const T*>(a.R);
  const T* bias = static_cast<const T*>(a.b);
  const T* s0 = static_cast<const T*>(a.s0);
  T* states = static_cast<T*>(a.states);

  // thread -> unit d0 + tid % 16 of batch row bt*16 + tid / 16 for the gate math; its operands are
  // requested before the product so that their latency hides behind it
  const int u = tid & 15, bl = tid >> 4;
  const int b = bt * 16 + bl, d = d0 + u;
  const bool evalid = b < B;
  const int be = evalid ? b : 0;
  const size_t idx = ((size_t)be * N + n) * D + d;
  float ry[GR], wx[GW], bb[GT - GR + 1], s[S], cc[NC > 0 ? NC : 1];
#pragma unroll
  for (int g = 0; g < GR; ++g) ry[g] = ld(bias + (size_t)(g * N + n) * D + d);
#pragma unroll
  for (int g = 0; g < GW; ++g) wx[g] = ld(Wx + (((size_t)be * Tn + t) * GW + g) * ND + (size_t)n * D + d);
#pragma unroll
  for (int g = GR; g < GT; ++g) bb[g - GR] = ld(bias + (size_t)(g * N + n) * D + d);
#pragma unroll
  for (int k = 0; k < S; ++k)
    s[k] = a.from_sfp ? a.sfp[(size_t)k * BND + idx] : ld(s0 + ((size_t)k * B + be) * ND + (size_t)n * D + d);

  // ---- R h_{t-1} of the tile: acc[g] = rows (g, n, d0..d0+15) x batch rows bt*16..+15 ----
  {
    const int bm = bt * 16 + r16;
    const bool bvalid = bm < B;
    const T* vrow = (t > 0 ? states + (size_t)(bvalid ? bm : 0) * Tn * ND + (size_t)(t - 1) * ND
                           : s0 + (size_t)(bvalid ? bm : 0) * ND) + (size_t)n * D;
    const int KS = D / X::KM;
    f32x4 acc[GR];
#pragma unroll
    for (int g = 0; g < GR; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
    // fp32: a fragment of v_mfma_f32_16x16x4_f32 is one float per lane, and a load of 4 bytes per lane and k-step
    // left the step waiting for hundreds of tiny loads (LSTM fp32 D = 1024: 52 us per step).  A lane takes 4
    // consecutive k with one 16-byte load instead (k = 16 kg + 4 q4 .. + 3) and MFMA i of the group uses element i of
    // every lane: both operands are read the same way, so every k still meets itself, in another order.
    if constexpr (sizeof(T) == 4) {
      const int KG = D / 16;
      for (int kg0 = w; kg0 < KG; kg0 += 16) {  // 4 groups of this wave per round, requested together
        float4 vf[4], af[4][GR];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int kg = kg0 + 4 * j;
          vf[j] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
          for (int g = 0; g < GR; ++g) af[j][g] = make_float4(0.f, 0.f, 0.f, 0.f);
          if (kg < KG) {  // uniform over the wave
            if (bvalid) vf[j] = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(vrow) + kg * 16 + q4 * 4);
#pragma unroll
            for (int g = 0; g < GR; ++g)
              af[j][g] = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(R) + ((size_t)(g * N + n) * D + d0 + r16) * D + kg * 16 + q4 * 4);
          }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int g = 0; g < GR; ++g) {
            acc[g] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[j][g].x, vf[j].x, acc[g], 0, 0, 0);
            acc[g] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[j][g].y, vf[j].y, acc[g], 0, 0, 0);
            acc[g] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[j][g].z, vf[j].z, acc[g], 0, 0, 0);
            acc[g] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[j][g].w, vf[j].w, acc[g], 0, 0, 0);
          }
      }
    }
    // 4 k-steps of this wave per round: all their fragments are requested before the first MFMA,
    // so a round costs one trip to L2 instead of four
    for (int ks0 = w; ks0 < (sizeof(T) == 4 ? 0 : KS); ks0 += 16) {
      Frag vf[4], af[4][GR];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int ks = ks0 + 4 * j;
        vf[j] = Frag{};
#pragma unroll
        for (int g = 0; g < GR; ++g) af[j][g] = Frag{};
        if (ks < KS) {  // uniform over the wave
          vf[j] = load_frag<T>(vrow, ks, q4);
#pragma unroll
          for (int g = 0; g < GR; ++g) af[j][g] = load_frag<T>(R + ((size_t)(g * N + n) * D + d0 + r16) * D, ks, q4);
          if (!bvalid) vf[j] = Frag{};
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int g = 0; g < GR; ++g) acc[g] = X::mfma(af[j][g], vf[j], acc[g]);
    }
#pragma unroll
    for (int g = 0; g < GR; ++g) *reinterpret_cast<f32x4*>(&red[w][g][lane * 4]) = acc[g];
  }
  __syncthreads();
  if (!evalid) return;
  const int src = red_index(u, bl);
#pragma unroll
  for (int g = 0; g < GR; ++g) ry[g] += red[0][g][src] + red[1][g][src] + red[2][g][src] + red[3][g][src];
  CM::fwd(ry, wx, bb, s, cc);
  s[0] = clamp_if(s[0], a.h_clip);
#pragma unroll
  for (int k = 0; k < S; ++k) {
    st_(states + (((size_t)k * B + b) * Tn + t) * ND + (size_t)n * D + d, s[k]);
    if (a.sfp) a.sfp[(size_t)k * BND + idx] = s[k];
  }
  if (a.training && NC > 0) {
    T* cache = static_cast<T*>(a.cache) + (((size_t)t * B + b) * N + n) * NC * D + d;
#pragma unroll
    for (int c = 0; c < NC; ++c) st_(cache + (size_t)c * D, cc[c]);
  }
}

// Reverse step t: the recurrent term R^T dg_{t+1} of the tile's 16 units (dg of the step above
// comes from the previous launch, in the storage type, as the product's operand), then the
// adjoint of step t for the same units, which leaves dg_t for the next launch.  t == -1: only the
// recurrent term of step 0, added to the running cotangent to give ds0.
struct AltStepBwdArgs {
  const void* Rt; const void* s0; const void* states; const void* cache; const void* dstates;
  void* dWx; void* dgx; void* ds0;
  const void* dg_in;  // [B][N][G_r*D] of step t+1
  void* dg_out;       // same for step t (the other of two buffers)
  float* dsr;         // [S][B][N][D] running cotangent without the recurrent term
  int B, T, N, D, t;
  int has_dg;         // 0: no recurrent term (first reverse step, or gradient_recurrent_cut)
  float g_clip;       // > 0: cotangent carried into h_t clamped to [-g_clip, g_clip]
};

template <int F, typename T>
__global__ void __launch_bounds__(256) alt_step_bwd_kernel(const AltStepBwdArgs a) {
  typedef Cell<F> C;
  typedef ST<T> X;
  typedef typename X::Frag Frag;
  typedef CellMath<F, X::FAST> CM;
  constexpr int GR = C::GR, GW = C::GW, GT = C::GT, S = C::S, NC = C::NC;
  __shared__ __attribute__((aligned(16))) float red[4][256];
  const int d0 = blockIdx.x * 16, n = blockIdx.y, bt = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int r16 = lane & 15, q4 = lane >> 4;
  const int D = a.D, N = a.N, B = a.B, Tn = a.T, t = a.t;
  const size_t ND = (size_t)N * D, BND = (size_t)B * ND;

  // operands of the adjoint first (thread -> unit d0 + tid % 16 of batch row bt*16 + tid / 16), so
  // that their latency hides behind the product
  const int u = tid & 15, bl = tid >> 4;
  const int b = bt * 16 + bl, d = d0 + u;
  const bool evalid = b < B;
  const int be = evalid ? b : 0;
  const size_t idx = ((size_t)be * N + n) * D + d;
  const T* s0 = static_cast<const T*>(a.s0);
  const T* states = static_cast<const T*>(a.states);
  const T* dstates = static_cast<const T*>(a.dstates);
  float cc[NC > 0 ? NC : 1], sp[S], sn[S], dso[S], ds[S], gr[GR], gw[GW], gb[GT];
#pragma unroll
  for (int k = 0; k < S; ++k) ds[k] = a.dsr[(size_t)k * BND + idx];
  if (t >= 0) {  // uniform
    const T* cache = static_cast<const T*>(a.cache) + (((size_t)t * B + be) * N + n) * NC * D + d;
#pragma unroll
    for (int c = 0; c < NC; ++c) cc[c] = ld(cache + (size_t)c * D);
#pragma unroll
    for (int k = 0; k < S; ++k) {
      const size_t so = (((size_t)k * B + be) * Tn + t) * ND + (size_t)n * D + d;
      sn[k] = ld(states + so);
      dso[k] = ld(dstates + so);
      sp[k] = t > 0 ? ld(states + so - ND) : ld(s0 + ((size_t)k * B + be) * ND + (size_t)n * D + d);
    }
  }

  if (a.has_dg) {  // uniform
    const int bm = bt * 16 + r16;
    const bool bvalid = bm < B;
    const int K = GR * D, KS = K / X::KM;
    const T* arow = static_cast<const T*>(a.Rt) + ((size_t)n * D + d0 + r16) * K;
    const T* vrow = static_cast<const T*>(a.dg_in) + ((size_t)(bvalid ? bm : 0) * N + n) * K;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    f32x4 acc2 = {0.f, 0.f, 0.f, 0.f};  // two chains: a dependent MFMA waits ~3x longer than an independent one
    if constexpr (sizeof(T) == 4) {  // (16-byte loads of 4 consecutive k per lane: see the forward kernel)
      const int KG = K / 16;
      for (int kg0 = w; kg0 < KG; kg0 += 32) {
        float4 vf[8], af[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int kg = kg0 + 4 * j, kc = kg < KG ? kg : KG - 1;
          vf[j] = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(vrow) + kc * 16 + q4 * 4);
          af[j] = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(arow) + kc * 16 + q4 * 4);
          if (!bvalid || kg >= KG) vf[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(af[j].x, vf[j].x, acc, 0, 0, 0);
          acc2 = __builtin_amdgcn_mfma_f32_16x16x4f32(af[j].y, vf[j].y, acc2, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(af[j].z, vf[j].z, acc, 0, 0, 0);
          acc2 = __builtin_amdgcn_mfma_f32_16x16x4f32(af[j].w, vf[j].w, acc2, 0, 0, 0);
        }
      }
    }
    for (int ks0 = w; ks0 < (sizeof(T) == 4 ? 0 : KS); ks0 += 32) {  // 8 k-steps of this wave per round, requested together
      Frag vf[8], af[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {  // out-of-range k-steps load the last one and are zeroed: branch-free (measured faster here)
        const int ks = ks0 + 4 * j, kc = ks < KS ? ks : KS - 1;
        vf[j] = load_frag<T>(vrow, kc, q4);
        af[j] = load_frag<T>(arow, kc, q4);
        if (!bvalid || ks >= KS) vf[j] = Frag{};
      }
#pragma unroll
      for (int j = 0; j < 8; j += 2) {
        acc = X::mfma(af[j], vf[j], acc);
        acc2 = X::mfma(af[j + 1], vf[j + 1], acc2);
      }
    }
    acc += acc2;
    *reinterpret_cast<f32x4*>(&red[w][lane * 4]) = acc;
    __syncthreads();
  }
  if (!evalid) return;
  float dh = 0.f;
  if (a.has_dg) {
    const int src = red_index(u, bl);
    dh = red[0][src] + red[1][src] + red[2][src] + red[3][src];
  }
  if (t < 0) {
    T* ds0 = static_cast<T*>(a.ds0);
#pragma unroll
    for (int k = 0; k < S; ++k) st_(ds0 + (size_t)k * BND + idx, ds[k] + (k == 0 ? dh : 0.f));
    return;
  }
  ds[0] = clamp_if(ds[0] + dh, a.g_clip);
  CM::bwd(cc, sp, sn, dso, ds, gr, gw, gb);
#pragma unroll
  for (int k = 0; k < S; ++k) a.dsr[(size_t)k * BND + idx] = ds[k];
  T* dg = static_cast<T*>(a.dg_out) + ((size_t)b * N + n) * GR * D + d;
#pragma unroll
  for (int g = 0; g < GR; ++g) st_(dg + (size_t)g * D, gr[g]);
  T* dWx = static_cast<T*>(a.dWx);
#pragma unroll
  for (int g = 0; g < GW; ++g) st_(dWx + (((size_t)b * Tn + t) * GW + g) * ND + (size_t)n * D + d, gw[g]);
  if (F == FRNN_GRU) st_(static_cast<T*>(a.dgx) + ((size_t)b * Tn + t) * ND + (size_t)n * D + d, gr[0]);
}

// partial bias sums: thread per bias element, rows split over blockIdx.y
struct AltBiasArgs {
  const void* src[4]; long ld[4];  // per bias gate: element (row r, n, d) at src + r*ld + n*D + d
  float* part;                     // [splits][G_t][N][D]
  int GT, N, D; long rows, rows_per_split;
};
// one thread sums 4 adjacent columns (one 8- or 16-byte load per row) over the rows of its split
template <typename T>
__global__ void __launch_bounds__(256) alt_bias_kernel(const AltBiasArgs a) {
  const size_t i4 = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t nb = (size_t)a.GT * a.N * a.D;
  if (i4 * 4 >= nb) return;
  const size_t i = i4 * 4;
  const int g = i / ((size_t)a.N * a.D);
  const size_t nd = i % ((size_t)a.N * a.D);
  const T* p = static_cast<const T*>(a.src[g]) + nd;
  const long r0 = (long)blockIdx.y * a.rows_per_split, r1 = min(a.rows, r0 + a.rows_per_split);
  float s[4] = {0.f, 0.f, 0.f, 0.f};
  for (long r = r0; r < r1; ++r) {
    float v[4];
    if constexpr (sizeof(T) == 2) {
      const uint2 w = *reinterpret_cast<const uint2*>(p + (size_t)r * a.ld[g]);
      Dw<2> d; d.v[0] = w.x; d.v[1] = w.y;
      unpack<4>(d, v, (T*)nullptr);
    } else {
      const float4 w = *reinterpret_cast<const float4*>(p + (size_t)r * a.ld[g]);
      v[0] = w.x; v[1] = w.y; v[2] = w.z; v[3] = w.w;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) s[e] += v[e];
  }
  *reinterpret_cast<float4*>(a.part + (size_t)blockIdx.y * nb + i) = make_float4(s[0], s[1], s[2], s[3]);
}

// ---------------------------------------------------------------------------------------------
// host drivers
// ---------------------------------------------------------------------------------------------
template <int F, typename T>
static int alt_forward_t(const AltProblem& p, const AltFwdBuffers& bf, hipStream_t st) {
  const dim3 grid(p.D / 16, p.N, (p.B + 15) / 16);
  for (int t = 0; t < p.T; ++t) {
    AltStepFwdArgs a{bf.Wx, bf.R, bf.b, bf.s0, bf.states, bf.cache, bf.sfp, p.B, p.T, p.N, p.D, t, p.training, p.h_clip,
                     (t > 0 || p.use_carry) ? 1 : 0};
    hipLaunchKernelGGL((alt_step_fwd_kernel<F, T>), grid, dim3(256), 0, st, a);
    const int e = (int)hipGetLastError();
    if (e) return e;
  }
  return 0;
}

template <int F, typename T>
static int alt_backward_t(const AltProblem& p, const AltBwdBuffers& bf, hipStream_t st) {
  constexpr int GR = Cell<F>::GR, S = Cell<F>::S;
  const size_t BND = (size_t)p.B * p.N * p.D;
  int e = launch_fill_zero(bf.dsr, (size_t)S * BND * sizeof(float), st);
  if (e) return e;
  const dim3 grid(p.D / 16, p.N, (p.B + 15) / 16);
  T* dg[2] = {static_cast<T*>(bf.dg), static_cast<T*>(bf.dg) + BND * GR};
  for (int t = p.T - 1; t >= -1; --t) {
    AltStepBwdArgs a{bf.Rt, bf.s0, bf.states, bf.cache, bf.dstates, bf.dWx, bf.dgx, bf.ds0,
                     dg[(t + 1) & 1], dg[t & 1], bf.dsr, p.B, p.T, p.N, p.D, t,
                     (t < p.T - 1 && !p.cut) ? 1 : 0, p.g_clip};
    hipLaunchKernelGGL((alt_step_bwd_kernel<F, T>), grid, dim3(256), 0, st, a);
    e = (int)hipGetLastError();
    if (e) return e;
  }
  return 0;
}

#define FRNN_ALT_DISPATCH(NAME, ...)                                                     \
  switch (p.function * 3 + p.dtype) {                                                    \
    case FRNN_LSTM * 3 + FRNN_BF16:  return NAME<FRNN_LSTM, bf16_t>(__VA_ARGS__);        \
    case FRNN_LSTM * 3 + FRNN_F32:   return NAME<FRNN_LSTM, float>(__VA_ARGS__);         \
    case FRNN_LSTM * 3 + FRNN_F16:   return NAME<FRNN_LSTM, half_t>(__VA_ARGS__);        \
    case FRNN_SLSTM * 3 + FRNN_BF16: return NAME<FRNN_SLSTM, bf16_t>(__VA_ARGS__);       \
    case FRNN_SLSTM * 3 + FRNN_F32:  return NAME<FRNN_SLSTM, float>(__VA_ARGS__);        \
    case FRNN_SLSTM * 3 + FRNN_F16:  return NAME<FRNN_SLSTM, half_t>(__VA_ARGS__);       \
    case FRNN_GRU * 3 + FRNN_BF16:   return NAME<FRNN_GRU, bf16_t>(__VA_ARGS__);         \
    case FRNN_GRU * 3 + FRNN_F32:    return NAME<FRNN_GRU, float>(__VA_ARGS__);          \
    case FRNN_GRU * 3 + FRNN_F16:    return NAME<FRNN_GRU, half_t>(__VA_ARGS__);         \
    case FRNN_ELMAN * 3 + FRNN_BF16: return NAME<FRNN_ELMAN, bf16_t>(__VA_ARGS__);       \
    case FRNN_ELMAN * 3 + FRNN_F32:  return NAME<FRNN_ELMAN, float>(__VA_ARGS__);        \
    case FRNN_ELMAN * 3 + FRNN_F16:  return NAME<FRNN_ELMAN, half_t>(__VA_ARGS__);       \
    case FRNN_ELMAN_CLIP * 3 + FRNN_BF16: return NAME<FRNN_ELMAN_CLIP, bf16_t>(__VA_ARGS__); \
    case FRNN_ELMAN_CLIP * 3 + FRNN_F32:  return NAME<FRNN_ELMAN_CLIP, float>(__VA_ARGS__);  \
    case FRNN_ELMAN_CLIP * 3 + FRNN_F16:  return NAME<FRNN_ELMAN_CLIP, half_t>(__VA_ARGS__); \
  }                                                                                      \
  return FRNN_E_ARG;

int alt_forward(const AltProblem& p, const AltFwdBuffers& bf, hipStream_t st) { FRNN_ALT_DISPATCH(alt_forward_t, p, bf, st) }
int alt_backward_scan(const AltProblem& p, const AltBwdBuffers& bf, hipStream_t st) { FRNN_ALT_DISPATCH(alt_backward_t, p, bf, st) }

int launch_bias_partial(int dtype, const void* const* src, const long* ld, int GT, int N, int D, long rows, int splits,
                        float* part, hipStream_t st) {
  AltBiasArgs a;
  for (int g = 0; g < 4; ++g) { a.src[g] = g < GT ? src[g] : nullptr; a.ld[g] = g < GT ? ld[g] : 0; }
  a.part = part; a.GT = GT; a.N = N; a.D = D; a.rows = rows; a.rows_per_split = (rows + splits - 1) / splits;
  const dim3 grid((unsigned)(((size_t)GT * N * D / 4 + 255) / 256), splits);  // D is a multiple of 16
  if (dtype == FRNN_BF16) hipLaunchKernelGGL(alt_bias_kernel<bf16_t>, grid, dim3(256), 0, st, a);
  else if (dtype == FRNN_F16) hipLaunchKernelGGL(alt_bias_kernel<half_t>, grid, dim3(256), 0, st, a);
  else hipLaunchKernelGGL(alt_bias_kernel<float>, grid, dim3(256), 0, st, a);
  return (int)hipGetLastError();
}

}  // namespace frnn
