// Alternating backend ("hip"): per time step one MFMA GEMM kernel over all heads, then one
// pointwise kernel; the recurrent matrix is re-read from L2/HBM every step, so any head
// dimension works.  Replaces flashrnn/flashrnn/alternating/flashrnn_forward.cu:150-267,
// flashrnn_backward.cu:267-431 and the four *_pointwise.cu files.
//
// Differences from the reference: the recurrent pre-activations stay fp32 between the two
// kernels (the reference rounds them to the storage type, flashrnn_forward.cu:176-181); tensors
// are read and written in the public layouts; everything runs on the caller's stream.
#include "frnn_alt.h"
#include "frnn_pointwise.h"

namespace frnn {

// ---------------------------------------------------------------------------------------------
// out[b][n][m] = sum_k A(n, m)[k] * V[b][n][k]      (M rows per head, K contraction, 16-row
// batch tiles).  One workgroup = one 16-row M tile x one batch tile; its 4 waves split K and
// reduce through LDS.  Operands go from global memory straight into MFMA fragments: both are
// contiguous in k.
//   row m of head n:  A + (m / D) * a_gstride + n * a_hstride + (m % D) * K
//   V element:        V + b * v_bstride + n * K + k
// ---------------------------------------------------------------------------------------------
struct AltGemmArgs {
  const void* A; size_t a_gstride, a_hstride;
  const void* V; size_t v_bstride;
  float* out;
  int B, N, D, M, K;
};

template <typename T>
__global__ void __launch_bounds__(256) alt_gemm_kernel(const AltGemmArgs a) {
  typedef ST<T> X;
  typedef typename X::Frag Frag;
  __shared__ f32x4 red[3][64];
  const int m0 = blockIdx.x * 16, n = blockIdx.y, bt = blockIdx.z;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int r16 = lane & 15, q4 = lane >> 4;
  const int m = m0 + r16;
  const T* arow = static_cast<const T*>(a.A) + (size_t)(m / a.D) * a.a_gstride + (size_t)n * a.a_hstride + (size_t)(m % a.D) * a.K;
  const int b = bt * 16 + r16;
  const bool bvalid = b < a.B;
  const T* vrow = static_cast<const T*>(a.V) + (size_t)(bvalid ? b : 0) * a.v_bstride + (size_t)n * a.K;
  const int KS = a.K / X::KM;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int ks = w; ks < KS; ks += 4) {
    const Frag af = load_frag<T>(arow, ks, q4);
    Frag vf = load_frag<T>(vrow, ks, q4);
    if (!bvalid) vf = Frag{};
    acc = X::mfma(af, vf, acc);
  }
  if (w > 0) red[w - 1][lane] = acc;
  __syncthreads();
  if (w == 0) {
    acc += red[0][lane]; acc += red[1][lane]; acc += red[2][lane];
    if (bvalid) *reinterpret_cast<f32x4*>(a.out + ((size_t)b * a.N + n) * a.M + m0 + q4 * 4) = acc;
  }
}

static int launch_alt_gemm(int dtype, const AltGemmArgs& a, hipStream_t st) {
  const dim3 grid(a.M / 16, a.N, (a.B + 15) / 16);
  if (dtype == FRNN_BF16) hipLaunchKernelGGL(alt_gemm_kernel<bf16_t>, grid, dim3(256), 0, st, a);
  else hipLaunchKernelGGL(alt_gemm_kernel<float>, grid, dim3(256), 0, st, a);
  return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------------------------
// pointwise kernels: one thread per (b, n, d)
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float ld(const bf16_t* p) { return (float)*p; }
__device__ __forceinline__ float ld(const float* p) { return *p; }
__device__ __forceinline__ void st_(bf16_t* p, float v) { *reinterpret_cast<unsigned short*>(p) = f2bf(v); }
__device__ __forceinline__ void st_(float* p, float v) { *p = v; }

struct AltPwArgs {
  const void* Wx; const void* b; const void* s0; void* states; void* cache;
  const float* ry;  // [B][N][G_r*D]
  float* sfp;       // [S][B][N][D] fp32 copy of the running state: the states tensor is the
                    // storage-type output, the recurrence itself is carried unrounded (only the h
                    // that feeds the GEMM is read back in the storage type), as in the fused path
  int B, T, N, D, t, training;
  float h_clip;     // > 0: new h clamped to [-h_clip, h_clip]
};

template <int F, typename T>
__global__ void __launch_bounds__(256) alt_pw_fwd_kernel(const AltPwArgs a) {
  typedef Cell<F> C;
  typedef CellMath<F, ST<T>::FAST> CM;
  constexpr int GR = C::GR, GW = C::GW, GT = C::GT, S = C::S, NC = C::NC;
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  const int D = a.D, N = a.N, B = a.B, Tn = a.T, t = a.t;
  if (idx >= (size_t)B * N * D) return;
  const int d = idx % D, n = (idx / D) % N, b = idx / ((size_t)D * N);
  const size_t ND = (size_t)N * D;
  const T* Wx = static_cast<const T*>(a.Wx);
  const T* bias = static_cast<const T*>(a.b);
  const T* s0 = static_cast<const T*>(a.s0);
  T* states = static_cast<T*>(a.states);
  float ry[GR], wx[GW], bb[GT - GR + 1], s[S], cc[NC > 0 ? NC : 1];
#pragma unroll
  for (int g = 0; g < GR; ++g) ry[g] = a.ry[((size_t)b * N + n) * GR * D + (size_t)g * D + d];
#pragma unroll
  for (int g = 0; g < GW; ++g) wx[g] = ld(Wx + (((size_t)b * Tn + t) * GW + g) * ND + (size_t)n * D + d);
#pragma unroll
  for (int g = 0; g < GR; ++g) ry[g] += ld(bias + (size_t)(g * N + n) * D + d);
#pragma unroll
  for (int g = GR; g < GT; ++g) bb[g - GR] = ld(bias + (size_t)(g * N + n) * D + d);
  const size_t BND = (size_t)B * ND;
#pragma unroll
  for (int k = 0; k < S; ++k)
    s[k] = t > 0 ? a.sfp[(size_t)k * BND + idx] : ld(s0 + ((size_t)k * B + b) * ND + (size_t)n * D + d);
  CM::fwd(ry, wx, bb, s, cc);
  s[0] = clamp_if(s[0], a.h_clip);
#pragma unroll
  for (int k = 0; k < S; ++k) {
    st_(states + (((size_t)k * B + b) * Tn + t) * ND + (size_t)n * D + d, s[k]);
    a.sfp[(size_t)k * BND + idx] = s[k];
  }
  if (a.training && NC > 0) {
    T* cache = static_cast<T*>(a.cache) + (((size_t)t * B + b) * N + n) * NC * D + d;
#pragma unroll
    for (int c = 0; c < NC; ++c) st_(cache + (size_t)c * D, cc[c]);
  }
}

struct AltPwBwdArgs {
  const void* s0; const void* states; const void* cache; const void* dstates;
  void* dWx; void* dgx;
  void* dg;        // [B][N][G_r*D] storage type: operand of the next GEMM
  float* dsr;      // [S][B][N][D] running cotangent without the recurrent term
  const float* dh; // [B][N][D] recurrent term R^T dg of the step above
  int B, T, N, D, t;
  float g_clip;    // > 0: cotangent carried into h_t clamped to [-g_clip, g_clip]
};

template <int F, typename T>
__global__ void __launch_bounds__(256) alt_pw_bwd_kernel(const AltPwBwdArgs a) {
  typedef Cell<F> C;
  typedef CellMath<F, ST<T>::FAST> CM;
  constexpr int GR = C::GR, GW = C::GW, GT = C::GT, S = C::S, NC = C::NC;
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  const int D = a.D, N = a.N, B = a.B, Tn = a.T, t = a.t;
  if (idx >= (size_t)B * N * D) return;
  const int d = idx % D, n = (idx / D) % N, b = idx / ((size_t)D * N);
  const size_t ND = (size_t)N * D, BND = (size_t)B * ND;
  const T* s0 = static_cast<const T*>(a.s0);
  const T* states = static_cast<const T*>(a.states);
  const T* dstates = static_cast<const T*>(a.dstates);
  float cc[NC > 0 ? NC : 1], sp[S], sn[S], dso[S], ds[S], gr[GR], gw[GW], gb[GT];
  const T* cache = static_cast<const T*>(a.cache) + (((size_t)t * B + b) * N + n) * NC * D + d;
#pragma unroll
  for (int c = 0; c < NC; ++c) cc[c] = ld(cache + (size_t)c * D);
#pragma unroll
  for (int k = 0; k < S; ++k) {
    const size_t so = (((size_t)k * B + b) * Tn + t) * ND + (size_t)n * D + d;
    sn[k] = ld(states + so);
    dso[k] = ld(dstates + so);
    sp[k] = t > 0 ? ld(states + so - ND) : ld(s0 + ((size_t)k * B + b) * ND + (size_t)n * D + d);
    ds[k] = a.dsr[(size_t)k * BND + idx];
  }
  ds[0] = clamp_if(ds[0] + a.dh[idx], a.g_clip);
  CM::bwd(cc, sp, sn, dso, ds, gr, gw, gb);
#pragma unroll
  for (int k = 0; k < S; ++k) a.dsr[(size_t)k * BND + idx] = ds[k];
  T* dg = static_cast<T*>(a.dg) + ((size_t)b * N + n) * GR * D + d;
#pragma unroll
  for (int g = 0; g < GR; ++g) st_(dg + (size_t)g * D, gr[g]);
  T* dWx = static_cast<T*>(a.dWx);
#pragma unroll
  for (int g = 0; g < GW; ++g) st_(dWx + (((size_t)b * Tn + t) * GW + g) * ND + (size_t)n * D + d, gw[g]);
  if (F == FRNN_GRU) st_(static_cast<T*>(a.dgx) + ((size_t)b * Tn + t) * ND + (size_t)n * D + d, gr[0]);
}

template <typename T>
__global__ void __launch_bounds__(256) alt_finish_kernel(const float* dsr, const float* dh, T* ds0, int S, size_t BND) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)S * BND) return;
  float v = dsr[i];
  if (i < BND) v += dh[i];
  st_(ds0 + i, v);
}

// partial bias sums: thread per bias element, rows split over blockIdx.y
struct AltBiasArgs {
  const void* src[4]; long ld[4];  // per bias gate: element (row r, n, d) at src + r*ld + n*D + d
  float* part;                     // [splits][G_t][N][D]
  int GT, N, D; long rows, rows_per_split;
};
template <typename T>
__global__ void __launch_bounds__(256) alt_bias_kernel(const AltBiasArgs a) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t nb = (size_t)a.GT * a.N * a.D;
  if (i >= nb) return;
  const int g = i / ((size_t)a.N * a.D);
  const size_t nd = i % ((size_t)a.N * a.D);
  const T* p = static_cast<const T*>(a.src[g]) + nd;
  const long r0 = (long)blockIdx.y * a.rows_per_split, r1 = min(a.rows, r0 + a.rows_per_split);
  float s = 0.f;
  for (long r = r0; r < r1; ++r) s += ld(p + (size_t)r * a.ld[g]);
  a.part[(size_t)blockIdx.y * nb + i] = s;
}

// ---------------------------------------------------------------------------------------------
// host drivers
// ---------------------------------------------------------------------------------------------
template <int F, typename T>
static int alt_forward_t(const AltProblem& p, const AltFwdBuffers& bf, hipStream_t st) {
  constexpr int GR = Cell<F>::GR;
  const size_t ND = (size_t)p.N * p.D;
  const unsigned pw_blocks = (unsigned)(((size_t)p.B * ND + 255) / 256);
  for (int t = 0; t < p.T; ++t) {
    AltGemmArgs g;
    g.A = bf.R; g.a_gstride = (size_t)p.N * p.D * p.D; g.a_hstride = (size_t)p.D * p.D;
    if (t == 0) { g.V = bf.s0; g.v_bstride = ND; }
    else { g.V = static_cast<const T*>(bf.states) + (size_t)(t - 1) * ND; g.v_bstride = (size_t)p.T * ND; }
    g.out = bf.ry; g.B = p.B; g.N = p.N; g.D = p.D; g.M = GR * p.D; g.K = p.D;
    int e = launch_alt_gemm(ST<T>::ID, g, st);
    if (e) return e;
    AltPwArgs a{bf.Wx, bf.b, bf.s0, bf.states, bf.cache, bf.ry, bf.sfp, p.B, p.T, p.N, p.D, t, p.training, p.h_clip};
    hipLaunchKernelGGL((alt_pw_fwd_kernel<F, T>), dim3(pw_blocks), dim3(256), 0, st, a);
    e = (int)hipGetLastError();
    if (e) return e;
  }
  return 0;
}

template <int F, typename T>
static int alt_backward_t(const AltProblem& p, const AltBwdBuffers& bf, hipStream_t st) {
  constexpr int GR = Cell<F>::GR, S = Cell<F>::S;
  const size_t ND = (size_t)p.N * p.D, BND = (size_t)p.B * ND;
  const unsigned pw_blocks = (unsigned)((BND + 255) / 256);
  int e = launch_fill_zero(bf.dsr, ((size_t)S * BND + BND) * sizeof(float), st);  // dsr and dh are adjacent
  if (e) return e;
  for (int t = p.T - 1; t >= 0; --t) {
    AltPwBwdArgs a{bf.s0, bf.states, bf.cache, bf.dstates, bf.dWx, bf.dgx, bf.dg, bf.dsr, bf.dh, p.B, p.T, p.N, p.D, t, p.g_clip};
    hipLaunchKernelGGL((alt_pw_bwd_kernel<F, T>), dim3(pw_blocks), dim3(256), 0, st, a);
    e = (int)hipGetLastError();
    if (e) return e;
    if (p.cut) continue;  // truncated backpropagation: dh stays zero
    AltGemmArgs g;
    g.A = bf.Rt; g.a_gstride = 0; g.a_hstride = (size_t)p.D * GR * p.D;
    g.V = bf.dg; g.v_bstride = (size_t)p.N * GR * p.D;
    g.out = bf.dh; g.B = p.B; g.N = p.N; g.D = p.D; g.M = p.D; g.K = GR * p.D;
    e = launch_alt_gemm(ST<T>::ID, g, st);
    if (e) return e;
  }
  hipLaunchKernelGGL(alt_finish_kernel<T>, dim3((unsigned)(((size_t)S * BND + 255) / 256)), dim3(256), 0, st,
                     (const float*)bf.dsr, (const float*)bf.dh, static_cast<T*>(bf.ds0), S, BND);
  return (int)hipGetLastError();
}

#define FRNN_ALT_DISPATCH(NAME, ...)                                                     \
  switch (p.function * 2 + p.dtype) {                                                    \
    case FRNN_LSTM * 2 + FRNN_BF16:  return NAME<FRNN_LSTM, bf16_t>(__VA_ARGS__);        \
    case FRNN_LSTM * 2 + FRNN_F32:   return NAME<FRNN_LSTM, float>(__VA_ARGS__);         \
    case FRNN_SLSTM * 2 + FRNN_BF16: return NAME<FRNN_SLSTM, bf16_t>(__VA_ARGS__);       \
    case FRNN_SLSTM * 2 + FRNN_F32:  return NAME<FRNN_SLSTM, float>(__VA_ARGS__);        \
    case FRNN_GRU * 2 + FRNN_BF16:   return NAME<FRNN_GRU, bf16_t>(__VA_ARGS__);         \
    case FRNN_GRU * 2 + FRNN_F32:    return NAME<FRNN_GRU, float>(__VA_ARGS__);          \
    case FRNN_ELMAN * 2 + FRNN_BF16: return NAME<FRNN_ELMAN, bf16_t>(__VA_ARGS__);       \
    case FRNN_ELMAN * 2 + FRNN_F32:  return NAME<FRNN_ELMAN, float>(__VA_ARGS__);        \
  }                                                                                      \
  return FRNN_E_ARG;

int alt_forward(const AltProblem& p, const AltFwdBuffers& bf, hipStream_t st) { FRNN_ALT_DISPATCH(alt_forward_t, p, bf, st) }
int alt_backward_scan(const AltProblem& p, const AltBwdBuffers& bf, hipStream_t st) { FRNN_ALT_DISPATCH(alt_backward_t, p, bf, st) }

int launch_bias_partial(int dtype, const void* const* src, const long* ld, int GT, int N, int D, long rows, int splits,
                        float* part, hipStream_t st) {
  AltBiasArgs a;
  for (int g = 0; g < 4; ++g) { a.src[g] = g < GT ? src[g] : nullptr; a.ld[g] = g < GT ? ld[g] : 0; }
  a.part = part; a.GT = GT; a.N = N; a.D = D; a.rows = rows; a.rows_per_split = (rows + splits - 1) / splits;
  const dim3 grid((unsigned)(((size_t)GT * N * D + 255) / 256), splits);
  if (dtype == FRNN_BF16) hipLaunchKernelGGL(alt_bias_kernel<bf16_t>, grid, dim3(256), 0, st, a);
  else hipLaunchKernelGGL(alt_bias_kernel<float>, grid, dim3(256), 0, st, a);
  return (int)hipGetLastError();
}

}  // namespace frnn
