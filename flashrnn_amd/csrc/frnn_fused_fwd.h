// Fused forward: one persistent kernel runs all T steps.
//
// Replaces FLASHRNNCellFusedForward, flashrnn/flashrnn/fused/flashrnn_fused_forward.cu:146-659.
//
// Work split.  A "unit tile" is 16 hidden units of one head with all their G_r gate rows.
// A wave owns UTW unit tiles and keeps their R rows (all K = D columns) in registers as MFMA
// A operands for the whole sequence.  A workgroup has WAVES waves; KW workgroups share one
// (head, 16-row batch tile) group: D = 16 * UTW * WAVES * KW.  Groups are independent.
//
// One step:  h_{t-1} (16 x D, storage type) sits in LDS in fragment order
//   -> per k-step one LDS read per lane, G_r*UTW MFMAs (A = R rows, B = h^T, fp32 acc)
//   -> lane (col b = lane%16, rows 4*(lane/16)..+3) holds every gate of 4 units of batch row b
//   -> gates, new states in fp32 registers; states / gate cache stored straight in the public
//      / private layouts; the new h goes to the other LDS buffer (KW == 1) or to the tagged
//      global exchange (KW > 1).
#pragma once
#include "frnn_exchange.h"
#include "frnn_pointwise.h"

namespace frnn {

struct FwdArgs {
  const void* Wx; const void* R; const void* b; const void* s0;
  void* states; void* cache;
  u64* ll; int* status;
  int B, T, N;
  int grp0, groups, groups_total;  // this launch handles groups [grp0, grp0 + groups)
  int training, spin_limit;
};

template <typename T> __device__ __forceinline__ typename ST<T>::Frag load_frag(const T* row, int ks, int kq);
template <> __device__ __forceinline__ bf16x8 load_frag<bf16_t>(const bf16_t* row, int ks, int kq) {
  return *reinterpret_cast<const bf16x8*>(row + ks * 32 + kq * 8);
}
template <> __device__ __forceinline__ float load_frag<float>(const float* row, int ks, int kq) {
  return row[ks * 4 + kq];
}

template <int F, typename T, int D, int WAVES, int UTW, int KW>
__global__ void __launch_bounds__(WAVES * 64) fused_fwd_kernel(const FwdArgs a) {
  typedef Cell<F> C;
  typedef ST<T> X;
  typedef CellMath<F, X::FAST> CM;
  typedef typename X::Vec4 Vec4;
  typedef typename X::Frag Frag;
  constexpr int GR = C::GR, GW = C::GW, GT = C::GT, S = C::S, NC = C::NC;
  constexpr int KS = D / X::KM, NT = WAVES * 64, UT_WG = WAVES * UTW;
  static_assert(UT_WG * KW * 16 == D, "tiling must cover the head");
  constexpr int LLW = 16 * D / X::EPW;  // 64-bit words per exchange slot
  constexpr int NP = (LLW + NT - 1) / NT;
  constexpr int NCA = NC > 0 ? NC : 1;

  __shared__ __attribute__((aligned(16))) T hbuf[2][16 * D];

  int grp_l, slice;
  if (!decode_block(a.groups, KW, grp_l, slice)) return;
  const int grp = a.grp0 + grp_l;
  const int N = a.N, Tn = a.T, B = a.B;
  const int n = grp % N, bt = grp / N;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int r16 = lane & 15, q4 = lane >> 4;
  const int bg = bt * 16 + r16;  // batch row of this lane's output column
  const bool bvalid = bg < B;
  const int rows_valid = min(16, B - bt * 16);
  const T* __restrict__ Wx = static_cast<const T*>(a.Wx);
  const T* __restrict__ R = static_cast<const T*>(a.R);
  const T* __restrict__ bias_g = static_cast<const T*>(a.b);
  const T* __restrict__ s0 = static_cast<const T*>(a.s0);
  T* __restrict__ states = static_cast<T*>(a.states);
  T* __restrict__ cache = static_cast<T*>(a.cache);
  const size_t ND = (size_t)N * D;

  int ub[UTW];
#pragma unroll
  for (int u = 0; u < UTW; ++u) ub[u] = (slice * UT_WG + w * UTW + u) * 16;

  // ---- resident operands ----------------------------------------------------------------
  Frag rf[UTW][GR][KS];
#pragma unroll
  for (int u = 0; u < UTW; ++u)
#pragma unroll
    for (int g = 0; g < GR; ++g) {
      const T* row = R + ((size_t)(g * N + n) * D + ub[u] + r16) * D;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) rf[u][g][ks] = load_frag<T>(row, ks, q4);
    }
  float bias[UTW][4][GT];
  float s[UTW][4][S];
#pragma unroll
  for (int u = 0; u < UTW; ++u) {
    const int d0 = ub[u] + q4 * 4;
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      float v[4];
      unpack4(*reinterpret_cast<const Vec4*>(bias_g + (size_t)(g * N + n) * D + d0), v);
#pragma unroll
      for (int i = 0; i < 4; ++i) bias[u][i][g] = v[i];
    }
#pragma unroll
    for (int k = 0; k < S; ++k) {
      float v[4] = {0.f, 0.f, 0.f, 0.f};
      if (bvalid) unpack4(*reinterpret_cast<const Vec4*>(s0 + ((size_t)k * B + bg) * ND + (size_t)n * D + d0), v);
#pragma unroll
      for (int i = 0; i < 4; ++i) s[u][i][k] = v[i];
    }
  }

  // ---- h_0 of the whole head -> LDS buffer 0 (rows beyond B: zeros, and they stay zero or
  //      private to their own MFMA column, so they never reach a valid row) ----------------
  for (int idx = tid; idx < 16 * D / 4; idx += NT) {
    const int row = idx / (D / 4), k0 = (idx % (D / 4)) * 4;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (bt * 16 + row < B) unpack4(*reinterpret_cast<const Vec4*>(s0 + (size_t)(bt * 16 + row) * ND + (size_t)n * D + k0), v);
    lds_write4(hbuf[0], row, k0, v);
    if (KW > 1) lds_write4(hbuf[1], row, k0, v);  // padded rows of buffer 1 must be finite too
  }

  int qpoll[NP];
  if (KW > 1) ll_plan<T, NP, NT>(tid, rows_valid, D, qpoll);
  u64* const llbase = a.ll + (size_t)grp * 2 * LLW;

  Vec4 wxA[UTW][GW], wxB[UTW][GW];
  auto load_wx = [&](Vec4 (&dst)[UTW][GW], int t) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < UTW; ++u)
#pragma unroll
      for (int g = 0; g < GW; ++g) {
        if (bvalid)
          dst[u][g] = *reinterpret_cast<const Vec4*>(Wx + (((size_t)bg * Tn + t) * GW + g) * ND + (size_t)n * D + ub[u] + q4 * 4);
        else
          dst[u][g] = Vec4{};
      }
  };
  load_wx(wxA, 0);
  __syncthreads();

  bool dead = false;
  // one time step: consumes `wc` (Wx of step t), prefetches Wx of step t+1 into `wn`
  auto step = [&](const int t, Vec4 (&wc)[UTW][GW], Vec4 (&wn)[UTW][GW]) __attribute__((always_inline)) {
    const int cur = t & 1;
    if (t > 0) {
      if (KW > 1) {
        const bool fail = ll_gather<T, NP>(llbase + (size_t)((t - 1) & 1) * LLW, qpoll, t - 1, hbuf[cur], a.status, a.spin_limit);
        if (__syncthreads_or(fail)) { dead = true; return; }
      } else {
        __syncthreads();
      }
    }
    if (t + 1 < Tn) load_wx(wn, t + 1);

    f32x4 acc[UTW][GR];
#pragma unroll
    for (int u = 0; u < UTW; ++u)
#pragma unroll
      for (int g = 0; g < GR; ++g) acc[u][g] = f32x4{0.f, 0.f, 0.f, 0.f};
    const Frag* hf = reinterpret_cast<const Frag*>(hbuf[cur]) + lane;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const Frag h = hf[ks * 64];
#pragma unroll
      for (int u = 0; u < UTW; ++u)
#pragma unroll
        for (int g = 0; g < GR; ++g) acc[u][g] = X::mfma(rf[u][g][ks], h, acc[u][g]);
    }

#pragma unroll
    for (int u = 0; u < UTW; ++u) {
      const int d0 = ub[u] + q4 * 4;
      float wxv[GW][4];
#pragma unroll
      for (int g = 0; g < GW; ++g) unpack4(wc[u][g], wxv[g]);
      float cv[NCA][4];
      float so[S][4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float ry[GR], wx[GW], cc[NCA];
#pragma unroll
        for (int g = 0; g < GR; ++g) ry[g] = acc[u][g][i];
#pragma unroll
        for (int g = 0; g < GW; ++g) wx[g] = wxv[g][i];
        CM::fwd(ry, wx, bias[u][i], s[u][i], cc);
#pragma unroll
        for (int c = 0; c < NC; ++c) cv[c][i] = cc[c];
#pragma unroll
        for (int k = 0; k < S; ++k) so[k][i] = s[u][i][k];
      }
      if (bvalid) {
#pragma unroll
        for (int k = 0; k < S; ++k) {
          Vec4 p; pack4(so[k], p);
          *reinterpret_cast<Vec4*>(states + (((size_t)k * B + bg) * Tn + t) * ND + (size_t)n * D + d0) = p;
        }
      }
      if (a.training && NC > 0) {
        // private layout [t][group][unit tile][value][16 rows][16 units]: 512 B runs per wave
        const size_t cb = ((((size_t)t * a.groups_total + grp) * (D / 16) + (ub[u] >> 4)) * NC) * 256 + r16 * 16 + q4 * 4;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          Vec4 p; pack4(cv[c], p);
          *reinterpret_cast<Vec4*>(cache + cb + (size_t)c * 256) = p;
        }
      }
      if (t + 1 < Tn) {
        if (KW == 1) lds_write4(hbuf[cur ^ 1], r16, d0, so[0]);
        else if (bvalid) ll_write4((T*)0, llbase + (size_t)(t & 1) * LLW, r16, d0, so[0], t);
      }
    }
  };

  int t = 0;
  for (; t + 1 < Tn && !dead; t += 2) {
    step(t, wxA, wxB);
    if (dead) break;
    step(t + 1, wxB, wxA);
  }
  if (!dead && t < Tn) step(t, wxA, wxB);

  if (dead) {
    // bounded wait ran out: report, and make the damage visible (NaN in every h of this
    // workgroup's units; the step that failed is not known exactly, so all steps are marked)
    if (tid == 0) __hip_atomic_store(a.status, (int)STATUS_WAIT_EXPIRED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (bvalid) {
      float nanv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) nanv[i] = __uint_as_float(0x7fc00000u);
      Vec4 p; pack4(nanv, p);
      for (int tt = 0; tt < Tn; ++tt)
#pragma unroll
        for (int u = 0; u < UTW; ++u)
          *reinterpret_cast<Vec4*>(states + ((size_t)bg * Tn + tt) * ND + (size_t)n * D + ub[u] + q4 * 4) = p;
    }
  }
}

}  // namespace frnn
