// Fused backward: one persistent kernel runs the reverse scan over all T steps.
//
// Replaces FLASHRNNCellFusedBackward, flashrnn/flashrnn/fused/flashrnn_fused_backward.cu:129-624
// and gradientBiasAggregationKernel (:626-665; the bias sums are kept in registers across T here).
//
// Same ownership as the forward kernel: a lane owns 4 units x 1 batch row of UTW unit tiles, and
// the KW workgroups of a (head, batch tile) group own D/KW units each.
// One reverse step t:
//   gate cache, s_{t-1}, s_t and the upstream cotangent of s_t (prefetched one step ahead)
//   -> per-element adjoint -> dg_t of the OWN units; dWx_t stored in the public layout; db summed
//      in registers
//   -> own dg_t (16 x G_r*D/KW, storage type) to LDS in fragment order, one workgroup barrier
//   -> MFMA over the own gate rows only (the contraction is split between the workgroups, the
//      reference's optional d_state_buffer scheme, flashrnn_fused_backward.cu:510-553):
//        part[p] = sum_{k own} Rt[p][k] dg_t[k]   for ALL previous units p of the head,
//      A = rows p of the transposed R, resident in registers
//   -> wave w keeps the partial sums of the tiles it owns itself and sends the others, as tagged
//      fp32 words, to wave w of the owning workgroup; it then polls its own inbox for the KW-1
//      partial sums of its tiles and adds everything to the running cotangent dh_{t-1}.
// Exchanging partial dh (D values per row) instead of dg (G_r*D values per row) moves 2-4x
// fewer bytes through L2 per step.
#pragma once
#include "frnn_exchange.h"
#include "frnn_fused_fwd.h"
#include "frnn_pointwise.h"

namespace frnn {

struct BwdArgs {
  const void* Rt;  // [N][D (previous unit p)][G_r*D (k = g*D + d)]
  const void* s0; const void* states; const void* cache; const void* dstates;
  void* dWx;       // [B,T,G_w,N,D]
  void* dgx;       // [B,T,N,D]: cotangent of R-side gates that have no Wx slot (gru: g); else null
  void* ds0;       // [S,B,N,D]
  float* dbp;      // [batch tiles][G_t][N][D] partial bias sums
  u64* ll; int* status;
  int B, T, N;
  int grp0, groups, groups_total;
  int spin_limit;
};

// 64-bit words of one inbox slot of one group: [dst wg][wave][tile][src wg][lane][4]
constexpr size_t bwd_inbox_words(int D, int KW) { return (size_t)KW * (D / 16) * 256; }

template <typename T> __device__ __forceinline__ typename ST<T>::Frag load_frag_at(const T* p);
template <> __device__ __forceinline__ bf16x8 load_frag_at<bf16_t>(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }
template <> __device__ __forceinline__ float load_frag_at<float>(const float* p) { return *p; }

template <int F, typename T, int D, int WAVES, int UTW, int KW>
__global__ void __launch_bounds__(WAVES * 64) fused_bwd_kernel(const BwdArgs a) {
  typedef Cell<F> C;
  typedef ST<T> X;
  typedef CellMath<F, X::FAST> CM;
  typedef typename X::Vec4 Vec4;
  typedef typename X::Frag Frag;
  constexpr int GR = C::GR, GW = C::GW, GT = C::GT, S = C::S, NC = C::NC;
  constexpr int NT = WAVES * 64, UT_WG = WAVES * UTW;
  static_assert(UT_WG * KW * 16 == D, "tiling must cover the head");
  constexpr int DL = D / KW;            // units owned by this workgroup
  constexpr int KDL = GR * DL;          // contraction length handled by this workgroup
  constexpr int KS = KDL / X::KM;
  static_assert(KDL % X::KM == 0 && DL % 8 == 0, "own gate rows must fill whole k-steps");
  constexpr int KE = X::KM / 4;         // consecutive k held by one lane of a fragment
  constexpr int NCA = NC > 0 ? NC : 1;
  constexpr int RC = KW == 1 ? 1 : ((KW - 1) < 3 ? (KW - 1) : 3);  // remote sources polled together
  constexpr size_t INW = bwd_inbox_words(D, KW);

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  T* const gbuf0 = reinterpret_cast<T*>(smem_raw);
  T* const gbuf1 = gbuf0 + 16 * KDL;

  int grp_l, slice;
  if (!decode_block(a.groups, KW, grp_l, slice)) return;
  const int grp = a.grp0 + grp_l;
  const int N = a.N, Tn = a.T, B = a.B;
  const int n = grp % N, bt = grp / N;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int r16 = lane & 15, q4 = lane >> 4;
  const int bg = bt * 16 + r16;
  const bool bvalid = bg < B;
  const T* __restrict__ Rt = static_cast<const T*>(a.Rt);
  const T* __restrict__ s0 = static_cast<const T*>(a.s0);
  const T* __restrict__ states = static_cast<const T*>(a.states);
  const T* __restrict__ cache = static_cast<const T*>(a.cache);
  const T* __restrict__ dstates = static_cast<const T*>(a.dstates);
  T* __restrict__ dWx = static_cast<T*>(a.dWx);
  T* __restrict__ dgx = static_cast<T*>(a.dgx);
  const size_t ND = (size_t)N * D;

  int ub[UTW];
#pragma unroll
  for (int u = 0; u < UTW; ++u) ub[u] = (slice * UT_WG + w * UTW + u) * 16;

  // rtf[r][u][ks]: rows p of the tiles at this wave's position in workgroup (slice + r) % KW,
  // columns = the own gate rows, local index kk = g*DL + (d - slice*DL)
  Frag rtf[KW][UTW][KS];
#pragma unroll
  for (int r = 0; r < KW; ++r) {
    const int x = (slice + r) % KW;
#pragma unroll
    for (int u = 0; u < UTW; ++u) {
      const T* row = Rt + ((size_t)n * D + (x * UT_WG + w * UTW + u) * 16 + r16) * (GR * D) + slice * DL;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int kk0 = ks * X::KM + q4 * KE;
        rtf[r][u][ks] = load_frag_at<T>(row + (kk0 / DL) * D + (kk0 % DL));
      }
    }
  }

  float ds[UTW][4][S];
  float dbacc[UTW][4][GT];
#pragma unroll
  for (int u = 0; u < UTW; ++u)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int k = 0; k < S; ++k) ds[u][i][k] = 0.f;
#pragma unroll
      for (int g = 0; g < GT; ++g) dbacc[u][i][g] = 0.f;
    }

  u64* const inbox = a.ll + (size_t)grp * 2 * INW;

  struct Pre { Vec4 cache[UTW][NCA], sp[UTW][S], sn[UTW][S], dso[UTW][S]; };
  Pre pa, pb;
  auto load_pre = [&](Pre& p, int t) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < UTW; ++u) {
      const int d0 = ub[u] + q4 * 4;
      const size_t cb = ((((size_t)t * a.groups_total + grp) * (D / 16) + (ub[u] >> 4)) * NC) * 256 + r16 * 16 + q4 * 4;
#pragma unroll
      for (int c = 0; c < NC; ++c) p.cache[u][c] = *reinterpret_cast<const Vec4*>(cache + cb + (size_t)c * 256);
#pragma unroll
      for (int k = 0; k < S; ++k) {
        if (bvalid) {
          const size_t so = (((size_t)k * B + bg) * Tn + t) * ND + (size_t)n * D + d0;
          p.sn[u][k] = *reinterpret_cast<const Vec4*>(states + so);
          p.dso[u][k] = *reinterpret_cast<const Vec4*>(dstates + so);
          p.sp[u][k] = t > 0 ? *reinterpret_cast<const Vec4*>(states + so - ND)
                             : *reinterpret_cast<const Vec4*>(s0 + ((size_t)k * B + bg) * ND + (size_t)n * D + d0);
        } else {
          p.sn[u][k] = Vec4{}; p.dso[u][k] = Vec4{}; p.sp[u][k] = Vec4{};
        }
      }
    }
  };
  load_pre(pa, Tn - 1);

  bool dead = false, fail = false;
  // one reverse step: consumes `pc` (operands of step t), prefetches those of step t-1 into `pn`
  auto step = [&](const int t, Pre& pc, Pre& pn) __attribute__((always_inline)) {
    T* const gb = (t & 1) ? gbuf1 : gbuf0;
#pragma unroll
    for (int u = 0; u < UTW; ++u) {
      const int d0 = ub[u] + q4 * 4;
      float cv[NCA][4], spv[S][4], snv[S][4], dsov[S][4];
#pragma unroll
      for (int c = 0; c < NC; ++c) unpack4(pc.cache[u][c], cv[c]);
#pragma unroll
      for (int k = 0; k < S; ++k) { unpack4(pc.sp[u][k], spv[k]); unpack4(pc.sn[u][k], snv[k]); unpack4(pc.dso[u][k], dsov[k]); }
      float dgr[GR][4], dgw[GW][4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float cc[NCA], sp[S], sn[S], dso[S], gr[GR], gw[GW], gb_[GT];
#pragma unroll
        for (int c = 0; c < NC; ++c) cc[c] = cv[c][i];
#pragma unroll
        for (int k = 0; k < S; ++k) { sp[k] = spv[k][i]; sn[k] = snv[k][i]; dso[k] = dsov[k][i]; }
        CM::bwd(cc, sp, sn, dso, ds[u][i], gr, gw, gb_);
        if (!bvalid) {  // padded batch rows contribute nothing
#pragma unroll
          for (int g = 0; g < GR; ++g) gr[g] = 0.f;
#pragma unroll
          for (int g = 0; g < GW; ++g) gw[g] = 0.f;
#pragma unroll
          for (int g = 0; g < GT; ++g) gb_[g] = 0.f;
#pragma unroll
          for (int k = 0; k < S; ++k) ds[u][i][k] = 0.f;
        }
#pragma unroll
        for (int g = 0; g < GR; ++g) dgr[g][i] = gr[g];
#pragma unroll
        for (int g = 0; g < GW; ++g) dgw[g][i] = gw[g];
#pragma unroll
        for (int g = 0; g < GT; ++g) dbacc[u][i][g] += gb_[g];
      }
      if (bvalid) {
#pragma unroll
        for (int g = 0; g < GW; ++g) {
          Vec4 p; pack4(dgw[g], p);
          *reinterpret_cast<Vec4*>(dWx + (((size_t)bg * Tn + t) * GW + g) * ND + (size_t)n * D + d0) = p;
        }
        if (F == FRNN_GRU) {
          Vec4 p; pack4(dgr[0], p);
          *reinterpret_cast<Vec4*>(dgx + ((size_t)bg * Tn + t) * ND + (size_t)n * D + d0) = p;
        }
      }
#pragma unroll
      for (int g = 0; g < GR; ++g) lds_write4(gb, r16, g * DL + (d0 - slice * DL), dgr[g]);
    }
    // the barrier also spreads a failed wait of the previous step to the whole workgroup
    if (__syncthreads_or(fail)) { dead = true; return; }
    if (t > 0) load_pre(pn, t - 1);

    f32x4 acc[KW][UTW];
#pragma unroll
    for (int r = 0; r < KW; ++r)
#pragma unroll
      for (int u = 0; u < UTW; ++u) acc[r][u] = f32x4{0.f, 0.f, 0.f, 0.f};
    const Frag* gf = reinterpret_cast<const Frag*>(gb) + lane;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const Frag g = gf[ks * 64];
#pragma unroll
      for (int r = 0; r < KW; ++r)
#pragma unroll
        for (int u = 0; u < UTW; ++u) acc[r][u] = X::mfma(rtf[r][u][ks], g, acc[r][u]);
    }
#pragma unroll
    for (int u = 0; u < UTW; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) ds[u][i][0] += acc[0][u][i];

    if constexpr (KW > 1) if (bvalid) {
      u64* const slot = inbox + (size_t)(t & 1) * INW;
      // send: partial sums of the tiles owned by workgroup (slice + r) % KW, same wave position
#pragma unroll
      for (int r = 1; r < KW; ++r) {
        const int x = (slice + r) % KW;
#pragma unroll
        for (int u = 0; u < UTW; ++u) {
          u64* dst = slot + ((((size_t)(x * WAVES + w) * UTW + u) * KW + slice) * 64 + lane) * 4;
#pragma unroll
          for (int i = 0; i < 4; ++i) ll_store(dst + i, ll_pack((float*)0, acc[r][u][i], t));
        }
      }
      // receive: KW-1 partial sums of the own tiles, RC sources at a time
      const u64* const mine = slot + ((size_t)(slice * WAVES + w) * UTW) * KW * 256 + (size_t)lane * 4;
#pragma unroll
      for (int r0 = 1; r0 < KW; r0 += RC) {
        u64 v[RC][UTW][4];
#pragma unroll
        for (int rr = 0; rr < RC; ++rr)
          if (r0 + rr < KW) {
            const int src = (slice + r0 + rr) % KW;
#pragma unroll
            for (int u = 0; u < UTW; ++u)
#pragma unroll
              for (int i = 0; i < 4; ++i) v[rr][u][i] = ll_load(mine + ((size_t)u * KW + src) * 256 + i);
          }
        for (int spins = 0; !fail;) {
          bool ok = true;
#pragma unroll
          for (int rr = 0; rr < RC; ++rr)
            if (r0 + rr < KW) {
              const int src = (slice + r0 + rr) % KW;
#pragma unroll
              for (int u = 0; u < UTW; ++u)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                  if (!ll_ok((float*)0, v[rr][u][i], t)) { ok = false; v[rr][u][i] = ll_load(mine + ((size_t)u * KW + src) * 256 + i); }
            }
          if (ok) break;
          if (++spins > a.spin_limit) fail = true;
          else if ((spins & 255) == 0 &&
                   __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != STATUS_OK) fail = true;
        }
#pragma unroll
        for (int rr = 0; rr < RC; ++rr)
          if (r0 + rr < KW) {
#pragma unroll
            for (int u = 0; u < UTW; ++u)
#pragma unroll
              for (int i = 0; i < 4; ++i) ds[u][i][0] += __uint_as_float((unsigned)v[rr][u][i]);
          }
      }
    }
  };

  int t = Tn - 1;
  for (; t >= 1 && !dead; t -= 2) {
    step(t, pa, pb);
    if (dead) break;
    step(t - 1, pb, pa);
  }
  if (!dead && t == 0) step(0, pa, pb);
  if (!dead && __syncthreads_or(fail)) dead = true;

  if (dead) {
    if (tid == 0) __hip_atomic_store(a.status, (int)STATUS_WAIT_EXPIRED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int u = 0; u < UTW; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int k = 0; k < S; ++k) ds[u][i][k] = __uint_as_float(0x7fc00000u);
  }

  // ---- cotangent of the initial state, bias partial sums ----------------------------------
  T* __restrict__ ds0 = static_cast<T*>(a.ds0);
#pragma unroll
  for (int u = 0; u < UTW; ++u) {
    const int d0 = ub[u] + q4 * 4;
    if (bvalid) {
#pragma unroll
      for (int k = 0; k < S; ++k) {
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = ds[u][i][k];
        Vec4 p; pack4(v, p);
        *reinterpret_cast<Vec4*>(ds0 + ((size_t)k * B + bg) * ND + (size_t)n * D + d0) = p;
      }
    }
#pragma unroll
    for (int g = 0; g < GT; ++g)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = dead ? __uint_as_float(0x7fc00000u) : dbacc[u][i][g];
        v += __shfl_xor(v, 1); v += __shfl_xor(v, 2); v += __shfl_xor(v, 4); v += __shfl_xor(v, 8);
        if (r16 == 0) a.dbp[(((size_t)bt * GT + g) * N + n) * D + d0 + i] = v;
      }
  }
}

}  // namespace frnn
