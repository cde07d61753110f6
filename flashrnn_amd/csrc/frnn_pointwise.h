// Per-element gate math of the four cells, forward and adjoint, in fp32 registers.
// Shared by the fused kernels (a lane owns a few elements) and the alternating kernels
// (a thread owns one element).
//
// Forward definitions follow flashrnn/flashrnn/vanilla/{lstm,gru,elman,slstm}.py; adjoints
// follow flashrnn/flashrnn/alternating/{lstm,gru,slstm,elman}_pointwise.cu (backward kernels).
// Two deliberate differences from the reference's native kernels, both on the side of accuracy:
//  * all arithmetic is fp32 whatever the storage type (the reference computes in the storage
//    type, flashrnn/flashrnn/fused/lstm_fused_pointwise.cuh:48-87);
//  * the sLSTM cache holds the stabilised forget gate exp(logsig(f)+m-m') and sigmoid(-f)
//    instead of the raw f (slstm_fused_pointwise.cuh:75), so that the backward pass does not
//    rebuild them from storage-rounded f and m.
#pragma once
#include "frnn_common.h"

namespace frnn {

template <bool FAST> struct Math {
  static __device__ __forceinline__ float exp(float x) { return FAST ? __expf(x) : expf(x); }
  static __device__ __forceinline__ float rcp(float x) { return FAST ? __builtin_amdgcn_rcpf(x) : 1.0f / x; }
  static __device__ __forceinline__ float sigmoid(float x) { return rcp(1.0f + exp(-x)); }
  static __device__ __forceinline__ float tanh(float x) {
    if (FAST) return 1.0f - 2.0f * rcp(1.0f + __expf(2.0f * x));
    return tanhf(x);
  }
  // log(sigmoid(x)) = min(x,0) - log1p(exp(-|x|))
  static __device__ __forceinline__ float logsigmoid(float x) {
    const float e = exp(-fabsf(x));
    return fminf(x, 0.0f) - (FAST ? __logf(1.0f + e) : log1pf(e));
  }
};

// fwd:  ry[GR] recurrent pre-activations WITH the bias of their gate slot already added (the
//       fused kernels fold it into the MFMA accumulator), wx[GW], bx = biases of the gate slots
//       that have no recurrent input (gru: the n gate), s[S] in/out, cache[NC] out
// bwd:  cache[NC], sp[S] = s_{t-1}, sn[S] = s_t, dso[S] upstream cotangent of s_t,
//       ds[S] in: running cotangent arriving from step t+1; out: cotangent for s_{t-1}
//       WITHOUT the recurrent term R^T dgr (the caller adds it to ds[0]);
//       dgr[GR] / dgw[GW] / dgb[GT]: cotangents of the R-side, Wx-side and bias pre-activations.
template <int F, bool FAST> struct CellMath;

template <bool FAST> struct CellMath<FRNN_LSTM, FAST> {
  typedef Math<FAST> M;
  static __device__ __forceinline__ void fwd(const float* ry, const float* wx, const float* b, float* s, float* cache) {
    const float i = M::sigmoid(wx[0] + ry[0]);
    const float f = M::sigmoid(wx[1] + ry[1]);
    const float z = M::tanh(wx[2] + ry[2]);
    const float o = M::sigmoid(wx[3] + ry[3]);
    const float c = f * s[1] + i * z;
    s[1] = c;
    s[0] = o * M::tanh(c);
    cache[0] = i; cache[1] = f; cache[2] = z; cache[3] = o;
  }
  static __device__ __forceinline__ void bwd(const float* cache, const float* sp, const float* sn, const float* dso,
                                             float* ds, float* dgr, float* dgw, float* dgb) {
    const float i = cache[0], f = cache[1], z = cache[2], o = cache[3];
    const float dy = dso[0] + ds[0];
    const float tc = M::tanh(sn[1]);
    const float dc = dso[1] + ds[1] + (1.0f - tc * tc) * o * dy;
    dgr[0] = i * (1.0f - i) * z * dc;
    dgr[1] = f * (1.0f - f) * sp[1] * dc;
    dgr[2] = (1.0f - z * z) * i * dc;
    dgr[3] = o * (1.0f - o) * tc * dy;
#pragma unroll
    for (int g = 0; g < 4; ++g) { dgw[g] = dgr[g]; dgb[g] = dgr[g]; }
    ds[0] = 0.0f;
    ds[1] = f * dc;
  }
};

template <bool FAST> struct CellMath<FRNN_SLSTM, FAST> {
  typedef Math<FAST> M;
  static __device__ __forceinline__ void fwd(const float* ry, const float* wx, const float* b, float* s, float* cache) {
    const float ir = wx[0] + ry[0];
    const float fr = wx[1] + ry[1];
    const float z = M::tanh(wx[2] + ry[2]);
    const float o = M::sigmoid(wx[3] + ry[3]);
    const float lfm = M::logsigmoid(fr) + s[3];
    // first step of a fresh sequence: n == 0 (per element, as the native reference kernels,
    // flashrnn/flashrnn/fused/slstm_fused_pointwise.cuh:54-62)
    const float mn = (s[2] == 0.0f) ? ir : fmaxf(ir, lfm);
    const float ig = M::exp(ir - mn);
    const float fg = M::exp(lfm - mn);
    const float c = fg * s[1] + ig * z;
    const float n = fmaxf(fg * s[2] + ig, 1.0f);
    s[0] = o * c * M::rcp(n);
    s[1] = c; s[2] = n; s[3] = mn;
    cache[0] = ig; cache[1] = fg; cache[2] = z; cache[3] = o; cache[4] = M::sigmoid(-fr);
  }
  static __device__ __forceinline__ void bwd(const float* cache, const float* sp, const float* sn, const float* dso,
                                             float* ds, float* dgr, float* dgw, float* dgb) {
    const float ig = cache[0], fg = cache[1], z = cache[2], o = cache[3], omf = cache[4];
    const float dy = dso[0] + ds[0];
    const float dyi = dy * M::rcp(sn[2]);
    const float dc = dso[1] + ds[1] + dyi * o;
    const float dn = dso[2] + ds[2] - dyi * sn[0];
    dgr[0] = ig * (z * dc + dn);
    dgr[1] = fg * (dc * sp[1] + dn * sp[2]) * omf;
    dgr[2] = dc * ig * (1.0f - z * z);
    dgr[3] = (1.0f - o) * sn[0] * dy;
#pragma unroll
    for (int g = 0; g < 4; ++g) { dgw[g] = dgr[g]; dgb[g] = dgr[g]; }
    // the stabiliser m is held constant (slstm_pointwise.cu:205): no cotangent flows into it
    ds[0] = 0.0f; ds[1] = fg * dc; ds[2] = fg * dn; ds[3] = 0.0f;
  }
};

template <bool FAST> struct CellMath<FRNN_GRU, FAST> {
  typedef Math<FAST> M;
  // R gates [g, r, z]; Wx gates [r, z, n]; bias gates [g, r, z, n]
  static __device__ __forceinline__ void fwd(const float* ry, const float* wx, const float* b, float* s, float* cache) {
    const float g = ry[0];
    const float r = M::sigmoid(wx[0] + ry[1]);
    const float z = M::sigmoid(wx[1] + ry[2]);
    const float nv = M::tanh(wx[2] + b[0] + r * g);
    s[0] = z * s[0] + (1.0f - z) * nv;
    cache[0] = g; cache[1] = r; cache[2] = z; cache[3] = nv;  // the candidate itself: the adjoint needs no tanh
  }
  static __device__ __forceinline__ void bwd(const float* cache, const float* sp, const float* sn, const float* dso,
                                             float* ds, float* dgr, float* dgw, float* dgb) {
    const float g = cache[0], r = cache[1], z = cache[2], nv = cache[3];
    const float dy = dso[0] + ds[0];
    const float dz = z * (1.0f - z) * dy * (sp[0] - nv);
    const float dn = dy * (1.0f - z) * (1.0f - nv * nv);
    const float dr = dn * g * r * (1.0f - r);
    const float dg = dn * r;
    dgr[0] = dg; dgr[1] = dr; dgr[2] = dz;
    dgw[0] = dr; dgw[1] = dz; dgw[2] = dn;
    dgb[0] = dg; dgb[1] = dr; dgb[2] = dz; dgb[3] = dn;
    ds[0] = z * dy;
  }
};

template <bool FAST> struct CellMath<FRNN_ELMAN, FAST> {
  typedef Math<FAST> M;
  static __device__ __forceinline__ void fwd(const float* ry, const float* wx, const float* b, float* s, float*) {
    s[0] = M::tanh(wx[0] + ry[0]);
  }
  static __device__ __forceinline__ void bwd(const float*, const float*, const float* sn, const float* dso,
                                             float* ds, float* dgr, float* dgw, float* dgb) {
    const float dy = dso[0] + ds[0];
    dgr[0] = (1.0f - sn[0] * sn[0]) * dy;
    dgw[0] = dgr[0]; dgb[0] = dgr[0];
    ds[0] = 0.0f;
  }
};

// Elman under forward_clipval: cache[0] is the unclamped tanh (the caller clamps s[0] after fwd)
template <bool FAST> struct CellMath<FRNN_ELMAN_CLIP, FAST> {
  typedef Math<FAST> M;
  static __device__ __forceinline__ void fwd(const float* ry, const float* wx, const float* b, float* s, float* cache) {
    s[0] = M::tanh(wx[0] + ry[0]);
    cache[0] = s[0];
  }
  static __device__ __forceinline__ void bwd(const float* cache, const float*, const float*, const float* dso,
                                             float* ds, float* dgr, float* dgw, float* dgb) {
    const float dy = dso[0] + ds[0];
    dgr[0] = (1.0f - cache[0] * cache[0]) * dy;
    dgw[0] = dgr[0]; dgb[0] = dgr[0];
    ds[0] = 0.0f;
  }
};

}  // namespace frnn
