// Shared definitions for the gfx950 FlashRNN kernels: ids, cell descriptors, storage-type
// traits (MFMA fragment shapes, tagged exchange words) and small device helpers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/flashrnn_hip.h"

namespace frnn {

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 half_t;
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned long long u64;

// ---------------------------------------------------------------------------------------
// Cell descriptors.  Gate-slot rule of the reference (flashrnn/flashrnn/flashrnn.py:148-158):
// R fills the first GR of the GI interacting slots, Wx the last GW, b covers all GT.
// NC = values cached per element for the backward pass (private layout; LSTM: the four activated
// gates, GRU: g, r, z and the candidate n, sLSTM: i', f', tanh z, sigmoid o, sigmoid(-f)).
// SPM / DSM = bit masks of the state planes that the adjoint reads at all: plane k of s_(t-1) (as the previous state of
// step t or as the new state of step t-1), plane k of the cotangent of the states.  The LSTM's adjoint never reads h, the
// sLSTM's neither m nor a cotangent of m.  A wave that loads operands for others (the reverse kernel's producer wave)
// skips the planes outside the masks; a lane that loads for itself needs no mask, its unused loads are never emitted.
// ---------------------------------------------------------------------------------------
template <int F> struct Cell;
template <> struct Cell<FRNN_LSTM>  { static constexpr int GR = 4, GW = 4, GT = 4, S = 2, NC = 4, SPM = 0x2, DSM = 0x3; };
template <> struct Cell<FRNN_SLSTM> { static constexpr int GR = 4, GW = 4, GT = 4, S = 4, NC = 5, SPM = 0x7, DSM = 0x7; };
template <> struct Cell<FRNN_GRU>   { static constexpr int GR = 3, GW = 3, GT = 4, S = 1, NC = 4, SPM = 0x1, DSM = 0x1; };
template <> struct Cell<FRNN_ELMAN> { static constexpr int GR = 1, GW = 1, GT = 1, S = 1, NC = 0, SPM = 0x1, DSM = 0x1; };
// Internal variant of the Elman cell for forward_clipval: the stored h is clamped, so the adjoint cannot
// rebuild tanh' from it and the forward pass caches the unclamped value, as the reference does
// (flashrnn/flashrnn/fused/elman_fused_pointwise.cuh:34-60).  Not a function id of the C ABI.
enum { FRNN_ELMAN_CLIP = 4 };
template <> struct Cell<FRNN_ELMAN_CLIP> { static constexpr int GR = 1, GW = 1, GT = 1, S = 1, NC = 1, SPM = 0x0, DSM = 0x1; };

struct CellDims { int GR, GW, GT, S, NC; };
inline CellDims cell_dims(int f) {
  switch (f) {
    case FRNN_LSTM:  return {4, 4, 4, 2, 4};
    case FRNN_SLSTM: return {4, 4, 4, 4, 5};
    case FRNN_GRU:   return {3, 3, 4, 1, 4};
    case FRNN_ELMAN: return {1, 1, 1, 1, 0};
    case FRNN_ELMAN_CLIP: return {1, 1, 1, 1, 1};
  }
  return {0, 0, 0, 0, 0};
}
inline int dtype_size(int dt) { return dt == FRNN_F32 ? 4 : 2; }

// Gate cache of the fused kernels: a value of s_(t-1) that the adjoint of step t needs may travel in the cache line of
// step t (the forward kernel has it in a register when it writes the line), so that the reverse kernel issues one load
// less per step (a vector memory instruction costs a wave ~30 cycles to issue, in front of the step's chain).
//   sLSTM, 16-bit types: c_(t-1) in the sixth slot, which the padding of its five values to whole dwords leaves free:
//          B16 T1024 N4 D192 backward 1.002 -> 0.977 ms, B16 T4096 N4 D192 fwd+bwd 7.97 -> 7.85, N3 D256 +-1 %.
//   LSTM:  measured with c_(t-1) as a fifth value for heads from 256 units on (4 -> 6 padded values, 12 instead of 8
//          bytes per element and step): backward D = 256 +1 %, D = 512 -2.6 %, D = 768 -1.5 %; not worth half as much
//          cache again, so its lines stay at four values.  fp32 lines have no padding.
// Returns the index of the carried state, or -1.  The layout depends on (function, storage type, head dim) only, never
// on the tiling.
constexpr int cache_carried_state(int function, int esize, int /*D*/) {
  return esize == 2 && function == FRNN_SLSTM ? 1 : -1;
}

// ---------------------------------------------------------------------------------------
// Storage-type traits.
//  KM   : K extent of one MFMA (bf16: v_mfma_f32_16x16x32_bf16, f32: v_mfma_f32_16x16x4_f32)
//  Frag : per-lane A/B operand of one MFMA
//  EPW  : elements carried by one 64-bit tagged exchange word
// Fragment order of a [16 rows x K] operand (row = batch for the streamed operand):
//  bf16, f16: element (row, k) -> ((k/32)*64 + ((k%32)/8)*16 + row)*8 + k%8
//  f32 : element (row, k) -> (k/4)*64 + (k%4)*16 + row
// so that lane l of k-step ks reads one contiguous Frag at (ks*64 + l).
// ---------------------------------------------------------------------------------------
template <typename T> struct ST;
struct ST16 {  // what the two 16-bit storage types share
  static constexpr int KM = 32, EPW = 2;
  static constexpr bool FAST = true;
  typedef uint2 Vec4;  // 4 packed elements
  static __device__ __forceinline__ int frag_elem(int row, int k) {
    return (((k >> 5) * 64 + ((k & 31) >> 3) * 16 + row) << 3) + (k & 7);
  }
};
template <> struct ST<bf16_t> : ST16 {
  static constexpr int ID = FRNN_BF16;
  typedef bf16x8 Frag;
  static __device__ __forceinline__ f32x4 mfma(Frag a, Frag b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct ST<half_t> : ST16 {
  static constexpr int ID = FRNN_F16;
  typedef f16x8 Frag;
  static __device__ __forceinline__ f32x4 mfma(Frag a, Frag b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};
template <> struct ST<float> {
  static constexpr int KM = 4, EPW = 1, ID = FRNN_F32;
#ifdef FRNN_F32_PRECISE
  static constexpr bool FAST = false;
#else
  static constexpr bool FAST = true;
#endif
  typedef float Frag;
  typedef float4 Vec4;
  static __device__ __forceinline__ int frag_elem(int row, int k) {
    return (k >> 2) * 64 + (k & 3) * 16 + row;
  }
  static __device__ __forceinline__ f32x4 mfma(Frag a, Frag b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
  }
};

// 16 consecutive k of a product on v_mfma_f32_4x4x1_16B_f32: k-th instruction with the A values (4 rows) of block
// k of `a` broadcast to all 16 blocks (CBSZ = 4, ABID = k: immediates of the instruction), B = b[k] (per block 4
// columns), accumulating round robin into the 4 chains acc[0..3] (first: the chains start from zero).
__device__ __forceinline__ void mfma_4x4x1_bcast16(float a, const float* b, f32x4 (&acc)[4], bool first) {
  const f32x4 z = {0.f, 0.f, 0.f, 0.f};
#define FRNN_K(i) acc[i & 3] = __builtin_amdgcn_mfma_f32_4x4x1f32(a, b[i], (first && i < 4) ? z : acc[i & 3], 4, i, 0);
  FRNN_K(0) FRNN_K(1) FRNN_K(2) FRNN_K(3) FRNN_K(4) FRNN_K(5) FRNN_K(6) FRNN_K(7)
  FRNN_K(8) FRNN_K(9) FRNN_K(10) FRNN_K(11) FRNN_K(12) FRNN_K(13) FRNN_K(14) FRNN_K(15)
#undef FRNN_K
}

__device__ __forceinline__ float bf2f(unsigned short u) { return __uint_as_float(((unsigned)u) << 16); }
__device__ __forceinline__ unsigned short f2bf(float f) {  // round to nearest even; NaN stays NaN
  unsigned u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (unsigned short)(u >> 16);
}

// ---------------------------------------------------------------------------------------
// E consecutive elements of the storage type as NDW dwords (bf16: two per dword, f32: one).
// ---------------------------------------------------------------------------------------
template <int N> struct Dw { unsigned v[N]; };
// dwords that hold E elements of T; a single bf16 (E = 1) still takes one dword in registers and
// is moved with 16-bit memory operations (the SUB flag below)
template <typename T, int E> struct NDW { static constexpr int value = (E * (int)sizeof(T) + 3) / 4; static constexpr bool SUB = E * (int)sizeof(T) < 4; };

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x3 __attribute__((ext_vector_type(3)));

// 16-bit storage types: the two elements of a dword <-> float, round to nearest even
template <typename T> struct H16;
template <> struct H16<bf16_t> {
  static __device__ __forceinline__ float lo(unsigned d) { return __uint_as_float(d << 16); }
  static __device__ __forceinline__ float hi(unsigned d) { return __uint_as_float(d & 0xffff0000u); }
  static __device__ __forceinline__ unsigned pack2(float a, float b) {  // v_cvt_pk_bf16_f32
    const bf16x2 h = __builtin_convertvector(f32x2{a, b}, bf16x2);
    return __builtin_bit_cast(unsigned, h);
  }
};
template <> struct H16<half_t> {
  static __device__ __forceinline__ float lo(unsigned d) { return (float)__builtin_bit_cast(half_t, (unsigned short)d); }
  static __device__ __forceinline__ float hi(unsigned d) { return (float)__builtin_bit_cast(half_t, (unsigned short)(d >> 16)); }
  static __device__ __forceinline__ unsigned pack2(float a, float b) {  // two v_cvt_f16_f32 (the packed convert rounds toward zero)
    const f16x2 h = {(half_t)a, (half_t)b};
    return __builtin_bit_cast(unsigned, h);
  }
};
__device__ __forceinline__ unsigned pack_bf16x2(float a, float b) { return H16<bf16_t>::pack2(a, b); }

template <int E, typename T> __device__ __forceinline__ void unpack16(const Dw<(E + 1) / 2>& d, float* o) {
  if constexpr (E == 1) { o[0] = H16<T>::lo(d.v[0]); }
  else {
#pragma unroll
    for (int k = 0; k < E / 2; ++k) { o[2 * k] = H16<T>::lo(d.v[k]); o[2 * k + 1] = H16<T>::hi(d.v[k]); }
  }
}
template <int E, typename T> __device__ __forceinline__ Dw<(E + 1) / 2> pack16(const float* i) {
  Dw<(E + 1) / 2> d;
  if constexpr (E == 1) { d.v[0] = H16<T>::pack2(i[0], 0.f); }
  else {
#pragma unroll
    for (int k = 0; k < E / 2; ++k) d.v[k] = H16<T>::pack2(i[2 * k], i[2 * k + 1]);
  }
  return d;
}
template <int E> __device__ __forceinline__ void unpack(const Dw<(E + 1) / 2>& d, float* o, bf16_t*) { unpack16<E, bf16_t>(d, o); }
template <int E> __device__ __forceinline__ void unpack(const Dw<(E + 1) / 2>& d, float* o, half_t*) { unpack16<E, half_t>(d, o); }
template <int E> __device__ __forceinline__ Dw<(E + 1) / 2> pack(const float* i, bf16_t*) { return pack16<E, bf16_t>(i); }
template <int E> __device__ __forceinline__ Dw<(E + 1) / 2> pack(const float* i, half_t*) { return pack16<E, half_t>(i); }
template <int E> __device__ __forceinline__ void unpack(const Dw<E>& d, float* o, float*) {
#pragma unroll
  for (int k = 0; k < E; ++k) o[k] = __uint_as_float(d.v[k]);
}
template <int E> __device__ __forceinline__ Dw<E> pack(const float* i, float*) {
  Dw<E> d;
#pragma unroll
  for (int k = 0; k < E; ++k) d.v[k] = __float_as_uint(i[k]);
  return d;
}

// x clamped to [-v, v] if v > 0, else x untouched (a select, not a branch; NaN stays NaN when off)
__device__ __forceinline__ float clamp_if(float x, float v) {
  const float c = fminf(fmaxf(x, -v), v);
  return v > 0.f ? c : x;
}

// ---------------------------------------------------------------------------------------
// Raw buffer access: one descriptor per tensor in SGPRs, 32-bit byte offsets.  An offset at or
// beyond the tensor's size makes a load return 0 and drops a store, so padded batch rows need
// no branch; kInvalidOff keeps such a lane out of range for any scalar offset below 2 GiB,
// which is why tensors handed to the fused kernels must be smaller than 2 GiB.
// ---------------------------------------------------------------------------------------
typedef __amdgpu_buffer_rsrc_t rsrc_t;
constexpr unsigned kInvalidOff = 0x80000000u;
__device__ __forceinline__ rsrc_t make_rsrc(const void* p, size_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)(bytes > 0x7fffffffu ? 0x7fffffffu : bytes), 0x00020000);
}
template <int N, bool SUB = false> __device__ __forceinline__ Dw<N> buf_load(rsrc_t r, unsigned voff, unsigned soff) {
  Dw<N> d;
  if constexpr (SUB) { static_assert(N == 1, "one 16-bit element"); d.v[0] = __builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, 0); }
  else if constexpr (N == 1) { d.v[0] = __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0); }
  else if constexpr (N == 2) { const u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0); d.v[0] = t.x; d.v[1] = t.y; }
  else { static_assert(N == 4, "1, 2 or 4 dwords"); const u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0); d.v[0] = t.x; d.v[1] = t.y; d.v[2] = t.z; d.v[3] = t.w; }
  return d;
}
// A buffer store of more than 8 bytes reads its data registers a cycle after it issues.  When the store takes its
// offset from an SGPR the compiler assumes that this cannot hurt and lets a vector instruction overwrite a data
// register in the very next slot; on gfx950 that instruction's result was what reached memory (seen as the LDS address
// of the next piece in the first dword of every 16-byte piece that a wave stored in a loop).  One independent
// instruction in between is enough: the s_nop below names the data registers as its inputs, so nothing can overwrite
// them before it, and it cannot move in front of the store.  Every store of 12 or 16 bytes in this library goes
// through these helpers; a test scans the generated code of every kernel for the pattern.
// (The data first pass through an empty asm that makes them opaque: a constant would otherwise be re-materialised
// into other registers for the s_nop, which then would not hold the store's own registers.)
template <int AUX = 0> __device__ __forceinline__ void store_b128_safe(unsigned a, unsigned b, unsigned c, unsigned d, rsrc_t r, unsigned voff, unsigned soff) {
  u32x4 v = {a, b, c, d};
  asm volatile("" : "+v"(v));  // (the register tuple itself, not the four values, is what the s_nop has to name)
  __builtin_amdgcn_raw_buffer_store_b128(v, r, voff, soff, AUX);
  asm volatile("s_nop 0" ::"v"(v));
}
__device__ __forceinline__ void store_b96_safe(unsigned a, unsigned b, unsigned c, rsrc_t r, unsigned voff, unsigned soff) {
  u32x3 v = {a, b, c};
  asm volatile("" : "+v"(v));
  __builtin_amdgcn_raw_buffer_store_b96(v, r, voff, soff, 0);
  asm volatile("s_nop 0" ::"v"(v));
}
template <int N, bool SUB = false> __device__ __forceinline__ void buf_store(const Dw<N>& d, rsrc_t r, unsigned voff, unsigned soff) {
  if constexpr (SUB) { static_assert(N == 1, "one 16-bit element"); __builtin_amdgcn_raw_buffer_store_b16((unsigned short)d.v[0], r, voff, soff, 0); }
  else if constexpr (N == 1) { __builtin_amdgcn_raw_buffer_store_b32(d.v[0], r, voff, soff, 0); }
  else if constexpr (N == 2) { __builtin_amdgcn_raw_buffer_store_b64(u32x2{d.v[0], d.v[1]}, r, voff, soff, 0); }
  else {
    static_assert(N == 4, "1, 2 or 4 dwords");
    store_b128_safe(d.v[0], d.v[1], d.v[2], d.v[3], r, voff, soff);
  }
}

// N dwords per lane with as few instructions as possible (pieces of 4, then 3, 2 or 1 dwords):
// every vector memory instruction costs a wave some 30 cycles of issue time, whatever its width
template <int N> __device__ __forceinline__ Dw<N> buf_load_wide(rsrc_t r, unsigned voff, unsigned soff) {
  Dw<N> d;
  constexpr int Q = N / 4 * 4, R = N % 4;
#pragma unroll
  for (int i = 0; i < Q; i += 4) {
    const u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(r, voff + i * 4, soff, 0);
    d.v[i] = t.x; d.v[i + 1] = t.y; d.v[i + 2] = t.z; d.v[i + 3] = t.w;
  }
  if constexpr (R == 3) { const u32x3 t = __builtin_amdgcn_raw_buffer_load_b96(r, voff + Q * 4, soff, 0); d.v[Q] = t.x; d.v[Q + 1] = t.y; d.v[Q + 2] = t.z; }
  else if constexpr (R == 2) { const u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(r, voff + Q * 4, soff, 0); d.v[Q] = t.x; d.v[Q + 1] = t.y; }
  else if constexpr (R == 1) { d.v[Q] = __builtin_amdgcn_raw_buffer_load_b32(r, voff + Q * 4, soff, 0); }
  return d;
}
template <int N> __device__ __forceinline__ void buf_store_wide(const Dw<N>& d, rsrc_t r, unsigned voff, unsigned soff) {
  constexpr int Q = N / 4 * 4, R = N % 4;
#pragma unroll
  for (int i = 0; i < Q; i += 4) {
    store_b128_safe(d.v[i], d.v[i + 1], d.v[i + 2], d.v[i + 3], r, voff + i * 4, soff);
  }
  if constexpr (R == 3) {
    store_b96_safe(d.v[Q], d.v[Q + 1], d.v[Q + 2], r, voff + Q * 4, soff);
  }
  else if constexpr (R == 2) __builtin_amdgcn_raw_buffer_store_b64(u32x2{d.v[Q], d.v[Q + 1]}, r, voff + Q * 4, soff, 0);
  else if constexpr (R == 1) __builtin_amdgcn_raw_buffer_store_b32(d.v[Q], r, voff + Q * 4, soff, 0);
}

// Gate cache of the fused kernels: the NC cached values of one (batch row, unit) are adjacent
// (padded to NCP, a whole number of dwords), units are the next index, so a lane moves all cached
// values of its E consecutive units with one or two instructions.
template <typename T, int NC> struct CacheBlk {
  static constexpr int NCP = sizeof(T) == 2 ? (NC + 1) / 2 * 2 : NC;
  template <int E> struct Words { static constexpr int value = E * NCP * (int)sizeof(T) / 4 > 0 ? E * NCP * (int)sizeof(T) / 4 : 1; };
};
// v[c][e] -> dwords, element (e, c) at flat index e*NCP + c
template <typename T, int NC, int E> __device__ __forceinline__ Dw<CacheBlk<T, NC>::template Words<E>::value>
cache_pack(const float (*v)[E]) {
  constexpr int NCP = CacheBlk<T, NC>::NCP, NW = CacheBlk<T, NC>::template Words<E>::value;
  Dw<NW> d;
  if constexpr (sizeof(T) == 4) {
#pragma unroll
    for (int i = 0; i < NW; ++i) d.v[i] = __float_as_uint(v[i % NCP][i / NCP]);
  } else {
#pragma unroll
    for (int i = 0; i < NW; ++i) {
      const int i0 = 2 * i, i1 = 2 * i + 1;
      const float a = (i0 % NCP) < NC ? v[i0 % NCP][i0 / NCP] : 0.f, b = (i1 % NCP) < NC ? v[i1 % NCP][i1 / NCP] : 0.f;
      d.v[i] = H16<T>::pack2(a, b);
    }
  }
  return d;
}
template <typename T, int NC, int E> __device__ __forceinline__ void
cache_unpack(const Dw<CacheBlk<T, NC>::template Words<E>::value>& d, float (*v)[E]) {
  constexpr int NCP = CacheBlk<T, NC>::NCP;
#pragma unroll
  for (int e = 0; e < E; ++e)
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int i = e * NCP + c;
      if constexpr (sizeof(T) == 4) v[c][e] = __uint_as_float(d.v[i]);
      else v[c][e] = (i & 1) ? H16<T>::hi(d.v[i / 2]) : H16<T>::lo(d.v[i / 2]);
    }
}

// 4 consecutive elements <-> 4 floats (vector form, used outside the time loops)
template <typename T> __device__ __forceinline__ void unpack4(uint2 v, float* o) {
  o[0] = H16<T>::lo(v.x); o[1] = H16<T>::hi(v.x); o[2] = H16<T>::lo(v.y); o[3] = H16<T>::hi(v.y);
}
template <typename T> __device__ __forceinline__ void unpack4(float4 v, float* o) { o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w; }

// ---------------------------------------------------------------------------------------
// Tagged exchange words ("data + step tag in one store"): a reader that sees the tag of the
// step it waits for has the data of that step; no separate flag, no fence.  32-bit stores
// are single-copy atomic, so each tagged element is validated on its own.
//  bf16, f16: 64-bit word = two (tag16 << 16 | element) halves;  f32: (tag32 << 32 | f32 bits).
// Tag of step t is never 0, so zero-filled memory never validates.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ unsigned tag16(int t) { return (unsigned)(t % 65535) + 1u; }
template <typename T> __device__ __forceinline__ u64 ll_pack16(float a, float b, int t) {
  const unsigned tg = tag16(t) << 16, ab = H16<T>::pack2(a, b);
  return (u64)(tg | (ab & 0xffffu)) | ((u64)(tg | (ab >> 16)) << 32);
}
__device__ __forceinline__ u64 ll_pack(bf16_t*, float a, float b, int t) { return ll_pack16<bf16_t>(a, b, t); }
__device__ __forceinline__ u64 ll_pack(half_t*, float a, float b, int t) { return ll_pack16<half_t>(a, b, t); }
__device__ __forceinline__ u64 ll_pack(float*, float a, int t) {
  return (u64)__float_as_uint(a) | ((u64)(unsigned)(t + 1) << 32);
}
__device__ __forceinline__ bool ll_ok16(u64 w, int t) {
  unsigned tg = tag16(t);
  return ((unsigned)(w >> 16) & 0xffffu) == tg && (unsigned)(w >> 48) == tg;
}
__device__ __forceinline__ bool ll_ok(bf16_t*, u64 w, int t) { return ll_ok16(w, t); }
__device__ __forceinline__ bool ll_ok(half_t*, u64 w, int t) { return ll_ok16(w, t); }
__device__ __forceinline__ bool ll_ok(float*, u64 w, int t) { return (unsigned)(w >> 32) == (unsigned)(t + 1); }
// payload as the 32 bits that go to LDS (bf16: two elements; f32: one)
__device__ __forceinline__ unsigned ll_payload16(u64 w) {
  return ((unsigned)w & 0xffffu) | (((unsigned)(w >> 32) & 0xffffu) << 16);
}
__device__ __forceinline__ unsigned ll_payload(bf16_t*, u64 w) { return ll_payload16(w); }
__device__ __forceinline__ unsigned ll_payload(half_t*, u64 w) { return ll_payload16(w); }
__device__ __forceinline__ unsigned ll_payload(float*, u64 w) { return (unsigned)w; }

// Partial sums of the backward exchange.  fp32 storage: (tag32 << 32 | f32 bits) as above.  16-bit
// storage: one 32-bit word (tag8 << 24 | the sum rounded to sign, 8 exponent and 15 mantissa bits):
// the operands of the sum carry 8 or 11 mantissa bits, and the exchange costs by the byte (measured:
// -18 % per step against 8-byte words).  Tag of step t is never 0 and differs from that of step
// t +- 2, the only older content a slot can hold.
struct Part64 { typedef u64 Word; };
struct Part32 { typedef unsigned Word; };
__device__ __forceinline__ u64 part_pack(Part64*, float a, int t) { return (u64)__float_as_uint(a) | ((u64)(unsigned)(t + 1) << 32); }
__device__ __forceinline__ bool ll_ok(Part64*, u64 w, int t) { return (unsigned)(w >> 32) == (unsigned)(t + 1); }
__device__ __forceinline__ float part_value(Part64*, u64 w) { return __uint_as_float((unsigned)w); }
__device__ __forceinline__ unsigned tag8(int t) { return (unsigned)(t % 255) + 1u; }
__device__ __forceinline__ unsigned part_pack(Part32*, float a, int t) {
  // round to nearest on the 8 dropped bits; a NaN is left as it is (the rounding add would carry a large
  // NaN payload out of the word and turn the NaN into a zero)
  const unsigned bits = __float_as_uint(a);
  return (tag8(t) << 24) | ((a != a ? bits : bits + 0x80u) >> 8);
}
__device__ __forceinline__ bool ll_ok(Part32*, unsigned w, int t) { return (w >> 24) == tag8(t); }
__device__ __forceinline__ float part_value(Part32*, unsigned w) { return __uint_as_float(w << 8); }
__device__ __forceinline__ unsigned ll_load(const unsigned* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ u64 ll_load(const u64* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Stores of tagged words, N per lane at `base + voff + i * STRIDE` bytes (base uniform, voff per lane).
// near == 0: agent scope (sc1), the store is written through to memory, where an agent-scope load of any
// compute unit finds it.  near == ~0: workgroup scope (sc0), the store is written through the compute unit's L1
// into the L2 of its XCD and stays there; the agent-scope loads of the other workgroups miss their L1 and meet
// it in that L2, provided they run on the same XCD (each XCD has an L2 of its own; a store left in another
// XCD's L2 is never seen).  Measured for an all-to-all exchange of one word per thread between 4 workgroups of
// one XCD: 1080 cycles per step against 1610-1980 with agent-scope stores (2 workgroups 840 against 1570,
// 8: 1420 against 2240).  The kernels pass near == ~0 only after xcd_handshake has shown that the workgroups of
// the group share an XCD.  `near` is a lane mask, all ones or zero: both forms of the store are issued, one of
// them with no lane enabled, inside one asm block.  A branch that the compiler sees splits the step's schedule and
// costs the kernels at the register limit spills; a scalar branch inside the block costs 35-60 cycles per store
// group (measured), which adds up where a wave sends to 31 other workgroups per step.
#define FRNN_SEL_HEAD "s_mov_b64 %[tmp], exec\n\ts_and_b64 exec, %[tmp], %[nr]\n\t"
#define FRNN_SEL_MID "s_andn2_b64 exec, %[tmp], %[nr]\n\t"
#define FRNN_SEL_TAIL "s_mov_b64 exec, %[tmp]"
#define FRNN_ST0(op, sc) op " %[o], %[v0], %[b] " sc "\n\t"
#define FRNN_ST1(op, sc) op " %[o], %[v1], %[b] offset:%[k1] " sc "\n\t"
#define FRNN_ST2(op, sc) op " %[o], %[v2], %[b] offset:%[k2] " sc "\n\t"
#define FRNN_ST3(op, sc) op " %[o], %[v3], %[b] offset:%[k3] " sc "\n\t"
#define FRNN_SEL_DEFINE(W, op)                                                                                   \
  template <int N, int STRIDE> __device__ __forceinline__ void ll_store_sel(const void* base, unsigned voff, const W* v, u64 near) { \
    static_assert(N == 1 || N == 2 || N == 4, "1, 2 or 4 words per lane");                                       \
    static_assert(3 * STRIDE < 4096, "immediate offsets");                                                      \
    u64 tmp;                                                                                                     \
    if constexpr (N == 1)                                                                                        \
      asm volatile(FRNN_SEL_HEAD FRNN_ST0(op, "sc0") FRNN_SEL_MID FRNN_ST0(op, "sc1") FRNN_SEL_TAIL                \
                   : [tmp] "=&s"(tmp) : [o] "v"(voff), [b] "s"(base), [v0] "v"(v[0]), [nr] "s"(near) : "scc");    \
    else if constexpr (N == 2)                                                                                   \
      asm volatile(FRNN_SEL_HEAD FRNN_ST0(op, "sc0") FRNN_ST1(op, "sc0") FRNN_SEL_MID FRNN_ST0(op, "sc1") FRNN_ST1(op, "sc1") FRNN_SEL_TAIL \
                   : [tmp] "=&s"(tmp) : [o] "v"(voff), [b] "s"(base), [v0] "v"(v[0]), [v1] "v"(v[1]), [k1] "n"(STRIDE), [nr] "s"(near) : "scc"); \
    else                                                                                                         \
      asm volatile(FRNN_SEL_HEAD FRNN_ST0(op, "sc0") FRNN_ST1(op, "sc0") FRNN_ST2(op, "sc0") FRNN_ST3(op, "sc0") FRNN_SEL_MID \
                   FRNN_ST0(op, "sc1") FRNN_ST1(op, "sc1") FRNN_ST2(op, "sc1") FRNN_ST3(op, "sc1") FRNN_SEL_TAIL    \
                   : [tmp] "=&s"(tmp) : [o] "v"(voff), [b] "s"(base), [v0] "v"(v[0]), [v1] "v"(v[1]), [v2] "v"(v[2]), [v3] "v"(v[3]), \
                      [k1] "n"(STRIDE), [k2] "n"(2 * STRIDE), [k3] "n"(3 * STRIDE), [nr] "s"(near) : "scc");     \
  }
FRNN_SEL_DEFINE(unsigned, "global_store_dword")
FRNN_SEL_DEFINE(u64, "global_store_dwordx2")
#undef FRNN_SEL_DEFINE

// The same for 4 destinations at once (4 uniform bases, one lane offset, N words each): the two switches of the lane
// mask cost ~40 cycles per block, which adds up for a wave that sends to 31 other workgroups per step.
#define FRNN_D(op, sc, d, e) op " %[o], %[v" #d #e "], %[b" #d "] offset:%[k" #e "] " sc "\n\t"
#define FRNN_D1(op, sc, d) FRNN_D(op, sc, d, 0)
#define FRNN_D2(op, sc, d) FRNN_D(op, sc, d, 0) FRNN_D(op, sc, d, 1)
#define FRNN_D4(op, sc, d) FRNN_D(op, sc, d, 0) FRNN_D(op, sc, d, 1) FRNN_D(op, sc, d, 2) FRNN_D(op, sc, d, 3)
#define FRNN_ALL(DN, op, sc) DN(op, sc, 0) DN(op, sc, 1) DN(op, sc, 2) DN(op, sc, 3)
#define FRNN_VROW(d) [v##d##0] "v"(v[d][0])
#define FRNN_VROW2(d) FRNN_VROW(d), [v##d##1] "v"(v[d][N > 1 ? 1 : 0])
#define FRNN_VROW4(d) FRNN_VROW2(d), [v##d##2] "v"(v[d][N > 2 ? 2 : 0]), [v##d##3] "v"(v[d][N > 3 ? 3 : 0])
#define FRNN_SEL4_DEFINE(W, op)                                                                                  \
  template <int N, int STRIDE> __device__ __forceinline__ void ll_store_sel4(const void* const (&base)[4], unsigned voff, const W (&v)[4][N], u64 near) { \
    static_assert(N == 1 || N == 2 || N == 4, "1, 2 or 4 words per lane and destination");                       \
    static_assert(3 * STRIDE < 4096, "immediate offsets");                                                      \
    u64 tmp;                                                                                                     \
    if constexpr (N == 1)                                                                                        \
      asm volatile(FRNN_SEL_HEAD FRNN_ALL(FRNN_D1, op, "sc0") FRNN_SEL_MID FRNN_ALL(FRNN_D1, op, "sc1") FRNN_SEL_TAIL \
                   : [tmp] "=&s"(tmp) : [o] "v"(voff), [b0] "s"(base[0]), [b1] "s"(base[1]), [b2] "s"(base[2]), [b3] "s"(base[3]), \
                     FRNN_VROW(0), FRNN_VROW(1), FRNN_VROW(2), FRNN_VROW(3), [k0] "n"(0), [nr] "s"(near) : "scc"); \
    else if constexpr (N == 2)                                                                                   \
      asm volatile(FRNN_SEL_HEAD FRNN_ALL(FRNN_D2, op, "sc0") FRNN_SEL_MID FRNN_ALL(FRNN_D2, op, "sc1") FRNN_SEL_TAIL \
                   : [tmp] "=&s"(tmp) : [o] "v"(voff), [b0] "s"(base[0]), [b1] "s"(base[1]), [b2] "s"(base[2]), [b3] "s"(base[3]), \
                     FRNN_VROW2(0), FRNN_VROW2(1), FRNN_VROW2(2), FRNN_VROW2(3), [k0] "n"(0), [k1] "n"(STRIDE), [nr] "s"(near) : "scc"); \
    else                                                                                                         \
      asm volatile(FRNN_SEL_HEAD FRNN_ALL(FRNN_D4, op, "sc0") FRNN_SEL_MID FRNN_ALL(FRNN_D4, op, "sc1") FRNN_SEL_TAIL \
                   : [tmp] "=&s"(tmp) : [o] "v"(voff), [b0] "s"(base[0]), [b1] "s"(base[1]), [b2] "s"(base[2]), [b3] "s"(base[3]), \
                     FRNN_VROW4(0), FRNN_VROW4(1), FRNN_VROW4(2), FRNN_VROW4(3),                                   \
                     [k0] "n"(0), [k1] "n"(STRIDE), [k2] "n"(2 * STRIDE), [k3] "n"(3 * STRIDE), [nr] "s"(near) : "scc"); \
  }
FRNN_SEL4_DEFINE(unsigned, "global_store_dword")
FRNN_SEL4_DEFINE(u64, "global_store_dwordx2")
#undef FRNN_SEL4_DEFINE
#undef FRNN_VROW4
#undef FRNN_VROW2
#undef FRNN_VROW
#undef FRNN_ALL
#undef FRNN_D4
#undef FRNN_D2
#undef FRNN_D1
#undef FRNN_D
#undef FRNN_ST3
#undef FRNN_ST2
#undef FRNN_ST1
#undef FRNN_ST0
#undef FRNN_SEL_TAIL
#undef FRNN_SEL_MID
#undef FRNN_SEL_HEAD

// largest divisor of n that is <= 8: k-steps whose LDS fragments are fetched together
constexpr int chunk_of(int n) { for (int c = 8; c > 1; --c) if (n % c == 0) return c; return 1; }

// status word values written by a kernel whose bounded wait ran out
enum { STATUS_OK = 0, STATUS_WAIT_EXPIRED = 1 };

// Workgroup -> (group, slice) mapping.  Workgroups are dispatched round-robin over the 8
// XCDs, so the KW workgroups of one (head, batch-tile) group take ids that are congruent
// mod 8 and share one XCD's L2.  grid = 8 * KW * ceil(groups / 8).
// Groups of more than 32 workgroups (fp32 gated cells beyond 512 units: one workgroup per compute unit, and an XCD has
// 32) spread over the whole device instead, consecutive ids, and exchange at agent scope.  grid = KW * groups.
constexpr int kXcdWorkgroups = 32;
__device__ __forceinline__ bool decode_block(int groups, int KW, int& grp, int& slice) {
  if (KW > kXcdWorkgroups) {
    grp = blockIdx.x / KW;
    slice = blockIdx.x % KW;
    return grp < groups;
  }
  const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
  grp = (q / KW) * 8 + xcd;
  slice = q % KW;
  return grp < groups;
}
inline int grid_for(int groups, int KW) { return KW > kXcdWorkgroups ? KW * groups : 8 * KW * ((groups + 7) / 8); }

}  // namespace frnn
