// Mailbox of the resident decode kernel: how tokens reach a kernel that stays on the device, and how the
// new states leave it.
//
// The reference decodes with one kernel launch per token that reloads R (flashrnn/flashrnn/flashrnn.py:957-985,
// alternating/flashrnn.h:97-101).  Here the forward kernel of a head dim is launched once, keeps R in its
// registers and the state in fp32 registers, and takes one token after the other from a ring of slots in a
// buffer of the caller:
//
//   ctrl     64 ints: status, stop word, exit reason, tokens done, sequence counters
//   exchange the slots through which the workgroups of a head pass h (heads of several workgroups)
//   inbox    SLOTS x [B][N][D] records of G_w tagged values: the Wx of one token, gate innermost
//   outbox   SLOTS x [B][N][D] records of S tagged values: the new states of that token
//
// A record holds the values of ONE element (batch row, head, unit), so the lane that owns the element fetches
// or stores it with one memory instruction.  Every value carries the tag of its token (16-bit types: a dword
// (tag16 << 16 | value); fp32: two dwords, value and tag32), so a reader that finds the tags of token t has
// the data of token t: no flag, no fence, and the writer may be any kernel of the caller (decode_exchange_kernel
// below is the one the library provides).  All accesses are agent scope.  Token t uses slot t % SLOTS; the
// caller may post token t + SLOTS only when it has collected token t.
#pragma once
#include "frnn_common.h"

namespace frnn {

enum { MB_STATUS = 0, MB_STOP = 1, MB_REASON = 2, MB_DONE = 3, MB_XERR = 4, MB_SEQ = 8, MB_TOK = 9, MB_CTRL_INTS = 64 };
// why the resident kernel ended (MB_REASON)
enum { MB_END_NONE = 0, MB_END_WAIT = 1, MB_END_IDLE = 2, MB_END_STOP = 3, MB_END_TOKENS = 4 };

constexpr int mb_pad(int n) { return n <= 1 ? 1 : n <= 2 ? 2 : 4; }
// dwords of a record of NV values of storage type T
template <typename T, int NV> struct MbRec {
  static constexpr int NVP = mb_pad(NV);
  static constexpr int DW = NVP * (sizeof(T) == 4 ? 2 : 1);
  static constexpr int BYTES = DW * 4;
};
inline int mb_rec_bytes(int dtype, int nv) { return mb_pad(nv) * (dtype == FRNN_F32 ? 8 : 4); }

// agent-scope (sc1) buffer accesses of N dwords, N = 1, 2, 4 or 8
template <int N> __device__ __forceinline__ Dw<N> mb_load(rsrc_t r, unsigned voff, unsigned soff) {
  Dw<N> d;
  if constexpr (N == 1) { d.v[0] = __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 16); }
  else if constexpr (N == 2) { const u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 16); d.v[0] = t.x; d.v[1] = t.y; }
  else {
    static_assert(N == 4 || N == 8, "1, 2, 4 or 8 dwords");
#pragma unroll
    for (int i = 0; i < N; i += 4) {
      const u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(r, voff + i * 4, soff, 16);
      d.v[i] = t.x; d.v[i + 1] = t.y; d.v[i + 2] = t.z; d.v[i + 3] = t.w;
    }
  }
  return d;
}
template <int N> __device__ __forceinline__ void mb_store(const Dw<N>& d, rsrc_t r, unsigned voff, unsigned soff) {
  if constexpr (N == 1) __builtin_amdgcn_raw_buffer_store_b32(d.v[0], r, voff, soff, 16);
  else if constexpr (N == 2) __builtin_amdgcn_raw_buffer_store_b64(u32x2{d.v[0], d.v[1]}, r, voff, soff, 16);
  else {
    static_assert(N == 4 || N == 8, "1, 2, 4 or 8 dwords");
#pragma unroll
    for (int i = 0; i < N; i += 4) {
      store_b128_safe<16>(d.v[i], d.v[i + 1], d.v[i + 2], d.v[i + 3], r, voff + i * 4, soff);
    }
  }
}

// record <-> values.  `bits` are the values in the storage type (16-bit types: in the low half of a dword).
template <typename T, int NV> __device__ __forceinline__ Dw<MbRec<T, NV>::DW> mb_pack(const unsigned* bits, int t) {
  Dw<MbRec<T, NV>::DW> d;
  constexpr int NVP = MbRec<T, NV>::NVP;
#pragma unroll
  for (int i = 0; i < NVP; ++i) {
    const unsigned v = i < NV ? bits[i] : 0u;
    if constexpr (sizeof(T) == 4) { d.v[2 * i] = v; d.v[2 * i + 1] = (unsigned)(t + 1); }
    else d.v[i] = (tag16(t) << 16) | (v & 0xffffu);
  }
  return d;
}
template <typename T, int NV> __device__ __forceinline__ bool mb_ok(const Dw<MbRec<T, NV>::DW>& d, int t) {
  constexpr int NVP = MbRec<T, NV>::NVP;
  bool ok = true;
#pragma unroll
  for (int i = 0; i < NVP; ++i) {
    if constexpr (sizeof(T) == 4) ok = ok & (d.v[2 * i + 1] == (unsigned)(t + 1));
    else ok = ok & ((d.v[i] >> 16) == tag16(t));
  }
  return ok;
}
// value i of a record as float (exact for every storage type)
template <typename T, int NV> __device__ __forceinline__ float mb_value(const Dw<MbRec<T, NV>::DW>& d, int i) {
  if constexpr (sizeof(T) == 4) return __uint_as_float(d.v[2 * i]);
  else return H16<T>::lo(d.v[i]);
}
// a float rounded to the storage type, as the dword that mb_pack takes (the rounding of the kernels' own stores)
template <typename T> __device__ __forceinline__ unsigned mb_bits(float v) {
  if constexpr (sizeof(T) == 4) return __float_as_uint(v);
  else return H16<T>::pack2(v, 0.f) & 0xffffu;
}

// Layout of the caller's buffer.  exch_bytes: what the kernel's tiling needs for the exchange between the
// workgroups of a head (0 for heads of one workgroup).
struct MbLayout {
  size_t exch_off, xcd_off, inbox_off, outbox_off, in_slot, out_slot, total, zero_bytes;
};
inline MbLayout mb_layout(int dtype, int B, int N, int D, int gw, int s, int slots, size_t exch_bytes, size_t xcd_bytes) {
  auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  MbLayout l;
  l.exch_off = up(MB_CTRL_INTS * 4);
  l.xcd_off = l.exch_off + up(exch_bytes);
  l.inbox_off = l.xcd_off + up(xcd_bytes);
  l.in_slot = up((size_t)B * N * D * mb_rec_bytes(dtype, gw));
  l.outbox_off = l.inbox_off + (size_t)slots * l.in_slot;
  l.out_slot = up((size_t)B * N * D * mb_rec_bytes(dtype, s));
  l.total = l.outbox_off + (size_t)slots * l.out_slot;
  l.zero_bytes = l.total;  // everything starts at zero: no tag of a token is 0
  return l;
}

// ---- the caller's side, as one kernel: posts `count` tokens and collects their new states ----------------
// Wx [B][count][G_w][N][D] and s_out [S][B][count][N][D] in the storage type (the public layouts of a sequence
// of `count` steps).  One thread per element.  The token numbers come from the mailbox itself (MB_TOK, advanced
// by `count` when the last workgroup of a launch leaves), so that the same launch can be replayed from a HIP
// graph.  The wait for a result is bounded: when it runs out the thread writes NaN and sets MB_XERR.
struct MbExchangeArgs {
  const void* Wx; void* s_out; void* mailbox;
  size_t inbox_off, outbox_off, in_slot, out_slot;
  int B, N, D, count, slots, spin_limit;
};
template <typename T, int GW, int S>
__global__ void __launch_bounds__(256) decode_exchange_kernel(const MbExchangeArgs a) {
  typedef MbRec<T, GW> RI;
  typedef MbRec<T, S> RO;
  int* const ctrl = static_cast<int*>(a.mailbox);
  __shared__ int tok_s;
  const unsigned ND = (unsigned)a.N * a.D, total = (unsigned)a.B * ND;
  const unsigned idx = blockIdx.x * 256u + threadIdx.x;
  const bool valid = idx < total;
  const unsigned b = valid ? idx / ND : 0, nd = valid ? idx % ND : 0;
  const T* __restrict__ Wx = static_cast<const T*>(a.Wx);
  T* __restrict__ so = static_cast<T*>(a.s_out);
  auto load_wx = [&](int c, unsigned* bits) __attribute__((always_inline)) {
#pragma unroll
    for (int g = 0; g < GW; ++g) {
      T v = T();
      if (valid) v = Wx[(((size_t)b * a.count + c) * GW + g) * ND + nd];
      if constexpr (sizeof(T) == 4) bits[g] = __float_as_uint(v);
      else bits[g] = (unsigned)__builtin_bit_cast(unsigned short, v);
    }
  };
  // (the first token's Wx is fetched while the token number is on its way)
  unsigned first[GW];
  load_wx(0, first);
  if (threadIdx.x == 0) tok_s = __hip_atomic_load(ctrl + MB_TOK, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  const int tok0 = tok_s;
  const rsrc_t rIn = make_rsrc(static_cast<char*>(a.mailbox) + a.inbox_off, (size_t)a.slots * a.in_slot);
  const rsrc_t rOut = make_rsrc(static_cast<char*>(a.mailbox) + a.outbox_off, (size_t)a.slots * a.out_slot);
  for (int c = 0; c < a.count; ++c) {
    const int t = tok0 + c;
    unsigned bits[GW];
    if (c == 0) {
#pragma unroll
      for (int g = 0; g < GW; ++g) bits[g] = first[g];
    } else {
      load_wx(c, bits);
    }
    mb_store<RI::DW>(mb_pack<T, GW>(bits, t), rIn, valid ? idx * RI::BYTES : kInvalidOff, (unsigned)(t % a.slots) * (unsigned)a.in_slot);
  }
  for (int c = 0; c < a.count; ++c) {
    const int t = tok0 + c;
    Dw<RO::DW> r;
    bool ok = false;
    for (int spins = 0; valid && a.spin_limit >= -1; ++spins) {
      r = mb_load<RO::DW>(rOut, idx * RO::BYTES, (unsigned)(t % a.slots) * (unsigned)a.out_slot);
      ok = mb_ok<T, S>(r, t);
      if (ok || spins > a.spin_limit) break;
      // the resident kernel has ended, or another thread has given up: look once more, then give up as well (so that a
      // dead session costs its caller one bounded wait, not one per token)
      if ((spins & 63) == 63 && (__hip_atomic_load(ctrl + MB_REASON, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0 ||
                                 __hip_atomic_load(ctrl + MB_XERR, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)) {
        r = mb_load<RO::DW>(rOut, idx * RO::BYTES, (unsigned)(t % a.slots) * (unsigned)a.out_slot);
        ok = mb_ok<T, S>(r, t);
        break;
      }
    }
    if (!valid) continue;
    if (!ok) __hip_atomic_store(ctrl + MB_XERR, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int k = 0; k < S; ++k) {
      T v;
      if constexpr (sizeof(T) == 4) v = ok ? __uint_as_float(r.v[2 * k]) : __uint_as_float(0x7fc00000u);
      else v = __builtin_bit_cast(T, (unsigned short)(ok ? (r.v[k] & 0xffffu) : (ST<T>::ID == FRNN_BF16 ? 0x7fc0u : 0x7e00u)));
      so[(((size_t)k * a.B + b) * a.count + c) * ND + nd] = v;
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    const int old = __hip_atomic_fetch_add(ctrl + MB_SEQ, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if ((old + 1) % (int)gridDim.x == 0)  // the last workgroup of this launch: every other one has read MB_TOK
      __hip_atomic_store(ctrl + MB_TOK, tok0 + a.count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// one word of the control block written from a stream (the stop word)
static __global__ void decode_ctrl_store_kernel(int* word, int value) {
  if (threadIdx.x == 0 && blockIdx.x == 0) __hip_atomic_store(word, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}


// Probe for frnn_streams_overlap: waits, bounded, for word 0 to become non-zero; word 1 = 1 if it did, 2 if not
static __global__ void overlap_spin_kernel(int* words, int limit) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  int seen = 2;
  for (int i = 0; i < limit; ++i) {
    if (__hip_atomic_load(words, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) { seen = 1; break; }
    __builtin_amdgcn_s_sleep(8);
  }
  __hip_atomic_store(words + 1, seen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace frnn
