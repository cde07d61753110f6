// Moving the per-step vector to every wave that needs it as an MFMA operand, and the lane
// ownership of the MFMA result.
//
// Within one workgroup the vector (h_{t-1} forward, the own dg_t backward) lives in LDS in MFMA
// fragment order, so a lane's operand for k-step ks is one contiguous read at (ks*64 + lane).
// Between the KW workgroups of one head data travels through small global buffers of tagged
// words: the producer's store carries data and step tag together, the consumer polls the words
// it needs until the tag matches.  That costs one trip through the coherent memory path instead
// of the store -> fence -> flag -> poll -> fence -> load chain of a flag barrier.  Two slots
// alternate by step parity: a workgroup can only write step t+2 after it has read all of step
// t+1, which every workgroup wrote only after reading step t, so slot (t & 1) is never
// overwritten while still in use.  Accesses are agent scope: workgroup-scope loads are served
// from the per-CU L1 and never see another compute unit's store (measured).  One all-to-all step
// between 4 workgroups costs ~1700 cycles when they share an XCD and ~2300 when they do not
// (measured), which is why the launch maps the workgroups of a head to one XCD.
//
// Ownership.  The 16x16 MFMA result gives lane l the 4 rows 4*(l/16)..+3 of column l%16, i.e.
// (with A = weight rows, B = streamed vector) 4 consecutive units of batch row l%16.
//   16-row tiles: a lane keeps its 4 elements.
//   8-row tiles: columns 8..15 are padding, so lanes 8..15 of every 16-lane row take elements
//   2,3 of the lane 8 below them (one DPP move each) and every lane does the gate math of 2
//   elements instead of 4.
//   4-row tiles: one more DPP move (row_shr:4) leaves one element per lane.
#pragma once
#include "frnn_common.h"

namespace frnn {

template <int TR> struct Own {  // TR = batch rows per tile: 16, 8 or 4
  static_assert(TR == 16 || TR == 8 || TR == 4, "tile rows");
  static constexpr int E = TR / 4;  // elements per lane per 16-unit tile
  static __device__ __forceinline__ int row(int r16) { return r16 & (TR - 1); }                   // batch row in the tile
  static __device__ __forceinline__ int sub(int r16, int q4) { return q4 * 4 + E * (r16 / TR); }  // first unit in the tile
};

// lanes 0..7 of a 16-lane row keep `lo`, lanes 8..15 receive `hi` of the lane 8 below (row_shr:8)
__device__ __forceinline__ float half_pick(float lo, float hi) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, lo), __builtin_bit_cast(int, hi),
                                                              0x118, 0xF, 0xC, false));
}
// lanes 0..3 and 8..11 keep `lo`, lanes 4..7 and 12..15 receive `hi` of the lane 4 below (row_shr:4)
__device__ __forceinline__ float quarter_pick(float lo, float hi) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, lo), __builtin_bit_cast(int, hi),
                                                              0x114, 0xF, 0xA, false));
}
template <int TR> __device__ __forceinline__ void own_elems(const f32x4& acc, float* out) {
  if constexpr (TR == 16) { out[0] = acc[0]; out[1] = acc[1]; out[2] = acc[2]; out[3] = acc[3]; }
  else if constexpr (TR == 8) { out[0] = half_pick(acc[0], acc[2]); out[1] = half_pick(acc[1], acc[3]); }
  else { out[0] = quarter_pick(half_pick(acc[0], acc[2]), half_pick(acc[1], acc[3])); }
}

// fp32 vector of a 4-row tile as the broadcast operand of v_mfma_f32_4x4x1_16B_f32: element (row, k) at
// k*4 + row, so that lane l reads the operand of the 16 k-values 16v .. 16v+15 with one access at 64v + l
__device__ __forceinline__ int lds_index4(int row, int k) { return k * 4 + row; }
// the same from the element's position in an exchange slot (fp32 fragment order, ST<float>::frag_elem)
__device__ __forceinline__ int lds_index4_of_word(int word) { return (((word >> 6) << 2) + ((word >> 4) & 3)) * 4 + (word & 15); }

// 4x4 transpose between the lanes of a quad and 4 registers: lane j of a quad passes r[i] = M[j][i] and
// gets r[i] = M[i][j] (two butterfly steps: partner lane ^ 1 with registers (0,1), (2,3), then lane ^ 2 with
// (0,2), (1,3))
__device__ __forceinline__ float quad_xor1(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1 /* quad_perm:[1,0,3,2] */, 0xF, 0xF, false));
}
__device__ __forceinline__ float quad_xor2(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E /* quad_perm:[2,3,0,1] */, 0xF, 0xF, false));
}
__device__ __forceinline__ void quad_transpose(float (&r)[4], int lane) {
  const bool b0 = lane & 1, b1 = lane & 2;
  {
    const float x0 = quad_xor1(b0 ? r[0] : r[1]), x1 = quad_xor1(b0 ? r[2] : r[3]);
    r[0] = b0 ? x0 : r[0]; r[1] = b0 ? r[1] : x0;
    r[2] = b0 ? x1 : r[2]; r[3] = b0 ? r[3] : x1;
  }
  {
    const float x0 = quad_xor2(b1 ? r[0] : r[2]), x1 = quad_xor2(b1 ? r[1] : r[3]);
    r[0] = b1 ? x0 : r[0]; r[2] = b1 ? r[2] : x0;
    r[1] = b1 ? x1 : r[1]; r[3] = b1 ? r[3] : x1;
  }
}

// LDS writes of E consecutive elements (row, k0..k0+E-1) in fragment order; k0 % E == 0
template <int E, typename T> __device__ __forceinline__ void lds_write16(T* buf, int row, int k0, const float* v) {
  const Dw<(E + 1) / 2> p = pack16<E, T>(v);
  unsigned* dst = reinterpret_cast<unsigned*>(buf + ST16::frag_elem(row, k0));
  if constexpr (E == 4) *reinterpret_cast<uint2*>(dst) = make_uint2(p.v[0], p.v[1]);
  else if constexpr (E == 2) dst[0] = p.v[0];
  else *reinterpret_cast<unsigned short*>(dst) = (unsigned short)p.v[0];
}
template <int E> __device__ __forceinline__ void lds_write(bf16_t* buf, int row, int k0, const float* v) { lds_write16<E>(buf, row, k0, v); }
template <int E> __device__ __forceinline__ void lds_write(half_t* buf, int row, int k0, const float* v) { lds_write16<E>(buf, row, k0, v); }
template <int E> __device__ __forceinline__ void lds_write(float* buf, int row, int k0, const float* v) {
#pragma unroll
  for (int i = 0; i < E; ++i) buf[ST<float>::frag_elem(row, k0 + i)] = v[i];
}

// tagged global stores of E consecutive elements (row, k0..) for step t into the slot that starts `slot_off`
// bytes behind `base` (base uniform; near: see ll_store_sel)
template <int E, typename T> __device__ __forceinline__ void ll_write16(const void* base, unsigned slot_off, int row, int k0, const float* v, int t, u64 near) {
  if constexpr (E == 1) {  // one 32-bit tagged half of a word; the other half belongs to another lane
    const unsigned wv[1] = {(tag16(t) << 16) | (H16<T>::pack2(v[0], 0.f) & 0xffffu)};
    ll_store_sel<1, 0>(base, slot_off + (unsigned)ST16::frag_elem(row, k0) * 4u, wv, near);
  } else {
    u64 wv[E / 2];
#pragma unroll
    for (int k = 0; k < E / 2; ++k) wv[k] = ll_pack16<T>(v[2 * k], v[2 * k + 1], t);
    ll_store_sel<E / 2, 8>(base, slot_off + (unsigned)(ST16::frag_elem(row, k0) >> 1) * 8u, wv, near);
  }
}
template <int E> __device__ __forceinline__ void ll_write(bf16_t*, const void* base, unsigned slot_off, int row, int k0, const float* v, int t, u64 near) { ll_write16<E, bf16_t>(base, slot_off, row, k0, v, t, near); }
template <int E> __device__ __forceinline__ void ll_write(half_t*, const void* base, unsigned slot_off, int row, int k0, const float* v, int t, u64 near) { ll_write16<E, half_t>(base, slot_off, row, k0, v, t, near); }
template <int E> __device__ __forceinline__ void ll_write(float*, const void* base, unsigned slot_off, int row, int k0, const float* v, int t, u64 near) {
  // (k0 is a multiple of E <= 4: the E elements sit in one group of 4 k, 16 words apart)
  u64 wv[E];
#pragma unroll
  for (int i = 0; i < E; ++i) wv[i] = ll_pack((float*)0, v[i], t);
  ll_store_sel<E, 128>(base, slot_off + (unsigned)ST<float>::frag_elem(row, k0) * 8u, wv, near);
}

// Do the KW workgroups of one group run on one XCD?  The launch places them on workgroup ids that are congruent
// mod 8, which the dispatcher hands to one XCD; this handshake checks it where it matters, once per launch: every
// workgroup publishes the id of its XCD (agent scope, visible anywhere) in the group's `words` (KW of them, zero at
// launch) and waits, bounded, for the others.  Called by the first wave of the workgroup; returns 1 if all ids
// agree (workgroup-scope exchange stores are then seen by the whole group), 0 if not, -1 if the wait ran out.
template <int KW>
__device__ __forceinline__ int xcd_handshake(int* words, int slice, int lane, int* status, int spin_limit) {
  static_assert(KW <= 64, "one lane per workgroup of the group");
  if (spin_limit < -1) return -1;  // host-side test hook: every wait gives up at once
  unsigned x;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(x));
  const int mine = (int)(x & 15u) + 1;
  if (lane == 0) __hip_atomic_store(words + slice, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  int v = mine;
  for (int spins = 0;; ++spins) {
    if (lane < KW) v = __hip_atomic_load(words + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (__all(v != 0)) break;
    if (spins > spin_limit) return -1;
    if ((spins & 63) == 63 &&
        __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != STATUS_OK) return -1;
  }
  return __all(v == mine) ? 1 : 0;
}

// The words thread `tid` of NT polls, for a [rows_valid x KDIM] vector without the `own` columns
// starting at `own0` (the workgroup's own slice, which it has in LDS already); -1 = none.
// PAIRS: entries 2j and 2j+1 of a thread are two adjacent words (16 bytes, fetched with one load).
template <typename T, int NP, int NT, bool PAIRS = false>
__device__ __forceinline__ void ll_plan(int tid, int rows_valid, int kdim, int own0, int own, int* q) {
  constexpr int CG = ST<T>::EPW == 2 ? 8 : 1;  // columns per enumerated group (bf16/f16: 4 words of 2)
  static_assert(!PAIRS || (ST<T>::EPW == 2 && NP % 2 == 0), "pairs: 16-bit types, an even number of words");
  const int tot = rows_valid * (kdim - own) / ST<T>::EPW;
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int qc = PAIRS ? 2 * tid + (i & 1) + (i >> 1) * 2 * NT : tid + i * NT;
    int r = qc, word;
    if (ST<T>::EPW == 2) {
      const int jj = r & 3; r >>= 2;
      const int b = r % rows_valid; r /= rows_valid;
      if (r >= own0 / CG) r += own / CG;
      word = (((r >> 2) * 64 + (r & 3) * 16 + b) << 2) + jj;
    } else {
      const int b = r % rows_valid; r /= rows_valid;
      if (r >= own0 / CG) r += own / CG;
      word = (r >> 2) * 64 + (r & 3) * 16 + b;
    }
    q[i] = qc < tot ? word : -1;
  }
}

// Poll NW tagged words (addresses base + off[i]; every lane polls NW words, lanes or entries
// with nothing to wait for pass need[i] = false and may point anywhere valid) until all carry the
// tag of step t.  Loads are unconditional and the exit test is a wave vote.  Returns true if the
// bounded wait ran out (or another workgroup already reported that).
template <typename TAG, int NW, int PD>
__device__ __forceinline__ bool poll_words(const u64* base, const int* off, const bool* need, int t, u64* out,
                                           int* status, int spin_limit, int first_delay) {
  static_assert(PD == 1, "one probe of the set in flight: more only add congestion (measured again with exact waits)");
  // the producers finish their step at about the same time as this wave: a probe sent at once
  // reaches memory before their stores and costs a whole extra round trip
  if (spin_limit < -1) return true;  // host-side test hook: every wait gives up at once
  for (int i = 0; i < first_delay; ++i) __builtin_amdgcn_s_sleep(1);
  for (int spins = 0;; ++spins) {
#pragma unroll
    for (int i = 0; i < NW; ++i) out[i] = ll_load(base + off[i]);
    // straight-line test of the whole set (bitwise, no short circuit: a short-circuit && turns into
    // a chain of divergent branches with a wait inside each)
    bool ok = true;
#pragma unroll
    for (int i = 0; i < NW; ++i) ok = ok & (!need[i] | ll_ok((TAG*)0, out[i], t));
    if (__all(ok)) return false;
    if (spins > spin_limit) return true;
    if ((spins & 63) == 63 &&
        __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != STATUS_OK) return true;
  }
}

// The same wait with a short-circuit test: the words are examined in the order their loads return
// and the first missing one sends the next probe at once, while the tail of the last one is still
// in flight.  Measured 3 % faster than the straight-line form for the 3-word sets of the backward
// exchange (and 4 % slower for the 2-word sets of the forward one).
template <typename TAG, int NW, typename W>
__device__ __forceinline__ bool poll_words_staggered(const W* base, const int* off, const bool* need, int t, W* out,
                                                     int* status, int spin_limit, int first_delay) {
  if (spin_limit < -1) return true;  // host-side test hook: every wait gives up at once
  for (int i = 0; i < first_delay; ++i) __builtin_amdgcn_s_sleep(1);
  W v[NW];
#pragma unroll
  for (int i = 0; i < NW; ++i) v[i] = ll_load(base + off[i]);
  for (int spins = 0;; ++spins) {
    bool ok = true;
#pragma unroll
    for (int i = 0; i < NW; ++i) ok = ok && (!need[i] || ll_ok((TAG*)0, v[i], t));
    if (__all(ok)) {
#pragma unroll
      for (int i = 0; i < NW; ++i) out[i] = v[i];
      return false;
    }
#pragma unroll
    for (int i = 0; i < NW; ++i) v[i] = ll_load(base + off[i]);
    if (spins > spin_limit) return true;
    if ((spins & 63) == 63 &&
        __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != STATUS_OK) return true;
  }
}
// The same wait in two halves: the first probe is sent by poll_issue, the caller does work that needs no
// memory result, poll_finish examines the probe and carries on probing as above.  A probe takes ~900 cycles to
// come back whether or not the words have arrived; work placed between the halves hides behind that trip.
template <int NW, typename W>
__device__ __forceinline__ void poll_issue(const W* base, const int* off, W* v) {
#pragma unroll
  for (int i = 0; i < NW; ++i) v[i] = ll_load(base + off[i]);
}
template <typename TAG, int NW, typename W>
__device__ __forceinline__ bool poll_finish(const W* base, const int* off, const bool* need, int t, W* v, W* out,
                                            int* status, int spin_limit) {
  if (spin_limit < -1) return true;  // host-side test hook: every wait gives up at once
  for (int spins = 0;; ++spins) {
    bool ok = true;
#pragma unroll
    for (int i = 0; i < NW; ++i) ok = ok && (!need[i] || ll_ok((TAG*)0, v[i], t));
    if (__all(ok)) {
#pragma unroll
      for (int i = 0; i < NW; ++i) out[i] = v[i];
      return false;
    }
#pragma unroll
    for (int i = 0; i < NW; ++i) v[i] = ll_load(base + off[i]);
    if (spins > spin_limit) return true;
    if ((spins & 63) == 63 &&
        __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != STATUS_OK) return true;
  }
}
constexpr int probe_depth(int) { return 1; }

// The same wait for pairs of adjacent words, each pair fetched with one 16-byte agent-scope load
// (raw buffer load, cache policy sc1): half the memory instructions per probe.  A 16-byte load is
// not one atomic access, which the protocol does not need: every 32-bit half carries its own tag.
template <typename TAG, int NW>
__device__ __forceinline__ bool poll_pairs(rsrc_t slot, unsigned soff, const int* off, const bool* need, int t, u64* out,
                                           int* status, int spin_limit, int first_delay) {
  static_assert(NW % 2 == 0, "pairs");
  if (spin_limit < -1) return true;  // host-side test hook: every wait gives up at once
  for (int i = 0; i < first_delay; ++i) __builtin_amdgcn_s_sleep(1);
  for (int spins = 0;; ++spins) {
#pragma unroll
    for (int i = 0; i < NW; i += 2) {
      const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(slot, (unsigned)off[i] * 8u, soff, 16 /* sc1 */);
      out[i] = (u64)v.x | ((u64)v.y << 32);
      out[i + 1] = (u64)v.z | ((u64)v.w << 32);
    }
    bool ok = true;
#pragma unroll
    for (int i = 0; i < NW; ++i) ok = ok & (!need[i] | ll_ok((TAG*)0, out[i], t));
    if (__all(ok)) return false;
    if (spins > spin_limit) return true;
    if ((spins & 63) == 63 &&
        __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != STATUS_OK) return true;
  }
}
// Word `off` of a vector of `tot` words in an LDS copy that starts `rot` words into the vector and wraps around
// (tot = 0: no rotation)
__device__ __forceinline__ unsigned lds_rotated(int off, int rot, int tot) {
  const unsigned d = (unsigned)(off - rot);
  return tot ? min(d, d + (unsigned)tot) : (unsigned)off;  // (off < rot: d wraps, d + tot is the index)
}
template <typename T, int NP>
__device__ __forceinline__ bool ll_gather_pairs(rsrc_t slots, unsigned soff, const int* q, int t, T* lds_dst,
                                                int* status, int spin_limit, int first_delay, int rot = 0, int tot = 0) {
  constexpr int CH = NP < 16 ? NP : 16;  // words polled together
  static_assert(NP % CH == 0 && CH % 2 == 0, "poll list must split into whole chunks of pairs");
  bool fail = false;
#pragma unroll
  for (int c0 = 0; c0 < NP; c0 += CH) {
    int off[CH]; bool need[CH]; u64 v[CH];
#pragma unroll
    for (int i = 0; i < CH; ++i) { need[i] = q[c0 + i] >= 0; off[i] = need[i] ? q[c0 + i] : 0; }
    fail = fail || poll_pairs<T, CH>(slots, soff, off, need, t, v, status, spin_limit, c0 == 0 ? first_delay : 0);
    if (!fail) {
      // (the list is a whole number of pairs: its length, rows x columns / 2, is even)
#pragma unroll
      for (int i = 0; i < CH; i += 2)
        if (need[i])
          *reinterpret_cast<uint2*>(reinterpret_cast<unsigned*>(lds_dst) + lds_rotated(off[i], rot, tot)) =
              make_uint2(ll_payload((T*)0, v[i]), ll_payload((T*)0, v[i + 1]));
    }
  }
  return fail;
}

// Forward gather: poll the planned words of slot, then copy their payloads to LDS.
// C4: the LDS vector is kept as [k][4 rows] (the fp32 4-row tiles, see lds_index4) instead of fragment order
template <typename T, int NP, bool C4 = false>
__device__ __forceinline__ bool ll_gather(const u64* slot, const int* q, int t, T* lds_dst,
                                          int* status, int spin_limit, int first_delay, int rot = 0, int tot = 0) {
  constexpr int CH = NP < 16 ? NP : 16;  // words polled together
  static_assert(NP % CH == 0, "poll list must split into whole chunks");
  bool fail = false;
#pragma unroll
  for (int c0 = 0; c0 < NP; c0 += CH) {
    int off[CH]; bool need[CH]; u64 v[CH];
#pragma unroll
    for (int i = 0; i < CH; ++i) { need[i] = q[c0 + i] >= 0; off[i] = need[i] ? q[c0 + i] : 0; }
    fail = fail || poll_words<T, CH, probe_depth(CH)>(slot, off, need, t, v, status, spin_limit, c0 == 0 ? first_delay : 0);
    if (!fail) {
#pragma unroll
      for (int i = 0; i < CH; ++i)
        if (need[i]) reinterpret_cast<unsigned*>(lds_dst)[C4 ? lds_index4_of_word(off[i]) : lds_rotated(off[i], rot, tot)] = ll_payload((T*)0, v[i]);
    }
  }
  return fail;
}

// Workgroup barrier that orders LDS accesses only.  __syncthreads() also waits for every global
// load and store the wave has in flight (s_waitcnt vmcnt(0)): inside the time loops that exposed
// the full HBM latency of the operand prefetch once per step (measured: ~1000 of 2200 cycles per
// reverse step at D = 64).  The steps exchange data between waves through LDS only (and between
// workgroups through the tagged words, which carry their own validity), so LDS order is all the
// barrier has to provide and the prefetches keep flying across it.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Workgroup barrier that also tells every wave whether any lane passed `fail`; `flag` is one LDS
// word that starts at 0 and is only ever set.  Costs one LDS read more than a plain barrier.
// The result is read back through readfirstlane so that the compiler knows it is wave-uniform
// and keeps the time-step counter (and every address derived from it) in scalar registers.
__device__ __forceinline__ bool barrier_or(bool fail, int* flag) {
  // an explicit LDS pointer: through a generic (or volatile) pointer the compiler emits a flat load,
  // which counts as a global access and drains every global load in flight before it returns
  typedef __attribute__((address_space(3))) int lds_int;
  lds_int* const f = (lds_int*)flag;
  if (fail) *f = 1;
  lds_barrier();  // also a compiler barrier: the read below is a fresh one
  return __builtin_amdgcn_readfirstlane(*f) != 0;
}

}  // namespace frnn
