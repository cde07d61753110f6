// Moving the per-step vector (h_{t-1} forward, dg_t backward) to every wave that needs it
// as an MFMA operand.
//
// Within one workgroup the vector lives in LDS in MFMA fragment order, so a lane's operand
// for k-step ks is one contiguous read at (ks*64 + lane).  Between the KW workgroups of one
// head it travels through a small global buffer of tagged words: the producer's store carries
// data and step tag together, the consumer polls the words it needs until the tag matches and
// copies the payload to LDS.  That costs one L2 round trip instead of the store -> fence ->
// flag -> poll -> fence -> load chain of a flag barrier.  Two slots alternate by step parity:
// a workgroup can only write step t+2 after it has read all of step t+1, which every workgroup
// wrote only after reading step t, so slot (t & 1) is never overwritten while still in use.
#pragma once
#include "frnn_common.h"

namespace frnn {

// LDS writes of 4 consecutive elements (row, k0..k0+3), k0 % 4 == 0, in fragment order
__device__ __forceinline__ void lds_write4(bf16_t* buf, int row, int k0, const float* v) {
  uint2 p; pack4(v, p);
  *reinterpret_cast<uint2*>(buf + ST<bf16_t>::frag_elem(row, k0)) = p;
}
__device__ __forceinline__ void lds_write4(float* buf, int row, int k0, const float* v) {
#pragma unroll
  for (int i = 0; i < 4; ++i) buf[ST<float>::frag_elem(row, k0 + i)] = v[i];
}

// tagged global stores of 4 consecutive elements (row, k0..k0+3) for step t
__device__ __forceinline__ void ll_write4(bf16_t*, u64* slot, int row, int k0, const float* v, int t) {
  const int q = ST<bf16_t>::frag_elem(row, k0) >> 1;
  ll_store(slot + q, ll_pack((bf16_t*)0, v[0], v[1], t));
  ll_store(slot + q + 1, ll_pack((bf16_t*)0, v[2], v[3], t));
}
__device__ __forceinline__ void ll_write4(float*, u64* slot, int row, int k0, const float* v, int t) {
#pragma unroll
  for (int i = 0; i < 4; ++i) ll_store(slot + ST<float>::frag_elem(row, k0 + i), ll_pack((float*)0, v[i], t));
}

// The words thread `tid` of NT polls, for a [rows_valid x KDIM] vector; -1 = none.
template <typename T, int NP, int NT>
__device__ __forceinline__ void ll_plan(int tid, int rows_valid, int kdim, int* q) {
  const int tot = rows_valid * kdim / ST<T>::EPW;
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int qc = tid + i * NT;
    int r = qc, word;
    if (ST<T>::EPW == 2) {
      const int jj = r & 3; r >>= 2;
      const int b = r % rows_valid; r /= rows_valid;
      word = (((r >> 2) * 64 + (r & 3) * 16 + b) << 2) + jj;
    } else {
      const int b = r % rows_valid; r /= rows_valid;
      word = (r >> 2) * 64 + (r & 3) * 16 + b;
    }
    q[i] = qc < tot ? word : -1;
  }
}

// Poll until every planned word carries the tag of step t, then copy payloads to LDS.
// Returns true if the bounded wait ran out (or another workgroup already reported that).
template <typename T, int NP>
__device__ __forceinline__ bool ll_gather(const u64* slot, const int* q, int t, T* lds_dst,
                                          int* status, int spin_limit) {
  u64 v[NP];
#pragma unroll
  for (int i = 0; i < NP; ++i)
    if (q[i] >= 0) v[i] = ll_load(slot + q[i]);
  bool fail = false;
  for (int spins = 0;;) {
    bool ok = true;
#pragma unroll
    for (int i = 0; i < NP; ++i)
      if (q[i] >= 0 && !ll_ok((T*)0, v[i], t)) { ok = false; v[i] = ll_load(slot + q[i]); }
    if (ok) break;
    if (++spins > spin_limit) { fail = true; break; }
    if ((spins & 255) == 0 &&
        __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != STATUS_OK) { fail = true; break; }
  }
  if (!fail) {
#pragma unroll
    for (int i = 0; i < NP; ++i)
      if (q[i] >= 0) reinterpret_cast<unsigned*>(lds_dst)[q[i]] = ll_payload((T*)0, v[i]);
  }
  return fail;
}

}  // namespace frnn
