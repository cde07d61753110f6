// Host-side declarations of the alternating backend (frnn_alt.hip).
#pragma once
#include "frnn_common.h"
#include "frnn_fused_fwd.h"  // load_frag
#include "frnn_grad.h"

namespace frnn {

struct AltProblem {
  int function, dtype, B, T, N, D, training; float h_clip, g_clip; int cut;
  int use_carry;  // forward: the first step takes its state from the fp32 side buffer, not from s0 (single-step calls)
};

struct AltFwdBuffers {
  const void* Wx; const void* R; const void* b; const void* s0;
  void* states; void* cache;
  float* sfp;  // [S][B][N][D] fp32 running state; may be null for a single step without carry
};

struct AltBwdBuffers {
  const void* Rt; const void* s0; const void* states; const void* cache; const void* dstates;
  void* dWx; void* dgx; void* ds0;
  void* dg;    // 2 x [B][N][G_r*D] storage type (steps of even / odd index)
  float* dsr;  // [S][B][N][D]
};

int alt_forward(const AltProblem& p, const AltFwdBuffers& bf, hipStream_t st);
int alt_backward_scan(const AltProblem& p, const AltBwdBuffers& bf, hipStream_t st);
int launch_bias_partial(int dtype, const void* const* src, const long* ld, int GT, int N, int D, long rows, int splits,
                        float* part, hipStream_t st);

}  // namespace frnn
