// Host-side declarations of the weight-gradient kernels (frnn_grad_gemm.hip).
#pragma once
#include "frnn_common.h"

namespace frnn {

struct GradGemmArgs {
  const void* gsrc[4];   // per recurrent gate g: cotangent of its pre-activation; element
                         // (row r = b*T + t, head n, unit d) at gsrc[g] + r*gld[g] + n*D + d
  long gld[4];           // row strides in elements
  const void* states_h;  // h of all steps, [B,T,N,D] (state 0 of the states tensor)
  const void* s0_h;      // initial h, [B,N,D]
  float* part;           // [splits][G_r][N][D][D] partial sums
  int B, T, N, D, GR;
  int rows_per_split;    // filled in by launch_grad_gemm
};

int launch_transpose_r(int dtype, const void* R, void* Rt, int N, int D, int GR, hipStream_t st);
int grad_gemm_splits(int dtype, int B, int T, int N, int D, int GR);
int launch_grad_gemm(int dtype, GradGemmArgs a, int splits, hipStream_t st);
int launch_grad_reduce(const float* part_r, int splits_r, size_t n_r, float* dR,
                       const float* part_b, int splits_b, size_t n_b, float* db, hipStream_t st);
int launch_fill_zero(void* p, size_t bytes, hipStream_t st);

}  // namespace frnn
