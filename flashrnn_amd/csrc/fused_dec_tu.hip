// One translation unit per (function, storage type): instantiates the resident decode kernel, i.e. the fused
// forward kernel in mailbox mode (4-row batch tiles), for every forward tiling in the plan table.
// Build with -DFRNN_F=<0..3> -DFRNN_DT=<0|1|2>.
#include "frnn_fused_fwd.h"
#include "frnn_launch.h"

namespace frnn {

template <>
int fused_dec_launch<FRNN_F, FRNN_DT>(const Plan& p, const FwdArgs& a, hipStream_t st) {
  const dim3 grid(grid_for(a.groups, p.kw));
#define FRNN_CASE(Dv, VAR, W, U, K, MTR)                                                     \
  if (p.D == Dv && p.waves == W && p.utw == U && p.kw == K) {                                 \
    hipLaunchKernelGGL((fused_fwd_kernel<FRNN_F, FRNN_TU_T, Dv, W, U, K, 4, true>), grid, dim3(W * 64), 0, st, a); \
    return (int)hipGetLastError();                                                            \
  }
  FRNN_TU_PLANS(FRNN_CASE)
#undef FRNN_CASE
  return FRNN_E_UNSUPPORTED;
}

}  // namespace frnn
