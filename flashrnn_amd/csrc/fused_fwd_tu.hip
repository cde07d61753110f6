// One translation unit per (function, storage type): instantiates the fused forward kernel for
// every tiling in the plan table.  Build with -DFRNN_F=<0..3> -DFRNN_DT=<0|1|2>.
#include "frnn_fused_fwd.h"
#include "frnn_launch.h"

namespace frnn {

template <>
int fused_fwd_launch<FRNN_F, FRNN_DT>(const Plan& p, const FwdArgs& a, hipStream_t st) {
  const dim3 grid(grid_for(a.groups, p.kw));
#define FRNN_CASE(Dv, VAR, W, U, K)                                                          \
  if (p.D == Dv && p.waves == W && p.utw == U && p.kw == K) {                                 \
    if (a.tile_rows == 4) hipLaunchKernelGGL((fused_fwd_kernel<FRNN_F, FRNN_TU_T, Dv, W, U, K, 4>), grid, dim3(W * 64), 0, st, a);       \
    else if (a.tile_rows == 8) hipLaunchKernelGGL((fused_fwd_kernel<FRNN_F, FRNN_TU_T, Dv, W, U, K, 8>), grid, dim3(W * 64), 0, st, a);  \
    else hipLaunchKernelGGL((fused_fwd_kernel<FRNN_F, FRNN_TU_T, Dv, W, U, K, 16>), grid, dim3(W * 64), 0, st, a);                       \
    return (int)hipGetLastError();                                                            \
  }
  FRNN_TU_PLANS(FRNN_CASE)
#undef FRNN_CASE
  return FRNN_E_UNSUPPORTED;
}

}  // namespace frnn
