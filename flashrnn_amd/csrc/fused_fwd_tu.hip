// One translation unit per (function, storage type): instantiates the fused forward kernel for
// every tiling in the plan table.  Build with -DFRNN_F=<0..3> -DFRNN_DT=<0|1|2>.
// A plan marked cooperative launches kernels whose workgroups wait for each other (K > 1) as
// cooperative kernels: the runtime then checks that the grid fits the device and runs one such
// kernel at a time, which makes calls that overlap on different streams safe (about 15 us per launch).
#include "frnn_fused_fwd.h"
#include "frnn_launch.h"

namespace frnn {

template <>
int fused_fwd_launch<FRNN_F, FRNN_DT>(const Plan& p, const FwdArgs& a, hipStream_t st) {
  const dim3 grid(grid_for(a.groups, p.kw));
#define FRNN_CASE(Dv, VAR, W, U, K)                                                          \
  if (p.D == Dv && p.waves == W && p.utw == U && p.kw == K) {                                 \
    auto kern = a.tile_rows == 4 ? fused_fwd_kernel<FRNN_F, FRNN_TU_T, Dv, W, U, K, 4>                       \
              : a.tile_rows == 8 ? fused_fwd_kernel<FRNN_F, FRNN_TU_T, Dv, W, U, K, 8>                       \
                                 : fused_fwd_kernel<FRNN_F, FRNN_TU_T, Dv, W, U, K, 16>;                     \
    if (K > 1 && p.cooperative) {                                                             \
      FwdArgs aa = a;                                                                         \
      void* args[] = {(void*)&aa};                                                            \
      return (int)hipLaunchCooperativeKernel((const void*)kern, grid, dim3(W * 64), args, 0, st); \
    }                                                                                         \
    hipLaunchKernelGGL(kern, grid, dim3(W * 64), 0, st, a);                                   \
    return (int)hipGetLastError();                                                            \
  }
  FRNN_TU_PLANS(FRNN_CASE)
#undef FRNN_CASE
  return FRNN_E_UNSUPPORTED;
}

}  // namespace frnn
