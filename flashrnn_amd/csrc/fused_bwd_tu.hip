// One translation unit per (function, storage type): instantiates the fused backward kernel for
// every tiling in the plan table.  Build with -DFRNN_F=<0..3> -DFRNN_DT=<0|1|2>.
#include "frnn_fused_bwd.h"
#include "frnn_launch.h"

namespace frnn {

template <>
int fused_bwd_launch<FRNN_F, FRNN_DT>(const Plan& p, const BwdArgs& a, hipStream_t st) {
  const dim3 grid(grid_for(a.groups, p.kw));
  const bool rc = p.recompute != 0;
  const size_t lds = bwd_lds_bytes(Cell<FRNN_F>::GR, p.D, p.waves, p.utw, p.kw, (int)sizeof(FRNN_TU_T), rc) + 16;
#define FRNN_CASE_(RCV, Dv, VAR, W, U, K)                                                               \
  if (rc == RCV && p.D == Dv && p.waves == W && p.utw == U && p.kw == K) {                               \
    auto kern = a.tile_rows == 4 ? fused_bwd_kernel<FRNN_F, FRNN_TU_T, Dv, W, U, K, 4, RCV>              \
              : a.tile_rows == 8 ? fused_bwd_kernel<FRNN_F, FRNN_TU_T, Dv, W, U, K, 8, RCV>              \
                                 : fused_bwd_kernel<FRNN_F, FRNN_TU_T, Dv, W, U, K, 16, RCV>;            \
    if (lds > 65536) {                                                                                   \
      hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
      if (e != hipSuccess) return (int)e;                                                                \
    }                                                                                                    \
    if (K > 1 && p.cooperative) { /* see fused_fwd_tu.hip */                                             \
      BwdArgs aa = a;                                                                                    \
      void* args[] = {(void*)&aa};                                                                       \
      return (int)hipLaunchCooperativeKernel((const void*)kern, grid, dim3(W * 64), args, lds, st);      \
    }                                                                                                    \
    hipLaunchKernelGGL(kern, grid, dim3(W * 64), lds, st, a);                                            \
    return (int)hipGetLastError();                                                                       \
  }
#define FRNN_CASE(Dv, VAR, W, U, K) FRNN_CASE_(false, Dv, VAR, W, U, K)
#define FRNN_CASE_RC(Dv, VAR, W, U, K) FRNN_CASE_(true, Dv, VAR, W, U, K)
  FRNN_TU_BWD_PLANS(FRNN_CASE)
  FRNN_TU_BWD_RC_PLANS(FRNN_CASE_RC)
#undef FRNN_CASE
#undef FRNN_CASE_RC
#undef FRNN_CASE_
  return FRNN_E_UNSUPPORTED;
}

}  // namespace frnn
