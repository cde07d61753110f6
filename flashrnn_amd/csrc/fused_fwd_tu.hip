// One translation unit per (function, storage type): instantiates the fused forward kernel for
// every tiling in the plan table.  Build with -DFRNN_F=<0..3> -DFRNN_DT=<0|1|2>.
// A plan marked cooperative launches kernels whose workgroups wait for each other (K > 1) as
// cooperative kernels: the runtime then checks that the grid fits the device and runs one such
// kernel at a time, which makes calls that overlap on different streams safe (about 15 us per launch).
#include "frnn_fused_fwd.h"
#include "frnn_launch.h"

namespace frnn {

// the kernel for a tile height, or null if the tiling is not compiled that tall (a template, so that the
// taller kernels of such a tiling are never instantiated)
template <int Dv, int W, int U, int K, int MTR> static void (*fwd_kernel_for(int tile_rows, int pst))(const FwdArgs) {
  if constexpr (fwd_producer_stores(Cell<FRNN_F>::GR, Dv, W, U, K, 4, (int)sizeof(FRNN_TU_T))) {
    if (tile_rows == 4 && pst) return fused_fwd_kernel<FRNN_F, FRNN_TU_T, Dv, W, U, K, 4, false, true>;
  }
  if (tile_rows == 4) return fused_fwd_kernel<FRNN_F, FRNN_TU_T, Dv, W, U, K, 4>;
  if constexpr (MTR >= 8) { if (tile_rows == 8) return fused_fwd_kernel<FRNN_F, FRNN_TU_T, Dv, W, U, K, 8>; }
  if constexpr (MTR >= 16) { if (tile_rows == 16) return fused_fwd_kernel<FRNN_F, FRNN_TU_T, Dv, W, U, K, 16>; }
  return nullptr;
}

template <>
int fused_fwd_launch<FRNN_F, FRNN_DT>(const Plan& p, const FwdArgs& a, hipStream_t st) {
  const dim3 grid(grid_for(a.groups, p.kw));
#define FRNN_CASE(Dv, VAR, W, U, K, MTR)                                                     \
  if (p.D == Dv && p.waves == W && p.utw == U && p.kw == K) {                                 \
    auto kern = fwd_kernel_for<Dv, W, U, K, MTR>(a.tile_rows, a.pst);                                \
    if (!kern) return FRNN_E_UNSUPPORTED;                                                     \
    /* (one more wave where the kernel has a producer wave: the same predicate as in the kernel) */ \
    const dim3 block((W + (fwd_producer_wave(Cell<FRNN_F>::GR, Dv, W, U, K, a.tile_rows, (int)sizeof(FRNN_TU_T)) ? 1 : 0)) * 64); \
    if (K > 1 && p.cooperative) {                                                             \
      FwdArgs aa = a;                                                                         \
      void* args[] = {(void*)&aa};                                                            \
      return (int)hipLaunchCooperativeKernel((const void*)kern, grid, block, args, 0, st);    \
    }                                                                                         \
    hipLaunchKernelGGL(kern, grid, block, 0, st, a);                                          \
    return (int)hipGetLastError();                                                            \
  }
  FRNN_TU_PLANS(FRNN_CASE)
#undef FRNN_CASE
  return FRNN_E_UNSUPPORTED;
}

}  // namespace frnn
