// One translation unit per (function, storage type): instantiates the fused backward kernel for
// every tiling in the plan table.  Build with -DFRNN_F=<0..3> -DFRNN_DT=<0|1|2>.
#include "frnn_fused_bwd.h"
#include "frnn_launch.h"

namespace frnn {

// the kernel for a tile height, or null if the tiling is not compiled that tall (a template, so that the
// taller kernels of such a tiling are never instantiated)
template <int Dv, int W, int U, int K, int MTR, bool RCV> static void (*bwd_kernel_for(int tile_rows, bool pst))(const BwdArgs) {
  if constexpr (bwd_producer_stores(Cell<FRNN_F>::GR, Cell<FRNN_F>::NC, Dv, W, U, K, 4, (int)sizeof(FRNN_TU_T), RCV)) {
    if (tile_rows == 4 && pst) return fused_bwd_kernel<FRNN_F, FRNN_TU_T, Dv, W, U, K, 4, RCV, true>;
  }
  if (tile_rows == 4) return fused_bwd_kernel<FRNN_F, FRNN_TU_T, Dv, W, U, K, 4, RCV>;
  if constexpr (MTR >= 8) { if (tile_rows == 8) return fused_bwd_kernel<FRNN_F, FRNN_TU_T, Dv, W, U, K, 8, RCV>; }
  if constexpr (MTR >= 16) { if (tile_rows == 16) return fused_bwd_kernel<FRNN_F, FRNN_TU_T, Dv, W, U, K, 16, RCV>; }
  return nullptr;
}

template <>
int fused_bwd_launch<FRNN_F, FRNN_DT>(const Plan& p, const BwdArgs& a, hipStream_t st) {
  const dim3 grid(grid_for(a.groups, p.kw));
  const bool rc = p.recompute != 0;
  // (one more wave and its hand-over buffers where the kernel has a producer wave: the same predicate as in the kernel)
  const bool pw = bwd_producer_wave(Cell<FRNN_F>::GR, Cell<FRNN_F>::NC, p.D, p.waves, p.utw, p.kw, a.tile_rows, (int)sizeof(FRNN_TU_T), rc);
  const bool pst = a.pst && !a.cut && bwd_producer_stores(Cell<FRNN_F>::GR, Cell<FRNN_F>::NC, p.D, p.waves, p.utw, p.kw, a.tile_rows, (int)sizeof(FRNN_TU_T), rc);  // (the truncated scan has no barrier per step to hand over at)
  // (wave pairs that split the destinations keep every fragment in registers: the two dg buffers only)
  const bool ds16 = sizeof(FRNN_TU_T) == 2 && bwd_dest_split(Cell<FRNN_F>::GR, p.D, p.waves, p.utw, p.kw, a.tile_rows, (int)sizeof(FRNN_TU_T), rc) > 1;
  const size_t lds = (ds16 ? (size_t)2 * 16 * Cell<FRNN_F>::GR * (p.D / p.kw) * sizeof(FRNN_TU_T)
                           : bwd_lds_bytes(Cell<FRNN_F>::GR, p.D, p.waves, p.utw, p.kw, (int)sizeof(FRNN_TU_T), rc)) + 16 +
                     (pw ? bwd_producer_bytes(Cell<FRNN_F>::NC + (cache_carried_state(FRNN_F, (int)sizeof(FRNN_TU_T), p.D) >= 0 ? 1 : 0), Cell<FRNN_F>::S, p.waves * p.utw, a.tile_rows, (int)sizeof(FRNN_TU_T)) : 0) +
                     (pst ? bwd_producer_store_bytes(Cell<FRNN_F>::GW, FRNN_F == FRNN_GRU, p.D, a.tile_rows, (int)sizeof(FRNN_TU_T)) : 0);
#define FRNN_CASE_(RCV, Dv, VAR, W, U, K, MTR)                                                          \
  if (rc == RCV && p.D == Dv && p.waves == W && p.utw == U && p.kw == K) {                               \
    auto kern = bwd_kernel_for<Dv, W, U, K, MTR, RCV>(a.tile_rows, pst);                                      \
    if (!kern) return FRNN_E_UNSUPPORTED;                                                                \
    if (lds > 65536) {                                                                                   \
      hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
      if (e != hipSuccess) return (int)e;                                                                \
    }                                                                                                    \
    if (K > 1 && p.cooperative) { /* see fused_fwd_tu.hip */                                             \
      BwdArgs aa = a;                                                                                    \
      void* args[] = {(void*)&aa};                                                                       \
      return (int)hipLaunchCooperativeKernel((const void*)kern, grid, dim3((W + (pw ? 1 : 0)) * 64), args, lds, st);      \
    }                                                                                                    \
    hipLaunchKernelGGL(kern, grid, dim3((W + (pw ? 1 : 0)) * 64), lds, st, a);                                            \
    return (int)hipGetLastError();                                                                       \
  }
#define FRNN_CASE(Dv, VAR, W, U, K, MTR) FRNN_CASE_(false, Dv, VAR, W, U, K, MTR)
#define FRNN_CASE_RC(Dv, VAR, W, U, K, MTR) FRNN_CASE_(true, Dv, VAR, W, U, K, MTR)
  FRNN_TU_BWD_PLANS(FRNN_CASE)
  FRNN_TU_BWD_RC_PLANS(FRNN_CASE_RC)
#undef FRNN_CASE
#undef FRNN_CASE_RC
#undef FRNN_CASE_
  return FRNN_E_UNSUPPORTED;
}

}  // namespace frnn
