// Declarations shared between the per-(function, dtype) kernel translation units and the API.
#pragma once
#include "frnn_common.h"
#include "frnn_plan.h"

namespace frnn {

struct FwdArgs;
struct BwdArgs;

// Each is defined in exactly one translation unit (fused_fwd_tu.hip / fused_bwd_tu.hip compiled
// with -DFRNN_F=<function> -DFRNN_DT=<dtype>).  Return: hipError_t, or FRNN_E_UNSUPPORTED if the
// plan is not compiled in.
template <int F, int DT> int fused_fwd_launch(const Plan& p, const FwdArgs& a, hipStream_t st);
template <int F, int DT> int fused_bwd_launch(const Plan& p, const BwdArgs& a, hipStream_t st);
// the forward kernel as a resident decode kernel (mailbox mode, 4-row tiles): fused_dec_tu.hip, functions 0..3
template <int F, int DT> int fused_dec_launch(const Plan& p, const FwdArgs& a, hipStream_t st);

// plan table lookup: function, dtype, D, variant -> plan; false if none.
// backward: 0 forward, 1 reverse scan with gate cache, 2 reverse scan in recompute mode
bool find_plan(int function, int dtype, int D, int variant, int backward, Plan* out);

}  // namespace frnn

#if defined(FRNN_F) && defined(FRNN_DT)
#if FRNN_DT == 0
#define FRNN_TU_T frnn::bf16_t
#elif FRNN_DT == 2
#define FRNN_TU_T frnn::half_t
#else
#define FRNN_TU_T float
#endif
#if FRNN_F == 0 || FRNN_F == 1
#if FRNN_DT != 1 && FRNN_F == 1
#define FRNN_TU_BWD_RC_PLANS FRNN_BWD_RC_PLANS_SLSTM_BF16
#elif FRNN_DT != 1
#define FRNN_TU_BWD_RC_PLANS FRNN_BWD_RC_PLANS_GR4_BF16
#else
#define FRNN_TU_BWD_RC_PLANS FRNN_BWD_RC_PLANS_GR4_F32
#endif
#elif FRNN_F == 2
#if FRNN_DT != 1
#define FRNN_TU_BWD_RC_PLANS FRNN_BWD_RC_PLANS_GR3_BF16
#else
#define FRNN_TU_BWD_RC_PLANS FRNN_BWD_RC_PLANS_GR3_F32
#endif
#else
#define FRNN_TU_BWD_RC_PLANS FRNN_BWD_RC_PLANS_NONE
#endif
#if FRNN_F == 0 || FRNN_F == 1
#if FRNN_DT != 1 && FRNN_F == 1
#define FRNN_TU_PLANS FRNN_PLANS_SLSTM_BF16
#define FRNN_TU_BWD_PLANS FRNN_BWD_PLANS_SLSTM_BF16
#elif FRNN_DT != 1
#define FRNN_TU_PLANS FRNN_PLANS_GR4_BF16
#define FRNN_TU_BWD_PLANS FRNN_BWD_PLANS_GR4_BF16
#elif FRNN_F == 1
#define FRNN_TU_PLANS FRNN_PLANS_GR4_F32
#define FRNN_TU_BWD_PLANS FRNN_BWD_PLANS_SLSTM_F32
#else
#define FRNN_TU_PLANS FRNN_PLANS_GR4_F32
#define FRNN_TU_BWD_PLANS FRNN_BWD_PLANS_GR4_F32
#endif
#elif FRNN_F == 2
#if FRNN_DT != 1
#define FRNN_TU_PLANS FRNN_PLANS_GR3_BF16
#define FRNN_TU_BWD_PLANS FRNN_BWD_PLANS_GR3_BF16
#else
#define FRNN_TU_PLANS FRNN_PLANS_GR3_F32
#define FRNN_TU_BWD_PLANS FRNN_BWD_PLANS_GR3_F32
#endif
#else
#if FRNN_DT != 1
#define FRNN_TU_PLANS FRNN_PLANS_GR1_BF16
#define FRNN_TU_BWD_PLANS FRNN_BWD_PLANS_GR1_BF16
#else
#define FRNN_TU_PLANS FRNN_PLANS_GR1_F32
#define FRNN_TU_BWD_PLANS FRNN_BWD_PLANS_GR1_F32
#endif
#endif
#endif
