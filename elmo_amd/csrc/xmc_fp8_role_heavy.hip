// Second translation unit of the library: the variants of the fused step kernel whose tile loop, with the reference's
// Philox recipe inlined twelve times per step or with the compensation terms of a head-Kahan layer, is larger than the
// compiler's default size limit for "#pragma unroll".  A loop that stays rolled indexes its register arrays (operands,
// accumulators) dynamically, i.e. through scratch memory, and runs eight times slower; this file is therefore compiled
// with -mllvm -pragma-unroll-threshold=1000000 (elmo_amd/build.py).  The other variants keep the default: with the
// higher limit the compiler schedules the plain kernel differently and it loses 6 % (measured, same device).
#define XMC_HEAVY_TU
#include <hip/hip_runtime.h>
#include "xmc_fp8_quad.hip"
#include "xmc_fp8_role.hip"

namespace xmc {

void role_heavy_set_lds() {
#define XMC_STEP_LDS(RMODE, WD, KT) \
  (void)hipFuncSetAttribute((const void*)fp8_step_role_kernel<RMODE, WD, KT>, hipFuncAttributeMaxDynamicSharedMemorySize, RLDS_BYTES)
  XMC_STEP_LDS(ROUND_SR_PHILOX, false, 0); XMC_STEP_LDS(ROUND_SR_PHILOX, true, 0);
  XMC_STEP_LDS(ROUND_RTN, false, 1); XMC_STEP_LDS(ROUND_RTN, false, 2);
  XMC_STEP_LDS(ROUND_SR_PHILOX, false, 1); XMC_STEP_LDS(ROUND_SR_PHILOX, false, 2);
  XMC_STEP_LDS(ROUND_SR_FAST, false, 1); XMC_STEP_LDS(ROUND_SR_FAST, false, 2);
#undef XMC_STEP_LDS
}

// kahan_type 0: round_mode must be ROUND_SR_PHILOX; kahan_type 1, 2: any rounding mode, no weight decay
void role_heavy_launch(int round_mode, bool weight_decay, int kahan_type, int grid, hipStream_t stream, const QuadParams& p) {
#define XMC_HEAVY_KT(RMODE)                                                                               \
  do {                                                                                                    \
    if (kahan_type == 1) fp8_step_role_kernel<RMODE, false, 1><<<grid, QNT, RLDS_BYTES, stream>>>(p);     \
    else fp8_step_role_kernel<RMODE, false, 2><<<grid, QNT, RLDS_BYTES, stream>>>(p);                     \
  } while (0)
  if (kahan_type == 0) {
    if (weight_decay) fp8_step_role_kernel<ROUND_SR_PHILOX, true, 0><<<grid, QNT, RLDS_BYTES, stream>>>(p);
    else fp8_step_role_kernel<ROUND_SR_PHILOX, false, 0><<<grid, QNT, RLDS_BYTES, stream>>>(p);
  } else if (round_mode == ROUND_RTN) {
    XMC_HEAVY_KT(ROUND_RTN);
  } else if (round_mode == ROUND_SR_PHILOX) {
    XMC_HEAVY_KT(ROUND_SR_PHILOX);
  } else {
    XMC_HEAVY_KT(ROUND_SR_FAST);
  }
#undef XMC_HEAVY_KT
}

}  // namespace xmc
