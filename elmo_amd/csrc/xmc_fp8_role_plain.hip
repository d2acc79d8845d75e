// Third translation unit of the library: the variants of the fused step kernel that the benchmark's headline runs
// (round to nearest and the fast stochastic rounding, no compensated head).  The kernel's speed depends on the order the
// compiler gives the vector instructions between the matrix instructions of a step; of the scheduler settings tried
// (same device, 200 launches each) the default took 0.4035 ms, -misched-cluster=0 0.4000 ms, with the AMDGPU register
// pressure trackers in addition 0.3962 ms, and the other strategies (max-ilp, max-memory-clause, iterative-ilp, top-down,
// no post-RA scheduler) 0.49-0.65 ms.  This file is compiled with the best of them (elmo_amd/build.py); the rest of the
// library keeps the defaults its kernels were tuned with.
#define XMC_HEAVY_TU
#include <hip/hip_runtime.h>
#include "xmc_fp8_quad.hip"
#include "xmc_fp8_role.hip"

namespace xmc {

void role_plain_set_lds() {
#define XMC_STEP_LDS(RMODE, WD) \
  (void)hipFuncSetAttribute((const void*)fp8_step_role_kernel<RMODE, WD, 0>, hipFuncAttributeMaxDynamicSharedMemorySize, RLDS_BYTES)
  XMC_STEP_LDS(ROUND_RTN, false); XMC_STEP_LDS(ROUND_RTN, true); XMC_STEP_LDS(ROUND_SR_FAST, false); XMC_STEP_LDS(ROUND_SR_FAST, true);
#undef XMC_STEP_LDS
}

// round_mode ROUND_RTN or ROUND_SR_FAST
void role_plain_launch(int round_mode, bool weight_decay, int grid, hipStream_t stream, const QuadParams& p) {
  if (round_mode == ROUND_RTN && weight_decay) fp8_step_role_kernel<ROUND_RTN, true, 0><<<grid, QNT, RLDS_BYTES, stream>>>(p);
  else if (round_mode == ROUND_RTN) fp8_step_role_kernel<ROUND_RTN, false, 0><<<grid, QNT, RLDS_BYTES, stream>>>(p);
  else if (weight_decay) fp8_step_role_kernel<ROUND_SR_FAST, true, 0><<<grid, QNT, RLDS_BYTES, stream>>>(p);
  else fp8_step_role_kernel<ROUND_SR_FAST, false, 0><<<grid, QNT, RLDS_BYTES, stream>>>(p);
}

}  // namespace xmc
