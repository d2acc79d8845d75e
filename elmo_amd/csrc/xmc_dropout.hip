// Dropout fused with the cast to e4m3: out[m][k] = e4m3(keep ? x[m][k] / (1 - p) : 0) with keep = rand(seed, m * cols + k) > p,
// rand = Triton's tl.rand (first Philox-4x32-10 word of counter (offset, 0, 0, 0) under the key (seed low, seed high),
// as a uniform fp32).  The reference holds this as a prototype applied to the A operand of its FP8 GEMM
// (src/triton_kernels/tma_gemm.py:7-13,34-38; its training loop applies nn.Dropout to the encoder output, model.py:135,165,
// and the classifier quantises afterwards, chunked_fp8xmc_clf.py:101): here it is one pass over the embedding that
// writes the e4m3 operand directly.  The cast saturates at +-448 like the other true-FP8 casts of this library.
#include "xmc_common.h"

namespace xmc {

// one thread per four consecutive elements of a row (cols % 4 == 0); x_type 0 = bf16, 1 = e4m3
__global__ __launch_bounds__(256) void dropout_quantize_kernel(const void* x, int x_type, long long n4, int cols, float p,
                                                              unsigned seed_lo, unsigned seed_hi, unsigned* out) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n4) return;
  float v[4];
  if (x_type == 0) {
    const uint2 raw = ((const uint2*)x)[i];
    v[0] = bf16_from_bits((unsigned short)(raw.x & 0xFFFFu)); v[1] = bf16_from_bits((unsigned short)(raw.x >> 16));
    v[2] = bf16_from_bits((unsigned short)(raw.y & 0xFFFFu)); v[3] = bf16_from_bits((unsigned short)(raw.y >> 16));
  } else {
    const unsigned raw = ((const unsigned*)x)[i];
    const floatx2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)raw, false), hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)raw, true);
    v[0] = lo.x; v[1] = lo.y; v[2] = hi.x; v[3] = hi.y;
  }
  const float keep_scale = 1.0f - p;
  const unsigned off0 = (unsigned)(4 * i);   // m * cols + k of the first element (the prototype computes it in int32)
#pragma unroll
  for (int q = 0; q < 4; q++) {
    int r = (int)philox_word0(off0 + (unsigned)q, seed_lo, seed_hi);
    r = r < 0 ? -r - 1 : r;
    const float u = (float)r * 4.6566127342e-10f;
    v[q] = u > p ? v[q] / keep_scale : 0.0f;
  }
  int packed = 0;
  packed = __builtin_amdgcn_cvt_pk_fp8_f32(clamp448(v[0]), clamp448(v[1]), packed, false);
  packed = __builtin_amdgcn_cvt_pk_fp8_f32(clamp448(v[2]), clamp448(v[3]), packed, true);
  out[i] = (unsigned)packed;
}

}  // namespace xmc
