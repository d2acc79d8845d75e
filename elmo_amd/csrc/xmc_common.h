// Shared device helpers and compile-time geometry for the gfx950 XMC classifier kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace xmc {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef int intx8 __attribute__((ext_vector_type(8)));
typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// ---- geometry of the FP8 kernels
constexpr int D = 768;            // input features (row length of W, bytes per FP8 row)
constexpr int BP = 128;           // padded batch rows
constexpr int TL = 64;            // labels per tile of the training kernels
constexpr int NT = 256;           // threads per workgroup of the inference kernel (4 wavefronts of 64)
constexpr int WS = D + 16;        // LDS row stride of a W tile in the inference kernel, bytes (49 x 16)
constexpr int MAX_CHUNKS = 64;
constexpr int MAX_POS = 32768;    // positives per step (per 256 batch rows on the tiled path): the rank sort keeps them all in LDS

// workspace of the fused step (byte offsets), all 256-byte aligned
constexpr int MAX_WG = 256;                                   // workgroups of the persistent step kernel
constexpr size_t WS_XQ = 0;                                   // FP8 logits operands   BP*D
constexpr size_t WS_XT = WS_XQ + (size_t)BP * D;              // bf16 grad_W operands  BP*D*2
constexpr size_t WS_KEYS = WS_XT + (size_t)BP * D * 2;        // sorted positive keys  MAX_POS*4
constexpr size_t WS_FLAGS = WS_KEYS + (size_t)MAX_POS * 4;    // 4096 ints: counters, XCC ids, error words (below)
constexpr size_t WS_PARTIAL = WS_FLAGS + 16384;               // MAX_WG * 12 * 512 * 16 bytes of grad_X partials
constexpr size_t WS_EXCH = WS_PARTIAL + (size_t)MAX_WG * 12 * 512 * 16;     // G exchange ring: 64 quads x 8 slots x 20 KiB
constexpr size_t WS_TILEPTR = WS_EXCH + (size_t)(MAX_WG / 4) * 8 * 20480;   // tile_ptr[num_tiles + 1], then the tile descriptors

// Layout of the 4096 ints at WS_FLAGS (all but the sticky word cleared at the start of every step):
//   [0, 1024)             tiles-published counters of the persistent step kernel: sixteen per quad
//   [QF_CNT2, +1024)      the same for the step's second launch (the head-Kahan layer runs the compensated tiles first)
//   [QF_XCC, QF_XCC+256)  XCC id every workgroup of the step kernel found itself on
//   [QF_ERR]              error word: bit 0 = a bounded wait expired, bit 1 = the workgroups of a quad were not placed on
//                         one XCD (their exchange of G through that XCD's L2 is then not coherent)
//   [QF_STICKY]           the error words of all steps since the caller last cleared it, OR-ed together by the step's
//                         last kernel; no kernel ever clears it
constexpr int QF_WORDS = 4096;
constexpr int QF_CNT2 = 2048;
constexpr int QF_XCC = 1024;
constexpr int QF_ERR = 2044;
constexpr int QF_STICKY = 2047;

// The step kernel assumes that workgroup g runs on XCD g % 8, and builds quads of four workgroups with equal g % 8:
// member m of quad q is workgroup ((q / 8) * 4 + m) * 8 + q % 8.
__host__ __device__ inline int quad_member_workgroup(int quad, int m) { return (((quad >> 3) << 2) + m) * 8 + (quad & 7); }
// true if the four members of `quad` did not all record the same XCC id
__host__ __device__ inline bool quad_xcc_mismatch(const int* xcc_ids, int quad) {
  const int id0 = xcc_ids[quad_member_workgroup(quad, 0)];
  return xcc_ids[quad_member_workgroup(quad, 1)] != id0 || xcc_ids[quad_member_workgroup(quad, 2)] != id0 ||
         xcc_ids[quad_member_workgroup(quad, 3)] != id0;
}

__device__ __forceinline__ float bf16_rt(float f) { return (float)(__bf16)f; }

// bf16(a) in the low half, bf16(b) in the high half (round to nearest even), one conversion instruction
__device__ __forceinline__ unsigned bf16_pack2(float a, float b) {
  const bf16x2 r = __builtin_convertvector(floatx2{a, b}, bf16x2);
  return __builtin_bit_cast(unsigned, r);
}

__device__ __forceinline__ unsigned short bf16_bits(float f) {
  __bf16 b = (__bf16)f;
  unsigned short u;
  __builtin_memcpy(&u, &b, 2);
  return u;
}
__device__ __forceinline__ float bf16_from_bits(unsigned short u) { return __uint_as_float((unsigned)u << 16); }

__device__ __forceinline__ float clamp448(float t) { return __builtin_fminf(__builtin_fmaxf(t, -448.0f), 448.0f); }

// Philox-4x32-10, counter (off,0,0,0), key (seed_lo, seed_hi); returns word 0.
__device__ __forceinline__ unsigned philox_word0(unsigned off, unsigned k0, unsigned k1) {
  unsigned c0 = off, c1 = 0, c2 = 0, c3 = 0;
#pragma unroll
  for (int r = 0; r < 10; r++) {
    // one 32 x 32 -> 64 bit multiply per product (both halves are needed)
    const unsigned long long p0 = (unsigned long long)0xD2511F53u * (unsigned long long)c0;
    const unsigned long long p1 = (unsigned long long)0xCD9E8D57u * (unsigned long long)c2;
    const unsigned hi0 = (unsigned)(p0 >> 32), lo0 = (unsigned)p0, hi1 = (unsigned)(p1 >> 32), lo1 = (unsigned)p1;
    c0 = hi1 ^ c1 ^ k0; c1 = lo1; c2 = hi0 ^ c3 ^ k1; c3 = lo0;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  return c0;
}

// Counter hash of the fast stochastic-rounding mode: one 32-bit mix per 4 consecutive weights of a row; the first
// weight takes the mix itself, the other three its products with odd constants.  idx = global_row * (D/4) + col/4.
// The caller's seed goes through a full 32-bit mixer once, on the host, before it reaches fast_mix: seeds that differ
// in a few bits (s and s + 1, say) must not give related words.
__host__ __device__ inline unsigned fast_seed(unsigned s) {
  s ^= s >> 16; s *= 0x7FEB352Du; s ^= s >> 15; s *= 0x846CA68Bu; s ^= s >> 16;
  return s;
}
__device__ __forceinline__ unsigned fast_mix(unsigned idx, unsigned seed) {
  unsigned h = idx * 0x9E3779B1u + seed;
  h ^= h >> 16; h *= 0x85EBCA77u; h ^= h >> 15;
  return h;
}
__device__ __forceinline__ unsigned fast_word(unsigned h, int i) {
  const unsigned k[4] = {1u, 0x27D4EB2Fu, 0x165667B1u, 0x9E3779B1u};
  return h * k[i];
}

// Dropout of the embedding inside the step (training.xmc dropout fused into the preparation of X; the reference keeps a
// prototype of this in src/triton_kernels/tma_gemm.py:7-13): element (b, k) is kept when rand(seed, b * D + k) > p, rand
// being Triton's tl.rand (first Philox-4x32-10 word of counter (offset, 0, 0, 0), key = seed, as a uniform fp32).
struct DropoutParams { float p; float keep_scale; unsigned seed_lo, seed_hi; };   // p == 0: no dropout

__device__ __forceinline__ bool dropout_keep(unsigned off, const DropoutParams& dp) {
  int r = (int)philox_word0(off, dp.seed_lo, dp.seed_hi);
  r = r < 0 ? -r - 1 : r;
  return (float)r * 4.6566127342e-10f > dp.p;
}
// the dropped-out embedding in the layer's type: bf16(keep ? x / (1 - p) : 0)
__device__ __forceinline__ unsigned short dropout_bf16(unsigned short raw, unsigned off, const DropoutParams& dp) {
  if (dp.p == 0.f) return raw;
  return dropout_keep(off, dp) ? bf16_bits(bf16_from_bits(raw) / dp.keep_scale) : (unsigned short)0;
}
// gradient with respect to the embedding in front of the dropout
__device__ __forceinline__ float dropout_backward(float g, unsigned off, const DropoutParams& dp) {
  if (dp.p == 0.f) return g;
  return dropout_keep(off, dp) ? g / dp.keep_scale : 0.f;
}

enum RoundMode { ROUND_RTN = 0, ROUND_SR_PHILOX = 1, ROUND_SR_FAST = 2 };

// Round four updated weights (fp32) of one row, columns col..col+3, to e4m3 codes packed in a dword.
//   RTN        round to nearest even, saturating at +-448
//   SR_PHILOX  bits(t) + (philox(seed, row*D+col) & 0xFFFFF), clear low 20 bits, then the RTN cast
//   SR_FAST    true stochastic rounding on the e4m3 grid (subnormals included) by the hardware
//              converter, random word from fast_mix/fast_word
template <int MODE>
__device__ __forceinline__ unsigned round4(float t0, float t1, float t2, float t3, unsigned row_in_chunk,
                                           unsigned grow, unsigned col, unsigned seed) {
  float t[4] = {t0, t1, t2, t3};
  if (MODE == ROUND_SR_PHILOX) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      unsigned r = philox_word0(row_in_chunk * (unsigned)D + col + i, seed, 0u) & 0xFFFFFu;
      t[i] = __uint_as_float((__float_as_uint(t[i]) + r) & 0xFFF00000u);
    }
  }
  int packed = 0;
  if (MODE == ROUND_SR_FAST) {
    unsigned h = fast_mix(grow * (unsigned)(D / 4) + (col >> 2), seed);
    packed = __builtin_amdgcn_cvt_sr_fp8_f32(clamp448(t[0]), fast_word(h, 0), packed, 0);
    packed = __builtin_amdgcn_cvt_sr_fp8_f32(clamp448(t[1]), fast_word(h, 1), packed, 1);
    packed = __builtin_amdgcn_cvt_sr_fp8_f32(clamp448(t[2]), fast_word(h, 2), packed, 2);
    packed = __builtin_amdgcn_cvt_sr_fp8_f32(clamp448(t[3]), fast_word(h, 3), packed, 3);
  } else {
    packed = __builtin_amdgcn_cvt_pk_fp8_f32(clamp448(t[0]), clamp448(t[1]), packed, false);
    packed = __builtin_amdgcn_cvt_pk_fp8_f32(clamp448(t[2]), clamp448(t[3]), packed, true);
  }
  return (unsigned)packed;
}

// 16-bit key of a bf16 value for the top-k selection: ascending key order == ascending value order, -0 below +0, and
// NaN of either sign above everything (torch.topk treats NaN as the largest value), all NaNs alike.
__device__ __forceinline__ unsigned topk_key(unsigned short bits) {
  if ((bits & 0x7FFFu) > 0x7F80u) return 0xFFFFu;
  return (bits & 0x8000u) ? (unsigned)(~bits & 0xFFFFu) : (unsigned)(bits | 0x8000u);
}
__device__ __forceinline__ unsigned short topk_bits(unsigned key) {   // key 0xFFFF gives back a NaN (0x7FFF)
  return (key & 0x8000u) ? (unsigned short)(key & 0x7FFFu) : (unsigned short)(~key & 0xFFFFu);
}

}  // namespace xmc
