// Fused FP8 extreme-classifier training step for gfx950 (MI355X).
//
// One persistent launch covers every label chunk of the layer.  Work unit = a tile of 64 consecutive
// label rows of one chunk (64 x 768 e4m3 bytes, contiguous in HBM).  Two workgroups on the same XCD
// form a pair and walk the same tile sequence: each brings the whole tile into LDS (the second read
// is served by that XCD's L2), both compute the full logits tile, and each owns one half of the 768
// input features for grad_X, grad_W and the in-place update, so every weight byte is read from HBM
// once and written once per step and neither logits nor gradients ever reach memory.
//
// Per tile (4 wavefronts, wavefront w owns batch rows 32w..32w+31 for the logits and features
// 96w..96w+95 of the workgroup's half for everything else):
//   1. logits  Z[l,b]  = sum_k W[l,k] Xq[b,k]        v_mfma_f32_16x16x128_f8f6f4, Xq operands in registers
//   2. G = bf16(sigmoid(bf16(Z)))  (-1 at positives)  written to LDS in [b][l] and [l][b] order
//   3. grad_X[b,k] += sum_l G[l,b] W[l,k]             v_mfma_f32_16x16x32_bf16, W read with
//                                                    ds_read_b64_tr_b8 (transposing LDS load), accumulators
//                                                    stay in registers for the whole launch
//   4. A[l,k]  = sum_b G[l,b] X[b,k]                 v_mfma_f32_16x16x32_bf16 (computed transposed)
//   5. W[l,k]  = round(W[l,k] - lr * A[l,k])          in LDS, then 16-byte stores of whole rows
// The next tile streams HBM -> LDS (global_load_lds, no registers) while the current one is processed.
// The update is in place, so a workgroup may only write its half of a tile back once its partner holds
// that tile in LDS: each workgroup publishes a tiles-loaded counter and checks its partner's before the
// write-back (normally already satisfied; the wait is bounded and raises an error word instead of hanging).
//
// Reference semantics: src/xmc_classifiers/chunked_fp8xmc_clf.py:81-123 with
// src/triton_kernels/matmul_kernel.py:204-239 (grad_X) and src/triton_kernels/fuse_kernel.py:63-113 (update).
#include "xmc_common.h"

namespace xmc {

struct StepParams {
  unsigned char* chunk[MAX_CHUNKS];   // device pointers of the chunk weight tensors [rows_per_chunk, 768] e4m3
  unsigned seed[MAX_CHUNKS];          // per-chunk rounding seed
  int num_chunks;
  int rows_per_chunk;
  int tiles_per_chunk;
  int num_tiles;
  const unsigned char* xq;            // logits operands (prep kernel layout)
  const bf16x8* xt;                   // grad_W operands (prep kernel layout)
  const unsigned* keys;               // sorted positives: label*256 + batch_row
  const int* tile_ptr;                // [num_tiles+1] offsets into keys
  floatx4* partial;                   // [gridDim.x][48][256] per-workgroup grad_X partial sums
  int* flags;                         // [npairs][2] tiles-loaded counters of the two workgroups of a pair; [npairs*2] = error word
  float zscale;                       // scale_w * scale_x applied to the logits accumulator
  float lr_eff;                       // lr / scale_w
  int batch;                          // real batch rows (<= BP)
};

#ifndef XMC_DBG_SKIP
#define XMC_DBG_SKIP 0   // timing experiments only: bit mask of phases to leave out (results are then wrong)
#endif
typedef __attribute__((address_space(3))) unsigned char lds_u8;
constexpr int SPIN_LIMIT = 1 << 20;   // polls of the partner's counter before giving up (error word set)

#define SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)   // nothing is scheduled across this point

// eight e4m3 codes -> eight bf16 values (exact)
__device__ __forceinline__ bf16x8 fp8x8_to_bf16x8(intx2 raw) {
  floatx2 f01 = __builtin_amdgcn_cvt_pk_f32_fp8(raw.x, false), f23 = __builtin_amdgcn_cvt_pk_f32_fp8(raw.x, true);
  floatx2 f45 = __builtin_amdgcn_cvt_pk_f32_fp8(raw.y, false), f67 = __builtin_amdgcn_cvt_pk_f32_fp8(raw.y, true);
  return bf16x8{(__bf16)f01.x, (__bf16)f01.y, (__bf16)f23.x, (__bf16)f23.y,
                (__bf16)f45.x, (__bf16)f45.y, (__bf16)f67.x, (__bf16)f67.y};
}

// transposing LDS read: within each group of 16 lanes, lanes 2j and 2j+1 point at the two 8-byte halves of
// a 16-byte row j (j = 0..7); lane i receives byte i of rows 0..7
__device__ __forceinline__ intx2 lds_tr8(const unsigned char* q) {
  return __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) intx2*)(__attribute__((address_space(3))) unsigned char*)q);
}

// 32 bytes from a 16-byte aligned LDS address
__device__ __forceinline__ intx8 lds_read32(const unsigned char* q) {
  intx4 lo = *(const intx4*)q, hi = *(const intx4*)(q + 16);
  return intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}

__device__ __forceinline__ void issue_tile_load(const unsigned char* gtile, int rows_valid, lds_u8* dst, int tid) {
  // LDS image = 64 rows x 49 chunks of 16 bytes (48 data + 1 pad); wave-instruction j fills chunks
  // [64j, 64j+63]; the pad chunk and rows past the end of the chunk re-read a valid address.
  const int last_row = rows_valid - 1;
#pragma unroll
  for (int s = 0; s < 13; s++) {
    int p = s * NT + tid;
    if (p < TL * 49) {
      int row = p / 49, c = p - row * 49;
      row = row < last_row ? row : last_row;
      c = c < 47 ? c : 47;
      const unsigned char* g = gtile + (size_t)row * D + c * 16;
      // inline assembly on purpose: the compiler would order every later LDS access behind a direct-to-LDS
      // load it knows about; completion is enforced by hand (s_waitcnt vmcnt(0) + barrier) before use
      const unsigned ldsoff = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(dst + (s * NT + (tid & ~63)) * 16));
      asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(ldsoff), "v"(g) : "memory", "m0");
    }
  }
}

template <int MODE>
__global__ __launch_bounds__(NT, 1) void fp8_step_kernel(const StepParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  unsigned char* wt0 = lds_raw;
  unsigned char* gt = lds_raw + 2 * WT_BYTES;
  unsigned char* gl = gt + BP * GT_S;

  const int tid = threadIdx.x;
  const int w = tid >> 6, lane = tid & 63, l16 = lane & 15, kg = lane >> 4;
  const int g = blockIdx.x;
  const int xcd = g & 7, j = g >> 3, h = j & 1;
  const int npairs = gridDim.x >> 1;
  const int pair = (j >> 1) * 8 + xcd;
  const int cw0 = HALF * h + WCOLS * w;          // first feature owned by this wavefront
  const int cb0 = cw0 / 16;

  // logits operands of this wavefront's 32 batch rows (re-read from L2 every tile: the register file is
  // taken by the grad_X accumulators)
  const intx8* xqw = (const intx8*)p.xq + (size_t)(w * 12) * 64 + lane;
  // ring of three K steps of logits operands (two 16-row batch blocks each); steps 0 and 1 are requested
  // before the tile loop and again at the end of every iteration, step ks+2 while step ks is consumed
  intx8 xqb[3][2];
  xqb[0][0] = xqw[0]; xqb[0][1] = xqw[6 * 64];
  xqb[1][0] = xqw[1 * 64]; xqb[1][1] = xqw[7 * 64];

  floatx4 acc2[8][6];
#pragma unroll
  for (int a = 0; a < 8; a++)
#pragma unroll
    for (int b = 0; b < 6; b++) acc2[a][b] = floatx4{0.f, 0.f, 0.f, 0.f};

  int t = pair;
  if (t < p.num_tiles) {
    int c = t / p.tiles_per_chunk, tj = t - c * p.tiles_per_chunk;
    int row0 = tj * TL;
    int rv = min(TL, p.rows_per_chunk - row0);
    issue_tile_load(p.chunk[c] + (size_t)row0 * D, rv, (lds_u8*)wt0, tid);
  }
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  int* flag_mine = p.flags + 2 * pair + h;
  int* flag_other = p.flags + 2 * pair + (h ^ 1);
  if (tid == 0) __hip_atomic_store(flag_mine, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

  for (int it = 0; t < p.num_tiles; t += npairs, it++) {
    unsigned char* wt = wt0 + (it & 1) * WT_BYTES;
    unsigned char* wtn = wt0 + ((it & 1) ^ 1) * WT_BYTES;
    const int c = t / p.tiles_per_chunk, tj = t - c * p.tiles_per_chunk;
    const int row0 = tj * TL;
    const int rows_valid = min(TL, p.rows_per_chunk - row0);
    unsigned char* gchunk = p.chunk[c];
    const unsigned seed = p.seed[c];
    const int p0 = p.tile_ptr[t], p1 = p.tile_ptr[t + 1];

    // ---- 1. logits: Z[64 x 32] for batch rows 32w..32w+31; 24 steps (ks major, row block minor), the LDS
    //         operand of step s+2 is requested before the two MFMAs of step s are issued
    floatx4 z[4][2];
#pragma unroll
    for (int rb = 0; rb < 4; rb++) { z[rb][0] = floatx4{0.f, 0.f, 0.f, 0.f}; z[rb][1] = floatx4{0.f, 0.f, 0.f, 0.f}; }
    if (!(XMC_DBG_SKIP & 1)) {
      const unsigned char* abase = wt + l16 * WS + kg * 32;
      intx8 ab[3];
      ab[0] = lds_read32(abase);
      ab[1] = lds_read32(abase + 16 * WS);
#pragma unroll
      for (int s = 0; s < 24; s++) {
        const int ks = s >> 2, rb = s & 3;
        if (s + 2 < 24) ab[(s + 2) % 3] = lds_read32(abase + 16 * ((s + 2) & 3) * WS + ((s + 2) >> 2) * 128);
        if (rb == 0 && ks + 2 < 6) {
          xqb[(ks + 2) % 3][0] = xqw[(size_t)(ks + 2) * 64];
          xqb[(ks + 2) % 3][1] = xqw[(size_t)(6 + ks + 2) * 64];
        }
        SCHED_FENCE();
        z[rb][0] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ab[s % 3], xqb[ks % 3][0], z[rb][0], 0, 0, 0, 0, 0, 0);
        z[rb][1] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ab[s % 3], xqb[ks % 3][1], z[rb][1], 0, 0, 0, 0, 0, 0);
        SCHED_FENCE();
      }
    }

    // ---- 2. G = bf16(sigmoid(bf16(Z))), zero for rows past the end of the chunk
    {
      const float nlog2e = -1.44269504088896340736f;
#pragma unroll
      for (int rb = 0; rb < 4; rb++) {
#pragma unroll
        for (int nb = 0; nb < 2; nb++) {
          const int b = 32 * w + 16 * nb + l16;
          const int r0 = 16 * rb + 4 * kg;
          unsigned short sb[4];
#pragma unroll
          for (int i = 0; i < 4; i++) {
            float zf = bf16_rt(z[rb][nb][i] * p.zscale);
            float sg = (XMC_DBG_SKIP & 2) ? zf : __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(zf * nlog2e));
            sb[i] = bf16_bits(sg);
          }
          if (rows_valid < TL) {
#pragma unroll
            for (int i = 0; i < 4; i++) sb[i] = (r0 + i < rows_valid) ? sb[i] : (unsigned short)0;
          }
#pragma unroll
          for (int i = 0; i < 4; i++) *(unsigned short*)(gl + (r0 + i) * GL_S + b * 2) = sb[i];
          uint2 v;
          v.x = (unsigned)sb[0] | ((unsigned)sb[1] << 16);
          v.y = (unsigned)sb[2] | ((unsigned)sb[3] << 16);
          *(uint2*)(gt + b * GT_S + r0 * 2) = v;
        }
      }
    }
    __syncthreads();

    // ---- stream the next tile into the other LDS buffer (every wavefront has finished reading it:
    //      its last readers were the write-back loads of the previous iteration)
    const int tn = t + npairs;
    if (tn < p.num_tiles && !(XMC_DBG_SKIP & 32)) {
      int cn = tn / p.tiles_per_chunk, tjn = tn - cn * p.tiles_per_chunk;
      int row0n = tjn * TL;
      issue_tile_load(p.chunk[cn] + (size_t)row0n * D, min(TL, p.rows_per_chunk - row0n), (lds_u8*)wtn, tid);
    }
    int seen = __hip_atomic_load(flag_other, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    // ---- positives of this tile: G -= 1 (set semantics: a repeated key is applied once)
    if (p1 > p0) {
      const unsigned label0 = (unsigned)(c * p.rows_per_chunk + row0);
      for (int e = p0 + tid; e < p1; e += NT) {
        unsigned key = p.keys[e];
        if (e > 0 && p.keys[e - 1] == key) continue;
        unsigned b = key & 255u, l = (key >> 8) - label0;
        if (b < (unsigned)BP && l < (unsigned)rows_valid) {
          unsigned short* q = (unsigned short*)(gl + l * GL_S + b * 2);
          unsigned short s2 = bf16_bits(bf16_from_bits(*q) - 1.0f);
          *q = s2;
          *(unsigned short*)(gt + b * GT_S + l * 2) = s2;
        }
      }
      __syncthreads();
    }

    // ---- 3. grad_X[128 x 96 of this wavefront] += G^T W; 12 steps (32-row K step major, 16-feature block
    //         minor); the transposed W read of step s+2 and the fp8->bf16 conversion of step s+1 are
    //         issued between the MFMAs of step s
    if (!(XMC_DBG_SKIP & 4)) {
      const unsigned char* wsrc = wt + (8 * kg + (l16 >> 1)) * WS + cw0 + (l16 & 1) * 8;
      const unsigned char* gsrc = gt + l16 * GT_S + kg * 16;
      bf16x8 ga[2][8];
#pragma unroll
      for (int mb = 0; mb < 8; mb++) ga[0][mb] = *(const bf16x8*)(gsrc + 16 * mb * GT_S);
      intx2 raw[3];
      raw[0] = lds_tr8(wsrc);
      raw[1] = lds_tr8(wsrc + 16);
      bf16x8 wb[2];
      wb[0] = fp8x8_to_bf16x8(raw[0]);
#pragma unroll
      for (int s = 0; s < 12; s++) {
        const int ks2 = s / 6, nn = s - ks2 * 6;
        if (s + 2 < 12) raw[(s + 2) % 3] = lds_tr8(wsrc + ((s + 2) / 6) * 32 * WS + ((s + 2) % 6) * 16);
        if (s < 4) {   // second K step's G^T operands, two per step
          ga[1][2 * s] = *(const bf16x8*)(gsrc + 16 * (2 * s) * GT_S + 64);
          ga[1][2 * s + 1] = *(const bf16x8*)(gsrc + 16 * (2 * s + 1) * GT_S + 64);
        }
        SCHED_FENCE();
#pragma unroll
        for (int mb = 0; mb < 8; mb++) {
          acc2[mb][nn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ga[ks2][mb], wb[s & 1], acc2[mb][nn], 0, 0, 0);
          if (mb == 1 && s + 1 < 12) wb[(s + 1) & 1] = fp8x8_to_bf16x8(raw[(s + 1) % 3]);
          if (mb == 1) SCHED_FENCE();
        }
        SCHED_FENCE();
      }
    }

    // ---- 4+5. A^T[96 x 64] = X^T G^T in six 16-feature groups; the update of group g-1 (VALU, in LDS) is
    //           issued between the MFMAs of group g.  G operands stay in registers for all six groups.
    {
      bf16x8 bg[4][4];   // [ks][nb]
#pragma unroll
      for (int ks = 0; ks < 4; ks++)
#pragma unroll
        for (int nb = 0; nb < 4; nb++) bg[ks][nb] = *(const bf16x8*)(gl + (16 * nb + l16) * GL_S + ks * 64 + kg * 16);
      const bf16x8* xsrc = p.xt + (size_t)cb0 * 4 * 64 + lane;
      bf16x8 ax[2][4];
#pragma unroll
      for (int ks = 0; ks < 4; ks++) ax[0][ks] = xsrc[ks * 64];
      floatx4 acc3[2][4];
      unsigned char* wrow = wt + l16 * WS + cw0 + 4 * kg;
      const unsigned grow0 = (unsigned)(c * p.rows_per_chunk + row0 + l16);
#pragma unroll
      for (int cg = 0; cg <= 6; cg++) {
        const int cur = cg & 1, prev = cur ^ 1;
        if (cg < 6) {
          if (cg + 1 < 6) {
#pragma unroll
            for (int ks = 0; ks < 4; ks++) ax[prev][ks] = xsrc[((cg + 1) * 4 + ks) * 64];
          }
#pragma unroll
          for (int nb = 0; nb < 4; nb++) acc3[cur][nb] = floatx4{0.f, 0.f, 0.f, 0.f};
        }
        unsigned wq[4];
        if (cg > 0 && !(XMC_DBG_SKIP & 16)) {
#pragma unroll
          for (int nb = 0; nb < 4; nb++) wq[nb] = *(const unsigned*)(wrow + 16 * nb * WS + 16 * (cg - 1));
        }
        SCHED_FENCE();
#pragma unroll
        for (int q = 0; q < 4; q++) {   // q = K step for the MFMAs, = row block for the update
          if (cg < 6 && !(XMC_DBG_SKIP & 8)) {
#pragma unroll
            for (int nb = 0; nb < 4; nb++)
              acc3[cur][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax[cur][q], bg[q][nb], acc3[cur][nb], 0, 0, 0);
          }
          if (cg > 0 && !(XMC_DBG_SKIP & 16)) {
            const int nb = q;
            floatx2 w01 = __builtin_amdgcn_cvt_pk_f32_fp8((int)wq[nb], false), w23 = __builtin_amdgcn_cvt_pk_f32_fp8((int)wq[nb], true);
            floatx4 a = acc3[prev][nb];
            float t0 = __builtin_fmaf(-p.lr_eff, a[0], w01.x), t1 = __builtin_fmaf(-p.lr_eff, a[1], w01.y);
            float t2 = __builtin_fmaf(-p.lr_eff, a[2], w23.x), t3 = __builtin_fmaf(-p.lr_eff, a[3], w23.y);
            const unsigned col = (unsigned)(cw0 + 16 * (cg - 1) + 4 * kg);
            *(unsigned*)(wrow + 16 * nb * WS + 16 * (cg - 1)) =
                round4<MODE>(t0, t1, t2, t3, (unsigned)(row0 + 16 * nb + l16), grow0 + 16 * nb, col, seed);
          }
          SCHED_FENCE();
        }
      }
    }
    // logits operands of the first two K steps of the next tile
    xqb[0][0] = xqw[0]; xqb[0][1] = xqw[6 * 64];
    xqb[1][0] = xqw[1 * 64]; xqb[1][1] = xqw[7 * 64];
    __builtin_amdgcn_s_waitcnt(0);   // next tile has landed in LDS (this thread's part)
    __syncthreads();
    if (tid == 0) __hip_atomic_store(flag_mine, it + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // the partner must hold this tile before its rows are overwritten
    for (int spin = 0; seen < it + 1 && !(XMC_DBG_SKIP & 128); spin++) {
      if (spin >= SPIN_LIMIT) { p.flags[2 * npairs] = 1; break; }
      __builtin_amdgcn_s_sleep(2);
      seen = __hip_atomic_load(flag_other, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // ---- write this workgroup's half of the updated tile back, 16 bytes per lane, whole 128-byte lines
#pragma unroll
    for (int s = 0; s < 6; s++) {
      int ch = s * NT + tid;
      int row = ch / 24, cc = ch - row * 24;
      if (row < rows_valid && !(XMC_DBG_SKIP & 64)) {
        uint4 v = *(const uint4*)(wt + row * WS + HALF * h + cc * 16);
        *(uint4*)(gchunk + (size_t)(row0 + row) * D + HALF * h + cc * 16) = v;
      }
    }
  }

  // ---- per-workgroup grad_X partial, summed in a fixed order by reduce_gx_kernel
  floatx4* dst = p.partial + (size_t)g * 48 * NT;
#pragma unroll
  for (int mb = 0; mb < 8; mb++)
#pragma unroll
    for (int nn = 0; nn < 6; nn++) dst[(mb * 6 + nn) * NT + tid] = acc2[mb][nn];
}

// grad_X = scale * sum over workgroups of the partials; writes fp32 and bf16 [batch, 768]
__global__ void reduce_gx_kernel(const floatx4* partial, int nwg, float scale, float* gx_f32, unsigned short* gx_bf16,
                                 int batch) {
  const int slot = blockIdx.x >> 1, h = blockIdx.x & 1;   // slot = mb*6+nn
  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, l16 = lane & 15, kg = lane >> 4;
  floatx4 s = {0.f, 0.f, 0.f, 0.f};
  for (int g = 0; g < nwg; g++) {
    if (((g >> 3) & 1) != h) continue;
    floatx4 v = partial[((size_t)g * 48 + slot) * NT + tid];
    s += v;
  }
  const int mb = slot / 6, nn = slot - mb * 6;
  const int col = HALF * h + WCOLS * w + 16 * nn + l16;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    int b = 16 * mb + 4 * kg + i;
    if (b < batch) {
      float v = s[i] * scale;
      if (gx_f32) gx_f32[(size_t)b * D + col] = v;
      if (gx_bf16) gx_bf16[(size_t)b * D + col] = bf16_bits(v);
    }
  }
}

// Build the operand images of X used by the step kernel.
//   xq: e4m3(X / scale_x) in v_mfma 16x16x128 B-operand order: [(w*2+nb)*6+ks][lane][32 bytes]
//   xt: bf16 X^T in v_mfma 16x16x32 A-operand order: [(col/16)*4+ks][lane][8 bf16], lane = (col%16) + 16*kg,
//       element j = X[32ks + 8kg + j][col]
__global__ void prep_x_kernel(const unsigned short* x, int batch, float inv_scale_x, unsigned char* xq, unsigned short* xt) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;   // one thread per (b, k4) group of 4 features
  if (i >= BP * (D / 4)) return;
  int b = i / (D / 4), k = (i - b * (D / 4)) * 4;
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  unsigned short raw[4] = {0, 0, 0, 0};
  if (b < batch) {
#pragma unroll
    for (int q = 0; q < 4; q++) { raw[q] = x[(size_t)b * D + k + q]; v[q] = bf16_from_bits(raw[q]) * inv_scale_x; }
  }
  int packed = 0;
  packed = __builtin_amdgcn_cvt_pk_fp8_f32(clamp448(v[0]), clamp448(v[1]), packed, false);
  packed = __builtin_amdgcn_cvt_pk_fp8_f32(clamp448(v[2]), clamp448(v[3]), packed, true);
  {
    int w = b >> 5, nb = (b >> 4) & 1, n = b & 15;
    int ks = k >> 7, kgq = (k >> 5) & 3, jq = k & 31;
    size_t off = ((size_t)((w * 2 + nb) * 6 + ks) * 64 + (n + 16 * kgq)) * 32 + jq;
    *(int*)(xq + off) = packed;
  }
#pragma unroll
  for (int q = 0; q < 4; q++) {
    int col = k + q;
    int ks = b >> 5, kgq = (b >> 3) & 3, jq = b & 7;
    size_t off = ((size_t)((col >> 4) * 4 + ks) * 64 + ((col & 15) + 16 * kgq)) * 8 + jq;
    xt[off] = raw[q];
  }
}

// tile_ptr[t] = first key whose label >= first label of tile t; tile_ptr[num_tiles] = first key past the last tile
__global__ void tile_ptr_kernel(const unsigned* keys, int n_pad, int rows_per_chunk, int tiles_per_chunk, int num_tiles,
                                int* tile_ptr) {
  int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t > num_tiles) return;
  unsigned long long label0;
  if (t == num_tiles) {
    label0 = (unsigned long long)(num_tiles / tiles_per_chunk) * rows_per_chunk;
  } else {
    int c = t / tiles_per_chunk, tj = t - c * tiles_per_chunk;
    label0 = (unsigned long long)c * rows_per_chunk + (unsigned long long)tj * TL;
  }
  unsigned long long bound = label0 << 8;
  int lo = 0, hi = n_pad;
  while (lo < hi) {
    int mid = (lo + hi) >> 1;
    if ((unsigned long long)keys[mid] < bound) lo = mid + 1; else hi = mid;
  }
  tile_ptr[t] = lo;
}

// Inference logits: out[b, label - col0] = bf16(zscale * sum_k Xq[b,k] W[label,k]) for the 32-label tiles
// [tile_begin, tile_end) of the chunk list (tile t = chunk t / tiles_per_chunk, rows 32 (t % tiles_per_chunk) ...).
struct ForwardParams {
  const unsigned char* chunk[MAX_CHUNKS];
  int rows_per_chunk, tiles_per_chunk;
  int tile_begin, tile_end;
  const unsigned char* xq;     // logits operands (prep kernel layout)
  float zscale;
  unsigned short* out;         // bf16 [batch][out_stride]
  long long out_stride;
  long long col0;              // label that column 0 of `out` stands for
  long long num_labels;        // labels at or past this one are not written
  int batch;
};

constexpr int FT = 32;                    // labels per tile of the inference kernel
constexpr int FB = FT * WS;               // one tile in LDS (rows of 48 + 1 pieces of 16 bytes)
constexpr int FWD_LDS = 3 * FB;           // three tiles in flight per workgroup; two workgroups share a compute unit
constexpr int FWD_DMA = 7;                // direct-to-LDS loads per wavefront and tile (8 rows x 49 pieces = 392 = 6 x 64 + 8)
constexpr int ZS = FT * 2 + 16;           // LDS row stride of the staged logits [b][32 labels] bf16, bytes

// Every wavefront fetches 8 rows of the tile with exactly FWD_DMA instructions (the wait counts below rely on it).
__device__ __forceinline__ void fwd_issue_tile(const unsigned char* gtile, int rows_valid, unsigned lds_off, int w, int lane) {
  const int last_row = rows_valid - 1;
#pragma unroll
  for (int j = 0; j < FWD_DMA; j++) {
    const int pl = 64 * j + lane;
    if (pl < 392) {
      const int pc = 392 * w + pl;
      int row = pc / 49, c = pc - row * 49;
      row = row < last_row ? row : last_row;   // rows past the end and the pad piece re-read a valid address
      c = c < 47 ? c : 47;
      const unsigned char* g = gtile + row * D + c * 16;
      const unsigned ldsoff = __builtin_amdgcn_readfirstlane(lds_off + (unsigned)(392 * w + 64 * j) * 16u);
      asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(ldsoff), "v"(g) : "memory", "m0");
    }
  }
}

// One workgroup streams its tiles through three LDS buffers, the loads two tiles ahead of the matrix products.  The
// accumulators go back through the buffer of the tile just used, so that a lane stores 16 consecutive bytes of one
// batch row.  Memory operations complete in order: "all but the newest FWD_DMA" means the tile after this one has
// landed and the stores of the tile before have left, whatever their number.
__device__ __forceinline__ void fp8_forward_body(const ForwardParams& p, unsigned char* lds_raw, int block, int nblocks) {
  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, l16 = lane & 15, kg = lane >> 4;
  const unsigned lds0 = (unsigned)(size_t)(lds_u8*)lds_raw;
  intx8 xq[2][6];
#pragma unroll
  for (int nb = 0; nb < 2; nb++)
#pragma unroll
    for (int ks = 0; ks < 6; ks++)
      xq[nb][ks] = *(const intx8*)(p.xq + ((size_t)((w * 2 + nb) * 6 + ks) * 64 + lane) * 32);
  __builtin_amdgcn_s_waitcnt(0);
  const int first = p.tile_begin + block;
  auto issue = [&](int t, int buf) {
    const int c = t / p.tiles_per_chunk, row0 = (t - c * p.tiles_per_chunk) * FT;
    fwd_issue_tile(p.chunk[c] + (size_t)row0 * D, min(FT, p.rows_per_chunk - row0), lds0 + (unsigned)buf * FB, w, lane);
  };
  if (first >= p.tile_end) return;
  issue(first, 0);
  if (first + nblocks < p.tile_end) {
    issue(first + nblocks, 1);
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(FWD_DMA) : "memory");
  } else {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  __syncthreads();
  int buf = 0;
  for (int t = first; t < p.tile_end; t += nblocks) {
    const int c = t / p.tiles_per_chunk, row0 = (t - c * p.tiles_per_chunk) * FT;
    const int rows_valid = min(FT, p.rows_per_chunk - row0);
    const long long label0 = (long long)c * p.rows_per_chunk + row0;
    unsigned char* wt = lds_raw + buf * FB;
    const bool more = t + 2 * nblocks < p.tile_end;
    if (more) issue(t + 2 * nblocks, buf == 0 ? 2 : buf - 1);
    floatx4 z[2][2];
#pragma unroll
    for (int rb = 0; rb < 2; rb++) { z[rb][0] = floatx4{0.f, 0.f, 0.f, 0.f}; z[rb][1] = floatx4{0.f, 0.f, 0.f, 0.f}; }
#pragma unroll
    for (int ks = 0; ks < 6; ks++)
#pragma unroll
      for (int rb = 0; rb < 2; rb++) {
        intx8 a = lds_read32(wt + (16 * rb + l16) * WS + ks * 128 + kg * 32);
        z[rb][0] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, xq[0][ks], z[rb][0], 0, 0, 0, 0, 0, 0);
        z[rb][1] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, xq[1][ks], z[rb][1], 0, 0, 0, 0, 0, 0);
      }
    __syncthreads();   // the weight tile has been read: its buffer now stages the logits
#pragma unroll
    for (int rb = 0; rb < 2; rb++)
#pragma unroll
      for (int nb = 0; nb < 2; nb++) {
        const int b = 32 * w + 16 * nb + l16;
        uint2 v;
        v.x = bf16_pack2(z[rb][nb][0] * p.zscale, z[rb][nb][1] * p.zscale);
        v.y = bf16_pack2(z[rb][nb][2] * p.zscale, z[rb][nb][3] * p.zscale);
        *(uint2*)(wt + b * ZS + (16 * rb + 4 * kg) * 2) = v;
      }
    if (more) asm volatile("s_waitcnt vmcnt(%0)" : : "n"(FWD_DMA) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();   // the next tile has landed for every wavefront; the staged logits are visible
    long long left = p.num_labels - label0;
    const int nvalid = (int)(left < rows_valid ? (left < 0 ? 0 : left) : rows_valid);
#pragma unroll
    for (int q = 0; q < 2; q++) {
      const int piece = tid + NT * q, b = piece >> 2, seg = piece & 3;
      if (b < p.batch) {
        unsigned short* orow = p.out + (size_t)b * p.out_stride + (label0 - p.col0);
        const unsigned short* zrow = (const unsigned short*)(wt + b * ZS);
        const int s = (int)((8u - (unsigned)(((uintptr_t)orow >> 1) & 7u)) & 7u);   // elements before a 16-byte boundary
        const int a = s + 8 * seg;
        if (a + 8 <= nvalid) {
          uint4 v;
          if (s == 0) {
            v = *(const uint4*)(zrow + a);
          } else {
            v.x = zrow[a] | ((unsigned)zrow[a + 1] << 16);
            v.y = zrow[a + 2] | ((unsigned)zrow[a + 3] << 16);
            v.z = zrow[a + 4] | ((unsigned)zrow[a + 5] << 16);
            v.w = zrow[a + 6] | ((unsigned)zrow[a + 7] << 16);
          }
          *(uint4*)(orow + a) = v;
        } else {
          for (int e = a; e < nvalid && e < a + 8; e++) orow[e] = zrow[e];
        }
        if (seg == 0)
          for (int e = 0; e < s && e < nvalid; e++) orow[e] = zrow[e];
      }
    }
    __syncthreads();   // the staged logits have been read: the buffer is free for the tile three ahead
    buf = buf == 2 ? 0 : buf + 1;
  }
}

__global__ __launch_bounds__(NT) void fp8_forward_kernel(const ForwardParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  fp8_forward_body(p, lds_raw, (int)blockIdx.x, (int)gridDim.x);
}

}  // namespace xmc
