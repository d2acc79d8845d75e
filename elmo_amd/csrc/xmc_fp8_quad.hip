// Fused FP8 extreme-classifier training step for gfx950 (MI355X): four compute units per tile stream.
//
// Work unit = a tile of 64 consecutive label rows of one chunk (64 x 768 e4m3 bytes, contiguous in HBM).
// Four workgroups on the same XCD (a "quad") walk the same tile sequence, one workgroup per compute unit,
// 8 wavefronts each.  Member m of the quad owns
//   * batch rows 32m..32m+31 for the logits and the sigmoid ("stage A"), and
//   * input features 192m..192m+191 for grad_X, grad_W and the in-place update ("stage B"),
// so no arithmetic is repeated and every weight byte is read from HBM once and written once per step.
// The only data the members exchange is G = sigmoid(logits) in bf16 (4.5 KiB per member and tile), through a
// small ring of slots in global memory that stays in the XCD's L2, guarded by per-member "tiles published"
// counters.  Stage A runs two tiles ahead of stage B, so the exchange latency is off the critical path.
// Neither logits nor gradients ever reach HBM; the X operands of all three GEMMs and the grad_X accumulators
// (96 KiB per compute unit) live in registers for the whole launch.
//
//   stage A(t): Z[64 x 32] = W_t Xq_m^T     v_mfma_f32_16x16x128_f8f6f4, W rows straight from L2 into registers,
//                                           K split over the two wavefront groups, partials summed through LDS
//               G = bf16(sigmoid(bf16(Z)))  stored to the exchange slot in [b][l] order
//   stage B(t): gather the four G parts into LDS (global_load_lds), subtract 1 at the positives
//               grad_X[128 x 192] += G^T W_t[:, own]   v_mfma_f32_16x16x32_bf16, W via ds_read_b64_tr_b8
//               A^T[192 x 64]     = X^T G^T             v_mfma_f32_16x16x32_bf16, G via ds_read_b64_tr_b16
//               W_t[:, own]       = round(W - lr A)     in LDS, then 16-byte stores
// A member may overwrite its columns of tile t only after every member has published G(t), i.e. has finished
// reading the rows of tile t; the counters guarantee it.  All waits on counters are bounded and raise an
// error word instead of hanging.
//
// Reference semantics: src/xmc_classifiers/chunked_fp8xmc_clf.py:81-123 with
// src/triton_kernels/matmul_kernel.py:204-239 (grad_X) and src/triton_kernels/fuse_kernel.py:63-113 (update).
#include "xmc_common.h"

namespace xmc {

constexpr int QNT = 512;                  // threads per workgroup (8 wavefronts)
constexpr int QCOLS = D / 4;              // features owned by one member (192)
constexpr int QWS = QCOLS + 16;           // LDS row stride of the own-column tile image (13 x 16 bytes)
constexpr int QWC_BYTES = TL * QWS;       // 13312
constexpr int QRING = 5;                  // own-column tile images in flight
constexpr int QPL_S = TL * 2 + 16;        // bytes per batch row of a G plane ([32 b][64 l] bf16 + pad)
constexpr int QPLANE = 5120;              // bytes per plane (32 x 144 = 4608, padded to 5 KiB)
constexpr int QG_BYTES = 4 * QPLANE;      // one gathered G tile
constexpr int QZ_BYTES = 8 * 2 * 64 * 16; // partial logits of the 8 wavefronts
constexpr int QSLOTS = 4;                 // exchange slots per quad
constexpr int QLDS_BYTES = QRING * QWC_BYTES + 2 * QG_BYTES + 2 * QZ_BYTES;
constexpr int QSPIN_LIMIT = 1 << 18;

struct QuadParams {
  unsigned char* chunk[MAX_CHUNKS];   // device pointers of the chunk weight tensors [rows_per_chunk, 768] e4m3
  unsigned seed[MAX_CHUNKS];          // per-chunk rounding seed
  int num_chunks;
  int rows_per_chunk;
  int tiles_per_chunk;
  int num_tiles;
  const unsigned char* xq;            // logits operands (prep_x_quad_kernel layout)
  const bf16x8* xt;                   // grad_W operands
  const unsigned* keys;               // sorted positives: label*256 + batch_row
  const int* tile_ptr;                // [num_tiles+1] offsets into keys
  floatx4* partial;                   // [gridDim.x][12][512] per-workgroup grad_X partial sums
  unsigned char* exch;                // [nquads][QSLOTS][4][QPLANE] G exchange ring
  int* flags;                         // [nquads][4] tiles-published counters; [nquads*4] error word; then xcc ids
  float zscale;                       // scale_w * scale_x applied to the logits accumulator
  float lr_eff;                       // lr / scale_w
  int batch;
};

#ifndef XMC_DBG_SKIP
#define XMC_DBG_SKIP 0   // timing experiments only: bit mask of phases to leave out (results are then wrong)
#endif
#ifndef XMC_DBG_TIMING
#define XMC_DBG_TIMING 0   // 1: workgroup 0 records wall-clock stamps of its first 48 iterations behind the flags
#endif
#define QSTAMP(k) do { if (XMC_DBG_TIMING && g == 0 && lane == 0 && i >= 8 && i < 14) \
    ((unsigned long long*)(lds_raw + QLDS_BYTES))[(w * 6 + (i - 8)) * 16 + (k)] = wall_clock64(); } while (0)
typedef __attribute__((address_space(3))) unsigned char qlds_u8;

// 16 bytes per lane from global memory straight into LDS at lds_wave_base + 16*lane (wave-uniform base).
// Issued through inline assembly on purpose: the compiler orders every later LDS access behind a direct-to-LDS
// load it knows about, which would serialise the prefetch.  Completion is enforced by hand (s_waitcnt vmcnt +
// barrier) before the data is read.  An operation the compiler does not count only makes its own counted
// waits stricter, never weaker, because vector memory operations retire in order.
__device__ __forceinline__ void q_lds_load16(const unsigned char* g, unsigned char* lds_wave_base) {
  const unsigned ldsoff = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(qlds_u8*)lds_wave_base);
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(ldsoff), "v"(g) : "memory", "m0");
}
// same, at device scope (sc1): served by the XCD's L2, never by this compute unit's L1, which may still hold
// the previous contents of an exchange slot
__device__ __forceinline__ void q_lds_load16_l2(const unsigned char* g, unsigned char* lds_wave_base) {
  const unsigned ldsoff = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(qlds_u8*)lds_wave_base);
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off sc1" : : "s"(ldsoff), "v"(g) : "memory", "m0");
}

__device__ __forceinline__ intx2 q_lds_tr8(const unsigned char* q) {
  return __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) intx2*)(qlds_u8*)q);
}
typedef short shortx4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ shortx4 q_lds_tr16(const unsigned char* q) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4*)(qlds_u8*)q);
}

__device__ __forceinline__ bf16x8 q_fp8x8_to_bf16x8(intx2 raw) {
  floatx2 f01 = __builtin_amdgcn_cvt_pk_f32_fp8(raw.x, false), f23 = __builtin_amdgcn_cvt_pk_f32_fp8(raw.x, true);
  floatx2 f45 = __builtin_amdgcn_cvt_pk_f32_fp8(raw.y, false), f67 = __builtin_amdgcn_cvt_pk_f32_fp8(raw.y, true);
  return bf16x8{(__bf16)f01.x, (__bf16)f01.y, (__bf16)f23.x, (__bf16)f23.y,
                (__bf16)f45.x, (__bf16)f45.y, (__bf16)f67.x, (__bf16)f67.y};
}

// Everything the kernel needs to know about one tile; wave-uniform, kept in scalar registers and computed
// several iterations before it is used so that the scalar-memory latency stays off the critical path.
struct QTile { unsigned char* base; int c, row0, rows_valid, p0, p1; unsigned seed; };

__device__ __forceinline__ QTile q_tile(const QuadParams& p, int t) {
  QTile q;
  const __attribute__((address_space(4))) int* ctile_ptr = (const __attribute__((address_space(4))) int*)p.tile_ptr;
  const bool valid = t < p.num_tiles;
  const int tt = valid ? t : 0;
  q.c = tt / p.tiles_per_chunk;
  q.row0 = (tt - q.c * p.tiles_per_chunk) * TL;
  q.rows_valid = min(TL, p.rows_per_chunk - q.row0);
  q.base = p.chunk[q.c] + (size_t)q.row0 * D;
  q.seed = p.seed[q.c];
  q.p0 = ctile_ptr[tt];
  q.p1 = valid ? ctile_ptr[tt + 1] : q.p0;
  return q;
}

template <int MODE>
__global__ __launch_bounds__(QNT) void fp8_step_quad_kernel(const QuadParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  unsigned char* wcol0 = lds_raw;
  unsigned char* gbuf0 = lds_raw + QRING * QWC_BYTES;
  unsigned char* zbuf0 = gbuf0 + 2 * QG_BYTES;

  const int tid = threadIdx.x;
  const int w = tid >> 6, lane = tid & 63, l16 = lane & 15, kg = lane >> 4;
  const int g = blockIdx.x;
  const int xcd = g & 7, j = g >> 3, m = j & 3;
  const int nquads = gridDim.x >> 2;
  const int quad = (j >> 2) * 8 + xcd;
  const int rb = w & 3, kh = w >> 2;       // logits: rows 16rb.., K half kh; afterwards batch block kh
  const int cgrp = w & 3, hi = w >> 2;     // gradients: features 48cgrp.. of this member, batch/row half hi
  const int n_it = quad < p.num_tiles ? (p.num_tiles - quad + nquads - 1) / nquads : 0;

  // the sorted keys are written before this kernel starts: read them through the scalar (constant) path
  const __attribute__((address_space(4))) unsigned* ckeys = (const __attribute__((address_space(4))) unsigned*)p.keys;
  int* flags = p.flags + quad * 4;
  int* errw = p.flags + nquads * 4;
  if (tid == 0) p.flags[nquads * 4 + 1 + g] = (int)(__builtin_amdgcn_s_getreg((3 << 11) | 20) & 15);   // XCC_ID

  // ---- resident operands
  intx8 xq[2][3];
#pragma unroll
  for (int nbk = 0; nbk < 2; nbk++)
#pragma unroll
    for (int ks3 = 0; ks3 < 3; ks3++)
      xq[nbk][ks3] = *(const intx8*)(p.xq + ((size_t)((((m * 2 + kh) * 2 + nbk) * 3 + ks3) * 64 + lane)) * 32);
  bf16x8 xt[3][4];
#pragma unroll
  for (int cg = 0; cg < 3; cg++)
#pragma unroll
    for (int ks = 0; ks < 4; ks++) xt[cg][ks] = p.xt[(size_t)(((4 * m + cgrp) * 3 + cg) * 4 + ks) * 64 + lane];
  floatx4 acc2[4][3];
#pragma unroll
  for (int a = 0; a < 4; a++)
#pragma unroll
    for (int b = 0; b < 3; b++) acc2[a][b] = floatx4{0.f, 0.f, 0.f, 0.f};

  // own-column tile image: 64 rows x 13 chunks of 16 bytes (12 data + 1 pad) = 13 wave-wide loads; every
  // wavefront issues exactly two (three of the sixteen are harmless repeats)
  auto issue_wcol = [&](int i, const QTile& q) {
    if (i >= n_it || (XMC_DBG_SKIP & 32)) return;
    unsigned char* dst = wcol0 + (i % QRING) * QWC_BYTES;
#pragma unroll
    for (int s = 0; s < 2; s++) {
      int piece = (w + 8 * s) % 13;
      int ch = piece * 64 + lane;
      int row = ch / 13, cc = ch - row * 13;
      row = min(row, q.rows_valid - 1);
      cc = min(cc, 11);
      q_lds_load16(q.base + (size_t)row * D + QCOLS * m + cc * 16, dst + piece * 1024);
    }
  };
  // rows of tile i as logits operands: lane (row 16rb + l16, k group kg) holds 32 consecutive bytes per K step
  auto load_a = [&](int i, const QTile& q, uint4 (&a)[6]) {
    if (i >= n_it || (XMC_DBG_SKIP & 512)) return;
    const unsigned char* src = q.base + (size_t)min(16 * rb + l16, q.rows_valid - 1) * D + kh * 384 + kg * 32;
#pragma unroll
    for (int ks3 = 0; ks3 < 3; ks3++) {
      a[2 * ks3] = *(const uint4*)(src + ks3 * 128);
      a[2 * ks3 + 1] = *(const uint4*)(src + ks3 * 128 + 16);
    }
  };
  // logits of tile i over this wavefront's K half, left in LDS (buffer i&1) for the other K half to add
  auto logits = [&](int i, const uint4 (&a)[6]) {
    if (i >= n_it) return;
    floatx4 z[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
    if (!(XMC_DBG_SKIP & 1))
#pragma unroll
    for (int ks3 = 0; ks3 < 3; ks3++) {
      intx8 av = intx8{(int)a[2 * ks3].x, (int)a[2 * ks3].y, (int)a[2 * ks3].z, (int)a[2 * ks3].w,
                       (int)a[2 * ks3 + 1].x, (int)a[2 * ks3 + 1].y, (int)a[2 * ks3 + 1].z, (int)a[2 * ks3 + 1].w};
      z[0] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, xq[0][ks3], z[0], 0, 0, 0, 0, 0, 0);
      z[1] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, xq[1][ks3], z[1], 0, 0, 0, 0, 0, 0);
    }
    unsigned char* zb = zbuf0 + (i & 1) * QZ_BYTES;
    *(floatx4*)(zb + ((w * 2 + 0) * 64 + lane) * 16) = z[0];
    *(floatx4*)(zb + ((w * 2 + 1) * 64 + lane) * 16) = z[1];
  };
  // after a barrier: G = bf16(sigmoid(bf16(Z))) - [positive] for rows 16rb.., batch block kh of this member,
  // stored to the exchange slot of tile i in [b][l] order (published later, once the stores have completed)
  auto sigmoid_store = [&](int i, const QTile& q) {
    if (i >= n_it) return;
    const unsigned char* zb = zbuf0 + (i & 1) * QZ_BYTES;
    floatx4 s0 = *(const floatx4*)(zb + ((rb * 2 + kh) * 64 + lane) * 16);         // K half 0
    floatx4 s1 = *(const floatx4*)(zb + (((rb + 4) * 2 + kh) * 64 + lane) * 16);   // K half 1
    const float nlog2e = -1.44269504088896340736f;
    const int r0 = 16 * rb + 4 * kg;
    float sg[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      float zf = bf16_rt((s0[e] + s1[e]) * p.zscale);
      float v = (XMC_DBG_SKIP & 2) ? zf : __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(zf * nlog2e));
      sg[e] = bf16_rt(v);
    }
    // positives of this tile (set semantics: a repeated key counts once); wave-uniform scalar loads
    const int p0 = q.p0, p1 = q.p1;
    if (p1 > p0) {
      const unsigned label0 = (unsigned)(q.c * p.rows_per_chunk + q.row0);
      const unsigned myb = (unsigned)(32 * m + 16 * kh + l16);
      for (int e = p0; e < p1; e++) {
        const unsigned key = ckeys[e];
        const unsigned prev = e > 0 ? ckeys[e - 1] : ~key;
        const unsigned l = (key >> 8) - label0 - (unsigned)r0;
        if (prev != key && (key & 255u) == myb && l < 4u) {
#pragma unroll
          for (int q4 = 0; q4 < 4; q4++)
            if (l == (unsigned)q4) sg[q4] = bf16_rt(sg[q4] - 1.0f);
        }
      }
    }
    unsigned short sb[4];
#pragma unroll
    for (int e = 0; e < 4; e++) sb[e] = (r0 + e < q.rows_valid) ? bf16_bits(sg[e]) : (unsigned short)0;
    uint2 v;
    v.x = (unsigned)sb[0] | ((unsigned)sb[1] << 16);
    v.y = (unsigned)sb[2] | ((unsigned)sb[3] << 16);
    unsigned char* plane = p.exch + ((size_t)((quad * QSLOTS + (i & (QSLOTS - 1))) * 4 + m)) * QPLANE;
    *(uint2*)(plane + (16 * kh + l16) * QPL_S + r0 * 2) = v;
  };
  // wait until every member has published at least `need` tiles (f: an earlier reading of the counters)
  auto wait_published = [&](int need, int f) {
    if (XMC_DBG_SKIP & 128) return;
    for (int spin = 0;; spin++) {
      int ok = f >= need;
      if (__builtin_amdgcn_read_exec() == __builtin_amdgcn_ballot_w64(ok)) break;
      if (spin >= QSPIN_LIMIT || ((spin & 1023) == 1023 && __hip_atomic_load(errw, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
        if (lane == 0) __hip_atomic_store(errw, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
      __builtin_amdgcn_s_sleep(2);
      f = __hip_atomic_load(flags + (lane & 3), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  };
  // gather the four G parts of tile i: 20 wave-wide loads of 1 KiB, three per wavefront (four repeats)
  auto issue_gather = [&](int i) {
    if (i >= n_it || (XMC_DBG_SKIP & 256)) return;
    const unsigned char* src = p.exch + ((size_t)((quad * QSLOTS + (i & (QSLOTS - 1))) * 4)) * QPLANE;
    unsigned char* dst = gbuf0 + (i & 1) * QG_BYTES;
#pragma unroll
    for (int s = 0; s < 3; s++) {
      int piece = (w + 8 * s) % 20;
      q_lds_load16_l2(src + piece * 1024 + lane * 16, dst + piece * 1024);
    }
  };

  // ---- prologue: own columns of tiles 0..3 in flight, logits of tiles 0..2, G of tiles 0 and 1 stored,
  //      gather of tile 0 issued
  uint4 areg[6];
  // inf[k] describes the tile k positions ahead of the current one
  QTile inf[5];
#pragma unroll
  for (int k = 0; k < 5; k++) inf[k] = q_tile(p, quad + nquads * k);
  issue_wcol(0, inf[0]); issue_wcol(1, inf[1]); issue_wcol(2, inf[2]); issue_wcol(3, inf[3]);
  load_a(0, inf[0], areg); logits(0, areg);
  load_a(1, inf[1], areg);
  __syncthreads();
  sigmoid_store(0, inf[0]); logits(1, areg);
  load_a(2, inf[2], areg);
  __syncthreads();
  sigmoid_store(1, inf[1]); logits(2, areg);
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (tid == 0 && n_it > 0) __hip_atomic_store(flags + m, min(2, n_it), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (n_it > 0) wait_published(1, 0);
  issue_gather(0);

  for (int i = 0; i < n_it; i++) {
    const QTile q = inf[0];
    const unsigned char* wc = wcol0 + (i % QRING) * QWC_BYTES;
    const unsigned char* gb = gbuf0 + (i & 1) * QG_BYTES;
    const unsigned seed = q.seed;
    // tile five positions ahead: its scalar loads complete under the wait below
    const QTile qnew = q_tile(p, quad + nquads * (i + 5));

    // everything issued during the previous iteration has landed: G of tile i, own columns up to tile i+3,
    // this member's G part of tile i+1; the K-half logits of tile i+2 are in LDS
    QSTAMP(0);
    __builtin_amdgcn_s_waitcnt(0);
    QSTAMP(1);
    __syncthreads();
    QSTAMP(2);
    if (tid == 0 && i + 1 < n_it) __hip_atomic_store(flags + m, i + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    sigmoid_store(i + 2, inf[2]);
    load_a(i + 3, inf[3], areg);
    issue_wcol(i + 4, inf[4]);
    QSTAMP(3);

    // ---- grad_X[64 batch rows of half hi x 48 features] += G^T W
    if (!(XMC_DBG_SKIP & 4))
#pragma unroll
    for (int ks2 = 0; ks2 < 2; ks2++) {
      bf16x8 ga[4];
#pragma unroll
      for (int mb = 0; mb < 4; mb++)
        ga[mb] = *(const bf16x8*)(gb + (2 * hi + (mb >> 1)) * QPLANE + (16 * (mb & 1) + l16) * QPL_S + ks2 * 64 + kg * 16);
#pragma unroll
      for (int nn = 0; nn < 3; nn++) {
        intx2 raw = q_lds_tr8(wc + (32 * ks2 + 8 * kg + (l16 >> 1)) * QWS + 48 * cgrp + 16 * nn + (l16 & 1) * 8);
        bf16x8 wb = q_fp8x8_to_bf16x8(raw);
#pragma unroll
        for (int mb = 0; mb < 4; mb++)
          acc2[mb][nn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ga[mb], wb, acc2[mb][nn], 0, 0, 0);
      }
    }
    QSTAMP(4);
    // an early look at the counters needed for the gather at the end of this iteration
    int fseen = __hip_atomic_load(flags + (lane & 3), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    // ---- A^T[48 features x 32 rows of half hi] = X^T G^T, then the update, straight from registers to memory.
    //      Row r = 4kg+e of feature block cg is feature 12kg + 4cg + e of the wavefront's 48, so that a lane
    //      ends up with 12 consecutive bytes of one weight row.
    {
      floatx4 acc3[3][2];
#pragma unroll
      for (int cg = 0; cg < 3; cg++) { acc3[cg][0] = floatx4{0.f, 0.f, 0.f, 0.f}; acc3[cg][1] = floatx4{0.f, 0.f, 0.f, 0.f}; }
      if (!(XMC_DBG_SKIP & 8))
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        bf16x8 bg[2];
#pragma unroll
        for (int nb = 0; nb < 2; nb++) {
          const unsigned char* src = gb + ks * QPLANE + (8 * kg + (l16 >> 2)) * QPL_S + (32 * hi + 16 * nb + 4 * (l16 & 3)) * 2;
          shortx4 lo = q_lds_tr16(src), hi4 = q_lds_tr16(src + 4 * QPL_S);
          typedef short shortx8 __attribute__((ext_vector_type(8)));
          shortx8 both = shortx8{lo[0], lo[1], lo[2], lo[3], hi4[0], hi4[1], hi4[2], hi4[3]};
          bg[nb] = __builtin_bit_cast(bf16x8, both);
        }
#pragma unroll
        for (int cg = 0; cg < 3; cg++) {
          acc3[cg][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xt[cg][ks], bg[0], acc3[cg][0], 0, 0, 0);
          acc3[cg][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xt[cg][ks], bg[1], acc3[cg][1], 0, 0, 0);
        }
      }
      QSTAMP(5);
      if (!(XMC_DBG_SKIP & 16))
#pragma unroll
      for (int nb = 0; nb < 2; nb++) {
        const int row = 32 * hi + 16 * nb + l16;
        const int lcol = 48 * cgrp + 12 * kg;
        const unsigned* wp = (const unsigned*)(wc + row * QWS + lcol);
        unsigned outw[3];
#pragma unroll
        for (int cg = 0; cg < 3; cg++) {
          const unsigned wq = wp[cg];
          floatx2 w01 = __builtin_amdgcn_cvt_pk_f32_fp8((int)wq, false), w23 = __builtin_amdgcn_cvt_pk_f32_fp8((int)wq, true);
          floatx4 a = acc3[cg][nb];
          float t0 = __builtin_fmaf(-p.lr_eff, a[0], w01.x), t1 = __builtin_fmaf(-p.lr_eff, a[1], w01.y);
          float t2 = __builtin_fmaf(-p.lr_eff, a[2], w23.x), t3 = __builtin_fmaf(-p.lr_eff, a[3], w23.y);
          outw[cg] = round4<MODE>(t0, t1, t2, t3, (unsigned)(q.row0 + row), (unsigned)(q.c * p.rows_per_chunk + q.row0 + row),
                                  (unsigned)(QCOLS * m + lcol + 4 * cg), seed);
        }
        if (row < q.rows_valid && !(XMC_DBG_SKIP & 64)) {
          unsigned* gp = (unsigned*)(q.base + (size_t)row * D + QCOLS * m + lcol);
          gp[0] = outw[0]; gp[1] = outw[1]; gp[2] = outw[2];
        }
      }
    }
    QSTAMP(7);

    // ---- G of the next tile (published by every member at the top of its current iteration or earlier)
    if (i + 1 < n_it) {
      wait_published(i + 2, fseen);
      QSTAMP(10);
      issue_gather(i + 1);
    }
    QSTAMP(11);
    // ---- logits three tiles ahead
    logits(i + 3, areg);
    QSTAMP(12);
#pragma unroll
    for (int k = 0; k < 4; k++) inf[k] = inf[k + 1];
    inf[4] = qnew;
  }
  if (XMC_DBG_TIMING && g == 0) {
    __syncthreads();
    for (int e = tid; e < 48 * 16; e += QNT)
      ((unsigned long long*)(p.flags + 1024))[e] = ((unsigned long long*)(lds_raw + QLDS_BYTES))[e];
  }
  // ---- per-workgroup grad_X partial, summed in a fixed order by reduce_gx_quad_kernel
  floatx4* dst = p.partial + (size_t)g * 12 * QNT;
#pragma unroll
  for (int mb = 0; mb < 4; mb++)
#pragma unroll
    for (int nn = 0; nn < 3; nn++) dst[(mb * 3 + nn) * QNT + tid] = acc2[mb][nn];
}

// grad_X = scale * sum over quads of the member partials; writes fp32 and bf16 [batch, 768]
__global__ __launch_bounds__(QNT) void reduce_gx_quad_kernel(const floatx4* partial, int nwg, float scale, float* gx_f32,
                                                             unsigned short* gx_bf16, int batch) {
  const int slot = blockIdx.x >> 2, m = blockIdx.x & 3;   // slot = mb*3+nn
  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, l16 = lane & 15, kg = lane >> 4;
  floatx4 s = {0.f, 0.f, 0.f, 0.f};
  for (int g = 0; g < nwg; g++) {
    if (((g >> 3) & 3) != m) continue;
    s += partial[((size_t)g * 12 + slot) * QNT + tid];
  }
  const int mb = slot / 3, nn = slot - mb * 3;
  const int col = QCOLS * m + 48 * (w & 3) + 16 * nn + l16;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    int b = 64 * (w >> 2) + 16 * mb + 4 * kg + i;
    if (b < batch) {
      float v = s[i] * scale;
      if (gx_f32) gx_f32[(size_t)b * D + col] = v;
      if (gx_bf16) gx_bf16[(size_t)b * D + col] = bf16_bits(v);
    }
  }
}

// Operand images of X for the quad kernel.
//   xq: e4m3(X / scale_x) in v_mfma 16x16x128 B-operand order, K split in halves:
//       operand index (((m*2 + kh)*2 + nbk)*3 + ks3), lane = (b%16) + 16*kg, byte j:
//       Xq[b = 32m + 16nbk + b%16][k = 384kh + 128ks3 + 32kg + j]
//   xt: bf16 X^T in v_mfma 16x16x32 A-operand order: [((col/48)*3 + cg)*4 + ks][lane][8 bf16], lane = r + 16*kg,
//       element j = X[32ks + 8kg + j][col] with col = 48*(col/48) + 12*(r/4) + 4*cg + r%4
__global__ void prep_x_quad_kernel(const unsigned short* x, int batch, float inv_scale_x, unsigned char* xq, unsigned short* xt) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;   // one thread per (b, group of 4 features)
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
    int m = b >> 5, nbk = (b >> 4) & 1, n = b & 15;
    int kh = k / 384, kr = k - kh * 384;
    int ks3 = kr >> 7, kgq = (kr >> 5) & 3, jq = kr & 31;
    size_t off = ((size_t)((((m * 2 + kh) * 2 + nbk) * 3 + ks3) * 64 + (n + 16 * kgq))) * 32 + jq;
    *(int*)(xq + off) = packed;
  }
#pragma unroll
  for (int q = 0; q < 4; q++) {
    int col = k + q;
    int G = col / 48, c48 = col - G * 48;
    int kq = c48 / 12, rem = c48 - kq * 12, cg = rem >> 2, r = 4 * kq + (rem & 3);
    int ks = b >> 5, kgq = (b >> 3) & 3, jq = b & 7;
    size_t off = ((size_t)((G * 3 + cg) * 4 + ks) * 64 + (r + 16 * kgq)) * 8 + jq;
    xt[off] = raw[q];
  }
}

}  // namespace xmc