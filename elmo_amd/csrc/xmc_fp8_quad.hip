// Fused FP8 extreme-classifier training step for gfx950 (MI355X): four compute units per tile stream.
//
// Work unit = a tile of 64 consecutive label rows of one chunk (64 x 768 e4m3 bytes, contiguous in HBM).
// Four workgroups on the same XCD (a "quad") walk the same tile sequence, one workgroup per compute unit,
// 4 wavefronts each (one per SIMD, 512 registers).  Member m of the quad owns
//   * label rows 16m..16m+15 of every tile for the logits and the sigmoid ("stage A"), and
//   * input features 192m..192m+191 for grad_X, grad_W and the in-place update ("stage B"),
// so no arithmetic is repeated and every weight byte is read from HBM once and written once per step.  A member
// reads 24 KiB per tile (its rows and its columns), always as whole 16-byte pieces of contiguous row segments
// sent straight to LDS: the vector memory path of a compute unit handles few cache lines per clock, and
// register loads in MFMA operand order (16 rows x 64 bytes per instruction) would keep it busy longer than
// the MFMAs run.
// The only data the members exchange is G = sigmoid(logits) - target in bf16 (4 KiB per member and tile),
// through a small ring of slots in global memory, guarded by per-member "tiles published" counters.  Stage A runs three tiles ahead of stage B, so neither the exchange nor the
// counters are on the critical path.  Neither logits nor gradients ever reach HBM; the X operands of all three
// GEMMs and the grad_X accumulators (96 KiB per compute unit) live in registers for the whole launch.
//
//   stage A(t): Z[16 x 128] = W_t[16m.., :] Xq^T  v_mfma_f32_16x16x128_f8f6f4; wavefront w takes batch rows 32w..32w+31,
//                                              the 16 W rows are read from LDS by all four wavefronts
//               G = bf16(sigmoid(bf16(Z))) - [positive], stored to the exchange slot in [b][l] order
//   stage B(t): the whole G tile arrives in LDS by global_load_lds; wavefront w takes features 48w..48w+47
//               grad_X[128 x 48] += G^T W_t      v_mfma_f32_16x16x32_bf16, W via ds_read_b64_tr_b8 + fp8->bf16
//               A^T[48 x 64]     = X^T G^T        v_mfma_f32_16x16x32_bf16, G via ds_read_b64_tr_b16
//               W_t              = round(W - lr A) from registers to memory, 12 bytes per lane
// A member may overwrite its columns of tile t only after every member has published G(t), i.e. has finished
// reading the rows of tile t; the counters guarantee it.  All waits on counters are bounded and raise an
// error word instead of hanging.
//
// Reference semantics: src/xmc_classifiers/chunked_fp8xmc_clf.py:81-123 with
// src/triton_kernels/matmul_kernel.py:204-239 (grad_X) and src/triton_kernels/fuse_kernel.py:63-113 (update).
#include "xmc_common.h"

namespace xmc {

constexpr int QNT = 256;                  // threads per workgroup (4 wavefronts)
constexpr int QCOLS = D / 4;              // features owned by one member (192)
constexpr int QWS = QCOLS + 16;           // LDS row stride of the own-column tile image (13 x 16 bytes)
constexpr int QWC_BYTES = TL * QWS;       // 13312
constexpr int QRING = 6;                  // own-column tile images in flight
constexpr int QPL_S = TL * 2 + 16;        // bytes per batch row of the G tile ([128 b][64 l] bf16 + pad)
constexpr int QG_BYTES = 20480;           // one G tile (128 x 144 = 18432), padded to 20 wave-wide loads
constexpr int QSLOTS = 8;                 // exchange slots per quad
constexpr int QLDS_G = QRING * QWC_BYTES; // LDS offset of the two gathered-G buffers
constexpr int QRS = D + 16;               // LDS row stride of the own-rows image (49 x 16 bytes)
constexpr int QROW_BYTES = 13 * 1024;     // 16 rows x 784 = 12544, padded to 13 wave-wide loads
constexpr int QRRING = 3;                 // own-rows images in flight
constexpr int QLDS_R = QLDS_G + 2 * QG_BYTES;
constexpr int QLDS_BYTES = QLDS_R + QRRING * QROW_BYTES;
constexpr int QSPIN_LIMIT = 1 << 18;
constexpr int QAHEAD = 4;                 // stage A runs this many tiles ahead of stage B
constexpr int QINF = QAHEAD + 3;          // tile descriptors held in scalar registers

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
  const uint4* desc;                  // [num_tiles][2] tile descriptors written by tile_desc_kernel
  floatx4* partial;                   // [gridDim.x][24][256] per-workgroup grad_X partial sums
  unsigned char* exch;                // [nquads][QSLOTS][QG_BYTES] G exchange ring
  int* flags;                         // [nquads][4] tiles-published counters; [nquads*4] error word; then xcc ids
  float zscale;                       // scale_w * scale_x applied to the logits accumulator
  float lr_eff;                       // lr / scale_w
  int batch;
};

#ifndef XMC_DBG_SKIP
#define XMC_DBG_SKIP 0   // timing experiments only: bit mask of phases to leave out (results are then wrong)
#endif
#ifdef XMC_TIMING   // timing experiments only: per-wavefront clock totals of the phases of the main loop
#define QT_DECL unsigned long long tprev = __builtin_amdgcn_s_memtime(); unsigned tacc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#define QT(k) { __builtin_amdgcn_sched_barrier(0); unsigned long long tn = __builtin_amdgcn_s_memtime(); tacc[k] += (unsigned)(tn - tprev); tprev = tn; __builtin_amdgcn_sched_barrier(0); }
#else
#define QT_DECL
#define QT(k)
#endif
#define QFENCE() __builtin_amdgcn_sched_barrier(0)   // nothing is scheduled across this point
typedef __attribute__((address_space(3))) unsigned char qlds_u8;
typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef short shortx8 __attribute__((ext_vector_type(8)));

// 16 bytes per lane from global memory straight into LDS at byte offset ldsoff + 16*lane (wave-uniform offset).
// Issued through inline assembly on purpose: the compiler orders every later LDS access behind a direct-to-LDS
// load it knows about, which would serialise the prefetch.  Completion is enforced by hand (s_waitcnt vmcnt +
// barrier) before the data is read.  An operation the compiler does not count only makes its own counted
// waits stricter, never weaker, because vector memory operations retire in order.
__device__ __forceinline__ void q_lds_load16(const unsigned char* g, unsigned ldsoff_) {
  const unsigned ldsoff = __builtin_amdgcn_readfirstlane(ldsoff_);
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(ldsoff), "v"(g) : "memory", "m0");
}
// same, at device scope (sc1): served by the XCD's L2, never by this compute unit's L1, which may still hold
// the previous contents of an exchange slot
__device__ __forceinline__ void q_lds_load16_l2(const unsigned char* g, unsigned ldsoff_) {
  const unsigned ldsoff = __builtin_amdgcn_readfirstlane(ldsoff_);
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off sc1" : : "s"(ldsoff), "v"(g) : "memory", "m0");
}

__device__ __forceinline__ bf16x8 q_fp8x8_to_bf16x8(intx2 raw) {
  floatx2 f01 = __builtin_amdgcn_cvt_pk_f32_fp8(raw.x, false), f23 = __builtin_amdgcn_cvt_pk_f32_fp8(raw.x, true);
  floatx2 f45 = __builtin_amdgcn_cvt_pk_f32_fp8(raw.y, false), f67 = __builtin_amdgcn_cvt_pk_f32_fp8(raw.y, true);
  return bf16x8{(__bf16)f01.x, (__bf16)f01.y, (__bf16)f23.x, (__bf16)f23.y,
                (__bf16)f45.x, (__bf16)f45.y, (__bf16)f67.x, (__bf16)f67.y};
}

// Everything the kernel needs to know about one tile; wave-uniform, kept in scalar registers.  The descriptors are
// precomputed by tile_desc_kernel and fetched with ordinary vector loads several iterations ahead, so that they
// travel in the same in-order queue as the other prefetches and never stall the wavefront the way a scalar load
// followed by an LDS wait would.
struct QTile { unsigned char* base; unsigned label0; int row0, rows_valid, p0, p1; unsigned seed; };

__device__ __forceinline__ QTile q_from_desc(uint4 d0, uint4 d1) {
  QTile q;
  const unsigned lo = __builtin_amdgcn_readfirstlane(d0.x), hi = __builtin_amdgcn_readfirstlane(d0.y);
  q.base = (unsigned char*)(((unsigned long long)hi << 32) | lo);
  q.seed = __builtin_amdgcn_readfirstlane(d0.z);
  q.p0 = (int)__builtin_amdgcn_readfirstlane(d0.w);
  q.p1 = (int)__builtin_amdgcn_readfirstlane(d1.x);
  q.row0 = (int)__builtin_amdgcn_readfirstlane(d1.y);
  q.rows_valid = (int)__builtin_amdgcn_readfirstlane(d1.z);
  q.label0 = __builtin_amdgcn_readfirstlane(d1.w);
  return q;
}

// desc[t] = {base pointer, seed, first key, one past last key | row in chunk, valid rows, first label, -}
__global__ void tile_desc_kernel(const QuadParams p, uint4* desc) {
  int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= p.num_tiles) return;
  const int c = t / p.tiles_per_chunk;
  const int row0 = (t - c * p.tiles_per_chunk) * TL;
  const unsigned long long base = (unsigned long long)(p.chunk[c] + (size_t)row0 * D);
  desc[2 * t] = uint4{(unsigned)base, (unsigned)(base >> 32), p.seed[c], (unsigned)p.tile_ptr[t]};
  desc[2 * t + 1] = uint4{(unsigned)p.tile_ptr[t + 1], (unsigned)row0, (unsigned)min(TL, p.rows_per_chunk - row0),
                          (unsigned)(c * p.rows_per_chunk + row0)};
}

template <int MODE>
__global__ __launch_bounds__(QNT, 1) void fp8_step_quad_kernel(const QuadParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  qlds_u8* lds = (qlds_u8*)lds_raw;

  const int tid = threadIdx.x;
  const int w = tid >> 6, lane = tid & 63, l16 = lane & 15, kg = lane >> 4;
  const int g = blockIdx.x;
  const int xcd = g & 7, j = g >> 3, m = j & 3;
  const int nquads = gridDim.x >> 2;
  const int quad = (j >> 2) * 8 + xcd;
  const int n_it = quad < p.num_tiles ? (p.num_tiles - quad + nquads - 1) / nquads : 0;

  // the sorted keys are written before this kernel starts: read them through the scalar (constant) path
  const __attribute__((address_space(4))) unsigned* ckeys = (const __attribute__((address_space(4))) unsigned*)p.keys;
  int* flags = p.flags + quad * 4;
  int* errw = p.flags + nquads * 4;
  if (tid == 0) p.flags[nquads * 4 + 1 + g] = (int)(__builtin_amdgcn_s_getreg((3 << 11) | 20) & 15);   // XCC_ID

  // ---- resident operands
  intx8 xq[2][6];      // logits: batch blocks 32w + 16nb.., K steps of 128
#pragma unroll
  for (int nb = 0; nb < 2; nb++)
#pragma unroll
    for (int ks = 0; ks < 6; ks++)
      xq[nb][ks] = *(const intx8*)(p.xq + ((size_t)(((w * 2 + nb) * 6 + ks) * 64 + lane)) * 32);
  bf16x8 xt[3][4];     // grad_W: feature blocks of this wavefront's 48 features, K steps of 32 batch rows
#pragma unroll
  for (int cg = 0; cg < 3; cg++)
#pragma unroll
    for (int ks = 0; ks < 4; ks++) xt[cg][ks] = p.xt[(size_t)(((4 * m + w) * 3 + cg) * 4 + ks) * 64 + lane];
  floatx4 acc2[8][3];  // grad_X[128 batch rows x 48 features]
#pragma unroll
  for (int a = 0; a < 8; a++)
#pragma unroll
    for (int b = 0; b < 3; b++) acc2[a][b] = floatx4{0.f, 0.f, 0.f, 0.f};

  QT_DECL
  // own-column tile image: 64 rows x 13 chunks of 16 bytes (12 data + 1 pad) = 13 wave-wide loads; every
  // wavefront issues exactly four (three of the sixteen are harmless repeats)
  auto wcol_piece = [&](int i, const QTile& q, int s) {
    if (i >= n_it || (XMC_DBG_SKIP & 32)) return;
    const unsigned dst = (unsigned)((i % QRING) * QWC_BYTES);
    int piece = (w + 4 * s) % 13;
    int ch = piece * 64 + lane;
    int row = ch / 13, cc = ch - row * 13;
    row = min(row, q.rows_valid - 1);
    cc = min(cc, 11);
    q_lds_load16(q.base + (size_t)row * D + QCOLS * m + cc * 16, dst + piece * 1024);
  };
  auto issue_wcol = [&](int i, const QTile& q) {
#pragma unroll
    for (int s = 0; s < 4; s++) wcol_piece(i, q, s);
  };
  // own-rows image: rows 16m..16m+15 of tile i, 16 x 49 chunks of 16 bytes (48 data + 1 pad) = 13 wave-wide loads
  auto rows_piece = [&](int i, const QTile& q, int s) {
    if (i >= n_it || (XMC_DBG_SKIP & 512)) return;
    const unsigned dst = (unsigned)(QLDS_R + (i % QRRING) * QROW_BYTES);
    int piece = (w + 4 * s) % 13;
    int ch = piece * 64 + lane;
    int row = ch / 49, cc = ch - row * 49;
    row = max(min(16 * m + min(row, 15), q.rows_valid - 1), 0);
    cc = min(cc, 47);
    q_lds_load16(q.base + (size_t)row * D + cc * 16, dst + piece * 1024);
  };
  auto issue_rows = [&](int i, const QTile& q) {
#pragma unroll
    for (int s = 0; s < 4; s++) rows_piece(i, q, s);
  };
  // stage A of tile i: logits of label rows 16m.. against batch rows 32w.., sigmoid minus target, store this
  // wavefront's part of G to the exchange slot (published later, once the stores have completed)
  auto stage_a = [&](int i, const QTile& q) {
    if (i >= n_it) return;
    floatx4 z[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
    if (!(XMC_DBG_SKIP & 1)) {
      // lane (row l16, k group kg) holds 32 consecutive bytes per K step
      const unsigned asrc = (unsigned)(QLDS_R + (i % QRRING) * QROW_BYTES) + l16 * QRS + kg * 32;
      intx4 alo[6], ahi[6];
#pragma unroll
      for (int ks = 0; ks < 6; ks++) {
        alo[ks] = *(const __attribute__((address_space(3))) intx4*)(lds + asrc + ks * 128);
        ahi[ks] = *(const __attribute__((address_space(3))) intx4*)(lds + asrc + ks * 128 + 16);
      }
#pragma unroll
      for (int ks = 0; ks < 6; ks++) {
        intx8 av = intx8{alo[ks].x, alo[ks].y, alo[ks].z, alo[ks].w, ahi[ks].x, ahi[ks].y, ahi[ks].z, ahi[ks].w};
        z[0] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, xq[0][ks], z[0], 0, 0, 0, 0, 0, 0);
        z[1] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, xq[1][ks], z[1], 0, 0, 0, 0, 0, 0);
      }
    }
    const float nlog2e = -1.44269504088896340736f;
    const int r0 = 16 * m + 4 * kg;   // this lane's label rows r0..r0+3; its batch rows are 32w + 16nb + l16
    float sg[2][4];
#pragma unroll
    for (int nb = 0; nb < 2; nb++)
#pragma unroll
      for (int e = 0; e < 4; e++) {
        float zf = bf16_rt(z[nb][e] * p.zscale);
        float v = (XMC_DBG_SKIP & 2) ? zf : __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(zf * nlog2e));
        sg[nb][e] = bf16_rt(v);
      }
    // positives of this tile (set semantics: a repeated key counts once); wave-uniform scalar loads
    if (q.p1 > q.p0) {
      const unsigned label0 = q.label0;
      for (int e = q.p0; e < q.p1; e++) {
        const unsigned key = ckeys[e];
        const unsigned prev = e > 0 ? ckeys[e - 1] : ~key;
        const unsigned l = (key >> 8) - label0 - (unsigned)r0;
        const unsigned bl = (key & 255u) - (unsigned)(32 * w) - (unsigned)l16;     // 0 or 16 for this lane's blocks
        if (prev != key && l < 4u && (bl == 0u || bl == 16u)) {
#pragma unroll
          for (int nb = 0; nb < 2; nb++)
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++)
              if (bl == (unsigned)(16 * nb) && l == (unsigned)q4) sg[nb][q4] = bf16_rt(sg[nb][q4] - 1.0f);
        }
      }
    }
    unsigned char* plane = p.exch + ((size_t)(quad * QSLOTS + (i & (QSLOTS - 1)))) * QG_BYTES + 32 * w * QPL_S;
#pragma unroll
    for (int nb = 0; nb < 2; nb++) {
      unsigned short sb[4];
#pragma unroll
      for (int e = 0; e < 4; e++) sb[e] = (r0 + e < q.rows_valid) ? bf16_bits(sg[nb][e]) : (unsigned short)0;
      uint2 v;
      v.x = (unsigned)sb[0] | ((unsigned)sb[1] << 16);
      v.y = (unsigned)sb[2] | ((unsigned)sb[3] << 16);
      *(uint2*)(plane + (16 * nb + l16) * QPL_S + r0 * 2) = v;
    }
  };
  // wait until every member has published at least `need` tiles (f: an earlier reading of the counters, which
  // normally suffices; the polling loop is kept out of the common path so that it costs no memory wait)
  auto wait_published = [&](int need, int f) {
    if (XMC_DBG_SKIP & 128) return;
    if (__builtin_amdgcn_read_exec() == __builtin_amdgcn_ballot_w64(f >= need)) return;
    for (int spin = 0;; spin++) {
      f = __hip_atomic_load(flags + (lane & 3), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (__builtin_amdgcn_read_exec() == __builtin_amdgcn_ballot_w64(f >= need)) break;
      if (spin >= QSPIN_LIMIT || ((spin & 1023) == 1023 && __hip_atomic_load(errw, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
        if (lane == 0) __hip_atomic_store(errw, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
      __builtin_amdgcn_s_sleep(2);
    }
  };
  // gather the G tile of tile i: 20 wave-wide loads of 1 KiB, five per wavefront
  auto gather_piece = [&](int i, int s) {
    if (i >= n_it || (XMC_DBG_SKIP & 256)) return;
    const unsigned char* src = p.exch + ((size_t)(quad * QSLOTS + (i & (QSLOTS - 1)))) * QG_BYTES;
    const unsigned dst = (unsigned)(QLDS_G + (i & 1) * QG_BYTES);
    int piece = w + 4 * s;
    // The slot was written by other compute units of this XCD and is read from the shared L2.  This compute unit's
    // own L1 may still hold the slot's previous contents, so the L1 (and only the L1) is invalidated first; nothing
    // else this kernel loads is ever reused from it.
    if (s == 0) asm volatile("buffer_inv sc0" ::: "memory");
    q_lds_load16(src + piece * 1024 + lane * 16, dst + piece * 1024);
  };
  auto issue_gather = [&](int i) {
#pragma unroll
    for (int s = 0; s < 5; s++) gather_piece(i, s);
  };

  // ---- prologue: own columns of tiles 0..4 in flight, stage A of the first QAHEAD tiles, own rows of the next two,
  //      gather of tile 0
  auto load_desc = [&](int i, uint4& d0, uint4& d1) {
    const int t = quad + nquads * i;
    const uint4* src = p.desc + 2 * (size_t)(t < p.num_tiles ? t : 0);
    d0 = src[0];
    d1 = src[1];
  };
  QTile inf[QINF];     // inf[k] describes the tile k positions ahead of the current one
#pragma unroll
  for (int k = 0; k < QINF; k++) {
    uint4 d0, d1;
    load_desc(k, d0, d1);
    inf[k] = q_from_desc(d0, d1);
  }
#pragma unroll
  for (int k = 0; k < 3; k++) issue_rows(k, inf[k]);
#pragma unroll
  for (int k = 0; k < 5; k++) issue_wcol(k, inf[k]);
#pragma unroll
  for (int k = 0; k < QAHEAD; k++) {
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    stage_a(k, inf[k]);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (k + 3 < QAHEAD + 2) issue_rows(k + 3, inf[k + 3]);
  }
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (tid == 0 && n_it > 0) __hip_atomic_store(flags + m, min(QAHEAD, n_it), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (n_it > 0) wait_published(1, 0);
  issue_gather(0);
  int fseen = __hip_atomic_load(flags + (lane & 3), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

  bool prev_full = false;
  for (int i = 0; i < n_it; i++) {
    const QTile q = inf[0];
    const unsigned wc = (unsigned)((i % QRING) * QWC_BYTES);
    const unsigned gb = (unsigned)(QLDS_G + (i & 1) * QG_BYTES);
    uint4 dnext0, dnext1;   // descriptor of the tile QINF positions ahead, fetched below
    // Vector memory operations retire in order.  The last four this wavefront issued in the previous iteration are
    // the stores of updated weights; everything older - G of tile i, own columns and own rows of the tiles ahead,
    // this member's G part of tile i+QAHEAD-1, the counters - was issued half an iteration earlier or more.
    // Leaving four operations in flight keeps the store latency off the critical path.  If the
    // previous tile was not full, fewer stores were issued and the count could cover loads, so all are waited for.
    if (prev_full) asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    QT(0)
    __syncthreads();
    prev_full = q.rows_valid == TL;
    if (tid == 0 && i > 0 && i + QAHEAD - 1 < n_it)
      __hip_atomic_store(flags + m, i + QAHEAD, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    QT(1)

    stage_a(i + QAHEAD, inf[QAHEAD]);
    QT(2)
    // G of the next tile was published by every member at least one full iteration ago, so the counters read at the
    // end of the previous iteration normally suffice
    if (i + 1 < n_it) wait_published(i + 2, fseen);
    // the 13 direct-to-LDS loads of this iteration (G of tile i+1, own rows of tile i+5, own columns of tile i+5),
    // issued one by one between the MFMAs below so that the memory pipeline never makes the wavefront wait
    auto mem_piece = [&](int k) {
      if (k < 5) gather_piece(i + 1, k);
      else if (k < 9) rows_piece(i + QAHEAD + 2, inf[QAHEAD + 2], k - 5);
      else if (k < 13) wcol_piece(i + 5, inf[5], k - 9);
      else load_desc(i + QINF, dnext0, dnext1);
    };
    QT(3)

    // ---- grad_X[128 x 48] += G^T W; 6 steps (32-row K step major, 16-feature block minor); the transposed W read
    //      of step s+2 and the fp8->bf16 conversion of step s+1 are issued between the MFMAs of step s
    if (!(XMC_DBG_SKIP & 4)) {
      const unsigned wsrc = wc + (8 * kg + (l16 >> 1)) * QWS + 48 * w + (l16 & 1) * 8;
      const unsigned gsrc = gb + l16 * QPL_S + kg * 16;
      bf16x8 ga[2][8];
#pragma unroll
      for (int mb = 0; mb < 8; mb++) ga[0][mb] = *(const bf16x8*)(lds + gsrc + 16 * mb * QPL_S);
      intx2 raw[3];
      raw[0] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) intx2*)(lds + wsrc));
      raw[1] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) intx2*)(lds + wsrc + 16));
      bf16x8 wb[2];
      wb[0] = q_fp8x8_to_bf16x8(raw[0]);
#pragma unroll
      for (int s = 0; s < 6; s++) {
        const int ks2 = s / 3, nn = s - ks2 * 3;
        if (s + 2 < 6)
          raw[(s + 2) % 3] = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
              (__attribute__((address_space(3))) intx2*)(lds + wsrc + ((s + 2) / 3) * 32 * QWS + ((s + 2) % 3) * 16));
        if (s < 2) {   // second K step's G^T operands, four per step
#pragma unroll
          for (int u = 0; u < 4; u++) {
            const int mb = 4 * s + u;
            ga[1][mb] = *(const bf16x8*)(lds + gsrc + 16 * mb * QPL_S + 64);
          }
        }
        QFENCE();
#pragma unroll
        for (int mb = 0; mb < 8; mb++) {
          acc2[mb][nn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ga[ks2][mb], wb[s & 1], acc2[mb][nn], 0, 0, 0);
          if (mb == 1 && s + 1 < 6) wb[(s + 1) & 1] = q_fp8x8_to_bf16x8(raw[(s + 1) % 3]);
          if (mb == 1) QFENCE();
          if (mb == 3) { mem_piece(2 * s); QFENCE(); }
          if (mb == 6) { mem_piece(2 * s + 1); QFENCE(); }
          if (mb == 7 && s == 4) { mem_piece(12); QFENCE(); }
          if (mb == 7 && s == 5) { mem_piece(13); QFENCE(); }
        }
        QFENCE();
      }
    } else {
#pragma unroll
      for (int k = 0; k < 14; k++) mem_piece(k);
    }

    QT(4)
    // the counters, read before this iteration's stores so that the wait at the top of the loop covers the load
    fseen = __hip_atomic_load(flags + (lane & 3), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // ---- A^T[48 features x 64 rows] = X^T G^T in four 16-row blocks; the update of block nb-1 (VALU, registers to
    //      memory) is issued between the MFMAs of block nb.  Row r = 4kg+e of feature block cg is feature
    //      12kg + 4cg + e of the wavefront's 48, so that a lane ends up with 12 consecutive bytes of one weight row.
    {
      const unsigned bsrc = gb + (8 * kg + (l16 >> 2)) * QPL_S + 4 * (l16 & 3) * 2;
      const unsigned wrow = wc + l16 * QWS + 48 * w + 12 * kg;
      const unsigned grow0 = q.label0 + (unsigned)l16;
      auto load_bg = [&](int nb, bf16x8 (&bg)[4]) {
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
          shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4*)(lds + bsrc + ks * 32 * QPL_S + 16 * nb * 2));
          shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4*)(lds + bsrc + ks * 32 * QPL_S + 16 * nb * 2 + 4 * QPL_S));
          bg[ks] = __builtin_bit_cast(bf16x8, shortx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]});
        }
      };
      bf16x8 bg[2][4];
      load_bg(0, bg[0]);
      floatx4 acc3[2][3];
      unsigned wq[2][3];
      unsigned outw[3];
#pragma unroll
      for (int nb = 0; nb <= 4; nb++) {
        const int cur = nb & 1, prev = cur ^ 1;
        if (nb + 1 < 4) load_bg(nb + 1, bg[prev]);
        if (nb < 4) {
#pragma unroll
          for (int cg = 0; cg < 3; cg++) {
            acc3[cur][cg] = floatx4{0.f, 0.f, 0.f, 0.f};
            wq[cur][cg] = *(const unsigned*)(lds + wrow + 16 * nb * QWS + 4 * cg);
          }
        }
        QFENCE();
#pragma unroll
        for (int cg = 0; cg < 3; cg++) {   // cg = feature block for the MFMAs and for the update
          if (nb < 4 && !(XMC_DBG_SKIP & 8)) {
#pragma unroll
            for (int ks = 0; ks < 4; ks++)
              acc3[cur][cg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xt[cg][ks], bg[cur][ks], acc3[cur][cg], 0, 0, 0);
          }
          if (nb > 0 && !(XMC_DBG_SKIP & 16)) {
            const int row = 16 * (nb - 1) + l16;
            const unsigned wv = wq[prev][cg];
            floatx2 w01 = __builtin_amdgcn_cvt_pk_f32_fp8((int)wv, false), w23 = __builtin_amdgcn_cvt_pk_f32_fp8((int)wv, true);
            floatx4 a = acc3[prev][cg];
            float t0 = __builtin_fmaf(-p.lr_eff, a[0], w01.x), t1 = __builtin_fmaf(-p.lr_eff, a[1], w01.y);
            float t2 = __builtin_fmaf(-p.lr_eff, a[2], w23.x), t3 = __builtin_fmaf(-p.lr_eff, a[3], w23.y);
            outw[cg] = round4<MODE>(t0, t1, t2, t3, (unsigned)(q.row0 + row), grow0 + 16 * (nb - 1),
                                    (unsigned)(QCOLS * m + 48 * w + 12 * kg + 4 * cg), q.seed);
            if (cg == 2 && row < q.rows_valid && !(XMC_DBG_SKIP & 64)) {
              unsigned* gp = (unsigned*)(q.base + (size_t)row * D + QCOLS * m + 48 * w + 12 * kg);
              gp[0] = outw[0]; gp[1] = outw[1]; gp[2] = outw[2];
            }
          }
          QFENCE();
        }
      }
    }

    QT(5)
    QT(6)
#pragma unroll
    for (int k = 0; k + 1 < QINF; k++) inf[k] = inf[k + 1];
    inf[QINF - 1] = q_from_desc(dnext0, dnext1);
  }

#ifdef XMC_TIMING
  if (lane == 0 && g < 96)
    for (int k = 0; k < 8; k++) p.flags[1024 + (g * 4 + w) * 8 + k] = (int)tacc[k];
#endif
  // ---- per-workgroup grad_X partial, summed in a fixed order by reduce_gx_quad_kernel
  floatx4* dst = p.partial + (size_t)g * 24 * QNT;
#pragma unroll
  for (int mb = 0; mb < 8; mb++)
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
    s += partial[((size_t)g * 24 + slot) * QNT + tid];
  }
  const int mb = slot / 3, nn = slot - mb * 3;
  const int col = QCOLS * m + 48 * w + 16 * nn + l16;
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

// Operand images of X for the quad kernel.
//   xq: e4m3(X / scale_x) in v_mfma 16x16x128 B-operand order: operand index ((b/16)*6 + ks), lane = (b%16) + 16*kg,
//       byte j: Xq[b][k = 128ks + 32kg + j]
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
    int ks = k >> 7, kgq = (k >> 5) & 3, jq = k & 31;
    size_t off = ((size_t)(((b >> 4) * 6 + ks) * 64 + ((b & 15) + 16 * kgq))) * 32 + jq;
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
