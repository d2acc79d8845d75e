// Fused FP8 extreme-classifier training step for gfx950 (MI355X): four compute units per tile stream.
//
// Work unit = a tile of 64 consecutive label rows of one chunk (64 x 768 e4m3 bytes, contiguous in HBM).
// Four workgroups on the same XCD (a "quad") walk the same tile sequence, one workgroup per compute unit,
// 8 wavefronts each (two per SIMD, 256 registers), so that while one wavefront of a SIMD waits - for the memory
// pipeline to accept a load, for LDS, for the matrix core - the other one issues.  Member m of the quad owns
//   * label rows 16m..16m+15 of every tile for the logits and the sigmoid ("stage A"), and
//   * input features 192m..192m+191 for grad_X, grad_W and the in-place update ("stage B"),
// so no arithmetic is repeated and every weight byte is read from HBM once and written once per step.  A member
// reads 24 KiB per tile (its rows and its columns), always as whole 16-byte pieces of contiguous row segments
// sent straight to LDS: the vector memory path of a compute unit handles few cache lines per clock, and
// register loads in MFMA operand order (16 rows x 64 bytes per instruction) would keep it busy longer than
// the MFMAs run.
// The only data the members exchange is G = sigmoid(logits) - target in bf16 (4 KiB per member and tile),
// through a small ring of slots in global memory, guarded by per-member "tiles published" counters.  Stage A runs
// QAHEAD tiles ahead of stage B, so neither the exchange nor the counters are on the critical path.  Neither logits
// nor gradients ever reach HBM; the X operands of all three GEMMs and the grad_X accumulators (96 KiB per compute
// unit) live in registers for the whole launch.
//
// Wavefront v = (fg = v % 4, h = v / 4):
//   stage A(t): Z[16 x 16] = W_t[16m.., :] Xq[16v.., :]^T   v_mfma_f32_16x16x128_f8f6f4, W rows read from LDS
//               G = bf16(sigmoid(bf16(Z))) - [positive], stored to the exchange slot in [b][l] order
//   stage B(t): the whole G tile arrives in LDS by global_load_lds
//               grad_X[64h.. x 48fg..] += G^T W_t   v_mfma_f32_16x16x32_bf16, W via ds_read_b64_tr_b8 + fp8->bf16
//               A^T[48fg.. x 32h..]     = X^T G^T    v_mfma_f32_16x16x32_bf16, G via ds_read_b64_tr_b16
//               W_t = round(W - lr A) from registers to memory, 12 bytes per lane and row
// Loads are direct-to-LDS, issued one at a time between the compute phases and consumed two iterations later: the
// wait in front of the per-tile barrier leaves the operations of the iteration just finished in flight, so neither
// the issue nor the latency of a load is waited for.  Tile descriptors come through the scalar path (they are
// constant during the launch); a snapshot of the counters arrives in LDS with the other loads.
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
constexpr int QRING = 6;                  // own-column tile images: in use, four landed or landing, one in flight
constexpr int QPL_S = TL * 2 + 16;        // bytes per batch row of the G tile ([128 b][64 l] bf16 + pad)
constexpr int QG_PIECES = (BP * QPL_S + 1023) / 1024;   // wave-wide loads per G tile (18)
constexpr int QG_BYTES = 20480;           // one G tile (128 x 144 = 18432), padded
constexpr int QSLOTS = 8;                 // exchange slots per quad
constexpr int QLDS_G = QRING * QWC_BYTES; // LDS offset of the two gathered-G buffers
constexpr int QRS = D + 32;               // LDS row stride of the own-rows image (50 x 16 bytes: with an even number of
                                          // 16-byte units per row the 16-byte operand reads of stage A have no bank conflicts)
constexpr int QROW_BYTES = 13 * 1024;     // 16 rows x 784 = 12544, padded to 13 wave-wide loads
constexpr int QRRING = 3;                 // own-rows images in flight
constexpr int QGBUF = 2;                  // gathered-G buffers: in use, in flight
constexpr int QLDS_R = QLDS_G + QGBUF * QG_BYTES;
constexpr int QLDS_M = QLDS_R + QRRING * QROW_BYTES;   // two snapshots of the counters, 16 bytes each; at +64 the abort word
constexpr int QLDS_BYTES = QLDS_M + 256;
constexpr int QSPIN_LIMIT = 1 << 18;
constexpr int QAHEAD = 5;                 // stage A runs this many tiles ahead of stage B
constexpr int QWAHEAD = QRING - 1;        // own columns are fetched this many tiles ahead

struct QuadParams {
  unsigned char* chunk[MAX_CHUNKS];   // device pointers of the chunk weight tensors [rows_per_chunk, 768] e4m3
  unsigned seed[MAX_CHUNKS];          // per-chunk rounding seed
  int num_chunks;
  int rows_per_chunk;
  int tiles_per_chunk;
  int num_tiles;
  const unsigned char* xq;            // logits operands (layout of prep_x_quad_thread)
  const bf16x8* xt;                   // grad_W operands
  const unsigned* keys;               // sorted positives: label*256 + batch_row
  const int* tile_ptr;                // [num_tiles+1] offsets into keys
  const uint4* desc;                  // [nquads][kmax][2] tile descriptors written by quad_desc_prep_kernel: the tiles of
                                      // one quad are consecutive entries, in the order the quad walks them
  int nquads;                         // quads of the step kernel's launch (grid / 4)
  int kmax;                           // descriptor entries per quad = ceil(num_tiles / nquads)
  floatx4* partial;                   // [gridDim.x][12][512] per-workgroup grad_X partial sums
  unsigned char* exch;                // [nquads][QSLOTS][QG_BYTES] G exchange ring
  int* flags;                         // [nquads][4] tiles-published counters; [QF_XCC + g] XCC ids; [QF_ERR] error word
  float zscale;                       // scale_w * scale_x applied to the logits accumulator
  float lr_eff;                       // lr / scale_w
  int batch;
};

#define QFENCE() __builtin_amdgcn_sched_barrier(0)   // nothing is scheduled across this point
typedef __attribute__((address_space(3))) unsigned char qlds_u8;
typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef short shortx8 __attribute__((ext_vector_type(8)));

// 16 bytes per lane from global memory straight into LDS at byte offset ldsoff + 16*lane (wave-uniform offset).
// Issued through inline assembly on purpose: the compiler orders every later LDS access behind a direct-to-LDS
// load it knows about, which would serialise the prefetch.  Completion is enforced by hand (s_waitcnt vmcnt +
// barrier) before the data is read.
__device__ __forceinline__ void q_lds_load16(const unsigned char* g, unsigned ldsoff_) {
  const unsigned ldsoff = __builtin_amdgcn_readfirstlane(ldsoff_);
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(ldsoff), "v"(g) : "memory", "m0");
}
// same with a wave-uniform base pointer and a 32-bit per-lane byte offset
__device__ __forceinline__ void q_lds_load16_sbase(const unsigned char* base, unsigned off, unsigned ldsoff_) {
  const unsigned ldsoff = __builtin_amdgcn_readfirstlane(ldsoff_);
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(ldsoff), "v"(off), "s"(base) : "memory", "m0");
}
// same, at device scope (sc1): never served by this compute unit's L1, which may still hold the previous contents
// of an exchange slot
__device__ __forceinline__ void q_lds_load16_l2(const unsigned char* g, unsigned ldsoff_) {
  const unsigned ldsoff = __builtin_amdgcn_readfirstlane(ldsoff_);
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off sc1" : : "s"(ldsoff), "v"(g) : "memory", "m0");
}
__device__ __forceinline__ void q_lds_load16_l2_sbase(const unsigned char* base, unsigned off, unsigned ldsoff_) {
  const unsigned ldsoff = __builtin_amdgcn_readfirstlane(ldsoff_);
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2 sc1" : : "s"(ldsoff), "v"(off), "s"(base) : "memory", "m0");
}
// 4 bytes per lane at device scope into LDS at ldsoff + 4*lane
__device__ __forceinline__ void q_lds_load4_l2(const void* g, unsigned ldsoff_) {
  const unsigned ldsoff = __builtin_amdgcn_readfirstlane(ldsoff_);
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, off sc1" : : "s"(ldsoff), "v"(g) : "memory", "m0");
}

// eight e4m3 codes -> eight bf16 values (exact), two per instruction
__device__ __forceinline__ bf16x8 q_fp8x8_to_bf16x8(intx2 raw) {
  bf16x2 c0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw.x, 1.0f, false), c1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw.x, 1.0f, true);
  bf16x2 c2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw.y, 1.0f, false), c3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw.y, 1.0f, true);
  return bf16x8{c0.x, c0.y, c1.x, c1.y, c2.x, c2.y, c3.x, c3.y};
}

// Everything the kernel needs to know about one tile; wave-uniform, kept in scalar registers.  The descriptors are
// precomputed by quad_desc_prep_kernel (32 bytes: {base pointer, valid rows, seed}, {first key, one past the last key,
// row in chunk, first label}) and read through the scalar (constant) path: they do not change during the launch.
struct QTile { unsigned char* base; unsigned label0; int row0, rows_valid, p0, p1; unsigned seed; };
typedef const __attribute__((address_space(4))) intx4 q_cdesc;

// base pointer and valid rows only
__device__ __forceinline__ q_cdesc* q_desc_ptr(q_cdesc* desc, int t) {
  return (q_cdesc*)((const __attribute__((address_space(4))) unsigned char*)desc + ((unsigned)t << 5));
}
__device__ __forceinline__ QTile q_desc_head(q_cdesc* desc, int t) {
  const intx4 d0 = q_desc_ptr(desc, t)[0];
  QTile q = {};
  q.base = (unsigned char*)(((unsigned long long)(unsigned)d0.y << 32) | (unsigned)d0.x);
  q.rows_valid = d0.z;
  q.seed = (unsigned)d0.w;
  return q;
}
__device__ __forceinline__ QTile q_desc_full(q_cdesc* desc, int t) {
  QTile q = q_desc_head(desc, t);
  const intx4 d1 = q_desc_ptr(desc, t)[1];
  q.p0 = d1.x;
  q.p1 = d1.y;
  q.row0 = d1.z;
  q.label0 = (unsigned)d1.w;
  return q;
}

// First of the two launches in front of the step kernel: clear the counters (flags, may be null) and sort the positives
// (key = label*256 + (batch row - row0) for the batch rows row0..row0+255 that lie below `batch`; every other entry, and
// labels outside the label space, -> 0xFFFFFFFF) by rank.  Workgroup b ranks keys 64b..64b+63 of the n_pad
// (a power of two, at least 64, or 0): every workgroup builds all keys in LDS, its four wavefronts each count the keys
// that precede the workgroup's own over a quarter of the set (equal keys: the one that comes first in the input
// precedes), and the sum of the four counts is the key's position in the output.  Grid: max(1, n_pad / 64) x 256
// threads, (n_pad + 256) * 4 bytes of LDS.
__global__ __launch_bounds__(256) void quad_sort_kernel(const int* coo, int nnz, int n_pad, int batch, int row0, unsigned* keys, int* flags) {
  extern __shared__ unsigned sk[];
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
  if (blockIdx.x == 0 && flags)
    for (int i = tid; i < QF_STICKY; i += 256) flags[i] = 0;
  if (n_pad == 0) return;
  // eight (row, label) pairs per thread in flight at a time: the loads miss every cache
  const int2* coo2 = (const int2*)coo;
  for (int i0 = tid; i0 < n_pad; i0 += 8 * 256) {
    int2 e[8];
#pragma unroll
    for (int u = 0; u < 8; u++) {
      const int i = i0 + u * 256;
      e[u] = i < nnz ? coo2[i] : int2{-1, -1};
    }
#pragma unroll
    for (int u = 0; u < 8; u++) {
      const int i = i0 + u * 256;
      const int r = e[u].x - row0, lab = e[u].y;
      if (i < n_pad) sk[i] = (r >= 0 && r < 256 && r + row0 < batch && lab >= 0 && lab < (1 << 24) - 1) ? (((unsigned)lab << 8) | (unsigned)r) : 0xFFFFFFFFu;
    }
  }
  __syncthreads();
  const int i0 = blockIdx.x * 64;
  const unsigned mine = sk[i0 + l];
  const int quarter = n_pad >> 2;
  // keys in front of the workgroup's own 64 precede on <=, keys behind them on <, the own 64 by position; each part
  // is a branch-free loop over groups of four so that several LDS reads are in flight
  const int jb = w * quarter, je = (w + 1) * quarter;
  const int e0 = min(je, max(jb, i0)), b2 = max(jb, min(je, i0 + 64));
  const uint4* sk4 = (const uint4*)sk;
  int rank = 0;
#pragma unroll 4
  for (int j = jb >> 2; j < e0 >> 2; j++) {
    const uint4 o = sk4[j];
    rank += (o.x <= mine) + (o.y <= mine) + (o.z <= mine) + (o.w <= mine);
  }
#pragma unroll 4
  for (int j = b2 >> 2; j < je >> 2; j++) {
    const uint4 o = sk4[j];
    rank += (o.x < mine) + (o.y < mine) + (o.z < mine) + (o.w < mine);
  }
  if (e0 < b2) {   // the part of the own 64 keys that lies in this wavefront's quarter
    const int me = i0 + l;
    for (int j = e0; j < b2; j += 4) {
      const uint4 o = sk4[j >> 2];
      rank += (o.x < mine || (o.x == mine && j < me)) + (o.y < mine || (o.y == mine && j + 1 < me)) +
              (o.z < mine || (o.z == mine && j + 2 < me)) + (o.w < mine || (o.w == mine && j + 3 < me));
    }
  }
  unsigned* part = sk + n_pad;
  part[tid] = (unsigned)rank;
  __syncthreads();
  if (w == 0) keys[part[l] + part[64 + l] + part[128 + l] + part[192 + l]] = mine;
}

__device__ __forceinline__ void prep_x_quad_thread(int i, const unsigned short* x, int batch, float inv_scale_x, unsigned char* xq,
                                                   unsigned short* xt);

// Second launch: blocks below desc_blocks write, for every tile,
//   desc[t] = {base pointer, valid rows, seed | first key, one past the last key, row in chunk, first label}
//   tile_ptr[t] = first key whose label >= first label of tile t (binary search in the sorted keys)
// and the remaining blocks build the operand images of X.
__global__ __launch_bounds__(256) void quad_desc_prep_kernel(const QuadParams p, int n_pad, int* tile_ptr, uint4* desc, int desc_blocks,
                                                             const unsigned short* x, float inv_scale_x, unsigned char* xq,
                                                             unsigned short* xt) {
  if ((int)blockIdx.x >= desc_blocks) {
    prep_x_quad_thread(((int)blockIdx.x - desc_blocks) * 256 + (int)threadIdx.x, x, p.batch, inv_scale_x, xq, xt);
    return;
  }
  // the sorted keys go to LDS first (n_pad * 4 bytes, then 257 search results): a binary search in global memory
  // is a chain of dependent cache misses
  extern __shared__ unsigned dk[];
  const int tid = threadIdx.x;
  for (int i0 = tid; i0 < n_pad; i0 += 8 * 256) {
    unsigned e[8];
#pragma unroll
    for (int u = 0; u < 8; u++) e[u] = i0 + u * 256 < n_pad ? p.keys[i0 + u * 256] : 0u;
#pragma unroll
    for (int u = 0; u < 8; u++)
      if (i0 + u * 256 < n_pad) dk[i0 + u * 256] = e[u];
  }
  __syncthreads();
  int* found = (int*)(dk + n_pad);
  const int t = blockIdx.x * 256 + tid;
  auto lower = [&](int tt) {   // first key of tile tt (tt >= num_tiles: first key past the last tile)
    if (tt > p.num_tiles) tt = p.num_tiles;
    const int c = tt / p.tiles_per_chunk, tj = tt - c * p.tiles_per_chunk;
    const unsigned long long bound = ((unsigned long long)c * p.rows_per_chunk + (unsigned long long)tj * TL) << 8;
    int lo = 0, hi = n_pad;
    while (lo < hi) {
      int mid = (lo + hi) >> 1;
      if ((unsigned long long)dk[mid] < bound) lo = mid + 1; else hi = mid;
    }
    return lo;
  };
  const int p0 = lower(t);
  found[tid] = p0;
  if (tid == 255) found[256] = lower(t + 1);
  __syncthreads();
  if (t > p.num_tiles) return;
  tile_ptr[t] = p0;
  if (t < p.num_tiles) {
    const int p1 = found[tid + 1];
    const int c = t / p.tiles_per_chunk;
    const int row0 = (t - c * p.tiles_per_chunk) * TL;
    const unsigned long long base = (unsigned long long)(p.chunk[c] + (size_t)row0 * D);
    // tile t is position t / nquads of quad t % nquads: a quad reads its descriptors as one contiguous run, so the
    // scalar cache serves all but one fetch in two
    const int slot = (t % p.nquads) * p.kmax + t / p.nquads;
    desc[2 * slot] = uint4{(unsigned)base, (unsigned)(base >> 32), (unsigned)min(TL, p.rows_per_chunk - row0), p.seed[c]};
    desc[2 * slot + 1] = uint4{(unsigned)p0, (unsigned)p1, (unsigned)row0, (unsigned)(c * p.rows_per_chunk + row0)};
  }
}

template <int MODE>
__global__ __launch_bounds__(QNT, 1) void fp8_step_quad_kernel(const QuadParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  qlds_u8* lds = (qlds_u8*)lds_raw;

  const int tid = threadIdx.x;
  const int v = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, l16 = lane & 15, kg = lane >> 4;
  const int fg = v & 3, h = v >> 2;
  const int g = blockIdx.x;
  const int xcd = g & 7, j = g >> 3, m = j & 3;
  const int nquads = gridDim.x >> 2;
  const int quad = (j >> 2) * 8 + xcd;
  const int n_it = quad < p.num_tiles ? (p.num_tiles - quad + nquads - 1) / nquads : 0;

  // the sorted keys are written before this kernel starts: read them through the scalar (constant) path
  const __attribute__((address_space(4))) unsigned* ckeys = (const __attribute__((address_space(4))) unsigned*)p.keys;
  int* flags = p.flags + quad * 4;
  int* errw = p.flags + QF_ERR;
  // the XCD this workgroup really runs on: reduce_gx_quad_kernel compares the four members of every quad
  if (tid == 0) p.flags[QF_XCC + g] = (int)(__builtin_amdgcn_s_getreg((3 << 11) | 20) & 15);   // XCC_ID
  // abort word of the workgroup: set by a wavefront whose bounded wait expired, read by all after the next barrier
  if (tid == 0) *(__attribute__((address_space(3))) int*)(lds + QLDS_M + 64) = 0;

  // ---- resident operands
  intx8 xq[6];         // logits: batch block 16v.., K steps of 128
#pragma unroll
  for (int ks = 0; ks < 6; ks++) xq[ks] = *(const intx8*)(p.xq + ((size_t)((v * 6 + ks) * 64 + lane)) * 32);
  bf16x8 xt[3][4];     // grad_W: feature blocks of this wavefront's 48 features, K steps of 32 batch rows
#pragma unroll
  for (int cg = 0; cg < 3; cg++)
#pragma unroll
    for (int ks = 0; ks < 4; ks++) xt[cg][ks] = p.xt[(size_t)(((4 * m + fg) * 3 + cg) * 4 + ks) * 64 + lane];
  floatx4 acc2[4][3];  // grad_X[64 batch rows x 48 features]
#pragma unroll
  for (int a = 0; a < 4; a++)
#pragma unroll
    for (int b = 0; b < 3; b++) acc2[a][b] = floatx4{0.f, 0.f, 0.f, 0.f};

  // Per-lane source rows and byte offsets of the wave-wide pieces this wavefront loads (pieces v and v+8 of an image).
  // own-column image: 64 rows x 13 chunks of 16 bytes (12 data + 1 pad) = 13 pieces of 1 KiB
  // own-rows image:   rows 16m..16m+15, 16 x 50 chunks of 16 bytes (48 data + 2 pad) = 13 pieces
  // The byte offsets are kept per lane for full tiles (nearly all): issuing a piece then costs no vector instruction.
  // A tile cut short by the end of its chunk recomputes them with the row clamped to the last valid one.
  auto wcol_offset = [&](int s, int last_row) {
    const int ch = (v + 8 * s) * 64 + lane, wr = ch / 13;
    return (unsigned)(min(wr, last_row) * D + QCOLS * m + min(ch - wr * 13, 11) * 16);
  };
  auto rows_offset = [&](int s, int last_row) {
    const int ch = (v + 8 * s) * 64 + lane, rr = ch / (QRS / 16);
    return (unsigned)(min(16 * m + min(rr, 15), last_row) * D + min(ch - rr * (QRS / 16), 47) * 16);
  };
  unsigned woff_full[2], roff_full[2];
#pragma unroll
  for (int s = 0; s < 2; s++) {
    woff_full[s] = wcol_offset(s, TL - 1);
    roff_full[s] = rows_offset(s, TL - 1);
  }
  q_cdesc* cdesc = (q_cdesc*)p.desc;
  // descriptor entry of position k in this quad's sequence; positions past the end fall back to entry 0 (tile 0),
  // whose data is loaded and never used
  auto tile_at = [&](int k) { return k < n_it ? quad * p.kmax + k : 0; };
  auto wcol_piece = [&](int slot, const QTile& q, int s) {
    if (v + 8 * s >= 13) return;
    if (q.rows_valid == TL) q_lds_load16_sbase(q.base, woff_full[s], (unsigned)(slot * QWC_BYTES + (v + 8 * s) * 1024));
    else q_lds_load16_sbase(q.base, wcol_offset(s, q.rows_valid - 1), (unsigned)(slot * QWC_BYTES + (v + 8 * s) * 1024));
  };
  auto rows_piece = [&](int slot, const QTile& q, int s) {
    if (v + 8 * s >= 13) return;
    if (q.rows_valid == TL) q_lds_load16_sbase(q.base, roff_full[s], (unsigned)(QLDS_R + slot * QROW_BYTES + (v + 8 * s) * 1024));
    else q_lds_load16_sbase(q.base, rows_offset(s, q.rows_valid - 1), (unsigned)(QLDS_R + slot * QROW_BYTES + (v + 8 * s) * 1024));
  };
  // the G tile of position i: 18 pieces of 1 KiB (pieces v, v+8, v+16)
  const unsigned char* gsrc_quad = p.exch + (size_t)quad * QSLOTS * QG_BYTES;   // wave-uniform; the lane part is an offset
  const unsigned gsrc_lane = (unsigned)(v * 1024 + lane * 16);
  auto gather_piece = [&](int i, int slot, int s) {
    if (v + 8 * s >= QG_PIECES) return;
    q_lds_load16_l2_sbase(gsrc_quad + (i & (QSLOTS - 1)) * QG_BYTES + s * 8192, gsrc_lane,
                          (unsigned)(QLDS_G + slot * QG_BYTES + (v + 8 * s) * 1024));
  };
  // snapshot of the four counters of iteration i (wavefront 0 only), read in the next iteration
  auto issue_snapshot = [&](int i) {
    if (v != 0) return;
    if (lane < 4) q_lds_load4_l2(flags + lane, (unsigned)(QLDS_M + (i & 1) * 16));
  };
  auto lds_i4 = [&](unsigned off) { return *(const __attribute__((address_space(3))) intx4*)(lds + off); };
  // stage A of the tile at position i: logits of label rows 16m.. against batch rows 16v.., sigmoid minus target, store
  // this wavefront's part of G to the exchange slot (published later, once the stores have completed)
  unsigned char* gdst_lane = p.exch + (size_t)quad * QSLOTS * QG_BYTES + (16 * v + l16) * QPL_S + (16 * m + 4 * kg) * 2;
  auto stage_a = [&](int i, int slot, const QTile& q) {
    floatx4 z = floatx4{0.f, 0.f, 0.f, 0.f};
    {
      // lane (row l16, k group kg) holds bytes 16kg..16kg+15 and 64+16kg..64+16kg+15 of every 128-byte K step (the X
      // image is built in the same order): two 16-byte reads whose lanes tile the LDS banks
      const unsigned asrc = (unsigned)(QLDS_R + slot * QROW_BYTES) + l16 * QRS + kg * 16;
      // the reads of three K steps are in flight at a time
      intx4 alo[6], ahi[6];
      auto rd = [&](int ks) {
        alo[ks] = *(const __attribute__((address_space(3))) intx4*)(lds + asrc + ks * 128);
        ahi[ks] = *(const __attribute__((address_space(3))) intx4*)(lds + asrc + ks * 128 + 64);
      };
      rd(0); rd(1); rd(2);
      QFENCE();
#pragma unroll
      for (int ks = 0; ks < 6; ks++) {
        if (ks + 3 < 6) rd(ks + 3);
        intx8 av = intx8{alo[ks].x, alo[ks].y, alo[ks].z, alo[ks].w, ahi[ks].x, ahi[ks].y, ahi[ks].z, ahi[ks].w};
        z = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, xq[ks], z, 0, 0, 0, 0, 0, 0);
        QFENCE();
      }
    }
    const float nlog2e = -1.44269504088896340736f;
    const int r0 = 16 * m + 4 * kg;   // this lane's label rows r0..r0+3; its batch row is 16v + l16
    // sigmoid of the bf16 logits, rounded to bf16 in pairs
    unsigned zb[2], sb[2];
#pragma unroll
    for (int e2 = 0; e2 < 2; e2++) {
      zb[e2] = bf16_pack2(z[2 * e2] * p.zscale, z[2 * e2 + 1] * p.zscale);
      const float z0 = __uint_as_float(zb[e2] << 16), z1 = __uint_as_float(zb[e2] & 0xFFFF0000u);
      sb[e2] = bf16_pack2(__builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(z0 * nlog2e)),
                          __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(z1 * nlog2e)));
    }
    // positives of this tile (set semantics: a repeated key counts once); wave-uniform scalar loads
    if (q.p1 > q.p0) {
      float sg[4] = {__uint_as_float(sb[0] << 16), __uint_as_float(sb[0] & 0xFFFF0000u), __uint_as_float(sb[1] << 16),
                     __uint_as_float(sb[1] & 0xFFFF0000u)};
      // The keys come eight at a time through the scalar path (one wait per eight; the first tiles of a chunk sorted
      // by label frequency hold hundreds of positives), and a key costs vector instructions only if it lies in this
      // wavefront's block (label rows 16m.., batch rows 16v..).  Up to seven keys behind the tile's last are read and
      // ignored; the buffer behind the keys belongs to the workspace.
      typedef unsigned q_keysx8 __attribute__((ext_vector_type(8), aligned(4)));
      const unsigned lbase = q.label0 + 16u * (unsigned)m;
      unsigned prev = q.p0 > 0 ? ckeys[q.p0 - 1] : ~ckeys[q.p0];
      for (int e0 = q.p0; e0 < q.p1; e0 += 8) {
        const q_keysx8 kk = *(const __attribute__((address_space(4))) q_keysx8*)(ckeys + e0);
#pragma unroll
        for (int j = 0; j < 8; j++) {
          const unsigned key = kk[j];
          const unsigned lrel = (key >> 8) - lbase;   // label row within this member's sixteen
          if (e0 + j < q.p1 && key != prev && lrel < 16u && ((key >> 4) & 15u) == (unsigned)v) {
            const bool mine = (unsigned)kg == (lrel >> 2) && (unsigned)l16 == (key & 15u);
            const unsigned q4 = lrel & 3u;   // wave-uniform: one of the lane's four labels
            if (q4 == 0u) sg[0] = mine ? bf16_rt(sg[0] - 1.0f) : sg[0];
            else if (q4 == 1u) sg[1] = mine ? bf16_rt(sg[1] - 1.0f) : sg[1];
            else if (q4 == 2u) sg[2] = mine ? bf16_rt(sg[2] - 1.0f) : sg[2];
            else sg[3] = mine ? bf16_rt(sg[3] - 1.0f) : sg[3];
          }
          prev = key;
        }
      }
      sb[0] = bf16_pack2(sg[0], sg[1]);
      sb[1] = bf16_pack2(sg[2], sg[3]);
    }
    if (q.rows_valid < TL) {   // rows past the end of the chunk contribute nothing
#pragma unroll
      for (int e2 = 0; e2 < 2; e2++) {
        if (r0 + 2 * e2 >= q.rows_valid) sb[e2] &= 0xFFFF0000u;
        if (r0 + 2 * e2 + 1 >= q.rows_valid) sb[e2] &= 0x0000FFFFu;
      }
    }
    *(uint2*)(gdst_lane + (i & (QSLOTS - 1)) * QG_BYTES) = uint2{sb[0], sb[1]};
  };
  // wait until every member has published at least `need` tiles (fmin: the smallest counter seen earlier, which
  // normally suffices; the polling loop is kept out of the common path)
  auto wait_published = [&](int need, int fmin) {
    if (fmin >= need) return;
    for (int spin = 0;; spin++) {
      int f = __hip_atomic_load(flags + (lane & 3), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (__builtin_amdgcn_read_exec() == __builtin_amdgcn_ballot_w64(f >= need)) break;
      if (spin >= QSPIN_LIMIT || ((spin & 1023) == 1023 && __hip_atomic_load(errw, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
        // give up: raise the error word (partners that wait for this workgroup see it and give up too) and the
        // workgroup's abort word; the iteration under way still has valid G, the next one is not started
        if (lane == 0) {
          __hip_atomic_fetch_or(errw, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          *(__attribute__((address_space(3))) int*)(lds + QLDS_M + 64) = 1;
        }
        break;
      }
      __builtin_amdgcn_s_sleep(2);
    }
  };

  // ---- prologue: own columns of the first QWAHEAD positions, stage A of the first QAHEAD positions, own rows of the
  //      next two, G of position 0
#pragma unroll
  for (int k = 0; k < 3; k++) {
    const QTile t = q_desc_head(cdesc, tile_at(k));
#pragma unroll
    for (int s = 0; s < 2; s++) rows_piece(k, t, s);
  }
#pragma unroll
  for (int k = 0; k < QWAHEAD; k++) {
    const QTile t = q_desc_head(cdesc, tile_at(k));
#pragma unroll
    for (int s = 0; s < 2; s++) wcol_piece(k, t, s);
  }
#pragma unroll
  for (int k = 0; k < QAHEAD; k++) {
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (k < n_it) stage_a(k, k % QRRING, q_desc_full(cdesc, tile_at(k)));
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (k + 3 < QAHEAD + 2) {
      const QTile t = q_desc_head(cdesc, tile_at(k + 3));
#pragma unroll
      for (int s = 0; s < 2; s++) rows_piece(k % QRRING, t, s);
    }
  }
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (tid == 0 && n_it > 0) __hip_atomic_store(flags + m, min(QAHEAD, n_it), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const int fboot = min(2, n_it);   // what the first iteration needs of the counters
  if (n_it > 0) wait_published(fboot, 0);
#pragma unroll
  for (int s = 0; s < 3; s++) gather_piece(0, 0, s);

  // Vector memory operations retire in order.  In a regular iteration every wavefront issues, in this order: the
  // snapshot of the counters (wavefront 0), its pieces of G of the next position, its pieces of the own columns
  // QWAHEAD and of the own rows QAHEAD+2 positions ahead, and two stores of updated weights; its part of G of position
  // i+QAHEAD is stored behind the first piece of G (h = 0) or behind the rows (h = 1).  The loads are spread over the
  // iteration so that the memory pipeline accepts each at once.  The wait in front of the barrier leaves the last four
  // (h = 0) or five (h = 1) operations in flight, which always include the rows - the only loads that miss the L2:
  // the snapshot and G, which the next iteration consumes, have landed; rows, columns and stores are not needed
  // before the iteration after.  A tile's rows and columns are fetched two iterations apart, so that the second fetch finds
  // the tile in the XCD's L2.  After an iteration that issued fewer operations (the last positions, a short tile)
  // everything is waited for.  Loads for positions past the end fetch tile 0 into buffers nobody reads.
  bool prev_regular = false;
  int s0 = 0, s1 = 1, s2 = 2;   // i % 3, (i+1) % 3, (i+2) % 3
  int w0 = 0;                   // i % QRING
  // descriptors of the next iteration: its tile, the tile of its stage A, the tiles whose rows and columns it fetches.
  // They are loaded in front of the weight update of the iteration before, where their latency hides behind LDS reads.
  QTile q_n = q_desc_full(cdesc, tile_at(0)), qa_n = q_desc_full(cdesc, tile_at(QAHEAD));
  QTile qr_n = q_desc_head(cdesc, tile_at(QAHEAD + 2)), qw_n = q_desc_head(cdesc, tile_at(QWAHEAD));
  for (int i = 0; i < n_it; i++) {
    if (!prev_regular) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    else if (h == 0) asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(5) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    // a wavefront gave up waiting in the iteration before: G of this position may be missing, nothing more is
    // computed or stored (the weights of the remaining tiles stay as they were; the error word tells the host)
    if (__builtin_amdgcn_readfirstlane(*(const __attribute__((address_space(3))) int*)(lds + QLDS_M + 64)) != 0) break;
    const QTile q = q_n, qa = qa_n, qr = qr_n, qw = qw_n;
    int fmin = fboot;
    if (i >= 1) {   // the counters as they were one iteration ago
      const intx4 fl = lds_i4((unsigned)(QLDS_M + ((i + 1) & 1) * 16));
      fmin = min(min((int)__builtin_amdgcn_readfirstlane(fl.x), (int)__builtin_amdgcn_readfirstlane(fl.y)),
                 min((int)__builtin_amdgcn_readfirstlane(fl.z), (int)__builtin_amdgcn_readfirstlane(fl.w)));
    }
    const int sl[3] = {s0, s1, s2};
    const int slot_rows = sl[(QAHEAD + 2) % 3], slot_a = sl[QAHEAD % 3];
    const int slot_wcol = w0 == 0 ? QRING - 1 : w0 - 1;   // (i + QWAHEAD) % QRING
    const unsigned wc = (unsigned)(w0 * QWC_BYTES);
    const unsigned gb = (unsigned)(QLDS_G + (i & 1) * QG_BYTES);
    const bool do_a = i + QAHEAD < n_it;
    prev_regular = q.rows_valid == TL && do_a;
    // G of the positions up to i+QAHEAD-2 was stored in iteration i-2 or earlier: complete by the wait above
    if (tid == 0 && i >= 2 && i + QAHEAD - 1 <= n_it)
      __hip_atomic_store(flags + m, i + QAHEAD - 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    issue_snapshot(i);
    if (i + 1 < n_it) wait_published(i + 2, fmin);
    // the loads of this iteration, one at a time between the phases below
    auto mem_piece = [&](int k) {
      if (k < 3) gather_piece(i + 1, (i + 1) & 1, k);
      else if (k < 5) wcol_piece(slot_wcol, qw, k - 3);
      else if (k < 7) rows_piece(slot_rows, qr, k - 5);
    };
    mem_piece(0);

    // The two wavefronts of a SIMD run stage A and grad_X in opposite orders, so that the LDS reads of one overlap
    // the MFMAs of the other.
    if (h == 0 && do_a) stage_a(i + QAHEAD, slot_a, qa);
    mem_piece(1);

    // ---- grad_X[64 x 48] += G^T W; 6 steps (32-row K step major, 16-feature block minor); the transposed W read of
    //      step s+2 and the fp8->bf16 conversion of step s+1 are issued between the MFMAs of step s
    {
      const unsigned wsrc = wc + (8 * kg + (l16 >> 1)) * QWS + 48 * fg + (l16 & 1) * 8;
      const unsigned gsrc = gb + (64 * h + l16) * QPL_S + kg * 16;
      bf16x8 ga[2][4];
#pragma unroll
      for (int ks2 = 0; ks2 < 2; ks2++)
#pragma unroll
        for (int mb = 0; mb < 4; mb++) ga[ks2][mb] = *(const bf16x8*)(lds + gsrc + 16 * mb * QPL_S + 64 * ks2);
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
        if (s + 1 < 6) wb[(s + 1) & 1] = q_fp8x8_to_bf16x8(raw[(s + 1) % 3]);
#pragma unroll
        for (int mb = 0; mb < 4; mb++)
          acc2[mb][nn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ga[ks2][mb], wb[s & 1], acc2[mb][nn], 0, 0, 0);
        mem_piece(2 + s);
      }
    }
    if (h != 0 && do_a) stage_a(i + QAHEAD, slot_a, qa);

    qa_n = q_desc_full(cdesc, tile_at(i + 1 + QAHEAD));
    qr_n = q_desc_head(cdesc, tile_at(i + 1 + QAHEAD + 2));
    qw_n = q_desc_head(cdesc, tile_at(i + 1 + QWAHEAD));
    q_n = q_desc_full(cdesc, tile_at(i + 1));
    // ---- A^T[48 features x 32 rows] = X^T G^T in two 16-row blocks, each followed by its update.  Row r = 4kg+e of
    //      feature block cg is feature 12kg + 4cg + e of the wavefront's 48, so that a lane ends up with 12
    //      consecutive bytes of one weight row.
    {
      const unsigned bsrc = gb + (8 * kg + (l16 >> 2)) * QPL_S + 4 * (l16 & 3) * 2;
      const unsigned wrow = wc + l16 * QWS + 48 * fg + 12 * kg;
      const unsigned grow0 = q.label0 + (unsigned)l16;
      bf16x8 bg[2][4];
      unsigned wq[2][3];
#pragma unroll
      for (int nb = 0; nb < 2; nb++) {
        const int nbg = 2 * h + nb;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
          shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4*)(lds + bsrc + ks * 32 * QPL_S + 16 * nbg * 2));
          shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4*)(lds + bsrc + ks * 32 * QPL_S + 16 * nbg * 2 + 4 * QPL_S));
          bg[nb][ks] = __builtin_bit_cast(bf16x8, shortx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]});
        }
#pragma unroll
        for (int cg = 0; cg < 3; cg++) wq[nb][cg] = *(const unsigned*)(lds + wrow + 16 * nbg * QWS + 4 * cg);
      }
      // all 24 matrix instructions first: the second block's run in the matrix pipe while the first block is updated
      floatx4 aa[2][3];
#pragma unroll
      for (int nb = 0; nb < 2; nb++)
#pragma unroll
        for (int cg = 0; cg < 3; cg++) {
          aa[nb][cg] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ks = 0; ks < 4; ks++) aa[nb][cg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xt[cg][ks], bg[nb][ks], aa[nb][cg], 0, 0, 0);
        }
      QFENCE();
#pragma unroll
      for (int nb = 0; nb < 2; nb++) {
        const int nbg = 2 * h + nb;
        const int row = 16 * nbg + l16;
        unsigned outw[3];
        float t[3][4];
#pragma unroll
        for (int cg = 0; cg < 3; cg++) {
          const floatx4 a = aa[nb][cg];
          const unsigned wv = wq[nb][cg];
          floatx2 w01 = __builtin_amdgcn_cvt_pk_f32_fp8((int)wv, false), w23 = __builtin_amdgcn_cvt_pk_f32_fp8((int)wv, true);
          t[cg][0] = __builtin_fmaf(-p.lr_eff, a[0], w01.x); t[cg][1] = __builtin_fmaf(-p.lr_eff, a[1], w01.y);
          t[cg][2] = __builtin_fmaf(-p.lr_eff, a[2], w23.x); t[cg][3] = __builtin_fmaf(-p.lr_eff, a[3], w23.y);
        }
        if (MODE == ROUND_SR_FAST) {
          // The converter does not saturate.  Results beyond +-448 are rare: the twelve values of a lane are clamped
          // only if some lane of the wavefront has one (six max3 and a compare instead of twelve med3).
          float mx = 0.f;
#pragma unroll
          for (int cg = 0; cg < 3; cg++) {
            mx = __builtin_fmaxf(__builtin_fmaxf(mx, __builtin_fabsf(t[cg][0])), __builtin_fabsf(t[cg][1]));
            mx = __builtin_fmaxf(__builtin_fmaxf(mx, __builtin_fabsf(t[cg][2])), __builtin_fabsf(t[cg][3]));
          }
          if (__builtin_amdgcn_ballot_w64(!(mx <= 448.0f)) != 0) {
#pragma unroll
            for (int cg = 0; cg < 3; cg++)
#pragma unroll
              for (int e = 0; e < 4; e++) t[cg][e] = clamp448(t[cg][e]);
          }
#pragma unroll
          for (int cg = 0; cg < 3; cg++) {
            const unsigned hsh = fast_mix((grow0 + 16 * nbg) * (unsigned)(D / 4) + (unsigned)((QCOLS * m + 48 * fg + 12 * kg + 4 * cg) >> 2), q.seed);
            int packed;
            asm volatile("" : "=v"(packed));   // every byte is written below
            packed = __builtin_amdgcn_cvt_sr_fp8_f32(t[cg][0], fast_word(hsh, 0), packed, 0);
            packed = __builtin_amdgcn_cvt_sr_fp8_f32(t[cg][1], fast_word(hsh, 1), packed, 1);
            packed = __builtin_amdgcn_cvt_sr_fp8_f32(t[cg][2], fast_word(hsh, 2), packed, 2);
            packed = __builtin_amdgcn_cvt_sr_fp8_f32(t[cg][3], fast_word(hsh, 3), packed, 3);
            outw[cg] = (unsigned)packed;
          }
        } else {
#pragma unroll
          for (int cg = 0; cg < 3; cg++)
            outw[cg] = round4<MODE>(t[cg][0], t[cg][1], t[cg][2], t[cg][3], (unsigned)(q.row0 + row), grow0 + 16 * nbg,
                                    (unsigned)(QCOLS * m + 48 * fg + 12 * kg + 4 * cg), q.seed);
        }
        if (row < q.rows_valid) {
          // the pointer comes out of scalar registers as an integer: say that it is global memory, or the store
          // becomes a flat one, which also counts as an LDS operation
          typedef __attribute__((address_space(1))) unsigned gu32;
          gu32* gp = (gu32*)(unsigned long long)(q.base + (size_t)row * D + QCOLS * m + 48 * fg + 12 * kg);
          gp[0] = outw[0]; gp[1] = outw[1]; gp[2] = outw[2];
        }
      }
    }
    { const int t = s0; s0 = s1; s1 = s2; s2 = t; }
    w0 = w0 == QRING - 1 ? 0 : w0 + 1;
  }

  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the last descriptor fetches still target LDS
  // ---- per-workgroup grad_X partial, summed in a fixed order by reduce_gx_quad_kernel
  floatx4* dst = p.partial + (size_t)g * 12 * QNT;
#pragma unroll
  for (int mb = 0; mb < 4; mb++)
#pragma unroll
    for (int nn = 0; nn < 3; nn++) dst[(mb * 3 + nn) * QNT + tid] = acc2[mb][nn];
}

// grad_X = scale * sum over quads of the member partials; writes fp32 and bf16 [batch, 768].  192 workgroups of 128
// threads: workgroup (slot, m, part) covers threads 128 part.. of the step kernel's workgroup layout.
__global__ __launch_bounds__(128) void reduce_gx_quad_kernel(const floatx4* partial, int nwg, float scale, float* gx_f32,
                                                             unsigned short* gx_bf16, int batch, int* flags) {
  // placement check: the members of a quad exchanged G through the L2 of one XCD, which holds only if all four ran there
  if (blockIdx.x == 0 && (int)threadIdx.x < (nwg >> 2) && quad_xcc_mismatch(flags + QF_XCC, (int)threadIdx.x))
    __hip_atomic_fetch_or(flags + QF_ERR, 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const int slot = blockIdx.x >> 4, m = (blockIdx.x >> 2) & 3;   // slot = mb*3+nn
  const int tid = (blockIdx.x & 3) * 128 + threadIdx.x, v = tid >> 6, lane = tid & 63, l16 = lane & 15, kg = lane >> 4;
  const int fg = v & 3, h = v >> 2;
  // the workgroups of member m, in a fixed order; eight loads in flight at a time
  floatx4 s = {0.f, 0.f, 0.f, 0.f};
  const int nq = nwg >> 5;   // quads per XCD
  for (int jq = 0; jq < nq; jq++) {
    floatx4 v[8];
#pragma unroll
    for (int x = 0; x < 8; x++) v[x] = partial[((size_t)(((jq * 4 + m) << 3) + x) * 12 + slot) * QNT + tid];
#pragma unroll
    for (int x = 0; x < 8; x++) s += v[x];
  }
  const int mb = slot / 3, nn = slot - mb * 3;
  const int col = QCOLS * m + 48 * fg + 16 * nn + l16;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    int b = 64 * h + 16 * mb + 4 * kg + i;
    if (b < batch) {
      float val = s[i] * scale;
      if (gx_f32) gx_f32[(size_t)b * D + col] = val;
      if (gx_bf16) gx_bf16[(size_t)b * D + col] = bf16_bits(val);
    }
  }
}

// Operand images of X for the quad kernel.
//   xq: e4m3(X / scale_x) in v_mfma 16x16x128 B-operand order: operand index ((b/16)*6 + ks), lane = (b%16) + 16*kg,
//       bytes 0..15: Xq[b][k = 128ks + 16kg + j], bytes 16..31: Xq[b][k = 128ks + 64 + 16kg + (j - 16)] (the order in which
//       stage A reads the weight rows from LDS)
//   xt: bf16 X^T in v_mfma 16x16x32 A-operand order: [((col/48)*3 + cg)*4 + ks][lane][8 bf16], lane = r + 16*kg,
//       element j = X[32ks + 8kg + j][col] with col = 48*(col/48) + 12*(r/4) + 4*cg + r%4
__device__ __forceinline__ void prep_x_quad_thread(int i, const unsigned short* x, int batch, float inv_scale_x, unsigned char* xq,
                                                   unsigned short* xt) {
  // one thread per (b, group of 4 features)
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
    // K step ks of 128 features; within it lane group kgq holds features 16kgq..16kgq+15 and 64+16kgq..64+16kgq+15
    int ks = k >> 7, pk = k & 127, kgq = (pk >> 4) & 3, jq = ((pk >> 6) << 4) | (pk & 15);
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
