// Shared pieces of the fused FP8 extreme-classifier training step for gfx950 (MI355X): parameters, geometry of the LDS
// images, direct-to-LDS loads, tile descriptors, and the two small kernels in front of the step kernel (sort of the
// positives; tile descriptors and operand images of X).  The step kernel itself is in xmc_fp8_role.hip.
//
// Work unit = a tile of 64 consecutive label rows of one chunk (64 x 768 e4m3 bytes, contiguous in HBM).  Four
// workgroups on the same XCD (a "quad") walk the same tile sequence, one workgroup per compute unit.  Member m of the
// quad owns label rows 16m..16m+15 of every tile for the logits and the sigmoid ("stage A"), and input features
// 192m..192m+191 for grad_X, grad_W and the in-place update ("stage B"), so no arithmetic is repeated and every weight
// byte is read from HBM once and written once per step.  A member reads 24 KiB per tile (its rows and its columns),
// always as whole 16-byte pieces of contiguous row segments sent straight to LDS: the vector memory path of a compute
// unit handles few cache lines per clock, and register loads in MFMA operand order (16 rows x 64 bytes per
// instruction) would keep it busy longer than the MFMAs run.
//
// Reference semantics: src/xmc_classifiers/chunked_fp8xmc_clf.py:81-123 with
// src/triton_kernels/matmul_kernel.py:204-239 (grad_X) and src/triton_kernels/fuse_kernel.py:63-113 (update).
#include "xmc_common.h"

namespace xmc {

constexpr int QNT = 512;                  // threads per workgroup (8 wavefronts)
constexpr int QCOLS = D / 4;              // features owned by one member (192)
constexpr int QWS = QCOLS + 16;           // LDS row stride of the own-column tile image (13 x 16 bytes)
constexpr int QWC_BYTES = TL * QWS;       // 13312
constexpr int QG_BYTES = 20480;           // stride of the exchange slots in global memory (a G tile takes 16 KiB of it)
constexpr int QSLOTS = 8;                 // exchange slots per quad
constexpr int QRS = D + 32;               // LDS row stride of the own-rows image (50 x 16 bytes: with an even number of
                                          // 16-byte units per row the 16-byte operand reads of stage A have no bank conflicts)
constexpr int QSPIN_LIMIT = 1 << 18;      // polls of a partner's counter before a workgroup gives up

struct QuadParams {
  unsigned char* chunk[MAX_CHUNKS];   // device pointers of the chunk weight tensors [rows_per_chunk, 768] e4m3
  unsigned seed[MAX_CHUNKS];          // per-chunk rounding seed
  int num_chunks;
  int rows_per_chunk;
  int tiles_per_chunk;
  int num_tiles;                      // tiles of all chunks
  int run_tiles;                      // tiles of this launch of the step kernel (all of them, the head's or the rest)
  const unsigned char* xq;            // logits operands (layout of prep_x_quad_thread)
  const bf16x8* xt;                   // grad_W operands
  const unsigned* keys;               // sorted positives: label*256 + batch_row
  const int* tile_ptr;                // [num_tiles+1] offsets into keys
  const uint4* desc;                  // [nquads][kmax][2] tile descriptors written by quad_desc_prep_kernel: the tiles of
                                      // one quad are consecutive entries, in the order the quad walks them
  int nquads;                         // quads of the step kernel's launch (grid / 4)
  int kmax;                           // descriptor entries per quad = ceil(run_tiles / nquads)
  floatx4* partial;                   // [gridDim.x][24][256] per-workgroup grad_X partial sums
  unsigned char* exch;                // [nquads][QSLOTS][QG_BYTES] G exchange ring
  int* flags;                         // [nquads][16] tiles-published counters; [QF_XCC + g] XCC ids; [QF_ERR] error word
  float zscale;                       // scale_w * scale_x applied to the logits accumulator
  float lr_eff;                       // lr / scale_w
  float wd_eff;                       // weight decay x scale_w (applied to the codes)
  int batch;
  // Head-Kahan layer (chunked_head_kahan_fp8xmc_clf.py:127-131): the first num_head rows of chunk 0 carry a compensation
  // term.  The tiles that contain such rows (the first head_tiles of chunk 0) are a launch of their own, with their own
  // descriptor table (kmax_head entries per quad, in front of the table of the other tiles) and counters.
  unsigned char* kahan;               // [num_head, 768] bf16 or e5m2, or null
  int num_head, head_tiles, kmax_head;
  int cnt_base;                       // first of this launch's tiles-published counters in flags
  int acc_init;                       // the grad_X partials continue from what the launch before left in `partial`
  int spin_limit;                     // polls of a partner's counter before a workgroup gives up (QSPIN_LIMIT; a test aid
                                      // lowers it to exercise the give-up path)
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

#ifndef XMC_HEAVY_TU   // the kernels below are compiled once, in the library's main translation unit
// First of the two launches in front of the step kernel: clear the counters (flags, may be null) and sort the positives
// (key = label*256 + (batch row - row0) for the batch rows row0..row0+255 that lie below `batch`; every other entry, and
// labels outside the label space, -> 0xFFFFFFFF) by rank.  Workgroup b ranks keys 64b..64b+63 of the n_pad
// (a power of two, at least 64, or 0): every workgroup builds all keys in LDS, its four wavefronts each count the keys
// that precede the workgroup's own over a quarter of the set (equal keys: the one that comes first in the input
// precedes), and the sum of the four counts is the key's position in the output.  Grid: max(1, n_pad / 64) x 256
// threads, (n_pad + 256) * 4 bytes of LDS.
// Labels are taken relative to label_base, and those outside [label_base, label_base + label_count) are dropped: a
// label space of 2^24 labels and more is sorted in segments of whole chunks (a key keeps 24 bits for the label).
__global__ __launch_bounds__(256) void quad_sort_kernel(const int* coo, int nnz, int n_pad, int batch, int row0, int label_base,
                                                        int label_count, unsigned* keys, int* flags) {
  extern __shared__ unsigned sk[];
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63;
  if (blockIdx.x == 0 && flags)
    for (int i = tid; i < QF_WORDS; i += 256)
      if (i != QF_STICKY) flags[i] = 0;
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
      const int r = e[u].x - row0;
      const long long lab = (long long)e[u].y - label_base;
      if (i < n_pad) sk[i] = (r >= 0 && r < 256 && r + row0 < batch && e[u].y >= 0 && lab >= 0 && lab < label_count && lab < (1 << 24) - 1) ? (((unsigned)lab << 8) | (unsigned)r) : 0xFFFFFFFFu;
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
                                                   unsigned short* xt, const DropoutParams& dp);

// Second launch: blocks below desc_blocks write, for every tile,
//   desc[t] = {base pointer, valid rows, seed | first key, one past the last key, row in chunk, first label}
//   tile_ptr[t] = first key whose label >= first label of tile t (binary search in the sorted keys)
// and the remaining blocks build the operand images of X.
__global__ __launch_bounds__(256) void quad_desc_prep_kernel(const QuadParams p, int n_pad, int* tile_ptr, uint4* desc, int desc_blocks,
                                                             const unsigned short* x, float inv_scale_x, unsigned char* xq,
                                                             unsigned short* xt, const DropoutParams dp) {
  if ((int)blockIdx.x >= desc_blocks) {
    prep_x_quad_thread(((int)blockIdx.x - desc_blocks) * 256 + (int)threadIdx.x, x, p.batch, inv_scale_x, xq, xt, dp);
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
    // With a compensated head its tiles have a table of their own in front; behind the head the row a tile records
    // counts from the head's end (the reference updates those rows through sliced tensors, so the offsets of its random
    // numbers restart there: chunked_head_kahan_fp8xmc_clf.py:130-131).
    const bool behind = t >= p.head_tiles;
    const int tl = behind ? t - p.head_tiles : t, km = behind ? p.kmax : p.kmax_head;
    const int slot = (behind ? p.nquads * p.kmax_head : 0) + (tl % p.nquads) * km + tl / p.nquads;
    const int row_rec = row0 - (behind && c == 0 ? p.num_head : 0);
    desc[2 * slot] = uint4{(unsigned)base, (unsigned)(base >> 32), (unsigned)min(TL, p.rows_per_chunk - row0), p.seed[c]};
    desc[2 * slot + 1] = uint4{(unsigned)p0, (unsigned)p1, (unsigned)row_rec, (unsigned)(c * p.rows_per_chunk + row0)};
  }
}

// Operand images of X for the step kernel.
//   xq: e4m3(X / scale_x) in v_mfma 16x16x128 B-operand order: operand index ((b/16)*6 + ks), lane = (b%16) + 16*kg,
//       bytes 0..15: Xq[b][k = 128ks + 16kg + j], bytes 16..31: Xq[b][k = 128ks + 64 + 16kg + (j - 16)] (the order in which
//       stage A reads the weight rows from LDS)
//   xt: bf16 X^T in v_mfma 16x16x32 A-operand order: [((col/48)*3 + cg)*4 + ks][lane][8 bf16], lane = r + 16*kg,
//       element j = X[32ks + 8kg + j][col] with col = 48*(col/48) + 12*(r/4) + 4*cg + r%4
__device__ __forceinline__ void prep_x_quad_thread(int i, const unsigned short* x, int batch, float inv_scale_x, unsigned char* xq,
                                                   unsigned short* xt, const DropoutParams& dp) {
  // one thread per (b, group of 4 features)
  if (i >= BP * (D / 4)) return;
  int b = i / (D / 4), k = (i - b * (D / 4)) * 4;
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  unsigned short raw[4] = {0, 0, 0, 0};
  if (b < batch) {
#pragma unroll
    for (int q = 0; q < 4; q++) {   // with dropout, both images are those of the dropped-out embedding
      raw[q] = dropout_bf16(x[(size_t)b * D + k + q], (unsigned)(b * D + k + q), dp);
      v[q] = bf16_from_bits(raw[q]) * inv_scale_x;
    }
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

#endif  // XMC_HEAVY_TU

}  // namespace xmc
