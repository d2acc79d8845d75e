// Inference logits of the FP8 extreme-classifier layer for gfx950 (MI355X), and two small kernels shared with the
// training paths: the e4m3 operand image of X (prep_x_kernel) and the first positive of every tile (tile_ptr_kernel).
//
// Reference semantics: src/xmc_classifiers/chunked_fp8xmc_clf.py:45-60 (xfc_forward).
#include "xmc_common.h"

namespace xmc {

typedef __attribute__((address_space(3))) unsigned char lds_u8;

// 32 bytes from a 16-byte aligned LDS address
__device__ __forceinline__ intx8 lds_read32(const unsigned char* q) {
  intx4 lo = *(const intx4*)q, hi = *(const intx4*)(q + 16);
  return intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}

// Operand images of X for the inference kernel (xt: a bf16 image in matrix-operand order that the kernel does not read).
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


// ---- Top-k of the inference logits without the logits in memory: two passes over the weights.
// Pass 1 (MODE 0) visits every tile_step-th tile; workgroup g keeps, per batch row, the largest logit of the tiles it
// visited (its tiles are spread over the whole label range) and writes these maxima as order keys to gmax[g][b].  The
// k-th largest of a row's maxima is at or below the row's k-th largest logit (k different groups each hold a logit at
// or above it): topk_bound_kernel stores it as the row's bound.  Pass 2 (MODE 1) visits every tile and appends the
// logits at or above the bound to the row's candidate list (label and key), in no particular order;
// topk_pick_kernel ranks the list.  A list holds SEL_CAP entries; the count keeps running past that, and the pick
// kernel reports a row whose count exceeded it.
constexpr int SEL_CAP = 1024;
constexpr int SEL_GROUPS = 512;          // most workgroups of pass 1
constexpr int SEL_QUEUE = 256;           // candidates a workgroup of pass 2 collects in LDS between two flushes
constexpr int SEL_FLUSH = 8;             // tiles between two flushes
constexpr int SEL_LDS = FWD_LDS + 16 + SEL_QUEUE * 8;

struct SelectParams {
  const unsigned char* chunk[MAX_CHUNKS];
  int rows_per_chunk, tiles_per_chunk;
  int n_visit, tile_step;        // the launch visits tiles j * tile_step, j in [0, n_visit)
  const unsigned char* xq;       // logits operands (prep kernel layout)
  float zscale;
  long long num_labels;          // labels at or past this one do not take part
  int batch;
  unsigned short* gmax;          // MODE 0: [gridDim.x][BP] keys
  const unsigned short* bound;   // MODE 1: [BP] keys
  unsigned* count;               // MODE 1: [BP]
  unsigned* cand_label;          // MODE 1: [BP][SEL_CAP]
  unsigned short* cand_key;      // MODE 1: [BP][SEL_CAP]
};

typedef unsigned short ushortx2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned pk_max_u16(unsigned a, unsigned b) {
  return __builtin_bit_cast(unsigned, __builtin_elementwise_max(__builtin_bit_cast(ushortx2, a), __builtin_bit_cast(ushortx2, b)));
}
// order keys of two packed bf16 values (topk_key per half, without its NaN rule: a NaN with the sign bit set gets a small key)
typedef short shortx2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned key_pair(unsigned w) {
  const unsigned neg = __builtin_bit_cast(unsigned, __builtin_bit_cast(shortx2, w) >> 15);   // 0xFFFF in the negative halves
  return w ^ (neg | 0x80008000u);
}

template <int MODE>
__global__ __launch_bounds__(NT) void fp8_forward_select_kernel(const SelectParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, l16 = lane & 15, kg = lane >> 4;
  const int block = blockIdx.x, nblocks = gridDim.x;
  const unsigned lds0 = (unsigned)(size_t)(lds_u8*)lds_raw;
  intx8 xq[2][6];
#pragma unroll
  for (int nb = 0; nb < 2; nb++)
#pragma unroll
    for (int ks = 0; ks < 6; ks++)
      xq[nb][ks] = *(const intx8*)(p.xq + ((size_t)((w * 2 + nb) * 6 + ks) * 64 + lane) * 32);
  unsigned bkey[2] = {0xFFFFu, 0xFFFFu}, bm1[2] = {0xFFFEFFFEu, 0xFFFEFFFEu};
  if (MODE == 1) {
#pragma unroll
    for (int nb = 0; nb < 2; nb++) {
      const int b = 32 * w + 16 * nb + l16;
      if (b < p.batch) {
        unsigned t = p.bound[b];
        t = t < 1u ? 1u : t;
        bkey[nb] = t;
        bm1[nb] = (t - 1u) * 0x00010001u;
      }
    }
  }
  __builtin_amdgcn_s_waitcnt(0);
  auto issue = [&](int j, int buf) {
    const int t = j * p.tile_step;
    const int c = t / p.tiles_per_chunk, row0 = (t - c * p.tiles_per_chunk) * FT;
    fwd_issue_tile(p.chunk[c] + (size_t)row0 * D, min(FT, p.rows_per_chunk - row0), lds0 + (unsigned)buf * FB, w, lane);
  };
  unsigned mx[2] = {0u, 0u};
  unsigned* q_cnt = (unsigned*)(lds_raw + FWD_LDS);
  unsigned long long* q_ent = (unsigned long long*)(lds_raw + FWD_LDS + 16);
  auto emit = [&](unsigned long long ent) {
    const unsigned b = (unsigned)(ent >> 48);
    const unsigned slot = atomicAdd(p.count + b, 1u);
    if (slot < (unsigned)SEL_CAP) {
      p.cand_label[(size_t)b * SEL_CAP + slot] = 0xFFFFFFFFu - (unsigned)ent;
      p.cand_key[(size_t)b * SEL_CAP + slot] = (unsigned short)(ent >> 32);
    }
  };
  int since = 0;
  if (MODE == 1) {
    if (tid == 0) *q_cnt = 0u;   // visible to all after the first barrier below
  }
  if (block < p.n_visit) {
    issue(block, 0);
    if (block + nblocks < p.n_visit) {
      issue(block + nblocks, 1);
      asm volatile("s_waitcnt vmcnt(%0)" : : "n"(FWD_DMA) : "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();
    int buf = 0;
    for (int j = block; j < p.n_visit; j += nblocks) {
      const int t = j * p.tile_step;
      const int c = t / p.tiles_per_chunk, row0 = (t - c * p.tiles_per_chunk) * FT;
      const int rows_valid = min(FT, p.rows_per_chunk - row0);
      const long long label0 = (long long)c * p.rows_per_chunk + row0;
      const long long left = p.num_labels - label0;
      const int nvalid = (int)(left < rows_valid ? (left < 0 ? 0 : left) : rows_valid);
      const unsigned char* wt = lds_raw + buf * FB;
      const bool more = j + 2 * nblocks < p.n_visit;
      // the buffer two ahead was read in the iteration before this one, which every wavefront has left (barrier below)
      if (more) issue(j + 2 * nblocks, buf == 0 ? 2 : buf - 1);
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
      // a lane holds, for batch rows 32w + 16nb + l16, the logits of tile rows 16rb + 4kg + e (e = 0..3): the bf16
      // values the dense kernel would store, two to a word
      unsigned wp[2][2][2];
#pragma unroll
      for (int rb = 0; rb < 2; rb++)
#pragma unroll
        for (int nb = 0; nb < 2; nb++) {
          if (p.zscale != 1.0f) z[rb][nb] *= p.zscale;   // the same product as the dense kernel's
          wp[rb][nb][0] = bf16_pack2(z[rb][nb][0], z[rb][nb][1]);
          wp[rb][nb][1] = bf16_pack2(z[rb][nb][2], z[rb][nb][3]);
        }
      if (MODE == 0) {
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
#pragma unroll
          for (int nb = 0; nb < 2; nb++)
#pragma unroll
            for (int hw = 0; hw < 2; hw++) {
              unsigned kw = key_pair(wp[rb][nb][hw]);
              if (nvalid < FT) {   // rows past the end of the chunk or of the labels do not count
                const int r = 16 * rb + 4 * kg + 2 * hw;
                kw &= (r < nvalid ? 0x0000FFFFu : 0u) | (r + 1 < nvalid ? 0xFFFF0000u : 0u);
              }
              mx[nb] = pk_max_u16(mx[nb], kw);
            }
      } else {
        unsigned hit[2][2][2], any = 0u, top = 0u;
#pragma unroll
        for (int rb = 0; rb < 2; rb++)
#pragma unroll
          for (int nb = 0; nb < 2; nb++)
#pragma unroll
            for (int hw = 0; hw < 2; hw++) {
              hit[rb][nb][hw] = pk_max_u16(key_pair(wp[rb][nb][hw]), bm1[nb]) ^ bm1[nb];   // non-zero: a key above bound - 1
              any |= hit[rb][nb][hw];
              top = pk_max_u16(top, wp[rb][nb][hw]);                                      // a half above 0xFF80: a NaN with the sign bit
            }
        const bool nan = pk_max_u16(top, 0xFF80FF80u) != 0xFF80FF80u;   // (a NaN without it has a key above every bound)
        if (__builtin_amdgcn_ballot_w64(any != 0u || nan) != 0) {
#pragma unroll
          for (int rb = 0; rb < 2; rb++)
#pragma unroll
            for (int nb = 0; nb < 2; nb++) {
              const int b = 32 * w + 16 * nb + l16;
#pragma unroll
              for (int hw = 0; hw < 2; hw++)
                if ((hit[rb][nb][hw] != 0u || nan) && b < p.batch) {
#pragma unroll
                  for (int e = 0; e < 2; e++) {
                    const int r = 16 * rb + 4 * kg + 2 * hw + e;
                    const unsigned key = topk_key((unsigned short)(wp[rb][nb][hw] >> (16 * e)));
                    if (key >= bkey[nb] && r < nvalid) {
                      const unsigned long long ent = ((unsigned long long)b << 48) | ((unsigned long long)key << 32) |
                                                     (unsigned long long)(0xFFFFFFFFu - (unsigned)(label0 + r));
                      const unsigned qs = atomicAdd(q_cnt, 1u);
                      if (qs < (unsigned)SEL_QUEUE) q_ent[qs] = ent;
                      else emit(ent);   // queue full (many logits at the bound): straight to the list
                    }
                  }
                }
            }
        }
      }
      if (more) asm volatile("s_waitcnt vmcnt(%0)" : : "n"(FWD_DMA) : "memory");
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();   // the next tile has landed for every wavefront, and this one has been read by all
      buf = buf == 2 ? 0 : buf + 1;
      if (MODE == 1 && (++since == SEL_FLUSH || j + nblocks >= p.n_visit)) {
        // Candidates wait in an LDS queue and move to the rows' lists every few tiles: the list slot comes from an
        // atomic whose result a wavefront has to wait for, together with its outstanding tile loads.  Nobody adds to the
        // queue between the barrier above and the one below.
        since = 0;
        const unsigned qn = *q_cnt < (unsigned)SEL_QUEUE ? *q_cnt : (unsigned)SEL_QUEUE;
        for (unsigned i = tid; i < qn; i += NT) emit(q_ent[i]);
        __syncthreads();
        if (tid == 0) *q_cnt = 0u;
        __syncthreads();
      }
    }
  }
  if (MODE == 0) {
#pragma unroll
    for (int nb = 0; nb < 2; nb++) {
      unsigned m = mx[nb] & 0xFFFFu, h = mx[nb] >> 16;
      m = m > h ? m : h;
      const unsigned o1 = __shfl_xor(m, 16, 64);
      m = m > o1 ? m : o1;
      const unsigned o2 = __shfl_xor(m, 32, 64);
      m = m > o2 ? m : o2;
      if (kg == 0) p.gmax[(size_t)block * BP + 32 * w + 16 * nb + l16] = (unsigned short)m;
    }
  }
}

}  // namespace xmc
