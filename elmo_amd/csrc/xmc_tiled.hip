// Three-kernel ("tiled") classifier step for gfx950, for the two modes of the reference that keep bf16 temporaries:
//   * bf16 weights          src/xmc_classifiers/chunked.py:85-131 with src/triton_kernels/stochastic_rounding_kernel.py:65-99
//   * simulated FP8 weights src/xmc_classifiers/chunked_fp8xmc_clf.py:98-99,110,115-116 with
//                           src/triton_kernels/fuse_kernel.py:134-199
// Per chunk, as the reference does: logits -> G (sigmoid minus targets, bf16, kept in HBM in both orientations),
// grad_X partial (split over label ranges, summed in a fixed order), grad_W + SGD update in place.  All three GEMMs
// are bf16 v_mfma_f32_16x16x32_bf16 with fp32 accumulation; e4m3 weights are widened exactly on load.  These modes are
// not the headline path: the kernels take their operands straight from global memory (L2) in MFMA operand order and
// stage only the one operand that needs a transposition (W in grad_X) through LDS.
#include "xmc_common.h"
#include <type_traits>

namespace xmc {

enum WType { W_E4M3 = 0, W_BF16 = 1 };
constexpr int T_SPLITS = 64;                       // label ranges of the grad_X kernel
constexpr int T_GROUP = 8;                         // most chunks one launch covers
constexpr int T_GROUP_ROWS = 65536;                // ... and most rows (the G buffers hold the rows of one launch)
struct TiledSeeds { unsigned s[T_GROUP]; };        // rounding seed of every chunk of a launch
// Chunks that lie one behind the other in memory and are a multiple of the tile height long are taken several per launch
// (small chunks leave a launch one tile per compute unit: prologue and tail then dominate).
__host__ __device__ inline int tiled_group(int num_chunks, int rows_per_chunk) {
  if (rows_per_chunk % TL != 0) return 1;
  int g = T_GROUP_ROWS / rows_per_chunk;
  g = g < T_GROUP ? g : T_GROUP;
  g = g < num_chunks ? g : num_chunks;
  return g < 1 ? 1 : g;
}
constexpr int T_WS2 = 48 * 2 + 16;                 // LDS row stride of a wavefront's W block, bytes

typedef short tshortx4 __attribute__((ext_vector_type(4)));
typedef short tshortx8 __attribute__((ext_vector_type(8)));

// The batch is processed in halves of up to 128 rows (1, 2 or 4 of them: up to 512 rows): logits per half, grad_X per
// pair of halves, grad_W summed over all halves in the update kernel.
constexpr int T_HALVES = 4;
__host__ __device__ inline int tiled_halves(int batch) { return batch <= BP ? 1 : batch <= 2 * BP ? 2 : 4; }
// workspace of the tiled path for `halves` batch halves (byte offsets, 256-byte aligned)
struct TiledLayout {
  size_t xb;     // X   [halves][128][768] bf16 in operand order, rows beyond the batch zero
  size_t xt;     // X^T [halves][768][128] bf16 in operand order
  size_t keys;   // sorted positive keys, one list of MAX_POS entries per pair of halves (key = label*256 + row in the pair)
  size_t gx;     // grad_X total, fp32 [halves*128][768]
  size_t part;   // grad_X partials [halves][T_SPLITS][128*768] fp32
  size_t g;      // per half: G then G^T, rows_pad x 128 bf16 each, in operand order; then tile_ptr per pair, loss shares
};
inline TiledLayout tiled_layout(int halves, int dd = D) {   // dd: features (768 or 1024)
  TiledLayout l;
  const size_t pairs = (size_t)(halves + 1) / 2;
  l.xb = 0;
  l.xt = l.xb + (size_t)halves * BP * dd * 2;
  l.keys = l.xt + (size_t)halves * BP * dd * 2;
  l.gx = l.keys + pairs * MAX_POS * 4 + 256;      // the kernels read up to seven keys past the end of a list
  l.part = l.gx + (size_t)halves * BP * dd * 4;
  l.g = l.part + (size_t)halves * T_SPLITS * BP * dd * 4;
  return l;
}

__device__ __forceinline__ bf16x8 t_fp8x8_to_bf16x8(intx2 raw) {
  bf16x2 c0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw.x, 1.0f, false), c1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw.x, 1.0f, true);
  bf16x2 c2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw.y, 1.0f, false), c3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(raw.y, 1.0f, true);
  return bf16x8{c0.x, c0.y, c1.x, c1.y, c2.x, c2.y, c3.x, c3.y};
}

// eight consecutive weights of a row, starting at element index idx (a multiple of 8), as bf16
template <int WT>
__device__ __forceinline__ bf16x8 t_load_w8(const void* w, size_t idx) {
  if (WT == W_BF16) return *(const bf16x8*)((const unsigned short*)w + idx);
  return t_fp8x8_to_bf16x8(*(const intx2*)((const unsigned char*)w + idx));
}

// X -> two zero-padded images per batch half, both in the order in which v_mfma_f32_16x16x32_bf16 takes its operands
// (element j of lane l16 + 16 kg is row l16, k = 8 kg + j of a 16 x 32 block), so that a wavefront's operand load is
// 1 KiB of consecutive bytes:
//   xb: X for the logits (optionally quantised to e4m3 and widened back, which makes the bf16 products equal to the FP8
//       ones of chunked_fp8xmc_clf.py:101-102): block (nb, ks) = batch rows 16nb.. x features 32ks..
//   xT: X^T for grad_W (never quantised): block (fblk, ks) = 16 features x batch rows 32ks.., the features of a block
//       chosen so that a lane of the update kernel owns consecutive ones
// (also clears the fp32 grad_X total, one entry per thread, and the loss shares if there are any: no launches for that)
// fp8_image: instead of the bf16 image, xb receives the e4m3 codes in the B-operand order of v_mfma_f32_16x16x128_f8f6f4
// (per half: [(16-row block)*6 + ks][lane = row % 16 + 16*((k / 32) % 4)][32 bytes], k = 128 ks + 32 (lane / 16) + byte).
// xt_split (two halves only): xT in the order of tiled_update2_kernel instead, [feature quarter][wavefront][block cg][K step
// of 32 batch rows, 8 over both halves][lane][8], row 4kq + e of block cg being feature 12kq + 4cg + e of the wavefront's 48.
// DD: features of the layer (768, or 1024 = 4 x 4 x 64; every kernel of this path takes it as its last template argument).
template <int DD>
__global__ void tiled_prep_x_kernel(const unsigned short* x, int batch, int halves, int quantize, int fp8_image, int xt_split,
                                    unsigned short* xb, unsigned short* xT, float* gx_total, float* loss_part, int n_loss,
                                    const DropoutParams dp) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= halves * BP * DD) return;
  gx_total[i] = 0.f;
  for (int j = i; j < n_loss; j += halves * BP * DD) loss_part[j] = 0.f;
  int b = i / DD, k = i - b * DD;
  unsigned short v = b < batch ? dropout_bf16(x[(size_t)b * DD + k], (unsigned)i, dp) : (unsigned short)0;
  unsigned short vq = v;
  int code = 0;
  if (quantize) {
    const float f = clamp448(bf16_from_bits(v));
    code = __builtin_amdgcn_cvt_pk_fp8_f32(f, f, 0, false);
    const floatx2 back = __builtin_amdgcn_cvt_pk_f32_fp8(code, false);
    vq = bf16_bits(back.x);
  }
  const int half = b >> 7, bh = b & 127;
  if (fp8_image)
    ((unsigned char*)xb)[(size_t)half * BP * DD + ((size_t)((bh >> 4) * (DD / 128) + (k >> 7)) * 64 + (bh & 15) + 16 * ((k >> 5) & 3)) * 32 + (k & 31)] =
        (unsigned char)(code & 0xFF);
  else
    xb[(size_t)half * BP * DD + ((size_t)((bh >> 4) * (DD / 32) + (k >> 5)) * 64 + (bh & 15) + 16 * ((k >> 3) & 3)) * 8 + (k & 7)] = vq;
  // feature k = 64 c + 16 kgk + 4 q + e sits in row 4 kgk + e of block 4 c + q: in the update kernel a lane then owns 16
  // consecutive features per step c of 64 features, and the four lanes of a label row 64 consecutive bytes
  const int kgk = (k >> 4) & 3, blk = 4 * (k >> 6) + ((k >> 2) & 3), e = k & 3;
  if (xt_split) {   // (768 features only)
    const int fbk = k / 192, r = k - fbk * 192;
    const int wq = r / 48, c48 = r - wq * 48, kq = c48 / 12, rem = c48 - kq * 12, cg = rem >> 2, rr = 4 * kq + (rem & 3);
    xT[((size_t)((((fbk * 4 + wq) * 3 + cg) * 8 + (b >> 5)) * 64 + rr + 16 * ((b >> 3) & 3))) * 8 + (b & 7)] = v;
  } else {
    xT[(size_t)half * BP * DD + ((size_t)(blk * (BP / 32) + (bh >> 5)) * 64 + (4 * kgk + e) + 16 * ((bh >> 3) & 3)) * 8 + (bh & 7)] = v;
  }
}

__global__ void tiled_zero_kernel(float* p, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

// ---- logits, sigmoid minus targets.  Persistent workgroups of 8 wavefronts; wavefront v keeps the X operand of batch
//      rows 16v..16v+15 of this half in registers (96 of them) for the whole launch.  The label rows stream through LDS
//      in sub-tiles of 32 rows (direct-to-LDS loads two sub-tiles ahead, three buffers, one barrier per sub-tile);
//      every wavefront multiplies the sub-tile with its batch rows.  Writes G twice, each in the operand order of its
//      reader so that a wavefront's operand load there is 1 KiB of consecutive bytes: for the update kernel blocks of
//      16 labels x 32 batch rows (lane = label + 16 * (batch row / 8), 8 batch rows per lane), for the grad_X kernel
//      blocks of 16 batch rows x 32 labels; rows beyond the chunk are written as zeros.
//      LOSS: also the sub-tile's share of the summed binary cross entropy of the bf16 logits z against the targets,
//      sum over labels and batch rows of max(z, 0) - [positive] z + log(1 + exp(-|z|)), the quantity that
//      _compute_loss of the reference is written to return (chunked.py:57-72), in fp32 and added per sub-tile for a
//      fixed-order sum.
constexpr int TLG_ROWS = 32;
template <int WT, int DD> struct TlgGeom {
  static constexpr int ROWB = WT == W_BF16 ? DD * 2 : DD;               // bytes of one weight row
  static constexpr int STRIDE = ROWB + 16;                               // LDS row stride
  static constexpr int SLOTS = STRIDE / 16;                              // 16-byte slots per LDS row, the last one padding
  static constexpr int PIECES = (TLG_ROWS * STRIDE + 1023) / 1024;       // wave-wide direct-to-LDS loads per sub-tile (49 or 25)
  static constexpr int BUF = PIECES * 1024;                              // bytes of one LDS buffer
  static constexpr int PER_WAVE = (PIECES + 7) / 8;                      // loads of wavefront 0 (7 or 4); the others issue at
  static constexpr int PER_WAVE_MIN = PIECES / 8;                        // least this many (6 or 3)
  static constexpr int NBUF = 3 * BUF + 64 + 8 * 1024 <= 160 * 1024 ? 3 : 2;   // LDS buffers: the loads run NBUF - 1 sub-tiles ahead
                                                                         // (two buffers for bf16 rows of 1024 features)
  static constexpr int STAGE0 = NBUF * BUF + 64;                         // 1 KiB per wavefront: its part of G, transposed
  static constexpr int LDS = STAGE0 + 8 * 1024;                          // the buffers, eight partial sums of the loss, staging
};

// 16 bytes per lane from global memory straight into LDS at byte offset ldsoff + 16*lane (wave-uniform offset).  Inline
// assembly: the compiler neither orders later LDS accesses behind it nor waits for it; completion is enforced by hand.
__device__ __forceinline__ void t_lds_load16(const unsigned char* g, unsigned ldsoff_) {
  const unsigned ldsoff = __builtin_amdgcn_readfirstlane(ldsoff_);
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(ldsoff), "v"(g) : "memory", "m0");
}

// Vector memory operations retire in order.  Per sub-tile a wavefront issues its loads of the sub-tile two steps ahead
// (always, past the end they fetch the last sub-tile again into a buffer nobody reads, so that the count is the same in
// every step) and then ten stores of G.  The wait at the top of a step leaves in flight what was issued after the
// loads of the sub-tile it is about to read.
template <int WT, bool LOSS, int DD>
__global__ __launch_bounds__(512, 1) void tiled_logits_kernel(const void* w, int rows, int nsub, const unsigned short* xb,
                                                              const unsigned* keys, const int* tile_ptr, unsigned label0_chunk,
                                                              unsigned short* glb, unsigned short* gbl, int batch, unsigned brow0,
                                                              float* loss_part) {
  typedef TlgGeom<WT, DD> G;
  constexpr int NB = G::NBUF;
  extern __shared__ __attribute__((aligned(16))) unsigned char tlg_lds[];
  __attribute__((address_space(3))) unsigned char* lds = (__attribute__((address_space(3))) unsigned char*)tlg_lds;
  // no static LDS in this kernel: the direct-to-LDS loads address LDS from byte 0
  __attribute__((address_space(3))) float* wsum = (__attribute__((address_space(3))) float*)(lds + NB * G::BUF);
  const int tid = threadIdx.x, v = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, l16 = lane & 15, kg = lane >> 4;
  // the sorted keys and the tile ranges were written by earlier launches: read them through the scalar (constant) path,
  // so that no vector-memory wait of this loop covers them
  const __attribute__((address_space(4))) unsigned* ckeys = (const __attribute__((address_space(4))) unsigned*)keys;
  const __attribute__((address_space(4))) int* ctile_ptr = (const __attribute__((address_space(4))) int*)tile_ptr;
  // source row and byte offset within the row of this lane's slot in pieces v, v+8, ..
  int prow[G::PER_WAVE], pcol[G::PER_WAVE];
#pragma unroll
  for (int s = 0; s < G::PER_WAVE; s++) {
    const int slot = (v + 8 * s) * 64 + lane;
    prow[s] = min(slot / G::SLOTS, TLG_ROWS - 1);
    pcol[s] = min(slot - (slot / G::SLOTS) * G::SLOTS, G::SLOTS - 2) * 16;
  }
  auto issue_sub = [&](int st, int buf) {
    const int s0 = min(st, nsub - 1) * TLG_ROWS;
#pragma unroll
    for (int s = 0; s < G::PER_WAVE; s++) {
      if (v + 8 * s < G::PIECES) {
        const int lr = min(s0 + prow[s], rows - 1);
        t_lds_load16((const unsigned char*)w + (size_t)lr * G::ROWB + pcol[s], (unsigned)(buf * G::BUF + (v + 8 * s) * 1024));
      }
    }
  };
  const float nlog2e = -1.44269504088896340736f;
  const int gs = (int)gridDim.x;
  __attribute__((address_space(3))) unsigned char* stg = lds + G::STAGE0 + v * 1024;
  issue_sub(blockIdx.x, 0);
  if (NB == 3) issue_sub(blockIdx.x + gs, 1);
  // the X operand of this wavefront's batch rows, behind the first sub-tiles in the memory pipeline
  bf16x8 xr[DD / 32];
#pragma unroll
  for (int ks = 0; ks < DD / 32; ks++) xr[ks] = *(const bf16x8*)(xb + ((size_t)(v * (DD / 32) + ks) * 64 + lane) * 8);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // from here on the loop counts its own operations: nothing is in flight
  int it = 0, b0 = 0, b2 = NB - 1;   // it % NB, (it + NB - 1) % NB
  for (int st = blockIdx.x; st < nsub; st += gs, it++) {
    // younger than the loads of this sub-tile: the loads of the next one and the stores of up to two steps
    // (three stores per wavefront and step: two of G^T, one of G); with two buffers only the stores of the step before
    if (NB == 2) {
      if (it > 0) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
    } else if (it == 0) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(G::PER_WAVE_MIN) : "memory");
    else if (it == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(G::PER_WAVE_MIN + 3) : "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(G::PER_WAVE_MIN + 6) : "memory");
    // range of positives of the enclosing 64-row tile: asked for here, needed after the MFMAs
    const int p0 = ctile_ptr[st >> 1], p1 = ctile_ptr[(st >> 1) + 1];
    __syncthreads();
    issue_sub(st + (NB - 1) * gs, b2);
    const int buf = b0;
    b0 = b0 == NB - 1 ? 0 : b0 + 1;
    b2 = b2 == NB - 1 ? 0 : b2 + 1;
    floatx4 acc[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
    const unsigned abase = (unsigned)(buf * G::BUF + l16 * G::STRIDE + kg * (WT == W_BF16 ? 16 : 8));
    // the LDS reads run three K steps ahead of the MFMAs (everything unrolled: xr must stay in registers)
    typedef typename std::conditional<WT == W_BF16, bf16x8, intx2>::type araw_t;
    araw_t araw[4][2];
    auto rd = [&](int ks, int lb) {
      if (WT == W_BF16) return *(const __attribute__((address_space(3))) araw_t*)(lds + abase + lb * 16 * G::STRIDE + ks * 64);
      else return *(const __attribute__((address_space(3))) araw_t*)(lds + abase + lb * 16 * G::STRIDE + ks * 32);
    };
#pragma unroll
    for (int ks = 0; ks < 3; ks++) { araw[ks][0] = rd(ks, 0); araw[ks][1] = rd(ks, 1); }
#pragma unroll
    for (int ks = 0; ks < DD / 32; ks++) {
      if (ks + 3 < DD / 32) { araw[(ks + 3) & 3][0] = rd(ks + 3, 0); araw[(ks + 3) & 3][1] = rd(ks + 3, 1); }
      __builtin_amdgcn_sched_barrier(0);   // keep the reads ahead of the MFMAs that do not need them yet
#pragma unroll
      for (int lb = 0; lb < 2; lb++) {
        bf16x8 a;
        if constexpr (WT == W_BF16) a = araw[ks & 3][lb];
        else a = t_fp8x8_to_bf16x8(araw[ks & 3][lb]);
        acc[lb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, xr[ks], acc[lb], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // acc[lb][e] = Z[label 32 st + 16 lb + 4kg + e][batch 16v + l16]
    float lsum = 0.f;
    float sg[2][4], zf[2][4];
#pragma unroll
    for (int lb = 0; lb < 2; lb++) {
      const int r0 = st * TLG_ROWS + 16 * lb;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        zf[lb][e] = bf16_rt(acc[lb][e]);
        sg[lb][e] = bf16_rt(__builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(zf[lb][e] * nlog2e)));
        if (LOSS && r0 + 4 * kg + e < rows && (int)brow0 + 16 * v + l16 < batch)
          lsum += __builtin_fmaxf(zf[lb][e], 0.f) + 0.69314718055994530942f * __builtin_amdgcn_logf(1.0f + __builtin_amdgcn_exp2f(-__builtin_fabsf(zf[lb][e]) * 1.44269504088896340736f));
      }
    }
    // Positives of the enclosing 64-row tile (set semantics: a repeated key counts once).  The keys come eight at a time
    // through the scalar path (the first tiles of a chunk sorted by label frequency hold hundreds), and a key costs vector
    // instructions only if it lies in this wavefront's block (the sub-tile's 32 labels, batch rows 16v.. of this half).
    // Up to seven keys behind the tile's last are read and ignored; the buffer behind the keys belongs to the workspace.
    if (p1 > p0) {
      typedef unsigned t_keysx8 __attribute__((ext_vector_type(8), aligned(4)));
      const unsigned lbase = label0_chunk + (unsigned)(st * TLG_ROWS);
      unsigned prev = p0 > 0 ? ckeys[p0 - 1] : ~ckeys[p0];
      for (int e0 = p0; e0 < p1; e0 += 8) {
        const t_keysx8 kk = *(const __attribute__((address_space(4))) t_keysx8*)(ckeys + e0);
#pragma unroll
        for (int j = 0; j < 8; j++) {
          const unsigned key = kk[j];
          const unsigned lrel = (key >> 8) - lbase;      // label within the sub-tile
          const unsigned b = (key & 255u) - brow0;       // batch row within this half
          if (e0 + j < p1 && key != prev && lrel < (unsigned)TLG_ROWS && (b >> 4) == (unsigned)v) {
            const bool mine = (unsigned)kg == ((lrel >> 2) & 3u) && (unsigned)l16 == (b & 15u);
            const unsigned sel = ((lrel >> 4) << 2) | (lrel & 3u);   // wave-uniform: label block and one of the lane's four labels
#pragma unroll
            for (int c = 0; c < 8; c++)
              if (sel == (unsigned)c) {
                if (LOSS && st * TLG_ROWS + 16 * (c >> 2) + 4 * kg + (c & 3) < rows) lsum -= mine ? zf[c >> 2][c & 3] : 0.f;
                sg[c >> 2][c & 3] = mine ? bf16_rt(sg[c >> 2][c & 3] - 1.0f) : sg[c >> 2][c & 3];
              }
          }
          prev = key;
        }
      }
    }
#pragma unroll
    for (int lb = 0; lb < 2; lb++) {
      const int r0 = st * TLG_ROWS + 16 * lb;
      unsigned short sb[4];
#pragma unroll
      for (int e = 0; e < 4; e++) sb[e] = (r0 + 4 * kg + e < rows) ? bf16_bits(sg[lb][e]) : (unsigned short)0;
      uint2 o;
      o.x = (unsigned)sb[0] | ((unsigned)sb[1] << 16);
      o.y = (unsigned)sb[2] | ((unsigned)sb[3] << 16);
      // G^T in operand order for grad_X: block (label / 32, batch block) of 16 batch rows x 32 labels
      *(uint2*)(gbl + ((size_t)(st * 8 + v) * 64 + l16 + 16 * (2 * lb + (kg >> 1))) * 8 + 4 * (kg & 1)) = o;
      // G for the update kernel: this wavefront's 32 labels x 16 batch rows, transposed through its own KiB of LDS
      // (label-major, 32 bytes per label)
#pragma unroll
      for (int e = 0; e < 4; e++)
        *(__attribute__((address_space(3))) unsigned short*)(stg + (16 * lb + 4 * kg + e) * 32 + 2 * l16) = sb[e];
    }
    {
      // ... and stored in the operand order of A = G X: block (16 labels, 32 batch rows) = 64 lanes x 8 batch rows,
      // lane = label + 16 * (batch row / 8).  This wavefront's batch rows are half of K step v / 2: lanes 0..31 store
      // the 512 contiguous bytes of the first label block, lanes 32..63 those of the second.
      const int lbo = lane >> 5, half = (lane >> 4) & 1;
      const intx4 gq = *(const __attribute__((address_space(3))) intx4*)(stg + (lane & 15) * 32 + 512 * lbo + 16 * half);
      *(intx4*)(glb + ((size_t)((2 * st + lbo) * 4 + (v >> 1)) * 64 + (lane & 15) + 16 * (2 * (v & 1) + half)) * 8) = gq;
    }
    if (LOSS) {
      // lanes of a wavefront, then the eight wavefronts, in a fixed order; the halves of the batch run one after the other
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) lsum += __shfl_xor(lsum, off, 64);
      if (lane == 0) wsum[v] = lsum;
      __syncthreads();
      if (tid == 0) loss_part[st] += ((wsum[0] + wsum[1]) + (wsum[2] + wsum[3])) + ((wsum[4] + wsum[5]) + (wsum[6] + wsum[7]));
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the last loads still target LDS
}

// ---- the same for the true-FP8 arithmetic with two batch halves per pass: the logits of e4m3 weights against e4m3(X)
//      are FP8 matrix products (chunked_fp8xmc_clf.py:101-102), so the rows go from LDS into v_mfma_f32_16x16x128_f8f6f4
//      as they are (no widening to bf16, a quarter of the matrix instructions per batch row) and wavefront v keeps the
//      e4m3 operand of batch rows 16v.. of BOTH halves (96 registers, as the bf16 operand of one half took): one pass over
//      the weights yields the G of 256 batch rows.  Tile loop, positives, rounding and both layouts of G as above; the
//      products are exact in fp32 either way, only the order of the fp32 sums differs from the bf16 form.
//      xq: e4m3 image of the pair's X in B-operand order, [half][(16-row block)*6 + ks][lane][32 bytes] (tiled_prep_x_kernel)
template <int DD>
__global__ __launch_bounds__(512, 1) void tiled_logits_fp8_kernel(const void* w, int rows, int nsub, const unsigned char* xq,
                                                                  const unsigned* keys, const int* tile_ptr, unsigned label0_chunk,
                                                                  unsigned short* glb, unsigned short* gbl, size_t g_half) {
  typedef TlgGeom<W_E4M3, DD> G;
  static_assert(G::NBUF == 3, "three buffers");
  constexpr int KS = DD / 128;   // K steps of the FP8 matrix instruction
  extern __shared__ __attribute__((aligned(16))) unsigned char tlg_lds[];
  __attribute__((address_space(3))) unsigned char* lds = (__attribute__((address_space(3))) unsigned char*)tlg_lds;
  const int tid = threadIdx.x, v = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, l16 = lane & 15, kg = lane >> 4;
  const __attribute__((address_space(4))) unsigned* ckeys = (const __attribute__((address_space(4))) unsigned*)keys;
  const __attribute__((address_space(4))) int* ctile_ptr = (const __attribute__((address_space(4))) int*)tile_ptr;
  int prow[G::PER_WAVE], pcol[G::PER_WAVE];
#pragma unroll
  for (int s = 0; s < G::PER_WAVE; s++) {
    const int slot = (v + 8 * s) * 64 + lane;
    prow[s] = min(slot / G::SLOTS, TLG_ROWS - 1);
    pcol[s] = min(slot - (slot / G::SLOTS) * G::SLOTS, G::SLOTS - 2) * 16;
  }
  auto issue_sub = [&](int st, int buf) {
    const int s0 = min(st, nsub - 1) * TLG_ROWS;
#pragma unroll
    for (int s = 0; s < G::PER_WAVE; s++) {
      if (v + 8 * s < G::PIECES) {
        const int lr = min(s0 + prow[s], rows - 1);
        t_lds_load16((const unsigned char*)w + (size_t)lr * G::ROWB + pcol[s], (unsigned)(buf * G::BUF + (v + 8 * s) * 1024));
      }
    }
  };
  const float nlog2e = -1.44269504088896340736f;
  const int gs = (int)gridDim.x;
  __attribute__((address_space(3))) unsigned char* stg = lds + G::STAGE0 + v * 1024;
  issue_sub(blockIdx.x, 0);
  issue_sub(blockIdx.x + gs, 1);
  intx8 xr[2][KS];   // the e4m3 operands of this wavefront's batch rows in either half
#pragma unroll
  for (int hf = 0; hf < 2; hf++)
#pragma unroll
    for (int ks = 0; ks < KS; ks++) xr[hf][ks] = *(const intx8*)(xq + (size_t)hf * BP * DD + ((size_t)(v * KS + ks) * 64 + lane) * 32);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // from here on the loop counts its own operations: nothing is in flight
  int it = 0, b0 = 0, b2 = 2;   // it % 3, (it + 2) % 3
  for (int st = blockIdx.x; st < nsub; st += gs, it++) {
    // younger than the loads of this sub-tile: the loads of the next one and the stores of up to two steps (six per
    // wavefront and step: per half two of G^T and one of G)
    if (it == 0) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(G::PER_WAVE_MIN) : "memory");
    else if (it == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(G::PER_WAVE_MIN + 6) : "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(G::PER_WAVE_MIN + 12) : "memory");
    const int p0 = ctile_ptr[st >> 1], p1 = ctile_ptr[(st >> 1) + 1];
    __syncthreads();
    issue_sub(st + 2 * gs, b2);
    const int buf = b0;
    b0 = b0 == 2 ? 0 : b0 + 1;
    b2 = b2 == 2 ? 0 : b2 + 1;
    floatx4 acc[2][2];   // [label block][half]
#pragma unroll
    for (int lb = 0; lb < 2; lb++) { acc[lb][0] = floatx4{0.f, 0.f, 0.f, 0.f}; acc[lb][1] = floatx4{0.f, 0.f, 0.f, 0.f}; }
    const unsigned abase = (unsigned)(buf * G::BUF + l16 * G::STRIDE + kg * 32);
    auto rd = [&](int ks, int lb) {
      const __attribute__((address_space(3))) intx4* q = (const __attribute__((address_space(3))) intx4*)(lds + abase + lb * 16 * G::STRIDE + ks * 128);
      const intx4 lo = q[0], hi = q[1];
      return intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };
    intx8 araw[3][2];   // the LDS reads run two K steps ahead of the matrix instructions
#pragma unroll
    for (int ks = 0; ks < 2; ks++) { araw[ks][0] = rd(ks, 0); araw[ks][1] = rd(ks, 1); }
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      if (ks + 2 < KS) { araw[(ks + 2) % 3][0] = rd(ks + 2, 0); araw[(ks + 2) % 3][1] = rd(ks + 2, 1); }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int lb = 0; lb < 2; lb++)
#pragma unroll
        for (int hf = 0; hf < 2; hf++)
          acc[lb][hf] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(araw[ks % 3][lb], xr[hf][ks], acc[lb][hf], 0, 0, 0, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    // acc[lb][hf][e] = Z[label 32 st + 16 lb + 4kg + e][batch 128 hf + 16v + l16]
#pragma unroll
    for (int hf = 0; hf < 2; hf++) {
      float sg[2][4];
#pragma unroll
      for (int lb = 0; lb < 2; lb++)
#pragma unroll
        for (int e = 0; e < 4; e++)
          sg[lb][e] = bf16_rt(__builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(bf16_rt(acc[lb][hf][e]) * nlog2e)));
      // positives of the enclosing 64-row tile, as in tiled_logits_kernel; the keys hold the row within the pair of halves
      if (p1 > p0) {
        typedef unsigned t_keysx8 __attribute__((ext_vector_type(8), aligned(4)));
        const unsigned lbase = label0_chunk + (unsigned)(st * TLG_ROWS);
        unsigned prev = p0 > 0 ? ckeys[p0 - 1] : ~ckeys[p0];
        for (int e0 = p0; e0 < p1; e0 += 8) {
          const t_keysx8 kk = *(const __attribute__((address_space(4))) t_keysx8*)(ckeys + e0);
#pragma unroll
          for (int j = 0; j < 8; j++) {
            const unsigned key = kk[j];
            const unsigned lrel = (key >> 8) - lbase;                  // label within the sub-tile
            const unsigned b = (key & 255u) - (unsigned)(BP * hf);     // batch row within this half
            if (e0 + j < p1 && key != prev && lrel < (unsigned)TLG_ROWS && (b >> 4) == (unsigned)v) {
              const bool mine = (unsigned)kg == ((lrel >> 2) & 3u) && (unsigned)l16 == (b & 15u);
              const unsigned sel = ((lrel >> 4) << 2) | (lrel & 3u);
#pragma unroll
              for (int c = 0; c < 8; c++)
                if (sel == (unsigned)c) sg[c >> 2][c & 3] = mine ? bf16_rt(sg[c >> 2][c & 3] - 1.0f) : sg[c >> 2][c & 3];
            }
            prev = key;
          }
        }
      }
      unsigned short* gl = glb + (size_t)hf * g_half;
      unsigned short* gb = gbl + (size_t)hf * g_half;
#pragma unroll
      for (int lb = 0; lb < 2; lb++) {
        const int r0 = st * TLG_ROWS + 16 * lb;
        unsigned short sb[4];
#pragma unroll
        for (int e = 0; e < 4; e++) sb[e] = (r0 + 4 * kg + e < rows) ? bf16_bits(sg[lb][e]) : (unsigned short)0;
        uint2 o;
        o.x = (unsigned)sb[0] | ((unsigned)sb[1] << 16);
        o.y = (unsigned)sb[2] | ((unsigned)sb[3] << 16);
        *(uint2*)(gb + ((size_t)(st * 8 + v) * 64 + l16 + 16 * (2 * lb + (kg >> 1))) * 8 + 4 * (kg & 1)) = o;
#pragma unroll
        for (int e = 0; e < 4; e++)
          *(__attribute__((address_space(3))) unsigned short*)(stg + (16 * lb + 4 * kg + e) * 32 + 2 * l16) = sb[e];
      }
      {
        const int lbo = lane >> 5, half = (lane >> 4) & 1;
        const intx4 gq = *(const __attribute__((address_space(3))) intx4*)(stg + (lane & 15) * 32 + 512 * lbo + 16 * half);
        *(intx4*)(gl + ((size_t)((2 * st + lbo) * 4 + (v >> 1)) * 64 + (lane & 15) + 16 * (2 * (v & 1) + half)) * 8) = gq;
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the last loads still target LDS
}

// sum of the per-workgroup loss shares in a fixed order (double precision), one workgroup
__global__ __launch_bounds__(256) void tiled_loss_kernel(const float* loss_part, int n, float* loss_out) {
  __shared__ double sh[256];
  double s = 0.0;
  for (int i = threadIdx.x; i < n; i += 256) s += (double)loss_part[i];
  sh[threadIdx.x] = s;
  __syncthreads();
  for (int off = 128; off > 0; off >>= 1) {
    if ((int)threadIdx.x < off) sh[threadIdx.x] += sh[threadIdx.x + off];
    __syncthreads();
  }
  if (threadIdx.x == 0) *loss_out = (float)sh[0];
}

// ---- grad_X partial of one label range: C[128 x 192] = G^T[128 x R] W[R x 192].  blockIdx = 8*(4*(split/8) + fb) + split%8; wavefront w
//      owns features 192fb + 48w.. (3 blocks of 16) against all 8 batch blocks.  Steps of 32 label rows: the step's
//      slice of W (32 rows x 192 features of this workgroup, whole 16-byte pieces of contiguous row segments) and its
//      8 KiB of G^T in operand order go straight to LDS, two steps ahead, in a ring of three stages; a compute unit's
//      memory path handles few cache lines per clock, and register loads in operand order touched four times as many.
//      The W operand comes back transposed (ds_read_b64_tr_b8 + exact fp8->bf16, or ds_read_b64_tr_b16).
//      With two batch halves (HV = 2) one pass over W serves both: the step's G^T of either half is staged, and the
//      workgroup's eight wavefronts are four per half; with one half they are four per four batch blocks (two wavefronts
//      per SIMD either way: one's LDS reads and conversions run under the other's matrix instructions).
template <int WT, int HV, int DD> struct TgxGeom {
  static constexpr int FB = DD / 4;                                       // features of a workgroup (192 or 256)
  static constexpr int FW = DD / 16;                                      // features of a wavefront (48 or 64)
  static constexpr int NN = FW / 16;                                      // ... in blocks of 16 (3 or 4)
  static constexpr int ROWB = WT == W_BF16 ? 2 * FB : FB;                 // bytes of this workgroup's features in one row
  static constexpr int STRIDE = ROWB + 16;                                // LDS row stride
  static constexpr int SLOTS = STRIDE / 16;                               // 16-byte slots per LDS row, the last one padding
  static constexpr int WPIECES = (32 * SLOTS + 63) / 64;                  // wave-wide loads of the W slice (7 or 13)
  static constexpr int PIECES = WPIECES + 8 * HV;                         // ... and of G^T (8 per batch half)
  static constexpr int WAVES = 8;                                         // four wavefronts (48 features each) per batch half or,
                                                                          // with one half, per four of its eight batch blocks
  static constexpr int NMB = 4 * HV;                                      // batch blocks of 16 rows per wavefront
  static constexpr int PER_WAVE = (PIECES + WAVES - 1) / WAVES;           // every wavefront issues this many per step (2 - 4)
  static constexpr int WBYTES = WPIECES * 1024;
  static constexpr int STAGE = WBYTES + 8192 * HV;
  static constexpr int LDS = 3 * STAGE;
};

//      A launch may cover several chunks that lie one behind the other in memory (cs rows each, a multiple of the tile
//      height; the last may be shorter): chunk k owns the partial slots k*spc .. k*spc+spc-1, and no label range crosses
//      a chunk boundary, so that each chunk's sum can be rounded by itself.
template <int WT, int HV, int DD>
__global__ __launch_bounds__(512) void tiled_gradx_kernel(const void* w, int rows, int rows_pad, int bound, int range, int cs, int spc,
                                                          const unsigned short* gbl, size_t g_half, floatx4* partial, size_t part_half) {
  typedef TgxGeom<WT, HV, DD> G;
  constexpr int NN = G::NN;
  extern __shared__ __attribute__((aligned(16))) unsigned char tgx_lds[];
  __attribute__((address_space(3))) unsigned char* lds = (__attribute__((address_space(3))) unsigned char*)tgx_lds;
  const unsigned lds0 = (unsigned)(size_t)lds;
  const int tid = threadIdx.x, wv = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, l16 = lane & 15, kg = lane >> 4;
  // this wavefront's 48 features of the quarter; its batch half, or with one half its four batch blocks
  const int fw = wv & 3, hw = HV == 2 ? wv >> 2 : 0, mb0 = HV == 2 ? 0 : 4 * (wv >> 2);
  // The four workgroups of a label range read the same G^T: they sit on one XCD (workgroups go to the XCDs round robin),
  // eight apart in launch order, so that three of the four reads are served by that XCD's L2.
  const int fb = ((int)blockIdx.x >> 3) & 3, split = ((int)blockIdx.x >> 5) * 8 + ((int)blockIdx.x & 7);
  const int ck = split / spc, lbeg = ck * cs + (split - ck * spc) * range;
  const int cend = min((ck + 1) * cs, bound);   // bound: the launch's rows rounded up to a tile
  if (lbeg >= cend) return;                     // the grid is rounded up to eight ranges; a short last chunk has fewer
  floatx4 acc[G::NMB][NN];
#pragma unroll
  for (int mb = 0; mb < G::NMB; mb++)
#pragma unroll
    for (int nn = 0; nn < NN; nn++) acc[mb][nn] = floatx4{0.f, 0.f, 0.f, 0.f};
  const int lend = min(lbeg + range, cend);
  const int nsteps = (lend - lbeg + 31) >> 5;
  // Every wavefront issues exactly PER_WAVE loads per step (pieces wv, wv + WAVES, ...; indices past the last piece repeat it),
  // so that "all but the newest PER_WAVE" means the step before has landed.  Steps past the end repeat the last one.
  auto issue_step = [&](int st, int stage) {
    const int l0 = lbeg + 32 * min(st, nsteps - 1);
#pragma unroll
    for (int j = 0; j < G::PER_WAVE; j++) {
      const int piece = min(wv + G::WAVES * j, G::PIECES - 1);
      if (piece < G::WPIECES) {
        const int ch = min(piece * 64 + lane, 32 * G::SLOTS - 1), row = ch / G::SLOTS, c16 = min(ch - row * G::SLOTS, G::SLOTS - 2);
        const int lr = min(l0 + row, rows - 1);   // rows past the end re-read a valid one (their G is zero)
        t_lds_load16((const unsigned char*)w + ((size_t)lr * DD + G::FB * fb) * (WT == W_BF16 ? 2 : 1) + 16 * c16,
                     lds0 + (unsigned)(stage * G::STAGE + piece * 1024));
      } else {
        const int gp = piece - G::WPIECES;   // piece gp & 7 of batch half gp >> 3
        t_lds_load16((const unsigned char*)(gbl + (size_t)(gp >> 3) * g_half + ((size_t)((l0 >> 5) * 8 + (gp & 7)) * 64 + lane) * 8),
                     lds0 + (unsigned)(stage * G::STAGE + G::WBYTES + gp * 1024));
      }
    }
  };
  if (nsteps > 0) {
    issue_step(0, 0);
    issue_step(1, 1);
  }
  int stage = 0;
  for (int st = 0; st < nsteps; st++) {
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(G::PER_WAVE) : "memory");
    __syncthreads();   // step st has landed for every wavefront; the stage of step st-1 is free
    issue_step(st + 2, stage == 0 ? 2 : stage - 1);
    const __attribute__((address_space(3))) unsigned char* wt = lds + stage * G::STAGE;
    const __attribute__((address_space(3))) unsigned char* gt = wt + G::WBYTES;
    bf16x8 ga[G::NMB];
#pragma unroll
    for (int mb = 0; mb < G::NMB; mb++)
      ga[mb] = *(const __attribute__((address_space(3))) bf16x8*)(gt + hw * 8192 + ((mb0 + mb) * 64 + lane) * 16);
    bf16x8 wb[NN];
#pragma unroll
    for (int nn = 0; nn < NN; nn++) {
      if (WT == W_BF16) {
        const unsigned off = (unsigned)((8 * kg + (l16 >> 2)) * G::STRIDE + (G::FW * fw + 16 * nn + 4 * (l16 & 3)) * 2);
        tshortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) tshortx4*)(wt + off));
        tshortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) tshortx4*)(wt + off + 4 * G::STRIDE));
        wb[nn] = __builtin_bit_cast(bf16x8, tshortx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]});
      } else {
        const unsigned off = (unsigned)((8 * kg + (l16 >> 1)) * G::STRIDE + G::FW * fw + 16 * nn + (l16 & 1) * 8);
        const intx2 raw = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) intx2*)(wt + off));
        wb[nn] = t_fp8x8_to_bf16x8(raw);
      }
    }
#pragma unroll
    for (int mb = 0; mb < G::NMB; mb++)
#pragma unroll
      for (int nn = 0; nn < NN; nn++) acc[mb][nn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ga[mb], wb[nn], acc[mb][nn], 0, 0, 0);
    stage = stage == 2 ? 0 : stage + 1;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the loads past the end still target LDS
  // acc[mb][nn][e] = C[batch 128hw + 16(mb0 + mb) + 4kg + e][feature FB fb + FW fw + 16nn + l16]
  floatx4* dst = partial + (size_t)hw * part_half + ((size_t)split * 4 + fb) * (8 * NN) * 256;
#pragma unroll
  for (int mb = 0; mb < G::NMB; mb++)
#pragma unroll
    for (int nn = 0; nn < NN; nn++) dst[((mb0 + mb) * NN + nn) * 256 + fw * 64 + lane] = acc[mb][nn];
}

// sum of the partials of one chunk and batch half in a fixed order; bf16 weights: the chunk's contribution is rounded to
// bf16 before it is added to the fp32 total (chunked.py:116).  Work of one wavefront; 384 of them cover a half.  It runs
// in the first workgroups of the chunk's update launch (the two do not depend on each other), so the sum costs no
// launch of its own and hides behind the update.
constexpr int tred_waves(int dd) { return 8 * (dd / 256) * 16; }   // (slot, feature quarter, wavefront): 384 or 512
template <int DD>
__device__ __forceinline__ void tiled_reduce_wave(int widx, int lane, const floatx4* partial, int nchunks, int spc, int cs, int range,
                                                  int bound, int round_bf16, float* gx_total) {
  // (slot, fb, wavefront of the grad_X kernel's layout); eight loads in flight
  const int slot = widx >> 4, fb = (widx >> 2) & 3, wv = widx & 3;
  const int tid = wv * 64 + lane, l16 = lane & 15, kg = lane >> 4;
  constexpr int NN = DD / 256, SL = 8 * NN;   // blocks of 16 features per wavefront; slots per (split, feature quarter)
  const int mb = slot / NN, nn = slot - mb * NN;
  const int col = (DD / 4) * fb + (DD / 16) * wv + 16 * nn + l16;
  floatx4 tot = {0.f, 0.f, 0.f, 0.f};
  for (int ck = 0; ck < nchunks; ck++) {   // the chunks of the launch, each summed (and rounded) by itself
    const int crows = min((ck + 1) * cs, bound) - ck * cs, splits = (crows + range - 1) / range;
    const floatx4* pc = partial + (size_t)ck * spc * 4 * SL * 256;
    floatx4 s = {0.f, 0.f, 0.f, 0.f};
    int sp = 0;
    for (; sp + 8 <= splits; sp += 8) {
      floatx4 v[8];
#pragma unroll
      for (int x = 0; x < 8; x++) v[x] = pc[(((size_t)(sp + x) * 4 + fb) * SL + slot) * 256 + tid];
#pragma unroll
      for (int x = 0; x < 8; x++) s += v[x];
    }
    for (; sp < splits; sp++) s += pc[(((size_t)sp * 4 + fb) * SL + slot) * 256 + tid];
#pragma unroll
    for (int i = 0; i < 4; i++) tot[i] += round_bf16 ? bf16_rt(s[i]) : s[i];
  }
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int b = 16 * mb + 4 * kg + i;
    gx_total[(size_t)b * DD + col] += tot[i];
  }
}

template <int DD>
__global__ void tiled_finalize_kernel(const float* gx_total, int batch, unsigned short* gx_bf16, float* gx_f32, const DropoutParams dp) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= batch * DD) return;
  const float v = dropout_backward(gx_total[i], (unsigned)i, dp);
  if (gx_f32) gx_f32[i] = v;
  gx_bf16[i] = bf16_bits(v);
}

// ---- grad_W and the SGD update of one chunk, in place.  blockIdx = tile*4 + fb; wavefront w owns label rows 16w..16w+15
//      of the tile and features 192fb.. (12 blocks of 16).  A^T[f][l] = sum_b X^T[f][b] G[l][b].  The rows of a feature
//      block are permuted (row 4kg+e of block nn = 4c+q is feature 192fb + 64c + 16kg + 4q + e, see tiled_prep_x_kernel)
//      so that a lane ends up with 16 consecutive features of one label row per step c, and the four lanes of a row
//      with 64 consecutive bytes.
//        bf16 weights : a = bf16(A); t = w - lr*a; RTN: bf16(t);  SR: bits(t) + (philox(seed, l*768+f) & 0xFFFF), clear 16 bits
//        e4m3 weights : t = w - lr*A;          RTN: e4m3(t); SR: add 20 bits, clear, same cast.  The cast is torch's (NaN above
//                       464; simulated FP8, chunked_fp8xmc_clf.py:116) or saturating at +-448 (true FP8, fuse_kernel.py:35).
//        head-Kahan (e4m3 weights, rows below num_head; fuse_kernel.py:202-262): t = (w + k) - lr*A, W' = round(t),
//                       k' = ((k + w) - W') - lr*A stored as bf16 (kahan_type 1) or e5m2 (2); rows behind the head take
//                       their random offsets from (row - num_head), as the reference's call on the sliced tensors does
// Four consecutive features of one row: old weights (bf16: two dwords, e4m3: one) and compensation terms in, new ones out.
template <int WT, int MODE>
__device__ __forceinline__ void t_update4(floatx4 a, const unsigned* wraw, const unsigned* kraw, bool head, int kahan_type, float lr,
                                          float wd, unsigned off0, unsigned fidx, unsigned seed, int saturate, unsigned* wout, unsigned* kout) {
  float wv4[4];
  if (WT == W_BF16) {
    wv4[0] = bf16_from_bits((unsigned short)(wraw[0] & 0xffffu)); wv4[1] = bf16_from_bits((unsigned short)(wraw[0] >> 16));
    wv4[2] = bf16_from_bits((unsigned short)(wraw[1] & 0xffffu)); wv4[3] = bf16_from_bits((unsigned short)(wraw[1] >> 16));
  } else {
    floatx2 w01 = __builtin_amdgcn_cvt_pk_f32_fp8((int)wraw[0], false), w23 = __builtin_amdgcn_cvt_pk_f32_fp8((int)wraw[0], true);
    wv4[0] = w01.x; wv4[1] = w01.y; wv4[2] = w23.x; wv4[3] = w23.y;
  }
  float kv[4] = {0.f, 0.f, 0.f, 0.f};
  if (head) {
    if (kahan_type == 1) {
      kv[0] = bf16_from_bits((unsigned short)(kraw[0] & 0xffffu)); kv[1] = bf16_from_bits((unsigned short)(kraw[0] >> 16));
      kv[2] = bf16_from_bits((unsigned short)(kraw[1] & 0xffffu)); kv[3] = bf16_from_bits((unsigned short)(kraw[1] >> 16));
    } else {
      floatx2 k01 = __builtin_amdgcn_cvt_pk_f32_bf8((int)kraw[0], false), k23 = __builtin_amdgcn_cvt_pk_f32_bf8((int)kraw[0], true);
      kv[0] = k01.x; kv[1] = k01.y; kv[2] = k23.x; kv[3] = k23.y;
    }
  }
  float t[4];
#pragma unroll
  for (int e = 0; e < 4; e++) {
    // the gradient plus the decay term wd * W in fp32 (wd = 0 leaves it as it is, bit for bit: weights are finite)
    a[e] = __builtin_fmaf(wd, wv4[e], WT == W_BF16 ? bf16_rt(a[e]) : a[e]);
    const float g = a[e];
    t[e] = __builtin_fmaf(-lr, g, head ? wv4[e] + kv[e] : wv4[e]);
    if (MODE == ROUND_SR_PHILOX) {
      const unsigned r = philox_word0(off0 + (unsigned)e, seed, 0u);
      const unsigned mask = WT == W_BF16 ? 0xFFFFu : 0xFFFFFu;
      t[e] = __uint_as_float((__float_as_uint(t[e]) + (r & mask)) & ~mask);
    }
  }
  if (WT == W_BF16) {
    if (MODE == ROUND_SR_FAST) {
      // the converter adds the upper half of the random word to the fp32 pattern and drops the lower 16 bits; the words
      // are those of the FP8 fast mode (one counter hash per four weights)
      typedef __bf16 t_bf16x2 __attribute__((ext_vector_type(2)));
      const unsigned hsh = fast_mix(fidx, seed);
      t_bf16x2 lo = {}, hi = {};
      lo = __builtin_amdgcn_cvt_sr_bf16_f32(lo, t[0], fast_word(hsh, 0), false);
      lo = __builtin_amdgcn_cvt_sr_bf16_f32(lo, t[1], fast_word(hsh, 1), true);
      hi = __builtin_amdgcn_cvt_sr_bf16_f32(hi, t[2], fast_word(hsh, 2), false);
      hi = __builtin_amdgcn_cvt_sr_bf16_f32(hi, t[3], fast_word(hsh, 3), true);
      wout[0] = __builtin_bit_cast(unsigned, lo);
      wout[1] = __builtin_bit_cast(unsigned, hi);
    } else {
      wout[0] = (unsigned)bf16_bits(t[0]) | ((unsigned)bf16_bits(t[1]) << 16);
      wout[1] = (unsigned)bf16_bits(t[2]) | ((unsigned)bf16_bits(t[3]) << 16);
    }
  } else {
    if (saturate) {
#pragma unroll
      for (int e = 0; e < 4; e++) t[e] = clamp448(t[e]);
    }
    int packed = 0;   // without the clamp: torch's cast gives NaN above 464 and so does the converter
    if (MODE == ROUND_SR_FAST) {
      // the fused kernel's mode: the converter rounds stochastically on the e4m3 grid, one counter hash per four
      // weights (fidx = global row * 192 + column / 4)
      const unsigned hsh = fast_mix(fidx, seed);
      packed = __builtin_amdgcn_cvt_sr_fp8_f32(t[0], fast_word(hsh, 0), packed, 0);
      packed = __builtin_amdgcn_cvt_sr_fp8_f32(t[1], fast_word(hsh, 1), packed, 1);
      packed = __builtin_amdgcn_cvt_sr_fp8_f32(t[2], fast_word(hsh, 2), packed, 2);
      packed = __builtin_amdgcn_cvt_sr_fp8_f32(t[3], fast_word(hsh, 3), packed, 3);
    } else {
      packed = __builtin_amdgcn_cvt_pk_fp8_f32(t[0], t[1], packed, false);
      packed = __builtin_amdgcn_cvt_pk_fp8_f32(t[2], t[3], packed, true);
    }
    wout[0] = (unsigned)packed;
    if (head) {
      floatx2 n01 = __builtin_amdgcn_cvt_pk_f32_fp8(packed, false), n23 = __builtin_amdgcn_cvt_pk_f32_fp8(packed, true);
      const float wn[4] = {n01.x, n01.y, n23.x, n23.y};
      float kn[4];
#pragma unroll
      for (int e = 0; e < 4; e++) kn[e] = __builtin_fmaf(-lr, a[e], (kv[e] + wv4[e]) - wn[e]);
      if (kahan_type == 1) {
        kout[0] = (unsigned)bf16_bits(kn[0]) | ((unsigned)bf16_bits(kn[1]) << 16);
        kout[1] = (unsigned)bf16_bits(kn[2]) | ((unsigned)bf16_bits(kn[3]) << 16);
      } else {
#pragma unroll
        for (int e = 0; e < 4; e++) kn[e] = __builtin_fminf(__builtin_fmaxf(kn[e], -57344.0f), 57344.0f);
        int pk = 0;
        pk = __builtin_amdgcn_cvt_pk_bf8_f32(kn[0], kn[1], pk, false);
        pk = __builtin_amdgcn_cvt_pk_bf8_f32(kn[2], kn[3], pk, true);
        kout[0] = (unsigned)pk;
      }
    }
  }
}

constexpr int TUP_TILES = 4;                       // tiles of 64 label rows that each group of four wavefronts processes
// A workgroup owns CS steps of 64 features (768 features: CS = 3, a feature quarter, with one or two batch halves; 1024
// features: CS = 2; CS = 1: 64 features, with four halves) and keeps their X^T operand blocks of every batch half in LDS:
// 16 KiB per step and half.
constexpr int tup_csteps(int halves, int dd = D) { return halves > 2 ? 1 : dd % 192 == 0 ? 3 : 2; }
constexpr int tup_xbytes(int halves, int dd = D) { return tup_csteps(halves, dd) * 4 * (BP / 32) * 1024; }
constexpr int tup_threads(int halves) { return halves == 1 ? 256 : 512; }
constexpr int tup_lds_bytes(int halves, int dd = D) { return halves * tup_xbytes(halves, dd); }

// Launched with tup_threads(HALVES) threads and tup_lds(HALVES) bytes of LDS: four wavefronts per tile, so that a
// compute unit runs at least eight wavefronts with one batch half (three workgroups) as with more (one workgroup of
// eight wavefronts, two tiles at a time).
// HALVES (batch halves: 1, 2 or 4) and KAHAN (a compensated head may be present) are template parameters: with run-time
// branches around the products the compiler issued every LDS operand read right in front of its matrix instruction.
template <int WT, int MODE, int HALVES, bool KAHAN, int DD>
__global__ __launch_bounds__(HALVES == 1 ? 256 : 512, HALVES == 1 ? 3 : HALVES == 2 ? 2 : 1) void tiled_update_kernel(
    void* w, int rows, int ntiles, const unsigned short* glb, size_t g_half_stride, const unsigned short* xT, float lr, float wd, TiledSeeds seeds,
    int cs, int saturate, void* kahan, int kahan_type, int num_head, unsigned label0, const floatx4* red_partial, size_t red_part_half,
    int red_nchunks, int red_spc, int red_range, int red_bound, int red_round_bf16, float* red_total) {
  static_assert(!KAHAN || WT == W_E4M3, "the compensated head belongs to the FP8 layer");
  // the first workgroups sum the chunk's grad_X partials (384 wavefronts per batch half), the others update the weights
  constexpr int CS = tup_csteps(HALVES, DD), XB = tup_xbytes(HALVES, DD), NFB = (DD / 64) / CS, WAVES = tup_threads(HALVES) / 64;
  constexpr int TRED_WAVES = tred_waves(DD), RED_BLOCKS = TRED_WAVES * HALVES / WAVES;
  if ((int)blockIdx.x < RED_BLOCKS) {
    const int widx = (int)blockIdx.x * WAVES + ((int)threadIdx.x >> 6), hh = widx / TRED_WAVES;
    tiled_reduce_wave<DD>(widx - hh * TRED_WAVES, (int)threadIdx.x & 63, red_partial + (size_t)hh * red_part_half, red_nchunks, red_spc, cs,
                      red_range, red_bound, red_round_bf16, red_total + (size_t)hh * BP * DD);
    return;
  }
  extern __shared__ __attribute__((aligned(16))) unsigned char tup_lds[];
  __attribute__((address_space(3))) unsigned char* lds = (__attribute__((address_space(3))) unsigned char*)tup_lds;
  const int tid = threadIdx.x, wv = (tid >> 6) & 3, sub = tid >> 8, nsub = (int)blockDim.x >> 8;
  const int lane = tid & 63, l16 = lane & 15, kg = lane >> 4;
  // fb: CS steps of 64 features.  The NFB workgroups of a tile group read the same rows of G: they sit on one XCD
  // (workgroups go to the XCDs round robin), eight apart in launch order, and share that XCD's L2.
  const int jb = (int)blockIdx.x - RED_BLOCKS, fb = (jb >> 3) % NFB, group = ((jb >> 3) / NFB) * 8 + (jb & 7);
  if (group * TUP_TILES * nsub >= ntiles) return;   // the grid is rounded up to eight tile groups
  // The X^T operand of these features goes to LDS once (it is contiguous in the image) and serves all tiles and
  // wavefronts of the workgroup; from global memory every MFMA would fetch its operand through L1 again.
#pragma unroll
  for (int hh = 0; hh < HALVES; hh++) {
    const intx4* src = (const intx4*)(xT + (size_t)hh * DD * BP + (size_t)fb * (XB / 2));
    for (int s = tid; s < XB / 16; s += (int)blockDim.x)
      *(__attribute__((address_space(3))) intx4*)(lds + hh * XB + s * 16) = src[s];
  }
  __syncthreads();
  // The G rows and the weights of the next tile are loaded before the products of the current one: a wavefront waits
  // for memory once per launch, not four times per tile.
  constexpr int WDW = WT == W_BF16 ? 8 : 4;   // dwords of 16 weights
  bf16x8 gf_n[HALVES][4];
  intx4 wr_n[CS][WDW / 4];
  auto load_tile = [&](int tile) {
    const int row = tile * TL + 16 * wv + l16;
    const bool live = tile < ntiles && row < rows;
#pragma unroll
    for (int hh = 0; hh < HALVES; hh++)
#pragma unroll
      for (int ks = 0; ks < 4; ks++)
        gf_n[hh][ks] = tile < ntiles ? *(const bf16x8*)(glb + hh * g_half_stride + ((size_t)((tile * 4 + wv) * 4 + ks) * 64 + lane) * 8) : bf16x8{};
#pragma unroll
    for (int c = 0; c < CS; c++) {
      const intx4* src = (const intx4*)((const unsigned char*)w + ((size_t)row * DD + 64 * (CS * fb + c) + 16 * kg) * (WT == W_BF16 ? 2 : 1));
#pragma unroll
      for (int q = 0; q < WDW / 4; q++) wr_n[c][q] = live ? src[q] : intx4{0, 0, 0, 0};
    }
  };
  load_tile(group * TUP_TILES * nsub + sub);
#pragma unroll 1
  for (int tt = 0; tt < TUP_TILES; tt++) {
  const int tile = (group * TUP_TILES + tt) * nsub + sub;
  if (tile >= ntiles) break;
  const int row = tile * TL + 16 * wv + l16;
  const bool live = row < rows;
  const bool head = KAHAN && kahan_type != 0 && row < num_head;
  // the launch may cover several chunks of cs rows (a multiple of the tile height): the tile's chunk gives the seed, and
  // the random offsets count rows from the chunk's first
  const int ck = __builtin_amdgcn_readfirstlane((tile * TL) / cs);
  const unsigned seed = seeds.s[ck];
  const int crow = row - ck * cs;
  const int orow = (WT == W_E4M3 && !head) ? crow - num_head : crow;   // row of the random offset
  bf16x8 gf[HALVES][4];
  intx4 wr_t[CS][WDW / 4];
#pragma unroll
  for (int hh = 0; hh < HALVES; hh++)
#pragma unroll
    for (int ks = 0; ks < 4; ks++) gf[hh][ks] = gf_n[hh][ks];
#pragma unroll
  for (int c = 0; c < CS; c++)
#pragma unroll
    for (int q = 0; q < WDW / 4; q++) wr_t[c][q] = wr_n[c][q];
  if (tt + 1 < TUP_TILES) load_tile(tile + nsub);
#pragma unroll
  for (int c = 0; c < CS; c++) {              // 16 consecutive features of this lane's row at a time
    const int col0 = 64 * (CS * fb + c) + 16 * kg;
    const size_t idx = (size_t)row * DD + col0;
    unsigned wr[WDW], wo[WDW], kr[8] = {0, 0, 0, 0, 0, 0, 0, 0}, ko[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int q = 0; q < WDW / 4; q++) {
      const intx4 v = wr_t[c][q];
      wr[4 * q] = (unsigned)v.x; wr[4 * q + 1] = (unsigned)v.y; wr[4 * q + 2] = (unsigned)v.z; wr[4 * q + 3] = (unsigned)v.w;
    }
#pragma unroll
    for (int q = 0; q < WDW; q++) wo[q] = 0;
    if (live && head) {
      const int kdw = kahan_type == 1 ? 8 : 4;
      const intx4* ksrc = (const intx4*)((const unsigned char*)kahan + idx * (kahan_type == 1 ? 2 : 1));
      const intx4 v0 = ksrc[0];
      kr[0] = (unsigned)v0.x; kr[1] = (unsigned)v0.y; kr[2] = (unsigned)v0.z; kr[3] = (unsigned)v0.w;
      if (kdw == 8) {
        const intx4 v1 = ksrc[1];
        kr[4] = (unsigned)v1.x; kr[5] = (unsigned)v1.y; kr[6] = (unsigned)v1.z; kr[7] = (unsigned)v1.w;
      }
    }
    // the four 16-feature products of this step: sixteen operand reads in flight (a batch of four or two products),
    // then their matrix instructions
    floatx4 acc[4];
    constexpr int QB = HALVES == 1 ? 4 : HALVES == 2 ? 2 : 1;
#pragma unroll
    for (int q0 = 0; q0 < 4; q0 += QB) {
      bf16x8 xa[QB][HALVES][4];
#pragma unroll
      for (int qq = 0; qq < QB; qq++)
#pragma unroll
        for (int hh = 0; hh < HALVES; hh++)
#pragma unroll
          for (int ks = 0; ks < 4; ks++)
            xa[qq][hh][ks] = *(const __attribute__((address_space(3))) bf16x8*)(lds + hh * XB +
                                                                                (((4 * c + q0 + qq) * (BP / 32) + ks) * 64 + lane) * 16);
#pragma unroll
      for (int qq = 0; qq < QB; qq++) {
        floatx4 a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int hh = 0; hh < HALVES; hh++)
#pragma unroll
          for (int ks = 0; ks < 4; ks++) a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[qq][hh][ks], gf[hh][ks], a, 0, 0, 0);
        acc[q0 + qq] = a;
      }
    }
    // acc[q][e] = A[label row][feature col0 + 4q + e]
    if (live) {
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const int wq = WT == W_BF16 ? 2 * q : q, kq = kahan_type == 1 ? 2 * q : q;
        t_update4<WT, MODE>(acc[q], wr + wq, kr + kq, head, kahan_type, lr, wd, (unsigned)orow * (unsigned)DD + (unsigned)(col0 + 4 * q),
                            (label0 + (unsigned)row) * (unsigned)(DD / 4) + (unsigned)((col0 + 4 * q) >> 2), seed, saturate, wo + wq,
                            ko + kq);
      }
    }
    if (live) {
      intx4* dst = (intx4*)((unsigned char*)w + idx * (WT == W_BF16 ? 2 : 1));
#pragma unroll
      for (int q = 0; q < WDW / 4; q++) dst[q] = intx4{(int)wo[4 * q], (int)wo[4 * q + 1], (int)wo[4 * q + 2], (int)wo[4 * q + 3]};
      if (head) {
        intx4* kdst = (intx4*)((unsigned char*)kahan + idx * (kahan_type == 1 ? 2 : 1));
        kdst[0] = intx4{(int)ko[0], (int)ko[1], (int)ko[2], (int)ko[3]};
        if (kahan_type == 1) kdst[1] = intx4{(int)ko[4], (int)ko[5], (int)ko[6], (int)ko[7]};
      }
    }
  }
  }
}


// ---- grad_W and the update for e4m3 weights and two batch halves, feature-split: in tiled_update_kernel a wavefront
//      owns 16 label rows and takes the X^T operand of every matrix instruction from LDS (96 reads of 1 KiB per tile, the
//      same ones in the four wavefronts of a tile: with 256 batch rows the LDS is the limit).  Here a wavefront owns 48
//      features of the workgroup's quarter and keeps their X^T operand for all 256 batch rows in registers (96 of them);
//      the tile's G - 32 KiB, already in operand order in memory - goes straight to LDS once per workgroup, two buffers,
//      and every wavefront reads its 32 blocks from there: a third of the LDS traffic.  A^T[48 features x 16 rows] per
//      row block, the features of a block permuted (row 4kg + e of block cg is feature 12kg + 4cg + e of the 48, see
//      tiled_prep_x_kernel) so that a lane ends up with 12 consecutive bytes of one weight row.  Persistent: stream s of
//      the launch walks tiles s, s + streams, ...; its four workgroups (one per feature quarter) sit on one XCD, eight
//      apart in launch order, and share the tile's G through that XCD's L2.  The first workgroups sum the grad_X
//      partials, as in tiled_update_kernel.  Same arithmetic, rounding modes and random words as there.
constexpr int TU2_GBUF = 32768;   // one tile's G: [half][row block][K step] blocks of 1 KiB
template <int MODE>
__global__ __launch_bounds__(256, 2) void tiled_update2_kernel(
    void* w, int rows, int ntiles, const unsigned short* glb, size_t g_half, const bf16x8* xt2, float lr, float wd, TiledSeeds seeds, int cs,
    int saturate, unsigned label0, const floatx4* red_partial, size_t red_part_half, int red_nchunks, int red_spc, int red_range,
    int red_bound, float* red_total) {
  constexpr int TRED_WAVES = tred_waves(D), RED_BLOCKS = TRED_WAVES * 2 / 4;   // (768 features only)
  if ((int)blockIdx.x < RED_BLOCKS) {
    const int widx = (int)blockIdx.x * 4 + ((int)threadIdx.x >> 6), hh = widx / TRED_WAVES;
    tiled_reduce_wave<D>(widx - hh * TRED_WAVES, (int)threadIdx.x & 63, red_partial + (size_t)hh * red_part_half, red_nchunks, red_spc, cs,
                      red_range, red_bound, 0, red_total + (size_t)hh * BP * D);
    return;
  }
  extern __shared__ __attribute__((aligned(16))) unsigned char tu2_lds[];
  __attribute__((address_space(3))) unsigned char* lds = (__attribute__((address_space(3))) unsigned char*)tu2_lds;
  const unsigned lds0 = (unsigned)(size_t)lds;
  const int tid = threadIdx.x, wv = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, l16 = lane & 15, kg = lane >> 4;
  const int jb = (int)blockIdx.x - RED_BLOCKS, fb = (jb >> 3) & 3, stream = (jb >> 5) * 8 + (jb & 7);
  const int nstreams = (((int)gridDim.x - RED_BLOCKS) >> 5) * 8;
  if (stream >= ntiles) return;
  bf16x8 xt[3][8];   // X^T of this wavefront's 48 features: feature blocks x K steps of 32 batch rows (both halves)
#pragma unroll
  for (int cg = 0; cg < 3; cg++)
#pragma unroll
    for (int ks = 0; ks < 8; ks++) xt[cg][ks] = xt2[(size_t)((((fb * 4 + wv) * 3 + cg) * 8 + ks) * 64 + lane)];
  // the tile's G: per half 16 KiB of consecutive memory; wavefront wv fetches pieces wv, wv + 4, ...
  auto issue_g = [&](int t, int buf) {
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const int p = wv + 4 * j, hf = p >> 4, q = p & 15;
      t_lds_load16((const unsigned char*)(glb + (size_t)hf * g_half + ((size_t)t * 16 + q) * 512) + lane * 16,
                   lds0 + (unsigned)(buf * TU2_GBUF + p * 1024));
    }
  };
  const int col0 = 192 * fb + 48 * wv + 12 * kg;   // this lane's 12 features
  // The weights come in through inline assembly like the pieces of G, so that the compiler counts none of the loads of
  // this loop and the waits below are the only ones: rows past the end read the last valid row (their result is not
  // stored).
  typedef unsigned tu2_x3 __attribute__((ext_vector_type(3)));
  auto load_w = [&](int t, tu2_x3 (&wr)[4]) {
#pragma unroll
    for (int rb = 0; rb < 4; rb++) {
      const int row = min(t * TL + 16 * rb + l16, rows - 1);
      const unsigned char* src = (const unsigned char*)w + (size_t)row * D + col0;
      asm volatile("global_load_dwordx3 %0, %1, off" : "=v"(wr[rb]) : "v"(src) : "memory");
    }
  };
  tu2_x3 wn[4];
  issue_g(stream, 0);
  load_w(stream, wn);
  int buf = 0;
  bool prev_full = false;   // the tile before stored all four row blocks: four stores are younger than this tile's loads
#pragma unroll 1
  for (int t = stream; t < ntiles; t += nstreams) {
    // This wavefront's pieces of G(t) and the weights of tile t have arrived (memory operations complete in order: all
    // but the four stores of the tile before, when it had that many); behind the barrier every wavefront's pieces are
    // there and nobody reads the other buffer any more.
    if (prev_full) asm volatile("s_waitcnt vmcnt(4)" : "+v"(wn[0]), "+v"(wn[1]), "+v"(wn[2]), "+v"(wn[3]) : : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" : "+v"(wn[0]), "+v"(wn[1]), "+v"(wn[2]), "+v"(wn[3]) : : "memory");
    __syncthreads();
    prev_full = (t + 1) * TL <= rows;
    unsigned wc[4][3];
#pragma unroll
    for (int rb = 0; rb < 4; rb++)
#pragma unroll
      for (int cg = 0; cg < 3; cg++) wc[rb][cg] = wn[rb][cg];
    if (t + nstreams < ntiles) {
      issue_g(t + nstreams, buf ^ 1);
      load_w(t + nstreams, wn);
    }
    // the launch may cover several chunks of cs rows (a multiple of the tile height): the tile's chunk gives the seed, and
    // the random offsets count rows from the chunk's first
    const int ck = __builtin_amdgcn_readfirstlane((t * TL) / cs);
    const unsigned seed = seeds.s[ck];
    const __attribute__((address_space(3))) unsigned char* gt = lds + buf * TU2_GBUF + lane * 16;
    // the products of row block rb + 1 are issued in front of the update of row block rb: they run in the matrix pipe
    // while the vector instructions of the update go through
    auto products = [&](int rb, floatx4 (&a)[3]) {
      bf16x8 bg[8];
#pragma unroll
      for (int k8 = 0; k8 < 8; k8++)
        bg[k8] = *(const __attribute__((address_space(3))) bf16x8*)(gt + ((k8 >> 2) * 16 + rb * 4 + (k8 & 3)) * 1024);
#pragma unroll
      for (int cg = 0; cg < 3; cg++) a[cg] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int k8 = 0; k8 < 8; k8++)
#pragma unroll
        for (int cg = 0; cg < 3; cg++) a[cg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xt[cg][k8], bg[k8], a[cg], 0, 0, 0);
    };
    floatx4 acc[2][3];
    products(0, acc[0]);
#pragma unroll
    for (int rb = 0; rb < 4; rb++) {
      if (rb + 1 < 4) products(rb + 1, acc[(rb + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
      const floatx4 (&a)[3] = acc[rb & 1];
      // a[cg][e] = A[label row 16rb + l16][feature col0 + 4cg + e]
      const int row = t * TL + 16 * rb + l16, orow = row - ck * cs;
      if (row < rows) {
        unsigned wo[3];
#pragma unroll
        for (int cg = 0; cg < 3; cg++)
          t_update4<W_E4M3, MODE>(a[cg], &wc[rb][cg], nullptr, false, 0, lr, wd, (unsigned)orow * (unsigned)D + (unsigned)(col0 + 4 * cg),
                                  (label0 + (unsigned)row) * (unsigned)(D / 4) + (unsigned)((col0 + 4 * cg) >> 2), seed, saturate, &wo[cg],
                                  nullptr);
        unsigned* dst = (unsigned*)((unsigned char*)w + (size_t)row * D + col0);
        dst[0] = wo[0]; dst[1] = wo[1]; dst[2] = wo[2];
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    buf ^= 1;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

}  // namespace xmc
