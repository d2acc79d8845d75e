// Fused FP8 extreme-classifier training step for gfx950 (MI355X), second generation: the four compute units of a quad
// share a tile stream as in xmc_fp8_quad.hip, but the two wavefronts of every SIMD have different jobs.
//
// Work unit = a tile of 64 consecutive label rows of one chunk (64 x 768 e4m3 bytes, contiguous in HBM).  Member m of
// a quad (four workgroups of 512 threads on one XCD, one per compute unit) owns label rows 16m..16m+15 of every tile
// for the logits ("stage A") and input features 192m..192m+191 for grad_X, grad_W and the update ("stage B").
//
//   wavefronts 0-3 ("A", one per SIMD): every vector-memory instruction of the tile loop (loads of weight rows, weight
//     columns, the G tiles of the partners and counters; stores of G and of the updated weights), and stage A for 32
//     batch rows each:
//       Z[16 labels x 32 rows] = W_t[16m.., :] Xq[32a.., :]^T  v_mfma_scale_f32_16x16x128_f8f6f4, Xq resident (96 registers)
//       G = bf16(sigmoid(bf16(Z))) - [positive], stored to the quad's exchange slot in global memory
//   wavefronts 4-7 ("B", one per SIMD): stage B for 48 features each, all 128 batch rows:
//       grad_X[128 x 48] += G^T W_t   v_mfma_f32_16x16x32_bf16, accumulators resident (96 registers)
//       A^T[48 x 64]      = X^T G^T    same instruction, X^T resident (48 registers)
//       W_t = round(W_t - lr A), 12 bytes per lane and row to an image of the tile's updated weights in LDS; the A
//       wavefronts store the image one iteration later, as whole 192-byte row segments
// A B wavefront issues no memory operation inside the tile loop and never waits for memory: its operands are in LDS
// when the per-tile barrier releases it.  The A wavefronts have slack (their matrix work is a fifth of a B
// wavefront's) and absorb the issue cost and latency of the loads and stores.
//
// The exchange: stage A runs RQ tiles ahead of stage B.  An A wavefront stores its part of G(t), waits for the stores at
// the end of the same iteration and then advances its own "tiles published" counter (sixteen counters per quad: member x
// A wavefront).  A wavefront a gathers block a of the next tile's G (the 4 KiB member a produced) after it has seen the
// four counters of member a's wavefronts, normally in a snapshot that arrived in LDS with the other loads of the
// iteration before; a bounded polling loop with an error word is the fallback.  The G tile is laid out member-major
// with a swizzle ([member][row'][quarter'] of 8 bytes) so that an A wavefront stores 512 contiguous bytes, the gather
// is a linear copy of 16 KiB, and both operand reads of stage B are free of LDS bank conflicts.
//
// Reference semantics: src/xmc_classifiers/chunked_fp8xmc_clf.py:81-123 with
// src/triton_kernels/matmul_kernel.py:204-239 (grad_X) and src/triton_kernels/fuse_kernel.py:63-113 (update).
#include "xmc_common.h"

namespace xmc {

constexpr int RQ = 4;                       // stage A runs this many tiles ahead of stage B
constexpr int RC_RING = RQ + 1;             // own-column images: in use, RQ - 1 landed, one landing
#ifndef XMC_NB_B
#define XMC_NB_B 3
#endif
#ifndef XMC_PD
#define XMC_PD 3
#endif
constexpr int NB_B = XMC_NB_B;              // A^T blocks (16 label rows) of a tile the B wavefronts take; the A wavefronts take the rest
// with a compensated head (KT != 0) the B wavefronts take all four: they alone then touch the compensation buffer, with
// ordinary loads and stores whose completion the compiler tracks (the A wavefronts count their loads by hand)
// With the reference's Philox recipe the update is a hundred vector instructions per weight and bounds the kernel: the
// two wavefronts of a SIMD then share it evenly.
constexpr int r_nbb(int kt, int mode) { return kt != 0 ? 4 : mode == ROUND_SR_PHILOX ? 2 : NB_B; }
constexpr int RR_RING = 3;                  // own-rows images: in use, landed, landing
constexpr int RG_BUF = 2;                   // gathered G tiles: in use, landing
constexpr int RG_BYTES = 16384;             // one G tile: 4 members x 128 rows x 32 bytes
constexpr int RO_RING = 2;                  // images of updated weights: being written, being stored to memory
constexpr int RO_BYTES = TL * QCOLS;         // image of updated weights: 64 rows x 192 bytes, no padding
constexpr int RROW_BYTES = 16 * QRS;        // own-rows image: 16 rows x 800 bytes (the 13th wave-wide piece is half a piece)
constexpr int RLDS_C = 0;
constexpr int RLDS_O = RLDS_C + RC_RING * QWC_BYTES;
constexpr int RLDS_G = RLDS_O + RO_RING * RO_BYTES;
constexpr int RLDS_R = RLDS_G + RG_BUF * RG_BYTES;
constexpr int RLDS_M = RLDS_R + RR_RING * RROW_BYTES;   // per A wavefront two snapshots of four counters (32 bytes); at +128 two abort words
constexpr int RLDS_BYTES = RLDS_M + 256;
// tiles-published counters: flags[p.cnt_base + quad*16 + member*4 + A wavefront]

static_assert(RLDS_BYTES <= 160 * 1024, "LDS budget");


// row permutation within sixteen rows of the G image: rows 8..11 and 12..15 trade places, so that the four row groups
// a transposing read touches (rows 8kg..8kg+3) fall into different halves of the LDS banks
__device__ __forceinline__ int g_row16(int r) { return r ^ ((r >> 1) & 4); }

// Everything a wavefront needs for the A^T blocks it takes (features 192m + 48f .. +47 of label rows 16nb..16nb+15):
// per-lane address parts, the resident X^T operand and the state of the update under way.
struct RBlockLane {
  unsigned bg_lane;      // G tile, transposing read: rows 8kg + l16/4, quarter l16%4
  unsigned wrow_lane;    // own-column image: old weights of row l16, 12 bytes
  unsigned orow_lane;    // image of updated weights: the same 12 bytes
  unsigned gcol;         // first of the lane's 12 features
  unsigned hash_lane;    // lane part of the random-word hash
};

// The compensation terms of one A^T block (head-Kahan layer): 12 per lane, raw (bf16: six dwords, e5m2: three), and
// whether the lane's row carries one at all.
struct RKahanBlock { unsigned raw[6]; bool head; int row; };

// piece c (0..7) of the update of A^T block nb (12 weights per lane): pieces 0-2 decode the old weights and form
// T = W - lr A, 3-5 make the random words' hashes, 6-7 round, 7 stores.  Split so that the vector instructions can be
// issued between matrix instructions.  With MODE.FP16_OVFL set the fp8 converters saturate, so nothing is clamped here.
//
// KT != 0 (compensation buffer of bf16 (1) or e5m2 (2) values, chunked_head_kahan_fp8xmc_clf.py:127-131 with
// fuse_kernel.py:237-262): on rows that carry a term k the update is
//   T = (W + k) - lr A,  W' = round(T),  k' = cast(((k + W) - W') - lr A)
// and on the other rows of the tile (behind the head's end) the plain update, whose random offsets count from that end.
template <int MODE, bool WD, int KT>
__device__ __forceinline__ void r_update_piece(int c, int nb, const floatx4 (&ab)[3], const unsigned (&wq)[3], float (&t)[3][4],
                                               unsigned (&hs)[3], unsigned (&outw)[3], unsigned (&knew)[6], const RBlockLane& bl, const QTile& q,
                                               unsigned hash_tile, float lr_eff, float wd_eff, int l16, qlds_u8* lds, unsigned oimg,
                                               const RKahanBlock& kb, unsigned char* kahan, int num_head) {
  // W + k of column group cg (exact decode of both; k = 0 on rows without a term)
  auto kahan_sum = [&](int cg, float (&s)[4]) {
    const unsigned wv = wq[cg];
    floatx2 w01 = __builtin_amdgcn_cvt_pk_f32_fp8((int)wv, false), w23 = __builtin_amdgcn_cvt_pk_f32_fp8((int)wv, true);
    float k[4];
    if (KT == 1) {
      k[0] = __uint_as_float(kb.raw[2 * cg] << 16); k[1] = __uint_as_float(kb.raw[2 * cg] & 0xFFFF0000u);
      k[2] = __uint_as_float(kb.raw[2 * cg + 1] << 16); k[3] = __uint_as_float(kb.raw[2 * cg + 1] & 0xFFFF0000u);
    } else {
      floatx2 k01 = __builtin_amdgcn_cvt_pk_f32_bf8((int)kb.raw[cg], false), k23 = __builtin_amdgcn_cvt_pk_f32_bf8((int)kb.raw[cg], true);
      k[0] = k01.x; k[1] = k01.y; k[2] = k23.x; k[3] = k23.y;
    }
    s[0] = w01.x + k[0]; s[1] = w01.y + k[1]; s[2] = w23.x + k[2]; s[3] = w23.y + k[3];
  };
  if (c < 3) {
    const int cg = c;
    const unsigned wv = wq[cg];
    floatx2 w01 = __builtin_amdgcn_cvt_pk_f32_fp8((int)wv, false), w23 = __builtin_amdgcn_cvt_pk_f32_fp8((int)wv, true);
    if (KT != 0) {
      float s[4];
      kahan_sum(cg, s);
#pragma unroll
      for (int e = 0; e < 4; e++) t[cg][e] = __builtin_fmaf(-lr_eff, ab[cg][e], s[e]);
    } else if (WD) {   // T = W - lr (A + wd W): the decayed gradient first, in fp32
      t[cg][0] = __builtin_fmaf(-lr_eff, __builtin_fmaf(wd_eff, w01.x, ab[cg][0]), w01.x);
      t[cg][1] = __builtin_fmaf(-lr_eff, __builtin_fmaf(wd_eff, w01.y, ab[cg][1]), w01.y);
      t[cg][2] = __builtin_fmaf(-lr_eff, __builtin_fmaf(wd_eff, w23.x, ab[cg][2]), w23.x);
      t[cg][3] = __builtin_fmaf(-lr_eff, __builtin_fmaf(wd_eff, w23.y, ab[cg][3]), w23.y);
    } else {
      t[cg][0] = __builtin_fmaf(-lr_eff, ab[cg][0], w01.x); t[cg][1] = __builtin_fmaf(-lr_eff, ab[cg][1], w01.y);
      t[cg][2] = __builtin_fmaf(-lr_eff, ab[cg][2], w23.x); t[cg][3] = __builtin_fmaf(-lr_eff, ab[cg][3], w23.y);
    }
  } else if (c < 6) {
    const int cg = c - 3;
    if (MODE == ROUND_SR_FAST) {
      // fast_mix(idx, seed) with idx = (label0 + 16nb + l16) * 192 + (gcol + 4cg) / 4: the product idx * 0x9E3779B1 is
      // the sum of a per-tile scalar, a per-lane constant and a literal
      unsigned h = bl.hash_lane + (hash_tile + (unsigned)(16 * nb * (D / 4) + cg) * 0x9E3779B1u);
      h ^= h >> 16; h *= 0x85EBCA77u; h ^= h >> 15;
      hs[cg] = h;
    }
    if (MODE == ROUND_SR_PHILOX) {
      // the reference's recipe on this column group's four targets, one Philox word after the other: the counter of
      // the next word passes through an opaque statement together with this word's result, so that the four chains of
      // ten rounds are not interleaved (forty live registers that this kernel does not have)
      const int row = 16 * nb + l16;
      const int rrow = KT != 0 ? (kb.head ? kb.row : kb.row - num_head) : q.row0 + row;
      unsigned off = (unsigned)rrow * (unsigned)D + bl.gcol + 4 * cg;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const unsigned r = philox_word0(off + e, q.seed, 0u) & 0xFFFFFu;
        unsigned tb = (__float_as_uint(t[cg][e]) + r) & 0xFFF00000u;
        asm volatile("" : "+v"(off), "+v"(tb));
        t[cg][e] = __uint_as_float(tb);
      }
    }
  } else {
#pragma unroll
    for (int cg = (c == 6 ? 0 : 2); cg < (c == 6 ? 2 : 3); cg++) {
      if (MODE == ROUND_SR_FAST) {
        int packed;
        asm volatile("" : "=v"(packed));   // every byte is written below
        packed = __builtin_amdgcn_cvt_sr_fp8_f32(t[cg][0], fast_word(hs[cg], 0), packed, 0);
        packed = __builtin_amdgcn_cvt_sr_fp8_f32(t[cg][1], fast_word(hs[cg], 1), packed, 1);
        packed = __builtin_amdgcn_cvt_sr_fp8_f32(t[cg][2], fast_word(hs[cg], 2), packed, 2);
        packed = __builtin_amdgcn_cvt_sr_fp8_f32(t[cg][3], fast_word(hs[cg], 3), packed, 3);
        outw[cg] = (unsigned)packed;
      } else {
        // round to nearest (the Philox recipe has been applied to T by now); the converter saturates
        int packed;
        asm volatile("" : "=v"(packed));   // every byte is written below
        packed = __builtin_amdgcn_cvt_pk_fp8_f32(t[cg][0], t[cg][1], packed, false);
        packed = __builtin_amdgcn_cvt_pk_fp8_f32(t[cg][2], t[cg][3], packed, true);
        outw[cg] = (unsigned)packed;
      }
      if (KT != 0) {
        float s[4], kn[4];
        kahan_sum(cg, s);
        floatx2 n01 = __builtin_amdgcn_cvt_pk_f32_fp8((int)outw[cg], false), n23 = __builtin_amdgcn_cvt_pk_f32_fp8((int)outw[cg], true);
        kn[0] = __builtin_fmaf(-lr_eff, ab[cg][0], s[0] - n01.x); kn[1] = __builtin_fmaf(-lr_eff, ab[cg][1], s[1] - n01.y);
        kn[2] = __builtin_fmaf(-lr_eff, ab[cg][2], s[2] - n23.x); kn[3] = __builtin_fmaf(-lr_eff, ab[cg][3], s[3] - n23.y);
        // this column group's new terms, packed; the block's 24 (bf16) or 12 (e5m2) bytes per lane go to memory together
        // behind the last column group (two stores or one instead of three: the buffer's rows are 1,536 or 768 bytes
        // apart, and what a scattered store costs is its cache lines, not its bytes)
        if (KT == 1) {
          knew[2 * cg] = bf16_pack2(kn[0], kn[1]); knew[2 * cg + 1] = bf16_pack2(kn[2], kn[3]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; e++) kn[e] = __builtin_fminf(__builtin_fmaxf(kn[e], -57344.0f), 57344.0f);
          int pk = 0;
          pk = __builtin_amdgcn_cvt_pk_bf8_f32(kn[0], kn[1], pk, false);
          pk = __builtin_amdgcn_cvt_pk_bf8_f32(kn[2], kn[3], pk, true);
          knew[cg] = (unsigned)pk;
        }
      }
    }
    if (KT != 0 && c == 7 && kb.head) {
      // (the lane's 24 or 12 bytes start at a multiple of 8 or 4 bytes: the vector types carry that alignment)
      typedef unsigned k_ux4 __attribute__((ext_vector_type(4), aligned(8)));
      typedef unsigned k_ux3 __attribute__((ext_vector_type(3), aligned(4)));
      if (KT == 1) {
        unsigned char* dst = kahan + ((size_t)kb.row * D + bl.gcol) * 2;
        *(k_ux4*)dst = k_ux4{knew[0], knew[1], knew[2], knew[3]};
        *(uint2*)(dst + 16) = uint2{knew[4], knew[5]};
      } else {
        *(k_ux3*)(kahan + (size_t)kb.row * D + bl.gcol) = k_ux3{knew[0], knew[1], knew[2]};
      }
    }
    if (c == 7) {
      // the block's 12 bytes per lane go to the image of updated weights in LDS (rows of 192 bytes);
      // the image is stored to memory as whole 192-byte row segments in the next iteration
      typedef unsigned uintx3 __attribute__((ext_vector_type(3)));
      *(__attribute__((address_space(3))) uintx3*)(lds + oimg + bl.orow_lane + 16 * nb * QCOLS) = uintx3{outw[0], outw[1], outw[2]};
    }
  }
}

template <int MODE, bool WD, int KT>
__global__ __launch_bounds__(QNT, 1) void fp8_step_role_kernel(const QuadParams p) {
  constexpr int NBB = r_nbb(KT, MODE);          // A^T blocks of a tile the B wavefronts take
  constexpr int NBA = 4 - NBB > 0 ? 4 - NBB : 1;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  qlds_u8* lds = (qlds_u8*)lds_raw;
  // fp8 conversions saturate at +-448 instead of returning NaN (MODE.FP16_OVFL; infinities and NaN still give NaN)
  asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 23, 1), 1");

  const int tid = threadIdx.x;
  const int v = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, l16 = lane & 15, kg = lane >> 4;
  const int g = blockIdx.x;
  const int xcd = g & 7, j = g >> 3, m = j & 3;
  const int nquads = gridDim.x >> 2;
  const int quad = (j >> 2) * 8 + xcd;
  const int n_it = quad < p.run_tiles ? (p.run_tiles - quad + nquads - 1) / nquads : 0;

  q_cdesc* cdesc = (q_cdesc*)p.desc;
  // descriptor entry of position k in this quad's sequence; positions past the end fall back to entry 0 (tile 0), whose
  // data is loaded and never used
  auto tile_at = [&](int k) { return k < n_it ? quad * p.kmax + k : 0; };
  unsigned char* exq = p.exch + (size_t)quad * QSLOTS * QG_BYTES;   // this quad's ring of exchange slots
  int* errw = p.flags + QF_ERR;
  typedef __attribute__((address_space(3))) int lds_int;
  // the XCD this workgroup really runs on: the reduction kernel compares the four members of every quad
  if (tid == 0) {
    p.flags[QF_XCC + g] = (int)(__builtin_amdgcn_s_getreg((3 << 11) | 20) & 15);   // XCC_ID
    *(lds_int*)(lds + RLDS_M + 128) = 0;
    *(lds_int*)(lds + RLDS_M + 132) = 0;
  }
  // abort word written during iteration i (a bounded wait expired): slot i & 1; everybody reads it behind the next barrier
  const unsigned abort_base = (unsigned)(RLDS_M + 128);

  // the wavefront's share of stage B: features 192m + 48f .. +47 (f = its SIMD)
  const int f = v & 3;
  RBlockLane bl;
  bl.bg_lane = (unsigned)((kg >> 1) * 512 + g_row16(8 * (kg & 1) + (l16 >> 2)) * 32 + (((((l16 >> 1) & 1) ^ (kg & 1)) << 1) | (l16 & 1)) * 8);
  bl.wrow_lane = (unsigned)(l16 * QWS + 48 * f + 12 * kg);
  bl.orow_lane = (unsigned)(l16 * QCOLS + 48 * f + 12 * kg);
  bl.gcol = (unsigned)(QCOLS * m + 48 * f + 12 * kg);
  bl.hash_lane = ((unsigned)l16 * (unsigned)(D / 4) + (bl.gcol >> 2)) * 0x9E3779B1u;
  bf16x8 xt[3][4];       // grad_W: feature blocks of this wavefront's 48 features, K steps of 32 batch rows
#pragma unroll
  for (int cg = 0; cg < 3; cg++)
#pragma unroll
    for (int ks = 0; ks < 4; ks++) xt[cg][ks] = p.xt[(size_t)(((4 * m + f) * 3 + cg) * 4 + ks) * 64 + lane];
  // operand of A^T block nb, K step ks (32 batch rows): two transposing reads
  auto read_bg = [&](unsigned gwl, unsigned gwh, int nb, int ks) {
    shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4*)(lds + gwl + nb * 4096 + ks * 1024));
    shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4*)(lds + gwh + nb * 4096 + ks * 1024));
    return __builtin_bit_cast(bf16x8, shortx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]});
  };

  if (v < 4) {
    // =========================================================================================== A wavefronts
    const int a = v;
    int* myflag = p.flags + p.cnt_base + quad * 16 + m * 4 + a;
    const int* srcflags = p.flags + p.cnt_base + quad * 16 + a * 4;
    const __attribute__((address_space(4))) unsigned* ckeys = (const __attribute__((address_space(4))) unsigned*)p.keys;

    intx8 xq[2][6];   // logits operands: batch blocks 2a, 2a+1, K steps of 128
#pragma unroll
    for (int blk = 0; blk < 2; blk++)
#pragma unroll
      for (int ks = 0; ks < 6; ks++) xq[blk][ks] = *(const intx8*)(p.xq + ((size_t)(((2 * a + blk) * 6 + ks) * 64 + lane)) * 32);

    // Per-lane byte offsets of the wave-wide 1 KiB pieces this wavefront loads.  own-column image: 64 rows x 13 chunks of
    // 16 bytes (12 data + 1 pad) = 13 pieces; own-rows image: rows 16m..16m+15, 16 x 50 chunks (48 data + 2 pad) = 13
    // pieces.  Wavefront a takes column pieces a, a+4, a+8 (and 12 if a == 0) and row pieces ra, ra+4, ra+8 (and 12 if
    // ra == 0) with ra = (a + 3) % 4, so that no wavefront has both extra pieces.
    const int ra = (a + 3) & 3;
    auto wcol_offset = [&](int s, int last_row) {
      const int ch = (a + 4 * s) * 64 + lane, wr = ch / 13;
      return (unsigned)(min(wr, last_row) * D + QCOLS * m + min(ch - wr * 13, 11) * 16);
    };
    auto rows_offset = [&](int s, int last_row) {
      const int ch = (ra + 4 * s) * 64 + lane, rr = ch / (QRS / 16);
      return (unsigned)(min(16 * m + min(rr, 15), last_row) * D + min(ch - rr * (QRS / 16), 47) * 16);
    };
    unsigned woff_full[4], roff_full[4];
#pragma unroll
    for (int s = 0; s < 4; s++) {
      woff_full[s] = wcol_offset(s, TL - 1);
      roff_full[s] = rows_offset(s, TL - 1);
    }
    auto wcol_piece = [&](int slot, const QTile& q, int s) {
      if (a + 4 * s >= 13) return;
      const unsigned off = q.rows_valid == TL ? woff_full[s] : wcol_offset(s, q.rows_valid - 1);
      q_lds_load16_sbase(q.base, off, (unsigned)(RLDS_C + slot * QWC_BYTES + (a + 4 * s) * 1024));
    };
    auto rows_piece = [&](int slot, const QTile& q, int s) {
      if (ra + 4 * s >= 13) return;
      const unsigned off = q.rows_valid == TL ? roff_full[s] : rows_offset(s, q.rows_valid - 1);
      if (ra + 4 * s == 12) {   // the last piece is half a piece: 32 chunks
        if (lane < 32) q_lds_load16_sbase(q.base, off, (unsigned)(RLDS_R + slot * RROW_BYTES + 12 * 1024));
      } else {
        q_lds_load16_sbase(q.base, off, (unsigned)(RLDS_R + slot * RROW_BYTES + (ra + 4 * s) * 1024));
      }
    };
    auto rows_pieces = [&](int slot, const QTile& q) {
#pragma unroll
      for (int s = 0; s < 4; s++) rows_piece(slot, q, s);
    };
    // block a (the part member a produced) of the G tile of position t, four pieces of 1 KiB, a linear copy
    const unsigned gsrc_lane = (unsigned)(a * 4096 + lane * 16);
    auto gather = [&](int t, int buf) {
#pragma unroll
      for (int s = 0; s < 4; s++)
        q_lds_load16_l2_sbase(exq + (t & (QSLOTS - 1)) * QG_BYTES + s * 1024, gsrc_lane,
                              (unsigned)(RLDS_G + buf * RG_BYTES + a * 4096 + s * 1024));
    };
    // the four counters of member a's wavefronts, as they are now, into LDS (read in the next iteration)
    auto issue_snapshot = [&](int i) {
      if (lane < 4) q_lds_load4_l2(srcflags + lane, (unsigned)(RLDS_M + a * 32 + (i & 1) * 16));
    };
    // wait until the four producers of block a have published at least `need` tiles
    auto wait_published = [&](int need, int fmin, int i) {
      if (fmin >= need) return;
      for (int spin = 0;; spin++) {
        int fl = __hip_atomic_load(srcflags + (lane & 3), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (__builtin_amdgcn_read_exec() == __builtin_amdgcn_ballot_w64(fl >= need)) break;
        if (spin >= p.spin_limit || ((spin & 1023) == 1023 && __hip_atomic_load(errw, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
          // give up: raise the error word (partners that wait for this workgroup see it and give up too) and the
          // workgroup's abort word; every wavefront leaves the loop behind the next barrier
          if (lane == 0) {
            __hip_atomic_fetch_or(errw, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            *(lds_int*)(lds + abort_base + (i & 1) * 4) = 1;
          }
          break;
        }
        __builtin_amdgcn_s_sleep(2);
      }
    };

    // Stage A of the tile at position t: logits of label rows 16m.. against batch rows 32a..32a+31, sigmoid minus target,
    // this wavefront's part of G to the exchange slot.  Lane (l16, kg) ends up with labels 16m + 4kg..+3 of batch rows
    // 32a + l16 and 32a + 16 + l16: eight bytes each, quarter kg of the row's 32 bytes in block m of the slot.
    // The matrix part takes a callback that runs once per K step: the caller spreads its loads over it.
    unsigned char* gdst_lane = exq + m * 4096 + (32 * a + g_row16(l16)) * 32 + ((((kg >> 1) ^ (l16 >> 3)) << 1) | (kg & 1)) * 8;
    auto stage_a_logits = [&](int slot, floatx4 (&z)[2], auto&& between) {
      // lane (row l16, k group kg) holds bytes 16kg..16kg+15 and 64+16kg..64+16kg+15 of every 128-byte K step (the X
      // image is built in the same order): two 16-byte reads whose lanes tile the LDS banks
      const unsigned asrc = (unsigned)(RLDS_R + slot * RROW_BYTES) + l16 * QRS + kg * 16;
      intx4 alo[6], ahi[6];
      auto rd = [&](int ks) {
        alo[ks] = *(const __attribute__((address_space(3))) intx4*)(lds + asrc + ks * 128);
        ahi[ks] = *(const __attribute__((address_space(3))) intx4*)(lds + asrc + ks * 128 + 64);
      };
      rd(0); rd(1); rd(2);
      QFENCE();
      z[0] = floatx4{0.f, 0.f, 0.f, 0.f}; z[1] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < 6; ks++) {
        if (ks + 3 < 6) rd(ks + 3);
        between(ks);
        intx8 av = intx8{alo[ks].x, alo[ks].y, alo[ks].z, alo[ks].w, ahi[ks].x, ahi[ks].y, ahi[ks].z, ahi[ks].w};
        z[0] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, xq[0][ks], z[0], 0, 0, 0, 0, 0, 0);
        z[1] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, xq[1][ks], z[1], 0, 0, 0, 0, 0, 0);
        QFENCE();
      }
    };
    auto stage_a_finish = [&](int t, const QTile& q, const floatx4 (&z)[2]) {
      const float nlog2e = -1.44269504088896340736f;
      const int r0 = 16 * m + 4 * kg;   // this lane's label rows r0..r0+3
      unsigned sb[2][2];
#pragma unroll
      for (int blk = 0; blk < 2; blk++)
#pragma unroll
        for (int e2 = 0; e2 < 2; e2++) {
          const unsigned zb = bf16_pack2(z[blk][2 * e2] * p.zscale, z[blk][2 * e2 + 1] * p.zscale);
          const float z0 = __uint_as_float(zb << 16), z1 = __uint_as_float(zb & 0xFFFF0000u);
          sb[blk][e2] = bf16_pack2(__builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(z0 * nlog2e)),
                                   __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(z1 * nlog2e)));
        }
      // positives of this tile (set semantics: a repeated key counts once); wave-uniform scalar loads, eight keys at a
      // time; a key costs vector instructions only if it lies in this wavefront's block (label rows 16m.., batch rows
      // 32a..).  Up to seven keys behind the tile's last are read and ignored; the buffer behind the keys belongs to
      // the workspace.
      if (q.p1 > q.p0) {
        float sg[2][4];
#pragma unroll
        for (int blk = 0; blk < 2; blk++) {
          sg[blk][0] = __uint_as_float(sb[blk][0] << 16); sg[blk][1] = __uint_as_float(sb[blk][0] & 0xFFFF0000u);
          sg[blk][2] = __uint_as_float(sb[blk][1] << 16); sg[blk][3] = __uint_as_float(sb[blk][1] & 0xFFFF0000u);
        }
        typedef unsigned q_keysx8 __attribute__((ext_vector_type(8), aligned(4)));
        const unsigned lbase = q.label0 + 16u * (unsigned)m;
        unsigned prev = q.p0 > 0 ? ckeys[q.p0 - 1] : ~ckeys[q.p0];
        for (int e0 = q.p0; e0 < q.p1; e0 += 8) {
          const q_keysx8 kk = *(const __attribute__((address_space(4))) q_keysx8*)(ckeys + e0);
#pragma unroll
          for (int jj = 0; jj < 8; jj++) {
            const unsigned key = kk[jj];
            const unsigned lrel = (key >> 8) - lbase;   // label row within this member's sixteen
            if (e0 + jj < q.p1 && key != prev && lrel < 16u && ((key >> 5) & 7u) == (unsigned)a) {
              const bool mine = (unsigned)kg == (lrel >> 2) && (unsigned)l16 == (key & 15u);
              const unsigned sel = ((key >> 4) & 1u) * 4u + (lrel & 3u);   // wave-uniform: block and one of the lane's four labels
#pragma unroll
              for (int blk = 0; blk < 2; blk++)
#pragma unroll
                for (int e = 0; e < 4; e++)
                  if (sel == (unsigned)(blk * 4 + e)) sg[blk][e] = mine ? bf16_rt(sg[blk][e] - 1.0f) : sg[blk][e];
            }
            prev = key;
          }
        }
#pragma unroll
        for (int blk = 0; blk < 2; blk++) {
          sb[blk][0] = bf16_pack2(sg[blk][0], sg[blk][1]);
          sb[blk][1] = bf16_pack2(sg[blk][2], sg[blk][3]);
        }
      }
      if (q.rows_valid < TL) {   // rows past the end of the chunk contribute nothing
#pragma unroll
        for (int blk = 0; blk < 2; blk++)
#pragma unroll
          for (int e2 = 0; e2 < 2; e2++) {
            if (r0 + 2 * e2 >= q.rows_valid) sb[blk][e2] &= 0xFFFF0000u;
            if (r0 + 2 * e2 + 1 >= q.rows_valid) sb[blk][e2] &= 0x0000FFFFu;
          }
      }
      unsigned char* dst = gdst_lane + (t & (QSLOTS - 1)) * QG_BYTES;
      *(uint2*)dst = uint2{sb[0][0], sb[0][1]};
      *(uint2*)(dst + 512) = uint2{sb[1][0], sb[1][1]};
    };

    // ---- prologue: rows and columns of the first RQ positions, their stage A, rows of the next two, G of position 0
#pragma unroll
    for (int k = 0; k < RR_RING; k++) rows_pieces(k, q_desc_head(cdesc, tile_at(k)));
#pragma unroll
    for (int k = 0; k < RQ; k++) {
      const QTile t = q_desc_head(cdesc, tile_at(k));
#pragma unroll
      for (int s = 0; s < 4; s++) wcol_piece(k, t, s);
    }
    // a wait the compiler knows of: without it, it takes the loads of xq above for outstanding wherever the loop below
    // uses them (it cannot see the waits written as inline assembly) and waits for all memory operations there
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();   // P1
    // stage A of positions 0..RQ-1; the rows image of position k + RR_RING replaces that of position k behind a barrier
#pragma unroll
    for (int k = 0; k < RQ; k++) {
      floatx4 z[2];
      if (k < n_it) {
        stage_a_logits(k % RR_RING, z, [](int) {});
        stage_a_finish(k, q_desc_full(cdesc, tile_at(k)), z);
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __syncthreads();   // P2.k: every A wavefront has read the rows image
      if (k + RR_RING < RQ + RR_RING - 1) rows_pieces(k % RR_RING, q_desc_head(cdesc, tile_at(k + RR_RING)));
      if (k + 1 < RQ && k + 1 >= RR_RING) {   // the next stage A reads an image that was just requested
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the stores of G included
    if (lane == 0 && n_it > 0) __hip_atomic_store(myflag, min(RQ, n_it), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (n_it > 0) {
      wait_published(1, 0, 1);   // an expiry here is seen behind the first barrier of the loop (slot 1 = "iteration -1")
      gather(0, 0);
    }
    issue_snapshot(1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    // descriptors of the next iteration: the tile of its stage A (whose columns it also fetches), the tile whose rows it
    // fetches and the tile of its share of stage B; loaded one iteration ahead through the scalar path
    QTile qa_n = q_desc_full(cdesc, tile_at(RQ)), qr_n = q_desc_head(cdesc, tile_at(RQ + RR_RING - 1)), qb_n = q_desc_full(cdesc, tile_at(0));
    unsigned char* qp_base = nullptr;   // the tile of the iteration before: base pointer and valid rows
    int qp_base_valid = 0;
    int sa = RQ % RR_RING;    // (i + RQ) % RR_RING, the rows image stage A reads
    int w0 = 0;               // i % RC_RING
    for (int i = 0; i < n_it; i++) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __syncthreads();
      const QTile qa = qa_n, qr = qr_n, qb = qb_n;
      const int abort_word = *(const lds_int*)(lds + abort_base + ((i + 1) & 1) * 4);
      // the counters as they were in the middle of the iteration before
      const intx4 fl = *(const __attribute__((address_space(3))) intx4*)(lds + RLDS_M + a * 32 + ((i + 1) & 1) * 16);
      if (__builtin_amdgcn_readfirstlane(abort_word) != 0) break;
      if (i + 1 < n_it) {
        const int fmin = min(min((int)__builtin_amdgcn_readfirstlane(fl.x), (int)__builtin_amdgcn_readfirstlane(fl.y)),
                             min((int)__builtin_amdgcn_readfirstlane(fl.z), (int)__builtin_amdgcn_readfirstlane(fl.w)));
        wait_published(i + 2, fmin, i);
        gather(i + 1, (i + 1) & 1);
      }
      // ---- stage A of position i + RQ, the columns of the same tile requested between its matrix instructions
      const bool do_a = i + RQ < n_it;
      const int wslot = w0 == 0 ? RC_RING - 1 : w0 - 1;   // (i + RQ) % RC_RING
      floatx4 z[2];
      stage_a_logits(sa, z, [&](int ks) { if (ks < 4) wcol_piece(wslot, qa, ks); });
      // the counters as they are now, for the next iteration; everything behind this point may stay in flight over the
      // barrier
      issue_snapshot(i);
      // ---- this wavefront's A^T blocks of position i: operands, matrix instructions
      const unsigned wc = (unsigned)(RLDS_C + w0 * QWC_BYTES);
      const unsigned gb = (unsigned)(RLDS_G + (i & 1) * RG_BYTES);
      const unsigned gwl = gb + bl.bg_lane, gwh = gb + (bl.bg_lane ^ 128u), wrow = wc + bl.wrow_lane;
      const unsigned oimg = (unsigned)(RLDS_O + (i & 1) * RO_BYTES);
      floatx4 aa[NBA][3];
      unsigned wq[NBA][3];
#pragma unroll
      for (int nb = NBB; nb < 4; nb++) {
        bf16x8 bg[4];
#pragma unroll
        for (int ks = 0; ks < 4; ks++) bg[ks] = read_bg(gwl, gwh, nb, ks);
#pragma unroll
        for (int cg = 0; cg < 3; cg++) wq[nb - NBB][cg] = *(const unsigned*)(lds + wrow + 16 * nb * QWS + 4 * cg);
#pragma unroll
        for (int ks = 0; ks < 4; ks++)
#pragma unroll
          for (int cg = 0; cg < 3; cg++)
            aa[nb - NBB][cg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xt[cg][ks], bg[ks], ks == 0 ? floatx4{0.f, 0.f, 0.f, 0.f} : aa[nb - NBB][cg], 0, 0, 0);
        QFENCE();
      }
      // descriptors of the next iteration: requested here, in front of a long stretch of vector work, because every wait
      // for an LDS read also waits for outstanding scalar loads
      qa_n = q_desc_full(cdesc, tile_at(i + 1 + RQ));
      qr_n = q_desc_head(cdesc, tile_at(i + 1 + RQ + RR_RING - 1));
      qb_n = q_desc_full(cdesc, tile_at(i + 1));
      if (do_a) stage_a_finish(i + RQ, qa, z);
      // the previous tile's updated weights, from their LDS image to memory: 12 wave-wide pieces of 16 bytes per lane,
      // three per A wavefront (chunk ch = (3a + jj) * 64 + lane is bytes 16 (ch % 12).. of row ch / 12)
      if (i > 0) {
#pragma unroll
        for (int jj = 0; jj < 3; jj++) {
          const int ch = (3 * a + jj) * 64 + lane, row = ch / 12;
          const unsigned off = (unsigned)(row * D + QCOLS * m + (ch - row * 12) * 16);
          const intx4 ov = *(const __attribute__((address_space(3))) intx4*)(lds + RLDS_O + ((i + 1) & 1) * RO_BYTES + ch * 16);
          if (qp_base_valid == TL) {
            // written through (system scope): the updated weights are not read again by this launch, and as ordinary
            // stores they push the exchanged G tiles and the weight tiles between their two fetches out of the XCD's
            // L2 (reads from memory 1.34 instead of 1.12 times the weights); same speed either way
            asm volatile("global_store_dwordx4 %0, %1, %2 sc0 sc1" : : "v"(off), "v"(ov), "s"(qp_base) : "memory");
          } else {
            // rows past the end of the chunk go to a place nobody reads (the padding behind an exchange slot), so that
            // the wavefront issues the same number of memory operations for every tile
            unsigned char* dst = row < qp_base_valid ? qp_base + off : exq + (size_t)(m * 2) * QG_BYTES + RG_BYTES + a * 1024 + lane * 16;
            asm volatile("global_store_dwordx4 %0, %1, off ; clamped rows" : : "v"(dst), "v"(ov) : "memory");
          }
        }
      }
      qp_base = qb.base; qp_base_valid = qb.rows_valid;
      // ---- the update of those blocks, with the rows of position i + RQ + 2 (the only loads that miss the L2) requested
      //      between its pieces
      {
        float t[3][4];
        unsigned hs[3], outw[3], knew[6];
        const RKahanBlock nok = {};
        const unsigned hash_tile = qb.label0 * (unsigned)(D / 4) * 0x9E3779B1u + qb.seed;
        const int rslot = sa == 0 ? RR_RING - 1 : sa - 1;   // (i + RQ + RR_RING - 1) % RR_RING
#pragma unroll
        for (int nb = NBB; nb < 4; nb++)
#pragma unroll
          for (int c = 0; c < 8; c++) {
            constexpr int every = 2 * NBA;
            const int pc = (nb - NBB) * 8 + c;
            if (pc % every == 0) rows_piece(rslot, qr, pc / every);
            r_update_piece<MODE, WD, 0>(c, nb, aa[nb - NBB], wq[nb - NBB], t, hs, outw, knew, bl, qb, hash_tile, p.lr_eff, p.wd_eff, l16, lds, oimg, nok, nullptr, 0);
          }
        if (NBB == 4) rows_pieces(rslot, qr);
      }
      // Loads and stores complete in order.  Waiting for all but the stores of G and the rows covers the gather, the
      // columns and the snapshot, all issued long before, and everything of the iteration before, whose stores of G can
      // now be published.
      {
        const int cnt = (do_a ? 2 : 0) + (i > 0 ? 3 : 0) + (ra == 0 ? 4 : 3);
        switch (cnt) {
          case 3: asm volatile("s_waitcnt vmcnt(3)" ::: "memory"); break;
          case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
          case 5: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
          case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
          case 7: asm volatile("s_waitcnt vmcnt(7)" ::: "memory"); break;
          case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
          default: asm volatile("s_waitcnt vmcnt(9)" ::: "memory"); break;
        }
      }
      if (lane == 0) __hip_atomic_store(myflag, min(i + RQ, n_it), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      sa = sa == RR_RING - 1 ? 0 : sa + 1;
      w0 = w0 == RC_RING - 1 ? 0 : w0 + 1;
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");   // the last loads still target LDS
    __syncthreads();   // the last tile's updated weights are in LDS: the B wavefronts store them
    return;
  }

  // ============================================================================================= B wavefronts
  const int s = f;       // features 192m + 48s .. +47
  floatx4 acc2[8][3];    // grad_X[128 batch rows x 48 features]
  {
    // a second launch of a step continues the sums of the first
    const floatx4* prev = p.partial + (size_t)g * 24 * 256;
#pragma unroll
    for (int mb = 0; mb < 8; mb++)
#pragma unroll
      for (int nn = 0; nn < 3; nn++)
        acc2[mb][nn] = p.acc_init ? prev[(mb * 3 + nn) * 256 + s * 64 + lane] : floatx4{0.f, 0.f, 0.f, 0.f};
  }

  // per-lane parts of the LDS addresses
  const unsigned ga_lane = (unsigned)((kg >> 1) * 4096 + g_row16(l16) * 32 + ((kg & 1) ^ (l16 >> 3)) * 16);           // grad_X operand
  const unsigned wtr_lane = (unsigned)((8 * kg + (l16 >> 1)) * QWS + 48 * s + (l16 & 1) * 8);                        // W columns, transposed read

  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();   // P1
#pragma unroll
  for (int k = 0; k < RQ; k++) {
    __syncthreads();   // P2.k
    if (k + 1 < RQ && k + 1 >= RR_RING) __syncthreads();
  }

  QTile q_n = q_desc_full(cdesc, tile_at(0)), q_p = q_n;
  int w0 = 0;   // i % RC_RING
  int n_done = 0;
  for (int i = 0; i < n_it; i++) {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __syncthreads();
    const QTile q = q_n;
    const unsigned oimg = (unsigned)(RLDS_O + (i & 1) * RO_BYTES);
    const unsigned wc = (unsigned)(RLDS_C + w0 * QWC_BYTES);
    const unsigned gb = (unsigned)(RLDS_G + (i & 1) * RG_BYTES);
    const unsigned gxa = gb + ga_lane, gwl = gb + bl.bg_lane, gwh = gb + (bl.bg_lane ^ 128u);
    const unsigned wtr = wc + wtr_lane, wrow = wc + bl.wrow_lane;
    const unsigned hash_tile = q.label0 * (unsigned)(D / 4) * 0x9E3779B1u + q.seed;

    // The tile is a sequence of 16 + 4 NBB steps of one LDS operand and three matrix instructions each.  The first
    // 8 NBB alternate:
    //   even step 8o + 2ks:      A^T block o (label rows 16o..), K step ks:  aa[cg] += X^T[cg][ks] * G^T   (operand: two transposing reads)
    //   odd  step 8o + 2j + 1:   grad_X step 4o + j
    // and the rest are the remaining grad_X steps; grad_X step x = K step x/8 (32 labels), batch block x%8:
    //   acc2[mb][nn] += G^T * W[nn]  (operand: one 16-byte read).
    // The operand of step k + 3 is requested in step k.  The vector work of the update of block o (12 weights per lane,
    // eight pieces) is spread over the steps behind the block's last, so that it issues between the matrix instructions.
    constexpr int NS = 16 + 4 * NBB, NALT = 8 * NBB;
    constexpr int PD = KT != 0 ? 2 : XMC_PD;   // operands are requested this many steps ahead (the head-Kahan variants
                                               // have no registers for a third operand in flight)
    bf16x8 op[NS + PD];
    auto request = [&](int k) {
      if (k >= NS) return;
      if (k < NALT && (k & 1) == 0) {
        op[k] = read_bg(gwl, gwh, k >> 3, (k & 7) >> 1);
      } else {
        const int x = k < NALT ? 4 * (k >> 3) + ((k & 7) >> 1) : NALT / 2 + (k - NALT);
        op[k] = *(const bf16x8*)(lds + gxa + (x >> 3) * 8192 + (x & 7) * 512);
      }
    };
    const int abort_word = *(const lds_int*)(lds + abort_base + ((i + 1) & 1) * 4);
#pragma unroll
    for (int k = 0; k < PD; k++) request(k);
    intx2 wraw[2][3];
#pragma unroll
    for (int ks2 = 0; ks2 < 2; ks2++)
#pragma unroll
      for (int nn = 0; nn < 3; nn++)
        wraw[ks2][nn] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) intx2*)(lds + wtr + ks2 * 32 * QWS + nn * 16));
    if (__builtin_amdgcn_readfirstlane(abort_word) != 0) break;
    n_done = i + 1;
    bf16x8 wb[2][3];

    floatx4 aa[2][3];       // A^T of the block in progress and of the one being rounded
    unsigned wq[2][3];      // their old weights
    float t[3][4];
    unsigned hs[3], outw[3], knew[6];
    RKahanBlock kb[2] = {};   // compensation terms of the block in progress and of the one being rounded
    // (this loop must be unrolled completely: its register arrays are indexed by k.  The variants with the Philox
    // recipe or a compensated head exceed the compiler's default size limit for "#pragma unroll" and are compiled in a
    // translation unit of their own, xmc_fp8_role_heavy.hip, with a higher limit.)
#pragma unroll
    for (int k = 0; k < NS; k++) {
      request(k + PD);
      // vector pieces of this step
      if (k == 0) {
#pragma unroll
        for (int nn = 0; nn < 3; nn++) wb[0][nn] = q_fp8x8_to_bf16x8(wraw[0][nn]);
      }
      if (k == 2) {
#pragma unroll
        for (int nn = 0; nn < 3; nn++) wb[1][nn] = q_fp8x8_to_bf16x8(wraw[1][nn]);
      }
      if (k < NALT && (k & 7) == 4) {   // old weights of the block in progress, read before its update starts
        const int o = k >> 3;
#pragma unroll
        for (int cg = 0; cg < 3; cg++) wq[o & 1][cg] = *(const unsigned*)(lds + wrow + 16 * o * QWS + 4 * cg);
      }
      if (KT != 0 && k < NALT && (k & 7) == 0) {
        const int o = k >> 3;
        {
          // the block's compensation terms: 24 (bf16) or 12 (e5m2) bytes per lane, from memory to registers; rows
          // behind the head's end (or the chunk's) read row 0 and count as zero
          RKahanBlock& kk = kb[o & 1];
          kk.row = q.row0 + 16 * o + l16;
          kk.head = kk.row < p.num_head;
          const unsigned char* src = p.kahan + ((size_t)(kk.head ? kk.row : 0) * D + bl.gcol) * (KT == 1 ? 2 : 1);
          if (KT == 1) {
#pragma unroll
            for (int cg = 0; cg < 3; cg++) {
              const uint2 kv = *(const uint2*)(src + 8 * cg);
              kk.raw[2 * cg] = kk.head ? kv.x : 0u; kk.raw[2 * cg + 1] = kk.head ? kv.y : 0u;
            }
          } else {
#pragma unroll
            for (int cg = 0; cg < 3; cg++) { const unsigned kv = *(const unsigned*)(src + 4 * cg); kk.raw[cg] = kk.head ? kv : 0u; }
          }
        }
      }
      if (k >= 8 && k < NALT) {
        const int o = (k >> 3) - 1;
        r_update_piece<MODE, WD, KT>(k & 7, o, aa[o & 1], wq[o & 1], t, hs, outw, knew, bl, q, hash_tile, p.lr_eff, p.wd_eff, l16, lds, oimg, kb[o & 1], p.kahan, p.num_head);
      } else if (k >= NALT && NBB > 0) {
        constexpr int per = NBB == 4 ? 8 : 8 / (16 - 4 * NBB);   // pieces per trailing step
        const int o = NBB - 1;
#pragma unroll
        for (int c = (k - NALT) * per; c < (k - NALT + 1) * per && c < 8; c++)
          r_update_piece<MODE, WD, KT>(c, o, aa[o & 1], wq[o & 1], t, hs, outw, knew, bl, q, hash_tile, p.lr_eff, p.wd_eff, l16, lds, oimg, kb[o & 1], p.kahan, p.num_head);
      }
      if (k < NALT && (k & 1) == 0) {
        const int o = k >> 3, ks = (k & 7) >> 1;
#pragma unroll
        for (int cg = 0; cg < 3; cg++)
          aa[o & 1][cg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xt[cg][ks], op[k], ks == 0 ? floatx4{0.f, 0.f, 0.f, 0.f} : aa[o & 1][cg], 0, 0, 0);
      } else {
        const int x = k < NALT ? 4 * (k >> 3) + ((k & 7) >> 1) : NALT / 2 + (k - NALT);
        const int ks2 = x >> 3, mb = x & 7;
#pragma unroll
        for (int nn = 0; nn < 3; nn++) acc2[mb][nn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(op[k], wb[ks2][nn], acc2[mb][nn], 0, 0, 0);
      }
      QFENCE();
    }
    if (NBB == 4) {
#pragma unroll
      for (int c = 0; c < 8; c++) r_update_piece<MODE, WD, KT>(c, 3, aa[1], wq[1], t, hs, outw, knew, bl, q, hash_tile, p.lr_eff, p.wd_eff, l16, lds, oimg, kb[1], p.kahan, p.num_head);
    }
    q_p = q;
    q_n = q_desc_full(cdesc, tile_at(i + 1));
    w0 = w0 == RC_RING - 1 ? 0 : w0 + 1;
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __syncthreads();   // every wavefront has written its part of the last tile's image
  // The image of the last tile's updated weights (64 rows x 192 bytes) goes to memory as 12 wave-wide stores of 16 bytes
  // per lane, three per B wavefront (the A wavefronts, which store the other tiles' images one iteration later, have
  // left): chunk ch = (3s + jj) * 64 + lane is bytes 16 (ch % 12).. of row ch / 12.
  if (n_done > 0) {
#pragma unroll
    for (int jj = 0; jj < 3; jj++) {
      const int ch = (3 * s + jj) * 64 + lane, row = ch / 12;
      const intx4 ov = *(const __attribute__((address_space(3))) intx4*)(lds + RLDS_O + ((n_done + 1) & 1) * RO_BYTES + ch * 16);
      if (row < q_p.rows_valid) *(intx4*)(q_p.base + (size_t)(row * D + QCOLS * m + (ch - row * 12) * 16)) = ov;
    }
  }

  // ---- per-workgroup grad_X partial, summed in a fixed order by reduce_gx_role_kernel: [24 blocks][4 B wavefronts][64 lanes]
  floatx4* dst = p.partial + (size_t)g * 24 * 256;
#pragma unroll
  for (int mb = 0; mb < 8; mb++)
#pragma unroll
    for (int nn = 0; nn < 3; nn++) dst[(mb * 3 + nn) * 256 + s * 64 + lane] = acc2[mb][nn];
}

#ifndef XMC_HEAVY_TU   // compiled once, in the library's main translation unit
// grad_X = scale * sum over quads of the member partials; writes fp32 and bf16 [batch, 768].  192 workgroups of 128
// threads: workgroup (block, m, part) covers lanes 128 part.. of the 256 B-wavefront lanes of a step workgroup.
__global__ __launch_bounds__(128) void reduce_gx_role_kernel(const floatx4* partial, int nwg, float scale, float* gx_f32,
                                                             unsigned short* gx_bf16, int batch, int* flags, const DropoutParams dp) {
  // placement check: the members of a quad exchanged G through the L2 of one XCD, which holds only if all four ran there
  if (blockIdx.x == 0) {
    if ((int)threadIdx.x < (nwg >> 2) && quad_xcc_mismatch(flags + QF_XCC, (int)threadIdx.x))
      __hip_atomic_fetch_or(flags + QF_ERR, 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    // the error word of this step joins the sticky word, which no kernel clears: a caller that looks at it only now and
    // then still learns of every failed step
    if (threadIdx.x == 0) {
      const int e = __hip_atomic_load(flags + QF_ERR, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (e != 0) __hip_atomic_fetch_or(flags + QF_STICKY, e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  const int blk = blockIdx.x >> 3, m = (blockIdx.x >> 1) & 3;   // blk = mb*3+nn
  const int t = (blockIdx.x & 1) * 128 + threadIdx.x, s = t >> 6, lane = t & 63, l16 = lane & 15, kg = lane >> 4;
  // the workgroups of member m, in a fixed order; eight loads in flight at a time
  floatx4 sum = {0.f, 0.f, 0.f, 0.f};
  const int nq = nwg >> 5;   // quads per XCD
  for (int jq = 0; jq < nq; jq++) {
    floatx4 pv[8];
#pragma unroll
    for (int x = 0; x < 8; x++) pv[x] = partial[((size_t)(((jq * 4 + m) << 3) + x) * 24 + blk) * 256 + t];
#pragma unroll
    for (int x = 0; x < 8; x++) sum += pv[x];
  }
  const int mb = blk / 3, nn = blk - mb * 3;
  const int col = QCOLS * m + 48 * s + 16 * nn + l16;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int b = 16 * mb + 4 * kg + i;
    if (b < batch) {
      const float val = dropout_backward(sum[i] * scale, (unsigned)(b * D + col), dp);
      if (gx_f32) gx_f32[(size_t)b * D + col] = val;
      if (gx_bf16) gx_bf16[(size_t)b * D + col] = bf16_bits(val);
    }
  }
}

#endif  // XMC_HEAVY_TU

// The variants of fp8_step_role_kernel with the reference's Philox recipe (XMC_ROUND_SR_PHILOX) or a compensated head
// (kahan_type 1, 2), defined in xmc_fp8_role_heavy.hip: opt in to the LDS size (once per device); launch.
void role_heavy_set_lds();
void role_heavy_launch(int round_mode, bool weight_decay, int kahan_type, int grid, hipStream_t stream, const QuadParams& p);
// The other variants (round to nearest, fast stochastic rounding), defined in xmc_fp8_role_plain.hip.
void role_plain_set_lds();
void role_plain_launch(int round_mode, bool weight_decay, int grid, hipStream_t stream, const QuadParams& p);

}  // namespace xmc
