// Running top-k over the label chunks of the inference logits (evaluate.py:158-159,235-236 take topk(100) / topk(5) of
// the dense [B, L] logits that xfc_forward returns, chunked_fp8xmc_clf.py:45-60).  The logits of one chunk at a time are
// written to a chunk-sized buffer and reduced to the k best per batch row, so the [B, L] matrix (172 MB at B = 128,
// L = 670 K) is never allocated.
//
// One workgroup per batch row and list (a row has two lists: a large group of chunks is split between two workgroups,
// and topk_finish_kernel merges the lists at the end).  Candidates = the k entries kept so far (from the chunks before, hence smaller label
// ids) followed by the chunk's logits in label order.  Radix select on a 16-bit key that orders bf16 values (two passes
// of 256 bins find the key T of the k-th largest), then everything above T is taken, entries equal to T are taken in
// candidate order until k are full (ties go to the smaller label id: a second radix select, on the label, among the
// chunk's entries equal to T), and the k entries are sorted by (value descending, label ascending).  NaN orders above every number, as in torch.topk.
// Once k entries are kept, their smallest value is a lower bound of the final k-th value: one pass over the chunk
// keeps only the logits at or above it, in LDS, and the selection passes run over that short list (the chunk is read
// again by every pass only when more than TOPK_CAP logits reach the bound).  The first chunk is therefore fed in two
// parts, a short prefix that fits the list and produces a bound, and the rest.
#include "xmc_common.h"

namespace xmc {

constexpr int TOPK_MAX = 128;   // largest k
constexpr int TOPK_NT = 1024;  // sixteen wavefronts keep enough loads in flight on the workgroup's compute unit
template <int N> struct TopkBins { static constexpr int value = N; };
typedef TopkBins<256> B256;
typedef TopkBins<1024> B1024;
constexpr int TOPK_CAP = 6144;  // chunk logits at or above the bound that one workgroup keeps in LDS
constexpr int TOPK_SMALL = 512; // candidates (kept entries included) that are ranked directly

// z: a row's logits of the chunk at z + row*stride, n_all of them valid (n_all <= 2^17; stride % 4 == 0; z 8-byte aligned)
// run_val/run_idx: [batch][2][TOPK_MAX] entries kept so far: every batch row has two lists, which topk_finish_kernel
// merges.  parts = 1: one workgroup per row adds all n_all logits to list 0 (have0 entries valid).  parts = 2: two
// workgroups per row, so that 128 rows fill 256 compute units; workgroup 2 row + p takes the first topk_split(n_all)
// logits (p = 0) or the rest (p = 1) and updates list p (have0 / have1 entries valid).  Lists are updated in place and
// stay sorted; within a list the entries kept from earlier launches have the smaller label ids.
__host__ __device__ __forceinline__ int topk_split(int n_all) { return ((n_all >> 1) + 3) & ~3; }
__global__ __launch_bounds__(TOPK_NT) void topk_chunk_kernel(const unsigned short* z, long long stride, int n_all, int label_base0, int k,
                                                             int parts, int have0, int have1, unsigned short* run_val, int* run_idx) {
  __shared__ unsigned hist[1024];
  __shared__ __attribute__((aligned(16))) unsigned sel_key[TOPK_MAX];
  __shared__ __attribute__((aligned(16))) int sel_idx[TOPK_MAX];
  __shared__ __attribute__((aligned(16))) unsigned cand_key[TOPK_CAP];
  __shared__ __attribute__((aligned(16))) int cand_idx[TOPK_CAP];   // index in the chunk (negative: an entry kept from earlier chunks)
  __shared__ unsigned s_bin, s_above, s_count, s_ncand, wtot[TOPK_NT / 64];
  const int tid = threadIdx.x;
  const int brow = parts == 2 ? (int)(blockIdx.x >> 1) : (int)blockIdx.x, part = parts == 2 ? (int)(blockIdx.x & 1) : 0;
  const int first = part == 0 ? 0 : topk_split(n_all);                      // this workgroup's range of the chunk
  const int n = parts == 2 ? (part == 0 ? topk_split(n_all) : n_all - first) : n_all;
  const int label_base = label_base0 + first;
  const int have = part == 0 ? have0 : have1;
  const unsigned short* row = z + (size_t)brow * stride + first;
  unsigned short* rv = run_val + ((size_t)brow * 2 + part) * TOPK_MAX;
  int* ri = run_idx + ((size_t)brow * 2 + part) * TOPK_MAX;
  const int total = n + have;
  const int kk = k < total ? k : total;
  const unsigned mykey = tid < have ? topk_key(rv[tid]) : 0u;   // this thread's entry of the running list
  const int myidx = tid < have ? ri[tid] : -1;
  const unsigned floor_key = have >= k ? topk_key(rv[k - 1]) : 0u;   // the list is sorted: entry k-1 is its smallest

  // visits every chunk element once, the workgroup reading 8 KiB of consecutive logits at a time, sixteen such loads in
  // flight (a compute unit runs one workgroup: nothing else hides the latency): f(key, index in chunk)
  auto for_each_global = [&](auto f) {
    constexpr int U = 16;
    for (int base = 0; base < n; base += U * 4 * TOPK_NT) {
      uint2 v[U];
#pragma unroll
      for (int u = 0; u < U; u++) {
        const int i = base + u * 4 * TOPK_NT + 4 * tid;
        v[u] = i + 4 <= n ? *(const uint2*)(row + i) : uint2{0u, 0u};
      }
#pragma unroll
      for (int u = 0; u < U; u++) {
        const int i = base + u * 4 * TOPK_NT + 4 * tid;
        if (i + 4 <= n) {
          f(topk_key((unsigned short)(v[u].x & 0xFFFFu)), i);
          f(topk_key((unsigned short)(v[u].x >> 16)), i + 1);
          f(topk_key((unsigned short)(v[u].y & 0xFFFFu)), i + 2);
          f(topk_key((unsigned short)(v[u].y >> 16)), i + 3);
        } else {
          for (int j = i; j < n; j++) f(topk_key(row[j]), j);
        }
      }
    }
  };
  // one pass over the chunk keeps the logits at or above the bound (key, index) in LDS; the selection then runs over
  // that list.  More than TOPK_CAP of them: every later pass reads the chunk again.
  if (tid == 0) s_ncand = 0;
  __syncthreads();
  for_each_global([&](unsigned key, int i) {
    const bool take = key >= floor_key;
    const unsigned long long m = __ballot(take);   // lanes of this wavefront that are here and take
    if (m != 0) {
      const int lane = tid & 63, leader = __ffsll((long long)m) - 1;
      unsigned base = 0;
      if (lane == leader) base = atomicAdd(&s_ncand, (unsigned)__popcll(m));
      base = __shfl(base, leader, 64);
      const unsigned slot = base + (unsigned)__popcll(m & ((1ull << lane) - 1ull));
      if (take && slot < (unsigned)TOPK_CAP) {
        cand_key[slot] = key;
        cand_idx[slot] = i;
      }
    }
  });
  __syncthreads();
  const bool listed = s_ncand <= (unsigned)TOPK_CAP;
  const int ncand = listed ? (int)s_ncand : 0;
  // rank of (key, idx) among m entries of (keys, idxs) in the order value descending, index ascending; m % 4 == 0
  auto rank_among = [&](const unsigned* keys, const int* idxs, int m, unsigned key, int idx) {
    int rank = 0;
    for (int j = 0; j < m; j += 4) {
      const uint4 kj = *(const uint4*)(keys + j);
      const int4 ij = *(const int4*)(idxs + j);
      rank += (kj.x > key || (kj.x == key && ij.x < idx)) ? 1 : 0;
      rank += (kj.y > key || (kj.y == key && ij.y < idx)) ? 1 : 0;
      rank += (kj.z > key || (kj.z == key && ij.z < idx)) ? 1 : 0;
      rank += (kj.w > key || (kj.w == key && ij.w < idx)) ? 1 : 0;
    }
    return rank;
  };
  if (listed && ncand + have <= TOPK_SMALL) {
    // few candidates (the usual case once a bound exists): the kept entries join the list, every entry finds its rank
    // among all of them and the first kk are written in place.  Kept entries have the smaller label ids.
    const int m = ncand + have, m4 = (m + 3) & ~3;
    if (tid < have) {
      cand_key[ncand + tid] = mykey;
      cand_idx[ncand + tid] = myidx - label_base;
    }
    if (tid < m4 - m) {   // padding that ranks after everything
      cand_key[m + tid] = 0u;
      cand_idx[m + tid] = 0x7FFFFFFF;
    }
    __syncthreads();
    for (int c = tid; c < m; c += TOPK_NT) {
      const unsigned key = cand_key[c];
      const int idx = cand_idx[c];
      const int rank = rank_among(cand_key, cand_idx, m4, key, idx);
      if (rank < kk) {
        rv[rank] = topk_bits(key);
        ri[rank] = label_base + idx;
      }
    }
    if (tid >= kk && tid < TOPK_MAX) {
      rv[tid] = 0xFF80;   // -inf
      ri[tid] = -1;
    }
    return;
  }
  auto for_each = [&](auto f) {
    if (listed) {
      for (int j = tid; j < ncand; j += TOPK_NT) f(cand_key[j], cand_idx[j]);
    } else {
      for_each_global([&](unsigned key, int i) { if (key >= floor_key) f(key, i); });
    }
  };
  auto clear_hist = [&]() {
    __syncthreads();
    for (int q = tid; q < 1024; q += TOPK_NT) hist[q] = 0;
    __syncthreads();
  };
  // exclusive prefix sum of one value per thread over the workgroup (thread order), and the total
  auto block_scan = [&](unsigned val, unsigned& total) {
    const int lane = tid & 63, wave = tid >> 6;
    unsigned x = val;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const unsigned y = __shfl_up(x, off, 64);
      if (lane >= off) x += y;
    }
    __syncthreads();
    if (lane == 63) wtot[wave] = x;
    __syncthreads();
    unsigned before = 0;
    total = 0;
#pragma unroll
    for (int q = 0; q < TOPK_NT / 64; q++) {
      if (q < wave) before += wtot[q];
      total += wtot[q];
    }
    return before + x - val;
  };
  // the bin in which the `want`-th candidate lies, counting from the top (down) or from the bottom: s_bin; s_above =
  // candidates in the bins before it.  Thread t looks at one bin (or bins / threads consecutive bins) in counting order.
  auto pick_bin = [&](unsigned want, auto bins_c, bool from_top) {
    __syncthreads();
    constexpr int bins = decltype(bins_c)::value;
    constexpr int per = bins > TOPK_NT ? bins / TOPK_NT : 1;
    unsigned local[per], sum = 0;
#pragma unroll
    for (int q = 0; q < per; q++) {
      const int pos = tid * per + q;
      local[q] = pos < bins ? hist[from_top ? bins - 1 - pos : pos] : 0u;
      sum += local[q];
    }
    unsigned total;
    unsigned before = block_scan(sum, total);
    if (tid == 0 && (want == 0 || total < want)) {   // nothing asked for, or fewer candidates than asked: the last bin in order
      s_bin = (unsigned)(want == 0 ? (from_top ? bins - 1 : 0) : (from_top ? 0 : bins - 1));
      s_above = want == 0 ? 0u : total - hist[from_top ? 0 : bins - 1];
    }
    if (want > 0 && total >= want) {
#pragma unroll
      for (int q = 0; q < per; q++) {
        if (before < want && want <= before + local[q]) {
          const int pos = tid * per + q;
          s_bin = (unsigned)(from_top ? bins - 1 - pos : pos);
          s_above = before;
        }
        before += local[q];
      }
    }
    __syncthreads();
  };

  clear_hist();
  for_each([&](unsigned key, int) { atomicAdd(&hist[key >> 8], 1u); });
  if (tid < have) atomicAdd(&hist[mykey >> 8], 1u);
  pick_bin((unsigned)kk, B256{}, true);
  const unsigned hi_bin = s_bin, above_hi = s_above;
  clear_hist();
  for_each([&](unsigned key, int) { if ((key >> 8) == hi_bin) atomicAdd(&hist[key & 255u], 1u); });
  if (tid < have && (mykey >> 8) == hi_bin) atomicAdd(&hist[mykey & 255u], 1u);
  pick_bin((unsigned)kk - above_hi, B256{}, true);
  const unsigned T = (hi_bin << 8) | s_bin;
  const unsigned n_gt = above_hi + s_above;          // candidates above T: all taken
  const unsigned need_eq = (unsigned)kk - n_gt;      // candidates equal to T still to take, in candidate order

  // equal candidates of the running list come first
  __syncthreads();
  if (tid == 0) s_count = 0;
  unsigned eq_run;
  const unsigned my_eq_rank = block_scan((tid < have && mykey == T) ? 1u : 0u, eq_run);   // the list is in candidate order
  const unsigned eq_from_run = eq_run < need_eq ? eq_run : need_eq;
  if (tid < have) {
    if (mykey > T || (mykey == T && my_eq_rank < need_eq)) {
      const unsigned slot = atomicAdd(&s_count, 1u);
      sel_key[slot] = mykey;
      sel_idx[slot] = myidx;
    }
  }
  // the chunk's candidates equal to T are taken up to the index limit that admits eq_chunk of them: a second radix
  // select, on the index (high bits i >> 10, then the low 10 bits), over those candidates only
  const unsigned eq_chunk = need_eq - eq_from_run;
  int idx_limit = -1;   // equal candidates with index <= idx_limit are taken
  if (eq_chunk > 0) {
    clear_hist();
    for_each([&](unsigned key, int i) { if (key == T) atomicAdd(&hist[i >> 10], 1u); });
    pick_bin(eq_chunk, B256{}, false);
    const unsigned hi_idx = s_bin, below_hi = s_above;
    clear_hist();
    for_each([&](unsigned key, int i) { if (key == T && (unsigned)(i >> 10) == hi_idx) atomicAdd(&hist[i & 1023], 1u); });
    pick_bin(eq_chunk - below_hi, B1024{}, false);
    idx_limit = (int)((hi_idx << 10) | s_bin);
  }
  __syncthreads();
  for_each([&](unsigned key, int i) {
    if (key > T || (key == T && i <= idx_limit)) {
      const unsigned slot = atomicAdd(&s_count, 1u);
      if (slot < (unsigned)TOPK_MAX) {
        sel_key[slot] = key;
        sel_idx[slot] = label_base + i;
      }
    }
  });
  __syncthreads();
  if (tid >= kk && tid < TOPK_MAX) {   // padding that ranks after everything
    sel_key[tid] = 0u;
    sel_idx[tid] = 0x7FFFFFFF;
  }
  __syncthreads();
  // exactly kk entries: sort by (value descending, label ascending) through ranks
  if (tid < kk) {
    const unsigned key = sel_key[tid];
    const int idx = sel_idx[tid];
    const int rank = rank_among(sel_key, sel_idx, (kk + 3) & ~3, key, idx);
    rv[rank] = topk_bits(key);
    ri[rank] = idx;
  }
  if (tid >= kk && tid < TOPK_MAX) {
    rv[tid] = 0xFF80;   // -inf
    ri[tid] = -1;
  }
}

// merges the two sorted lists of every batch row (have0 and have1 entries valid, have0 + have1 >= k, all label ids
// distinct) and writes the first k entries to the outputs [batch][k]: an entry's position is its index in its own list
// plus the number of entries of the other list that come before it (value descending, label ascending).
// One workgroup of 2 * TOPK_MAX threads per row.
__global__ __launch_bounds__(2 * TOPK_MAX) void topk_finish_kernel(const unsigned short* run_val, const int* run_idx, int k, int have0,
                                                                  int have1, unsigned short* out_val, int* out_idx) {
  __shared__ __attribute__((aligned(16))) unsigned fkey[2][TOPK_MAX];
  __shared__ __attribute__((aligned(16))) int fidx[2][TOPK_MAX];
  const int b = blockIdx.x, list = threadIdx.x / TOPK_MAX, j = threadIdx.x - list * TOPK_MAX;
  const int mine = list == 0 ? have0 : have1;
  const bool valid = j < mine;
  const unsigned short bits = valid ? run_val[((size_t)b * 2 + list) * TOPK_MAX + j] : (unsigned short)0;
  const int idx = valid ? run_idx[((size_t)b * 2 + list) * TOPK_MAX + j] : 0x7FFFFFFF;
  const unsigned key = valid ? topk_key(bits) : 0u;   // an entry that is not there comes before nothing
  fkey[list][j] = key;
  fidx[list][j] = idx;
  __syncthreads();
  if (!valid) return;
  int pos = j;
#pragma unroll 8
  for (int o = 0; o < TOPK_MAX; o += 4) {
    const uint4 ko = *(const uint4*)&fkey[list ^ 1][o];
    const int4 io = *(const int4*)&fidx[list ^ 1][o];
    pos += (ko.x > key || (ko.x == key && io.x < idx)) ? 1 : 0;
    pos += (ko.y > key || (ko.y == key && io.y < idx)) ? 1 : 0;
    pos += (ko.z > key || (ko.z == key && io.z < idx)) ? 1 : 0;
    pos += (ko.w > key || (ko.w == key && io.w < idx)) ? 1 : 0;
  }
  if (pos < k) {
    out_val[(size_t)b * k + pos] = bits;
    out_idx[(size_t)b * k + pos] = idx;
  }
}


// ---- the two small kernels of the two-pass top-k (fp8_forward_select_kernel produces gmax and the candidate lists)

// The k-th largest of the 16-bit keys that the threads of a workgroup hold (one per thread; `valid` false = no key), or
// 0 if fewer than k are valid: the largest T with at least k keys >= T, found bit by bit from the top.  Every thread of
// the workgroup calls this; wcnt = 2 x WAVES words of LDS.
template <int WAVES>
__device__ __forceinline__ unsigned block_kth_key(unsigned key, bool valid, int k, unsigned* wcnt) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  unsigned T = 0u;
#pragma unroll 1
  for (int bit = 15; bit >= 0; bit--) {
    const unsigned c = T | (1u << bit);
    const unsigned long long m = __ballot(valid && key >= c);
    unsigned* mine = wcnt + ((bit & 1) ? WAVES : 0);   // alternating halves: a slow reader is never overtaken by a writer
    if (lane == 0) mine[wave] = (unsigned)__popcll(m);
    __syncthreads();
    unsigned total = 0;
#pragma unroll
    for (int q = 0; q < WAVES; q++) total += mine[q];
    if (total >= (unsigned)k) T = c;
  }
  return T;
}

// bound[b] = k-th largest of the `groups` maxima gmax[g][b] of batch row b (groups >= k); rows at or past `batch` get
// a bound nothing reaches.  Also clears the candidate counts and the status word.  One workgroup of TOPK_GROUPS threads
// per row of the padded batch.
constexpr int TOPK_GROUPS = 512;
__global__ __launch_bounds__(TOPK_GROUPS) void topk_bound_kernel(const unsigned short* gmax, int groups, int k, int batch,
                                                                 unsigned short* bound, unsigned* count, int* status) {
  __shared__ unsigned wcnt[2 * (TOPK_GROUPS / 64)];
  const int b = blockIdx.x, g = threadIdx.x;
  if (g == 0) {
    count[b] = 0u;
    if (b == 0) *status = 0;
    if (b >= batch) bound[b] = 0xFFFFu;
  }
  if (b >= batch) return;
  const unsigned key = g < groups ? (unsigned)gmax[(size_t)g * BP + b] : 0u;
  const unsigned T = block_kth_key<TOPK_GROUPS / 64>(key, g < groups, k, wcnt);
  if (g == 0) bound[b] = (unsigned short)T;
}

// Picks the k best of the candidate list of batch row b (label and key per entry, all labels different) and writes
// them to the outputs [batch][k]: value descending, label ascending among equal values; labels as int32 or, with
// idx64, as int64.  The k-th largest key T is found first; the entries at or above it (k plus the ties at T) are then
// ranked against each other, several threads sharing the comparisons of one entry.  status |= 1 if a row collected
// more candidates than its list holds (the outputs of that call are then not to be used), |= 2 if a row has fewer than k.
constexpr int TOPK_LIST = 1024;   // == SEL_CAP of the producing kernel
__global__ __launch_bounds__(TOPK_LIST) void topk_pick_kernel(const unsigned* cand_label, const unsigned short* cand_key,
                                                              const unsigned* count, int k, unsigned short* out_val, void* out_idx,
                                                              int idx64, int* status) {
  __shared__ __attribute__((aligned(16))) unsigned long long ent[TOPK_LIST];
  __shared__ unsigned rank[TOPK_LIST];
  __shared__ unsigned wcnt[2 * (TOPK_LIST / 64)];
  __shared__ unsigned s_m;
  const int b = blockIdx.x, tid = threadIdx.x;
  const unsigned have = count[b];
  const int n = have < (unsigned)TOPK_LIST ? (int)have : TOPK_LIST;
  if (tid == 0) {
    if (have > (unsigned)TOPK_LIST || n < k) atomicOr(status, have > (unsigned)TOPK_LIST ? 1 : 2);
    s_m = 0u;
  }
  rank[tid] = 0u;
  const unsigned key = tid < n ? (unsigned)cand_key[(size_t)b * TOPK_LIST + tid] : 0u;
  const unsigned label = tid < n ? cand_label[(size_t)b * TOPK_LIST + tid] : 0u;
  const unsigned T = block_kth_key<TOPK_LIST / 64>(key, tid < n, k, wcnt);   // its barriers also publish s_m and rank
  if (tid < n && key >= T) {
    // key << 32 | ~label: larger = better value, then smaller label
    ent[atomicAdd(&s_m, 1u)] = ((unsigned long long)key << 32) | (unsigned long long)(0xFFFFFFFFu - label);
  }
  __syncthreads();
  const int m = (int)s_m;                       // >= min(k, n) entries, all different
  int mp = 64;
  while (mp < m) mp <<= 1;                      // threads per slice; TOPK_LIST / mp slices share an entry's comparisons
  const int slices = TOPK_LIST / mp, i = tid & (mp - 1), sl = tid / mp;
  const int per = (m + slices - 1) / slices, j0 = sl * per, j1 = j0 + per < m ? j0 + per : m;
  if (i < m) {
    const unsigned long long mine = ent[i];
    unsigned r = 0;
    for (int j = j0; j < j1; j++) r += ent[j] > mine ? 1u : 0u;
    if (r != 0u) atomicAdd(&rank[i], r);
  }
  __syncthreads();
  if (tid < m) {
    const unsigned r = rank[tid];
    if (r < (unsigned)k) {
      const unsigned long long mine = ent[tid];
      const int lab = (int)(0xFFFFFFFFu - (unsigned)mine);
      out_val[(size_t)b * k + r] = topk_bits((unsigned)(mine >> 32));
      if (idx64) ((long long*)out_idx)[(size_t)b * k + r] = lab;
      else ((int*)out_idx)[(size_t)b * k + r] = lab;
    }
  }
  if (tid >= m && tid < k) {   // fewer than k candidates (reported above): -inf, label -1
    out_val[(size_t)b * k + tid] = 0xFF80;
    if (idx64) ((long long*)out_idx)[(size_t)b * k + tid] = -1;
    else ((int*)out_idx)[(size_t)b * k + tid] = -1;
  }
}

}  // namespace xmc
