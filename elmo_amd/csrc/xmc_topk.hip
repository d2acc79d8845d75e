// Running top-k over the label chunks of the inference logits (evaluate.py:158-159,235-236 take topk(100) / topk(5) of
// the dense [B, L] logits that xfc_forward returns, chunked_fp8xmc_clf.py:45-60).  The logits of one chunk at a time are
// written to a chunk-sized buffer and reduced to the k best per batch row, so the [B, L] matrix (172 MB at B = 128,
// L = 670 K) is never allocated.
//
// One workgroup per batch row.  Candidates = the k entries kept so far (from the chunks before, hence smaller label
// ids) followed by the chunk's logits in label order.  Radix select on a 16-bit key that orders bf16 values (two passes
// of 256 bins find the key T of the k-th largest), then everything above T is taken, entries equal to T are taken in
// candidate order until k are full (ties go to the smaller label id), and the k entries are sorted by (value
// descending, label ascending).  NaN orders above every number, as in torch.topk.
#include "xmc_common.h"

namespace xmc {

constexpr int TOPK_MAX = 128;   // largest k
constexpr int TOPK_NT = 256;

// ascending key order == ascending value order
__device__ __forceinline__ unsigned topk_key(unsigned short bits) {
  return (bits & 0x8000u) ? (unsigned)(~bits & 0xFFFFu) : (unsigned)(bits | 0x8000u);
}
__device__ __forceinline__ unsigned short topk_bits(unsigned key) {
  return (key & 0x8000u) ? (unsigned short)(key & 0x7FFFu) : (unsigned short)(~key & 0xFFFFu);
}

// z: this row's logits of the chunk at z + row*stride, n of them valid (n % 4 may be anything; stride % 4 == 0)
// run_key/run_idx: [batch][TOPK_MAX] entries kept so far, `have` of them valid; updated in place, sorted
__global__ __launch_bounds__(TOPK_NT) void topk_chunk_kernel(const unsigned short* z, long long stride, int n, int label_base, int k,
                                                             int have, unsigned short* run_val, int* run_idx) {
  __shared__ unsigned hist[256];
  __shared__ unsigned scan[TOPK_NT];
  __shared__ unsigned sel_key[TOPK_MAX];
  __shared__ int sel_idx[TOPK_MAX];
  __shared__ unsigned s_bin, s_above, s_count;
  const int tid = threadIdx.x;
  const unsigned short* row = z + (size_t)blockIdx.x * stride;
  unsigned short* rv = run_val + (size_t)blockIdx.x * TOPK_MAX;
  int* ri = run_idx + (size_t)blockIdx.x * TOPK_MAX;
  const int total = n + have;
  const int kk = k < total ? k : total;
  // thread t owns the chunk elements [lo, hi): contiguous, so that candidate order is label order
  const int per = ((n + TOPK_NT - 1) / TOPK_NT + 3) & ~3;
  const int lo = min(tid * per, n), hi = min(lo + per, n);
  const unsigned mykey = tid < have ? topk_key(rv[tid]) : 0u;   // this thread's entry of the running list
  const int myidx = tid < have ? ri[tid] : -1;

  // visits every chunk element of this thread: f(key, index in chunk)
  auto for_each = [&](auto f) {
    int i = lo;
    for (; i + 4 <= hi; i += 4) {
      const uint2 v = *(const uint2*)(row + i);
      f(topk_key((unsigned short)(v.x & 0xFFFFu)), i);
      f(topk_key((unsigned short)(v.x >> 16)), i + 1);
      f(topk_key((unsigned short)(v.y & 0xFFFFu)), i + 2);
      f(topk_key((unsigned short)(v.y >> 16)), i + 3);
    }
    for (; i < hi; i++) f(topk_key(row[i]), i);
  };
  // finds, from the top, the bin in which the `want`-th candidate lies: s_bin, and s_above = candidates in higher bins
  auto pick_bin = [&](unsigned want) {
    __syncthreads();
    if (tid == 0) {
      unsigned above = 0;
      int b = 255;
      for (; b > 0; b--) {
        if (above + hist[b] >= want) break;
        above += hist[b];
      }
      s_bin = (unsigned)b;
      s_above = above;
    }
    __syncthreads();
  };

  hist[tid] = 0;
  __syncthreads();
  for_each([&](unsigned key, int) { atomicAdd(&hist[key >> 8], 1u); });
  if (tid < have) atomicAdd(&hist[mykey >> 8], 1u);
  pick_bin((unsigned)kk);
  const unsigned hi_bin = s_bin, above_hi = s_above;
  __syncthreads();
  hist[tid] = 0;
  __syncthreads();
  for_each([&](unsigned key, int) { if ((key >> 8) == hi_bin) atomicAdd(&hist[key & 255u], 1u); });
  if (tid < have && (mykey >> 8) == hi_bin) atomicAdd(&hist[mykey & 255u], 1u);
  pick_bin((unsigned)kk - above_hi);
  const unsigned T = (hi_bin << 8) | s_bin;
  const unsigned n_gt = above_hi + s_above;          // candidates above T: all taken
  const unsigned need_eq = (unsigned)kk - n_gt;      // candidates equal to T still to take, in candidate order

  // equal candidates of the running list come first
  unsigned eq_run = 0;
  __syncthreads();
  if (tid == 0) s_count = 0;
  scan[tid] = (tid < have && mykey == T) ? 1u : 0u;
  __syncthreads();
  if (tid == 0) {
    unsigned c = 0;
    for (int i = 0; i < have; i++) { unsigned f = scan[i]; scan[i] = c; c += f; }
    s_above = c;   // reused: equal entries in the running list
  }
  __syncthreads();
  eq_run = s_above;
  const unsigned eq_from_run = eq_run < need_eq ? eq_run : need_eq;
  if (tid < have) {
    if (mykey > T || (mykey == T && scan[tid] < need_eq)) {
      const unsigned slot = atomicAdd(&s_count, 1u);
      sel_key[slot] = mykey;
      sel_idx[slot] = myidx;
    }
  }
  __syncthreads();
  // equal candidates of the chunk, in label order: exclusive scan of the per-thread counts
  unsigned my_eq = 0;
  for_each([&](unsigned key, int) { my_eq += key == T ? 1u : 0u; });
  scan[tid] = my_eq;
  __syncthreads();
  if (tid == 0) {
    unsigned c = 0;
    for (int i = 0; i < TOPK_NT; i++) { unsigned f = scan[i]; scan[i] = c; c += f; }
  }
  __syncthreads();
  unsigned eq_rank = scan[tid];
  const unsigned eq_chunk = need_eq - eq_from_run;
  for_each([&](unsigned key, int i) {
    bool take = key > T;
    if (key == T) { take = eq_rank < eq_chunk; eq_rank++; }
    if (take) {
      const unsigned slot = atomicAdd(&s_count, 1u);
      sel_key[slot] = key;
      sel_idx[slot] = label_base + i;
    }
  });
  __syncthreads();
  // exactly kk entries: sort by (value descending, label ascending) through ranks
  if (tid < kk) {
    const unsigned key = sel_key[tid];
    const int idx = sel_idx[tid];
    int rank = 0;
    for (int j = 0; j < kk; j++) {
      const unsigned kj = sel_key[j];
      rank += (kj > key || (kj == key && sel_idx[j] < idx)) ? 1 : 0;
    }
    rv[rank] = topk_bits(key);
    ri[rank] = idx;
  }
  if (tid >= kk && tid < TOPK_MAX) {
    rv[tid] = 0xFF80;   // -inf
    ri[tid] = -1;
  }
}

// copies the first k entries of the running lists to the outputs [batch][k]
__global__ void topk_finish_kernel(const unsigned short* run_val, const int* run_idx, int batch, int k, unsigned short* out_val, int* out_idx) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= batch * k) return;
  const int b = i / k, j = i - b * k;
  out_val[i] = run_val[(size_t)b * TOPK_MAX + j];
  out_idx[i] = run_idx[(size_t)b * TOPK_MAX + j];
}

}  // namespace xmc
