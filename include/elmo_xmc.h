/* C ABI of the MI355X (gfx950) extreme-classifier step library, libelmo_xmc.so.
 *
 * Every entry point takes raw device pointers, sizes and a HIP stream (passed as void*), enqueues its
 * kernels on that stream and returns immediately with a status code (0 = ok, negative = error, see
 * xmc_error_string).  Nothing here allocates or frees device memory, synchronises the device or copies
 * to the host: the caller owns every buffer, including the workspace.
 *
 * The entry points replace, for the FP8 layer of the reference
 *   src/xmc_classifiers/chunked_fp8xmc_clf.py:81-123   Fp8XMCBCEChunkedLayer.xfc_forward_backward
 *   src/xmc_classifiers/chunked_fp8xmc_clf.py:45-60    Fp8XMCBCEChunkedLayer.xfc_forward
 * and the kernels those call
 *   torch._scaled_mm (:101-102), sigmoid_/index_put (:107-108),
 *   src/triton_kernels/matmul_kernel.py:342-353 large_k_matmul,
 *   src/triton_kernels/fuse_kernel.py:116-131 matmul_update.
 */
#ifndef ELMO_XMC_H
#define ELMO_XMC_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  XMC_OK = 0,
  XMC_ERR_NULL = -1,        /* a required pointer is null */
  XMC_ERR_SHAPE = -2,       /* unsupported shape (features != 768 - tiled path: 768 or 1024 -, batch > 128 or not a multiple of 16, rows % 16 != 0, ...) */
  XMC_ERR_ALIGN = -3,       /* a device pointer is not 16-byte aligned */
  XMC_ERR_RANGE = -4,       /* too many chunks / positives / labels for this build */
  XMC_ERR_WORKSPACE = -5,   /* workspace smaller than xmc_workspace_bytes() */
  XMC_ERR_MODE = -6,        /* unknown rounding mode */
  XMC_ERR_LAUNCH = -7,      /* HIP reported a launch failure */
  XMC_ERR_DEVICE = -8       /* not a gfx950 device / too few compute units */
};

/* rounding of the updated weights (fuse_kernel.py:107-113 is XMC_ROUND_SR_PHILOX) */
enum {
  XMC_ROUND_RTN = 0,        /* round to nearest even, saturating at +-448 */
  XMC_ROUND_SR_PHILOX = 1,  /* the reference bit recipe: Philox-4x32-10 word per element, add 20 bits, mask, cast */
  XMC_ROUND_SR_FAST = 2     /* unbiased stochastic rounding on the e4m3 (or bf16) grid (hardware converter, counter hash) */
};

int xmc_version(void);
/* Build aid (no counterpart in the reference): digest of the sources this library was compiled from, as
 * elmo_amd/build.py computes it, or "unknown".  A test compares it with the sources in the tree. */
const char* xmc_source_hash(void);
const char* xmc_error_string(int status);

/* Bytes of workspace the step needs for `num_chunks` chunks of `rows_per_chunk` rows (features fixed at 768).
 * Returns 0 for an unsupported shape. */
size_t xmc_workspace_bytes(int num_chunks, int rows_per_chunk);

/* One training step over all chunks: logits, sigmoid minus sparse targets, grad_X, grad_W and the in-place
 * SGD update (chunked_fp8xmc_clf.py:91-123).
 *   chunk_ptrs      host array of num_chunks device pointers, each [rows_per_chunk, 768] e4m3fn, updated in place
 *   x_bf16          device [batch, 768] bf16 (not modified); batch % 16 == 0, batch <= 128
 *   labels_coo      device [nnz, 2] int32 (row-in-batch, label id in the padded label space), any order, duplicates allowed;
 *                   8-byte aligned (the pairs are read whole); entries outside the batch or the label space are ignored
 *   lr              learning rate (xmc_lr[0])
 *   seeds           host array of num_chunks seeds (one torch.randint(0, 1e6) per chunk in the reference, :113)
 *   round_mode      XMC_ROUND_*
 *   scale_w/scale_x per-tensor scales: weight = scale_w * code, Xq = e4m3(X / scale_x); the reference uses 1, 1
 *   grad_x_bf16     device [batch, 768] bf16 out (self.grad_input, :122)
 *   grad_x_f32      device [batch, 768] fp32 out, or null
 * Asynchronous on `stream`; allocates nothing and never synchronises.  The fused kernel is persistent: one workgroup
 * per compute unit, and the four workgroups that share a tile stream wait for one another through counters in the
 * workspace, so all of them must be running at the same time.  Give the step the whole device while it runs: a kernel
 * of another stream that keeps compute units occupied for more than about ten milliseconds makes the waiting
 * workgroups give up (every wait is bounded; nothing hangs).  A workgroup that gives up stops before its next tile, so
 * no weight is ever updated from missing data; the step is incomplete and the error word (xmc_step_error_word,
 * xmc_step_error_offset) is non-zero.  One step at a time per workspace.
 */
int xmc_fp8_step(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, const void* x_bf16, int batch,
                 int features, const int32_t* labels_coo, int nnz, float lr, const uint32_t* seeds, int round_mode,
                 float scale_w, float scale_x, void* grad_x_bf16, float* grad_x_f32, void* workspace,
                 size_t workspace_bytes, void* stream);

/* xmc_fp8_step with three more arguments (no counterpart in the reference's FP8 layer, whose kernels take neither):
 *   weight_decay  T = W - lr (A + weight_decay * W) in fp32 before the rounding: the decay the reference applies to fp32 /
 *                 fp16 weights (chunked.py:122-124) and accepts but ignores for low-precision ones
 *                 (stochastic_rounding_kernel.py:91-99).  0 = xmc_fp8_step.
 *   dropout_p, dropout_seed
 *                 dropout of the embedding inside the step (prototype in the reference: src/triton_kernels/tma_gemm.py:7-13,
 *                 34-38): element (b, k) is kept when tl.rand(dropout_seed, b * 768 + k) > dropout_p, X' = bf16(keep ? X /
 *                 (1 - p) : 0); logits, grad_W and the update use X' (the logits' operand is e4m3(X' / scale_x)), and
 *                 grad_x is the gradient with respect to X: (dL/dX') * keep / (1 - p).  The same result as a dropout
 *                 layer with this mask in front of xmc_fp8_step, without its launches.  dropout_p = 0: xmc_fp8_step.
 * Everything else as xmc_fp8_step, bit for bit when the three are zero. */
int xmc_fp8_step_ex(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, const void* x_bf16, int batch,
                    int features, const int32_t* labels_coo, int nnz, float lr, const uint32_t* seeds, int round_mode,
                    float scale_w, float scale_x, float weight_decay, float dropout_p, unsigned long long dropout_seed,
                    void* grad_x_bf16, float* grad_x_f32, void* workspace, size_t workspace_bytes, void* stream);

/* The fused step of the head-Kahan layer (src/xmc_classifiers/chunked_head_kahan_fp8xmc_clf.py:95-133, update of the
 * head rows: :127-129 with src/triton_kernels/fuse_kernel.py:202-262): as xmc_fp8_step with scales 1, and the first
 * num_head rows of chunk 0 carry a compensation term,
 *     T = (W + k) - lr A,   W' = round(T),   k' = cast(((k + W) - W') - lr A).
 * The rows of chunk 0 behind the head are updated as the reference updates them, through tensors sliced at num_head
 * (:130-131): the offsets of XMC_ROUND_SR_PHILOX's random numbers count from there.
 *   kahan        device [num_head, 768], updated in place: bf16 (kahan_type 1) or float8_e5m2 (kahan_type 2, saturating
 *                cast), 16-byte aligned
 *   num_head     1 .. rows_per_chunk
 * The tiles that hold head rows run as a launch of their own in front of the other tiles' launch.  Same status codes. */
int xmc_fp8_kahan_step(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, const void* x_bf16, int batch,
                       int features, const int32_t* labels_coo, int nnz, float lr, const uint32_t* seeds, int round_mode,
                       void* kahan, int kahan_type, int num_head, void* grad_x_bf16, float* grad_x_f32, void* workspace,
                       size_t workspace_bytes, void* stream);

/* Inference logits (chunked_fp8xmc_clf.py:45-60): out[b, label] = bf16(scale * sum_k e4m3(X/scale_x)[b,k] * W[label,k])
 * for label < num_labels (the padding rows of the last chunk are dropped, :60).
 *   out_bf16        device [batch, out_stride] bf16, out_stride >= num_labels; any alignment works, rows that start
 *                   on 32-byte boundaries (out_stride % 16 == 0) are written fastest
 */
int xmc_fp8_forward(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, const void* x_bf16, int batch,
                    int features, float scale_w, float scale_x, void* out_bf16, long long out_stride,
                    long long num_labels, void* workspace, size_t workspace_bytes, void* stream);

/* xmc_fp8_forward without a workspace argument.  It has no counterpart in the reference: it is for callers that cannot
 * allocate device memory for a workspace (code under HIP graph capture, serving loops and harnesses that forbid
 * hipMalloc).  The operand images of X that xmc_fp8_forward keeps in the caller's workspace live in a static device array
 * of the library instead (294,912 bytes per GPU, held until the process ends), so the limits are those of the array:
 * features == 768 and batch <= 128 (a multiple of 16); anything larger returns XMC_ERR_SHAPE.  The call allocates and
 * frees nothing.  Every call on a GPU uses that GPU's one array: calls that overlap on the same GPU (two streams, two
 * threads) race on it and must be serialised by the caller.  Outputs are bit-identical to xmc_fp8_forward's. */
int xmc_fp8_forward_static(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, const void* x_bf16, int batch,
                           int features, float scale_w, float scale_x, void* out_bf16, long long out_stride,
                           long long num_labels, void* stream);

/* Bytes of the scratch buffer of xmc_fp8_forward_topk: the logits of one segment of labels (as many whole chunks as
 * give at most 2^17 labels, or a 2^17-row piece of a larger chunk) and the running lists (two of 128 entries per batch
 * row).  Any rows_per_chunk that is a multiple of 16. */
size_t xmc_topk_scratch_bytes(int rows_per_chunk);

/* Inference with the top-k taken chunk by chunk: what the evaluation loop computes as
 * xfc_forward(embed).topk(k) (evaluate.py:158-159,235-236 on chunked_fp8xmc_clf.py:45-60) without the dense
 * [batch, num_labels] logits: the logits of a few chunks at a time go to `scratch` and are merged into the k best per row.
 *   out_val_bf16    device [batch, k] bf16, descending; equal values ordered by ascending label id
 *   out_idx         device [batch, k] int32 label ids (< num_labels: the padding rows of the last chunk are dropped)
 *   k               1..128, at most num_labels;  batch, x_bf16, scales, workspace: as xmc_fp8_forward
 */
int xmc_fp8_forward_topk(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, const void* x_bf16, int batch,
                         int features, float scale_w, float scale_x, long long num_labels, int k, void* out_val_bf16,
                         int32_t* out_idx, void* workspace, size_t workspace_bytes, void* scratch, size_t scratch_bytes,
                         void* stream);

/* Bytes of the scratch buffer of xmc_fp8_forward_topk_fused (a constant, below 1 MB: per-group maxima, bounds, counts and
 * 1,024 candidates per batch row). */
size_t xmc_topk_fused_scratch_bytes(void);

/* The same result as xmc_fp8_forward_topk (evaluate.py:158-159,235-236 on chunked_fp8xmc_clf.py:45-60) with the
 * selection inside the logits kernel: no logits reach memory.  Two passes over the weights: the first visits one tile
 * in 4..16 and yields, per batch row, a lower bound of the k-th largest logit; the second visits every tile and keeps
 * the logits at or above the bound (a few hundred per row), which a last kernel ranks.
 *   out_idx  device [batch, k] label ids, int32, or int64 (what torch.topk returns) with idx_int64 != 0
 *   status   device int32, written by the call's kernels: 0 = outputs valid; bit 0 = a row had more than 1,024 logits
 *            at or above its bound (massive ties, e.g. constant logits): the outputs of this call are then not to be
 *            used, and xmc_fp8_forward_topk gives the result; bit 1 = a row found fewer than k (not expected).
 *   returns XMC_ERR_RANGE (nothing launched) when the labels are too few for a useful bound (fewer than 4 k tiles of
 *   32 labels, i.e. num_labels below about 128 k): such shapes belong to xmc_fp8_forward_topk.  Other arguments as
 *   xmc_fp8_forward_topk.
 */
int xmc_fp8_forward_topk_fused(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, const void* x_bf16, int batch,
                               int features, float scale_w, float scale_x, long long num_labels, int k, void* out_val_bf16,
                               void* out_idx, int idx_int64, void* workspace, size_t workspace_bytes, void* scratch,
                               size_t scratch_bytes, int32_t* status, void* stream);

/* Dropout fused with the cast to e4m3 (the reference's prototype `_dropout` on the FP8 GEMM's A operand,
 * src/triton_kernels/tma_gemm.py:7-13,34-38): out[m][k] = e4m3(keep ? x[m][k] / (1 - p) : 0), keep = tl.rand(seed,
 * m * cols + k) > p (Philox-4x32-10 word 0 of counter (offset, 0, 0, 0), key = seed, as Triton's uniform fp32), the cast
 * saturating at +-448.
 *   x        device [rows, cols] contiguous, bf16 (x_type 0) or e4m3 (x_type 1, what the prototype takes); cols % 4 == 0
 *   p        drop probability, 0 <= p < 1;  out_e4m3: device [rows, cols] bytes;  rows * cols < 2^31
 */
int xmc_dropout_quantize(const void* x, int x_type, int rows, int cols, float p, unsigned long long seed, void* out_e4m3,
                         void* stream);

/* Test aid (no counterpart in the reference): sets how often a workgroup of the fused step polls a partner's counter
 * before it gives up (see xmc_fp8_step), for all later calls of the process, and returns the previous value; a negative
 * `limit` restores the default (2^18 polls).  With a limit of 0 every wait that is not satisfied at once expires: the
 * step then ends early with bit 0 of its error word set, every kernel still exits normally, and the tiles it did not
 * reach keep their old weights.  The tests use it to exercise the give-up path. */
int xmc_debug_spin_limit(int limit);

/* Benchmarking aid (no counterpart in the reference): the next xmc_fp8_step call records these two HIP events
 * (hipEvent_t, created by the caller) immediately before and after its fused step kernel, on the call's stream,
 * then forgets them.  Pass nulls to cancel. */
int xmc_profile_events(void* start_event, void* stop_event);

/* weight types of the tiled path */
enum {
  XMC_WEIGHT_E4M3 = 0,      /* simulated-FP8 mode of the FP8 layer (chunked_fp8xmc_clf.py:98-99,110,115-116) */
  XMC_WEIGHT_BF16 = 1       /* bf16 layer (chunked.py:85-131) */
};

/* Bytes of workspace xmc_tiled_step needs for batches of up to max_batch rows (1..512). */
size_t xmc_tiled_workspace_bytes(int num_chunks, int rows_per_chunk, int max_batch);
/* The same for a layer of `features` inputs (768 or 1024; the function above is this one at 768).  0 for any other
 * width. */
size_t xmc_tiled_workspace_bytes_ex(int num_chunks, int rows_per_chunk, int max_batch, int features);

/* One training step of the modes in which the reference keeps bf16 temporaries, three kernels per chunk as there:
 *   XMC_WEIGHT_BF16  XMCBCECHUNKEDLayer.xfc_forward_backward (chunked.py:76-133) with sgd_update
 *                    (stochastic_rounding_kernel.py:91-99): bf16 logits, grad_X partial rounded to bf16 per chunk,
 *                    grad_W rounded to bf16, W = SR16(W - lr*A) (XMC_ROUND_SR_PHILOX) or bf16(W - lr*A) (XMC_ROUND_RTN)
 *   XMC_WEIGHT_E4M3  Fp8XMCBCEChunkedLayer with simulated_fp8 (chunked_fp8xmc_clf.py:98-99,110,115-116;
 *                    fuse_kernel.py:184-199): logits from the un-quantised bf16 X, W = e4m3_torch(SR20(W - lr*A)),
 *                    where the final cast does not saturate (NaN above 464)
 *   features         768 or 1024 (d below); XMC_ERR_SHAPE otherwise.  The workspace is sized by
 *                    xmc_tiled_workspace_bytes_ex for the same width
 *   chunk_ptrs       host array of device pointers to the chunks' first rows; [rows, d] row-major each; all chunks
 *                    have rows_per_chunk rows except the last (rows_last_chunk <= rows_per_chunk); any row count
 *   labels_coo       as xmc_fp8_step; label id = chunk * rows_per_chunk + row.  The label space may exceed the 2^24 labels
 *                    the sort keys of xmc_fp8_step hold (up to 2^31 - 1 labels, a chunk below 2^24 - 1 rows): the
 *                    positives are then sorted once per segment of whole chunks with fewer than 2^24 - 1 labels
 *   round_mode       XMC_ROUND_RTN, XMC_ROUND_SR_PHILOX, or XMC_ROUND_SR_FAST with the random words of xmc_fp8_step's
 *                    mode of that name (bf16 weights: the hardware converter to bf16, which adds the upper 16 bits of the
 *                    word to the fp32 pattern); batch: 1..512, any value (processed in one, two or four halves of 128 rows)
 *   quantize_x       e4m3 weights: 0 = logits from the un-quantised X (simulated FP8), 1 = from e4m3(X) (true FP8, :101)
 *   saturate         e4m3 weights: 0 = final cast as torch (NaN above 464, :116), 1 = saturating at +-448 (fuse_kernel.py:35)
 *   kahan, kahan_type, num_head
 *                    head-Kahan update of Fp8XMCBCEChunkedHeadKahanLayer (chunked_head_kahan_fp8xmc_clf.py:41-48,127-131;
 *                    fuse_kernel.py:202-262), e4m3 weights only: device buffer [num_head, d] of bf16 (kahan_type 1) or
 *                    e5m2 (kahan_type 2) for the first num_head rows of chunk 0, updated in place; kahan_type 0 = none
 *   loss_out         device float or null.  Not null: receives the summed binary cross entropy of the step's bf16 logits
 *                    against the targets, sum over labels and batch rows of max(z,0) - [positive] z + log(1 + exp(-|z|)),
 *                    which is what _compute_loss of the reference is written to return (chunked.py:57-72; its caller
 *                    passes the weights where the logits belong, chunked.py:109, so the reference itself never returns
 *                    this value).  fp32 per element, summed in a fixed order.
 */
int xmc_tiled_step(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, int rows_last_chunk, int weight_type,
                   const void* x_bf16, int batch, int features, const int32_t* labels_coo, int nnz, float lr,
                   const uint32_t* seeds, int round_mode, int quantize_x, int saturate, void* kahan, int kahan_type,
                   int num_head, void* grad_x_bf16, float* grad_x_f32, float* loss_out, void* workspace,
                   size_t workspace_bytes, void* stream);

/* xmc_tiled_step with weight decay and dropout of the embedding, defined as for xmc_fp8_step_ex (for bf16 weights the
 * decay term joins the bf16-rounded gradient in fp32: T = W - lr (bf16(A) + weight_decay * W)).  With a head-Kahan
 * buffer (kahan_type != 0) both must be zero, as in the reference's layer: XMC_ERR_MODE otherwise. */
int xmc_tiled_step_ex(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, int rows_last_chunk, int weight_type,
                      const void* x_bf16, int batch, int features, const int32_t* labels_coo, int nnz, float lr,
                      const uint32_t* seeds, int round_mode, int quantize_x, int saturate, void* kahan, int kahan_type,
                      int num_head, float weight_decay, float dropout_p, unsigned long long dropout_seed, void* grad_x_bf16,
                      float* grad_x_f32, float* loss_out, void* workspace, size_t workspace_bytes, void* stream);

/* Measurement aid (no counterpart in the reference): copies `bytes` (a multiple of 16) from src to dst with a plain
 * grid-stride kernel.  Memory-traffic counters are calibrated against this launch of known size. */
int xmc_copy_probe(void* dst, const void* src, size_t bytes, void* stream);

/* Reads back the error word the last fused step on this workspace left there (every step clears it when it starts):
 *   bit 0  a workgroup gave up waiting for its partners (see xmc_fp8_step); it and, in turn, its partners stopped at
 *          that tile: the weights of the tiles they had not reached are unchanged, grad_X is incomplete
 *   bit 1  the four workgroups of some quad did not run on one XCD (a partition mode or dispatch order the kernel
 *          does not expect): the G they exchanged through that XCD's L2 may have been stale, the step is invalid
 * Synchronises the stream: meant for tests, debugging and a check where the training loop synchronises anyway. */
int xmc_step_error_word(const void* workspace, int num_chunks, int rows_per_chunk, void* stream);

/* Byte offset of that error word (one int32) inside the workspace. */
size_t xmc_step_error_offset(void);

/* Byte offset of the sticky error word (one int32) inside the workspace (no counterpart in the reference): the last
 * kernel of every fused step ORs the step's error word into it, and no kernel ever clears it.  It is for callers that
 * do not want to synchronise after every step: zero the word once after allocating the workspace, copy it to pinned
 * host memory behind any step (or every few steps) without waiting, and look at a copy whenever one has arrived - a
 * failure of any step since the word was last zeroed is still in it.  Zero it again after handling a failure. */
size_t xmc_step_sticky_error_offset(void);

/* Diagnostics of the placement assumption of the fused kernel (no counterpart in the reference).  The kernel builds
 * quads out of workgroups g with equal g % 8 and expects them on one XCD; every workgroup records the XCC id it really
 * ran on.  xmc_step_workgroups: number of workgroups the fused kernel is launched with on the current device.
 * xmc_step_xcc_ids: copies the ids of the first `count` workgroups of the last step to host memory (synchronises).
 * xmc_quad_placement_check: host-only; number of quads whose four members recorded different ids (0 = fine) - the
 * comparison the device makes at the end of every step before it raises bit 1 of the error word. */
int xmc_step_workgroups(void);
int xmc_step_xcc_ids(const void* workspace, int32_t* ids_host, int count, void* stream);
int xmc_quad_placement_check(const int32_t* xcc_ids_host, int num_workgroups);

#ifdef __cplusplus
}
#endif
#endif
