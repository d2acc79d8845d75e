// extern "C" surface of libelmo_xmc.so: argument validation, workspace carving and kernel launches.
// Declarations and the reference interfaces they replace: include/elmo_xmc.h.
#include "../../include/elmo_xmc.h"
#include "xmc_fp8_forward.hip"
#include "xmc_fp8_quad.hip"
#include "xmc_fp8_role.hip"
#include "xmc_tiled.hip"
#include "xmc_topk.hip"
#include "xmc_dropout.hip"
#include <stdlib.h>
#include <atomic>
#include <mutex>

using namespace xmc;

// Operand images of X for xmc_fp8_forward_static, the entry point that takes no workspace: e4m3 X in MFMA operand order
// (BP*D bytes), then the bf16 image the same preparation kernel writes (BP*D*2 bytes).  Every GPU the library runs on
// holds its own copy of this array until the process ends.  In host code the name stands for the symbol only, never for
// device memory: the address kernels get is the one hipGetSymbolAddress returned for the current device.
constexpr size_t FWD_STATIC_XQ = 0;
constexpr size_t FWD_STATIC_XT = (size_t)BP * D;
constexpr size_t FWD_STATIC_BYTES = FWD_STATIC_XT + (size_t)BP * D * 2;   // 294,912
static __device__ __align__(256) unsigned char scratch[FWD_STATIC_BYTES];

namespace {

struct DeviceInfo { int ok; int cus; unsigned char* scratch_ptr; };

// Filled once per device, by the first call on it; std::call_once makes concurrent first calls of several host threads
// wait for the one that fills the slot, and publishes the finished slot to all of them.
DeviceInfo g_device_info[64];
std::once_flag g_device_once[64];

void fill_device_info(int dev) {
  DeviceInfo di = {-1, 0, nullptr};
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, dev) != hipSuccess) { g_device_info[dev] = di; return; }
  di.cus = prop.multiProcessorCount;
  di.ok = (__builtin_strncmp(prop.gcnArchName, "gfx950", 6) == 0) ? 1 : -1;
  // this device's copy of the static scratch array (device `dev` is current here); stays null if the lookup fails
  void* sp = nullptr;
  di.scratch_ptr = (di.ok == 1 && hipGetSymbolAddress(&sp, HIP_SYMBOL(scratch)) == hipSuccess) ? (unsigned char*)sp : nullptr;
  // opt in to the full 160 KiB of LDS once per device
  role_plain_set_lds();
  role_heavy_set_lds();
  (void)hipFuncSetAttribute((const void*)fp8_forward_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, FWD_LDS);
  (void)hipFuncSetAttribute((const void*)fp8_forward_select_kernel<0>, hipFuncAttributeMaxDynamicSharedMemorySize, SEL_LDS);
  (void)hipFuncSetAttribute((const void*)fp8_forward_select_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize, SEL_LDS);
  (void)hipFuncSetAttribute((const void*)quad_sort_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (MAX_POS + 256) * 4);
  (void)hipFuncSetAttribute((const void*)quad_desc_prep_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (MAX_POS + 257) * 4);
#define XMC_TILED_ATTR(DD)                                                                                                                        \
  (void)hipFuncSetAttribute((const void*)tiled_gradx_kernel<W_BF16, 1, DD>, hipFuncAttributeMaxDynamicSharedMemorySize, TgxGeom<W_BF16, 1, DD>::LDS); \
  (void)hipFuncSetAttribute((const void*)tiled_gradx_kernel<W_E4M3, 1, DD>, hipFuncAttributeMaxDynamicSharedMemorySize, TgxGeom<W_E4M3, 1, DD>::LDS); \
  (void)hipFuncSetAttribute((const void*)tiled_gradx_kernel<W_BF16, 2, DD>, hipFuncAttributeMaxDynamicSharedMemorySize, TgxGeom<W_BF16, 2, DD>::LDS); \
  (void)hipFuncSetAttribute((const void*)tiled_gradx_kernel<W_E4M3, 2, DD>, hipFuncAttributeMaxDynamicSharedMemorySize, TgxGeom<W_E4M3, 2, DD>::LDS); \
  (void)hipFuncSetAttribute((const void*)tiled_logits_kernel<W_BF16, true, DD>, hipFuncAttributeMaxDynamicSharedMemorySize, TlgGeom<W_BF16, DD>::LDS); \
  (void)hipFuncSetAttribute((const void*)tiled_logits_kernel<W_BF16, false, DD>, hipFuncAttributeMaxDynamicSharedMemorySize, TlgGeom<W_BF16, DD>::LDS); \
  (void)hipFuncSetAttribute((const void*)tiled_logits_kernel<W_E4M3, true, DD>, hipFuncAttributeMaxDynamicSharedMemorySize, TlgGeom<W_E4M3, DD>::LDS); \
  (void)hipFuncSetAttribute((const void*)tiled_logits_kernel<W_E4M3, false, DD>, hipFuncAttributeMaxDynamicSharedMemorySize, TlgGeom<W_E4M3, DD>::LDS); \
  (void)hipFuncSetAttribute((const void*)tiled_logits_fp8_kernel<DD>, hipFuncAttributeMaxDynamicSharedMemorySize, TlgGeom<W_E4M3, DD>::LDS)
  XMC_TILED_ATTR(D);
  XMC_TILED_ATTR(1024);
#undef XMC_TILED_ATTR
  (void)hipFuncSetAttribute((const void*)tiled_update2_kernel<ROUND_RTN>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * TU2_GBUF);
  (void)hipFuncSetAttribute((const void*)tiled_update2_kernel<ROUND_SR_PHILOX>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * TU2_GBUF);
  (void)hipFuncSetAttribute((const void*)tiled_update2_kernel<ROUND_SR_FAST>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * TU2_GBUF);
  // the update kernels with two batch halves keep 96 KiB of operands in LDS, more than the default limit
#define XMC_UPD_ATTR_D(WTYPE, RMODE, KH, DD) (void)hipFuncSetAttribute((const void*)tiled_update_kernel<WTYPE, RMODE, 2, KH, DD>, hipFuncAttributeMaxDynamicSharedMemorySize, tup_lds_bytes(2, DD))
#define XMC_UPD_ATTR(WTYPE, RMODE, KH) XMC_UPD_ATTR_D(WTYPE, RMODE, KH, D); XMC_UPD_ATTR_D(WTYPE, RMODE, KH, 1024)
  XMC_UPD_ATTR(W_BF16, ROUND_RTN, false); XMC_UPD_ATTR(W_BF16, ROUND_SR_PHILOX, false); XMC_UPD_ATTR(W_BF16, ROUND_SR_FAST, false);
  XMC_UPD_ATTR(W_E4M3, ROUND_RTN, false); XMC_UPD_ATTR(W_E4M3, ROUND_SR_PHILOX, false); XMC_UPD_ATTR(W_E4M3, ROUND_SR_FAST, false);
  XMC_UPD_ATTR(W_E4M3, ROUND_RTN, true); XMC_UPD_ATTR(W_E4M3, ROUND_SR_PHILOX, true); XMC_UPD_ATTR(W_E4M3, ROUND_SR_FAST, true);
#undef XMC_UPD_ATTR_D
#undef XMC_UPD_ATTR
  g_device_info[dev] = di;
}

DeviceInfo device_info() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return DeviceInfo{-1, 0, nullptr};
  std::call_once(g_device_once[dev], fill_device_info, dev);
  return g_device_info[dev];
}

// polls of a partner's counter before a workgroup of the fused step gives up (xmc_debug_spin_limit)
std::atomic<int> g_spin_limit{QSPIN_LIMIT};

// optional event pair recorded around the next launch of the fused step kernel by the calling thread (benchmarking aid)
thread_local hipEvent_t g_prof_start = nullptr, g_prof_stop = nullptr;

inline bool aligned16(const void* q) { return ((uintptr_t)q & 15) == 0; }

int check_common(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, const void* x, int batch, int features,
                 const void* workspace, size_t workspace_bytes) {
  if (!chunk_ptrs || !x || !workspace) return XMC_ERR_NULL;
  if (features != D || batch <= 0 || batch > BP || batch % 16 != 0) return XMC_ERR_SHAPE;
  if (rows_per_chunk <= 0 || rows_per_chunk % 16 != 0) return XMC_ERR_SHAPE;
  if (num_chunks <= 0 || num_chunks > MAX_CHUNKS) return XMC_ERR_RANGE;
  if ((long long)num_chunks * rows_per_chunk > 0x7FFFFFFFLL) return XMC_ERR_RANGE;   // the fused step has a lower limit of its own
  for (int c = 0; c < num_chunks; c++) {
    if (!chunk_ptrs[c]) return XMC_ERR_NULL;
    if (!aligned16(chunk_ptrs[c])) return XMC_ERR_ALIGN;
  }
  if (!aligned16(x) || ((uintptr_t)workspace & 255) != 0) return XMC_ERR_ALIGN;
  if (workspace_bytes < xmc_workspace_bytes(num_chunks, rows_per_chunk)) return XMC_ERR_WORKSPACE;
  return XMC_OK;
}

// plain 16-byte-per-lane copy: the known-size reference against which memory counters are calibrated
__global__ __launch_bounds__(256) void copy_probe_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n16) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256) dst[i] = src[i];
}

int launch_status() { return hipGetLastError() == hipSuccess ? XMC_OK : XMC_ERR_LAUNCH; }

// xmc_fp8_forward_topk takes the labels in segments of at most 2^17: as many whole chunks as fit (fewer, larger
// launches), or, for a chunk that is larger than that by itself, pieces of it of 2^17 rows
constexpr int TOPK_SEG = 1 << 17;
int topk_group(int rows_per_chunk) { const int g = TOPK_SEG / rows_per_chunk; return g < 1 ? 1 : g; }
long long topk_segment_rows(int rows_per_chunk) {
  return rows_per_chunk > TOPK_SEG ? (long long)TOPK_SEG : (long long)topk_group(rows_per_chunk) * rows_per_chunk;
}
size_t topk_zbuf_bytes(int rows_per_chunk) {
  return ((size_t)BP * (size_t)topk_segment_rows(rows_per_chunk) * 2 + 255) / 256 * 256;
}

// The launches of the inference logits, shared by xmc_fp8_forward (operand images in the caller's workspace) and
// xmc_fp8_forward_static (operand images in this device's copy of the static array); shapes are checked by the callers.
int forward_launch(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, const void* x_bf16, int batch, float scale_w,
                   float scale_x, void* out_bf16, long long out_stride, long long num_labels, unsigned char* xq,
                   unsigned short* xt, hipStream_t stream) {
  if (!out_bf16) return XMC_ERR_NULL;
  if (num_labels <= 0 || out_stride < num_labels || num_labels > (long long)num_chunks * rows_per_chunk) return XMC_ERR_SHAPE;
  if (!(scale_w > 0.f) || !(scale_x > 0.f)) return XMC_ERR_SHAPE;
  DeviceInfo di = device_info();
  if (di.ok != 1) return XMC_ERR_DEVICE;
  prep_x_kernel<<<(BP * (D / 4) + 255) / 256, 256, 0, stream>>>((const unsigned short*)x_bf16, batch, 1.0f / scale_x, xq, xt);
  ForwardParams fp;
  for (int c = 0; c < MAX_CHUNKS; c++) fp.chunk[c] = c < num_chunks ? (const unsigned char*)chunk_ptrs[c] : nullptr;
  fp.rows_per_chunk = rows_per_chunk;
  fp.tiles_per_chunk = (rows_per_chunk + FT - 1) / FT;
  const int last_chunk = (int)((num_labels - 1) / rows_per_chunk);
  fp.tile_begin = 0;
  fp.tile_end = last_chunk * fp.tiles_per_chunk + (int)((num_labels - (long long)last_chunk * rows_per_chunk + FT - 1) / FT);
  fp.xq = xq;
  fp.zscale = scale_w * scale_x;
  fp.out = (unsigned short*)out_bf16;
  fp.out_stride = out_stride;
  fp.col0 = 0;
  fp.num_labels = num_labels;
  fp.batch = batch;
  const int grid = fp.tile_end < 2 * di.cus ? fp.tile_end : 2 * di.cus;   // two workgroups fit the LDS of a compute unit
  fp8_forward_kernel<<<grid, NT, FWD_LDS, stream>>>(fp);
  return launch_status();
}

}  // namespace

extern "C" {

int xmc_version(void) { return 1; }

#ifndef XMC_SOURCE_HASH
#define XMC_SOURCE_HASH "unknown"
#endif
const char* xmc_source_hash(void) { return XMC_SOURCE_HASH; }

const char* xmc_error_string(int status) {
  switch (status) {
    case XMC_OK: return "ok";
    case XMC_ERR_NULL: return "null pointer";
    case XMC_ERR_SHAPE: return "unsupported shape (features must be 768, batch a multiple of 16 and <= 128, rows per chunk a multiple of 16)";
    case XMC_ERR_ALIGN: return "device pointer not sufficiently aligned";
    case XMC_ERR_RANGE: return "too many chunks, labels or positives";
    case XMC_ERR_WORKSPACE: return "workspace too small";
    case XMC_ERR_MODE: return "unknown rounding mode";
    case XMC_ERR_LAUNCH: return "kernel launch failed";
    case XMC_ERR_DEVICE: return "current device is not a gfx950 GPU with at least 16 compute units";
    default: return "unknown status";
  }
}

size_t xmc_workspace_bytes(int num_chunks, int rows_per_chunk) {
  if (num_chunks <= 0 || num_chunks > MAX_CHUNKS || rows_per_chunk <= 0) return 0;
  size_t tiles = (size_t)num_chunks * ((rows_per_chunk + TL - 1) / TL);
  // tile_ptr, then 32-byte tile descriptors, one run per quad (up to MAX_WG / 4 runs, each rounded up to whole entries)
  // (two tables with a compensated head)
  return WS_TILEPTR + ((tiles + 1) * 4 + 255) / 256 * 256 + (tiles + MAX_WG / 2) * 32;
}

int xmc_fp8_step(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, const void* x_bf16, int batch,
                 int features, const int32_t* labels_coo, int nnz, float lr, const uint32_t* seeds, int round_mode,
                 float scale_w, float scale_x, void* grad_x_bf16, float* grad_x_f32, void* workspace,
                 size_t workspace_bytes, void* stream_) {
  return xmc_fp8_step_ex(chunk_ptrs, num_chunks, rows_per_chunk, x_bf16, batch, features, labels_coo, nnz, lr, seeds, round_mode,
                         scale_w, scale_x, 0.0f, 0.0f, 0ull, grad_x_bf16, grad_x_f32, workspace, workspace_bytes, stream_);
}

}  // extern "C"

// The fused step behind xmc_fp8_step, xmc_fp8_step_ex and xmc_fp8_kahan_step.  kahan_type 0: no compensated head.
static int fused_step(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, const void* x_bf16, int batch,
                      int features, const int32_t* labels_coo, int nnz, float lr, const uint32_t* seeds, int round_mode,
                      float scale_w, float scale_x, float weight_decay, float dropout_p, unsigned long long dropout_seed,
                      void* kahan, int kahan_type, int num_head,
                      void* grad_x_bf16, float* grad_x_f32, void* workspace, size_t workspace_bytes, void* stream_) {
  int st = check_common(chunk_ptrs, num_chunks, rows_per_chunk, x_bf16, batch, features, workspace, workspace_bytes);
  if (st != XMC_OK) return st;
  // a sort key keeps 24 bits for the label (xmc_tiled_step takes larger label spaces in segments)
  if ((long long)num_chunks * rows_per_chunk >= (1LL << 24) - 1) return XMC_ERR_RANGE;
  if (!grad_x_bf16 || (nnz > 0 && !labels_coo)) return XMC_ERR_NULL;
  if (((uintptr_t)labels_coo & 7) != 0) return XMC_ERR_ALIGN;   // read as (row, label) pairs
  if (nnz < 0 || nnz > MAX_POS) return XMC_ERR_RANGE;
  if (round_mode < XMC_ROUND_RTN || round_mode > XMC_ROUND_SR_FAST) return XMC_ERR_MODE;
  if (round_mode != XMC_ROUND_RTN && !seeds) return XMC_ERR_NULL;
  if (!(scale_w > 0.f) || !(scale_x > 0.f)) return XMC_ERR_SHAPE;
  if (!(weight_decay >= 0.f) || !(dropout_p >= 0.f) || !(dropout_p < 1.f)) return XMC_ERR_SHAPE;
  if (kahan_type < 0 || kahan_type > 2) return XMC_ERR_MODE;
  if (kahan_type != 0) {
    if (!kahan) return XMC_ERR_NULL;
    if (!aligned16(kahan)) return XMC_ERR_ALIGN;
    if (num_head <= 0 || num_head > rows_per_chunk) return XMC_ERR_SHAPE;
  } else {
    num_head = 0;
  }
  DeviceInfo di = device_info();
  if (di.ok != 1 || di.cus < 16) return XMC_ERR_DEVICE;
  hipStream_t stream = (hipStream_t)stream_;
  unsigned char* ws = (unsigned char*)workspace;
  const DropoutParams dp = {dropout_p, 1.0f - dropout_p, (unsigned)(dropout_seed & 0xFFFFFFFFull), (unsigned)(dropout_seed >> 32)};

  const int grid = di.cus < MAX_WG ? di.cus : MAX_WG;   // one workgroup per compute unit
  const int tiles_per_chunk = (rows_per_chunk + TL - 1) / TL;
  const int num_tiles = num_chunks * tiles_per_chunk;
  int n_pad = 0;
  if (nnz > 0) { n_pad = 64; while (n_pad < nnz) n_pad <<= 1; }

  {
    QuadParams p;
    for (int c = 0; c < MAX_CHUNKS; c++) {
      p.chunk[c] = c < num_chunks ? (unsigned char*)chunk_ptrs[c] : nullptr;
      p.seed[c] = (c < num_chunks && seeds) ? (round_mode == XMC_ROUND_SR_FAST ? fast_seed(seeds[c]) : seeds[c]) : 0u;
    }
    p.num_chunks = num_chunks;
    p.rows_per_chunk = rows_per_chunk;
    p.tiles_per_chunk = tiles_per_chunk;
    p.num_tiles = num_tiles;
    p.run_tiles = num_tiles;
    p.xq = ws + WS_XQ;
    p.xt = (const bf16x8*)(ws + WS_XT);
    p.keys = (const unsigned*)(ws + WS_KEYS);
    p.tile_ptr = (const int*)(ws + WS_TILEPTR);
    p.partial = (floatx4*)(ws + WS_PARTIAL);
    p.exch = ws + WS_EXCH;
    uint4* desc = (uint4*)(ws + WS_TILEPTR + ((size_t)(num_tiles + 1) * 4 + 255) / 256 * 256);
    p.desc = desc;
    p.flags = (int*)(ws + WS_FLAGS);
    p.zscale = scale_w * scale_x;
    p.lr_eff = lr / scale_w;
    p.wd_eff = weight_decay * scale_w;   // T = c - (lr / s) (A + wd s c) for codes c = W / s
    p.batch = batch;
    int qgrid = grid / 32 * 32;   // whole quads on every XCD
    if (qgrid < 32) return XMC_ERR_DEVICE;
    p.nquads = qgrid >> 2;
    // with a compensated head the tiles that hold its rows run first, as a launch of their own
    const int head_tiles = (num_head + TL - 1) / TL, rest_tiles = num_tiles - head_tiles;
    p.kahan = (unsigned char*)kahan;
    p.num_head = num_head;
    p.head_tiles = head_tiles;
    p.kmax_head = (head_tiles + p.nquads - 1) / p.nquads;
    p.kmax = (rest_tiles + p.nquads - 1) / p.nquads;
    p.cnt_base = 0;
    p.acc_init = 0;
    p.spin_limit = g_spin_limit.load(std::memory_order_relaxed);
    quad_sort_kernel<<<n_pad > 0 ? n_pad / 64 : 1, 256, (size_t)(n_pad + 256) * 4, stream>>>(
        labels_coo, nnz, n_pad, batch, 0, 0, num_chunks * rows_per_chunk, (unsigned*)(ws + WS_KEYS), (int*)(ws + WS_FLAGS));
    const int desc_blocks = (num_tiles + 1 + 255) / 256;
    quad_desc_prep_kernel<<<desc_blocks + (BP * (D / 4) + 255) / 256, 256, (size_t)(n_pad + 257) * 4, stream>>>(
        p, n_pad, (int*)(ws + WS_TILEPTR), desc, desc_blocks, (const unsigned short*)x_bf16, 1.0f / scale_x, ws + WS_XQ,
        (unsigned short*)(ws + WS_XT), dp);
    if (g_prof_start) (void)hipEventRecord(g_prof_start, stream);
    QuadParams ph = p;   // the head's launch
    ph.run_tiles = head_tiles;
    ph.kmax = p.kmax_head;
    p.run_tiles = rest_tiles;
    p.desc = desc + 2 * (size_t)p.nquads * p.kmax_head;
    if (head_tiles > 0) { p.cnt_base = QF_CNT2; p.acc_init = 1; }
    // the variants with the Philox recipe or a compensated head live in the library's second translation unit
    if (kahan_type != 0) role_heavy_launch(round_mode, false, kahan_type, qgrid, stream, ph);
    if (rest_tiles > 0) {
      const bool wd = weight_decay != 0.f;
      if (round_mode == XMC_ROUND_SR_PHILOX) role_heavy_launch(round_mode, wd, 0, qgrid, stream, p);
      else role_plain_launch(round_mode, wd, qgrid, stream, p);
    }
    if (g_prof_stop) (void)hipEventRecord(g_prof_stop, stream);
    g_prof_start = g_prof_stop = nullptr;
    reduce_gx_role_kernel<<<192, 128, 0, stream>>>((const floatx4*)(ws + WS_PARTIAL), qgrid, scale_w, grad_x_f32,
                                                 (unsigned short*)grad_x_bf16, batch, (int*)(ws + WS_FLAGS), dp);
  }
  return launch_status();
}

extern "C" {

int xmc_fp8_step_ex(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, const void* x_bf16, int batch,
                    int features, const int32_t* labels_coo, int nnz, float lr, const uint32_t* seeds, int round_mode,
                    float scale_w, float scale_x, float weight_decay, float dropout_p, unsigned long long dropout_seed,
                    void* grad_x_bf16, float* grad_x_f32, void* workspace, size_t workspace_bytes, void* stream_) {
  return fused_step(chunk_ptrs, num_chunks, rows_per_chunk, x_bf16, batch, features, labels_coo, nnz, lr, seeds, round_mode,
                    scale_w, scale_x, weight_decay, dropout_p, dropout_seed, nullptr, 0, 0, grad_x_bf16, grad_x_f32, workspace,
                    workspace_bytes, stream_);
}

int xmc_fp8_kahan_step(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, const void* x_bf16, int batch,
                       int features, const int32_t* labels_coo, int nnz, float lr, const uint32_t* seeds, int round_mode,
                       void* kahan, int kahan_type, int num_head, void* grad_x_bf16, float* grad_x_f32, void* workspace,
                       size_t workspace_bytes, void* stream_) {
  if (kahan_type != 1 && kahan_type != 2) return XMC_ERR_MODE;
  return fused_step(chunk_ptrs, num_chunks, rows_per_chunk, x_bf16, batch, features, labels_coo, nnz, lr, seeds, round_mode,
                    1.0f, 1.0f, 0.0f, 0.0f, 0ull, kahan, kahan_type, num_head, grad_x_bf16, grad_x_f32, workspace,
                    workspace_bytes, stream_);
}

int xmc_fp8_forward(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, const void* x_bf16, int batch,
                    int features, float scale_w, float scale_x, void* out_bf16, long long out_stride,
                    long long num_labels, void* workspace, size_t workspace_bytes, void* stream_) {
  int st = check_common(chunk_ptrs, num_chunks, rows_per_chunk, x_bf16, batch, features, workspace, workspace_bytes);
  if (st != XMC_OK) return st;
  unsigned char* ws = (unsigned char*)workspace;
  return forward_launch(chunk_ptrs, num_chunks, rows_per_chunk, x_bf16, batch, scale_w, scale_x, out_bf16, out_stride,
                        num_labels, ws + WS_XQ, (unsigned short*)(ws + WS_XT), (hipStream_t)stream_);
}

int xmc_fp8_forward_static(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, const void* x_bf16, int batch,
                           int features, float scale_w, float scale_x, void* out_bf16, long long out_stride,
                           long long num_labels, void* stream_) {
  // the same checks as xmc_fp8_forward, without a workspace; the static array holds the operand images of at most
  // BP = 128 batch rows of D = 768 features, which is also the limit of xmc_fp8_forward
  if (!chunk_ptrs || !x_bf16) return XMC_ERR_NULL;
  if (features != D || batch <= 0 || batch > BP || batch % 16 != 0) return XMC_ERR_SHAPE;
  if (rows_per_chunk <= 0 || rows_per_chunk % 16 != 0) return XMC_ERR_SHAPE;
  if (num_chunks <= 0 || num_chunks > MAX_CHUNKS) return XMC_ERR_RANGE;
  if ((long long)num_chunks * rows_per_chunk > 0x7FFFFFFFLL) return XMC_ERR_RANGE;
  for (int c = 0; c < num_chunks; c++) {
    if (!chunk_ptrs[c]) return XMC_ERR_NULL;
    if (!aligned16(chunk_ptrs[c])) return XMC_ERR_ALIGN;
  }
  if (!aligned16(x_bf16)) return XMC_ERR_ALIGN;
  const DeviceInfo di = device_info();
  if (di.ok != 1 || !di.scratch_ptr) return XMC_ERR_DEVICE;
  return forward_launch(chunk_ptrs, num_chunks, rows_per_chunk, x_bf16, batch, scale_w, scale_x, out_bf16, out_stride,
                        num_labels, di.scratch_ptr + FWD_STATIC_XQ, (unsigned short*)(di.scratch_ptr + FWD_STATIC_XT),
                        (hipStream_t)stream_);
}

size_t xmc_topk_scratch_bytes(int rows_per_chunk) {
  if (rows_per_chunk <= 0 || rows_per_chunk % 16 != 0) return 0;
  // logits of one group of chunks [128][group * rows] bf16, then the running lists, two per batch row: values
  // [128][2][128] bf16, label ids [128][2][128] int32
  return topk_zbuf_bytes(rows_per_chunk) + 2 * ((size_t)BP * TOPK_MAX * 2 + (size_t)BP * TOPK_MAX * 4);
}

int xmc_fp8_forward_topk(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, const void* x_bf16, int batch,
                         int features, float scale_w, float scale_x, long long num_labels, int k, void* out_val_bf16,
                         int32_t* out_idx, void* workspace, size_t workspace_bytes, void* scratch, size_t scratch_bytes,
                         void* stream_) {
  int st = check_common(chunk_ptrs, num_chunks, rows_per_chunk, x_bf16, batch, features, workspace, workspace_bytes);
  if (st != XMC_OK) return st;
  if (!out_val_bf16 || !out_idx || !scratch) return XMC_ERR_NULL;
  if (((uintptr_t)scratch & 255) != 0) return XMC_ERR_ALIGN;
  if (scratch_bytes < xmc_topk_scratch_bytes(rows_per_chunk)) return XMC_ERR_WORKSPACE;
  if (num_labels <= 0 || num_labels > (long long)num_chunks * rows_per_chunk) return XMC_ERR_SHAPE;
  if (k <= 0 || k > TOPK_MAX || k > num_labels) return XMC_ERR_SHAPE;
  if (!(scale_w > 0.f) || !(scale_x > 0.f)) return XMC_ERR_SHAPE;
  DeviceInfo di = device_info();
  if (di.ok != 1) return XMC_ERR_DEVICE;
  hipStream_t stream = (hipStream_t)stream_;
  unsigned char* ws = (unsigned char*)workspace;
  unsigned short* zbuf = (unsigned short*)scratch;
  unsigned short* run_val = (unsigned short*)((unsigned char*)scratch + topk_zbuf_bytes(rows_per_chunk));
  int* run_idx = (int*)(run_val + (size_t)BP * 2 * TOPK_MAX);
  prep_x_kernel<<<(BP * (D / 4) + 255) / 256, 256, 0, stream>>>((const unsigned short*)x_bf16, batch, 1.0f / scale_x, ws + WS_XQ,
                                                              (unsigned short*)(ws + WS_XT));
  ForwardParams fp;
  for (int c = 0; c < MAX_CHUNKS; c++) fp.chunk[c] = c < num_chunks ? (const unsigned char*)chunk_ptrs[c] : nullptr;
  fp.rows_per_chunk = rows_per_chunk;
  fp.tiles_per_chunk = (rows_per_chunk + FT - 1) / FT;
  fp.xq = ws + WS_XQ;
  fp.zscale = scale_w * scale_x;
  const int group = topk_group(rows_per_chunk);
  const long long seg_rows = topk_segment_rows(rows_per_chunk);
  fp.out = zbuf;
  fp.out_stride = seg_rows;
  fp.num_labels = num_labels;
  fp.batch = batch;
  // Every batch row keeps two lists.  Large segments are split between two workgroups per row (one list each), so that
  // 128 rows occupy all compute units; small ones go to list 0.  A list without k entries yet is first given a short
  // piece (4,096 logits, which fit the workgroup's candidate store): that leaves k entries whose smallest value bounds
  // the rest.
  int have[2] = {0, 0};
  auto select = [&](const unsigned short* zp, int n, int base, int parts) {
    topk_chunk_kernel<<<batch * parts, TOPK_NT, 0, stream>>>(zp, seg_rows, n, base, k, parts, have[0], have[1], run_val, run_idx);
    const int n0 = parts == 2 ? topk_split(n) : n;
    have[0] = have[0] + n0 < k ? have[0] + n0 : k;
    have[1] = have[1] + (n - n0) < k ? have[1] + (n - n0) : k;
  };
  // one segment: the logits of tiles [tile_begin, tile_end) into the scratch buffer, then their n labels from `base` on
  auto segment = [&](int tile_begin, int tile_end, long long base, int n) {
    fp.tile_begin = tile_begin;
    fp.tile_end = tile_end;
    fp.col0 = base;
    const int tiles = tile_end - tile_begin;
    fp8_forward_kernel<<<tiles < 2 * di.cus ? tiles : 2 * di.cus, NT, FWD_LDS, stream>>>(fp);
    int done = 0;
    if (n > 32768) {          // two workgroups per row
      if (have[0] < k || have[1] < k) {
        done = 8192;
        select(zbuf, done, (int)base, 2);
      }
      select(zbuf + done, n - done, (int)base + done, 2);
    } else {
      if (have[0] < k && n > 8192) {
        done = 4096;
        select(zbuf, done, (int)base, 1);
      }
      select(zbuf + done, n - done, (int)base + done, 1);
    }
  };
  if (rows_per_chunk <= TOPK_SEG) {
    for (int c = 0; c < num_chunks; c += group) {
      const long long base = (long long)c * rows_per_chunk;
      if (base >= num_labels) break;
      const int n = (int)(num_labels - base < seg_rows ? num_labels - base : seg_rows);     // padding rows are dropped
      const int full = n / rows_per_chunk, rest = n - full * rows_per_chunk;                // whole chunks, rows of the last one
      segment(c * fp.tiles_per_chunk, c * fp.tiles_per_chunk + full * fp.tiles_per_chunk + (rest + FT - 1) / FT, base, n);
    }
  } else {
    for (int c = 0; c < num_chunks; c++)
      for (int r0 = 0; r0 < rows_per_chunk; r0 += TOPK_SEG) {       // TOPK_SEG is a multiple of the tile height
        const long long base = (long long)c * rows_per_chunk + r0;
        if (base >= num_labels) break;
        long long n = rows_per_chunk - r0 < TOPK_SEG ? rows_per_chunk - r0 : TOPK_SEG;
        if (n > num_labels - base) n = num_labels - base;
        segment(c * fp.tiles_per_chunk + r0 / FT, c * fp.tiles_per_chunk + r0 / FT + (int)((n + FT - 1) / FT), base, (int)n);
      }
  }
  topk_finish_kernel<<<batch, 2 * TOPK_MAX, 0, stream>>>(run_val, run_idx, k, have[0], have[1], (unsigned short*)out_val_bf16, out_idx);
  return launch_status();
}

// scratch of xmc_fp8_forward_topk_fused: group maxima, bounds, counts, candidate labels and keys
constexpr size_t SELS_GMAX = 0;
constexpr size_t SELS_BOUND = SELS_GMAX + (size_t)SEL_GROUPS * BP * 2;
constexpr size_t SELS_COUNT = SELS_BOUND + 256;
constexpr size_t SELS_LABEL = SELS_COUNT + (size_t)BP * 4;
constexpr size_t SELS_KEY = SELS_LABEL + (size_t)BP * SEL_CAP * 4;
constexpr size_t SELS_BYTES = SELS_KEY + (size_t)BP * SEL_CAP * 2;
static_assert(SEL_CAP == TOPK_LIST && SEL_GROUPS == TOPK_GROUPS, "the two top-k kernels share these sizes");

size_t xmc_topk_fused_scratch_bytes(void) { return SELS_BYTES; }

// tiles pass 1 skips between two it visits: the k-th largest of the group maxima of a 1/step sample leaves about
// k * step candidates per row, which have to stay well below the list size; at least four groups per wanted entry
static int topk_fused_step(int tiles, int k) {
  int step = 16;
  while (step > 1 && (k * step > SEL_CAP / 2 || tiles / step < 4 * k)) step >>= 1;
  return tiles / step >= 4 * k ? step : 0;
}

int xmc_fp8_forward_topk_fused(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, const void* x_bf16, int batch,
                               int features, float scale_w, float scale_x, long long num_labels, int k, void* out_val_bf16,
                               void* out_idx, int idx_int64, void* workspace, size_t workspace_bytes, void* scratch,
                               size_t scratch_bytes, int32_t* status, void* stream_) {
  int st = check_common(chunk_ptrs, num_chunks, rows_per_chunk, x_bf16, batch, features, workspace, workspace_bytes);
  if (st != XMC_OK) return st;
  if (!out_val_bf16 || !out_idx || !scratch || !status) return XMC_ERR_NULL;
  if (((uintptr_t)scratch & 255) != 0 || ((uintptr_t)status & 3) != 0 || ((uintptr_t)out_idx & (idx_int64 ? 7 : 3)) != 0) return XMC_ERR_ALIGN;
  if (scratch_bytes < SELS_BYTES) return XMC_ERR_WORKSPACE;
  if (num_labels <= 0 || num_labels > (long long)num_chunks * rows_per_chunk) return XMC_ERR_SHAPE;
  if (k <= 0 || k > TOPK_MAX || k > num_labels) return XMC_ERR_SHAPE;
  if (!(scale_w > 0.f) || !(scale_x > 0.f)) return XMC_ERR_SHAPE;
  SelectParams sp;
  sp.rows_per_chunk = rows_per_chunk;
  sp.tiles_per_chunk = (rows_per_chunk + FT - 1) / FT;
  const int last_chunk = (int)((num_labels - 1) / rows_per_chunk);
  const int tiles = last_chunk * sp.tiles_per_chunk + (int)((num_labels - (long long)last_chunk * rows_per_chunk + FT - 1) / FT);
  const int step = topk_fused_step(tiles, k);
  if (step == 0) return XMC_ERR_RANGE;   // too few labels for a useful bound: xmc_fp8_forward_topk takes these
  DeviceInfo di = device_info();
  if (di.ok != 1) return XMC_ERR_DEVICE;
  hipStream_t stream = (hipStream_t)stream_;
  unsigned char* ws = (unsigned char*)workspace;
  unsigned char* sc = (unsigned char*)scratch;
  prep_x_kernel<<<(BP * (D / 4) + 255) / 256, 256, 0, stream>>>((const unsigned short*)x_bf16, batch, 1.0f / scale_x, ws + WS_XQ,
                                                              (unsigned short*)(ws + WS_XT));
  for (int c = 0; c < MAX_CHUNKS; c++) sp.chunk[c] = c < num_chunks ? (const unsigned char*)chunk_ptrs[c] : nullptr;
  sp.xq = ws + WS_XQ;
  sp.zscale = scale_w * scale_x;
  sp.num_labels = num_labels;
  sp.batch = batch;
  sp.gmax = (unsigned short*)(sc + SELS_GMAX);
  sp.bound = (const unsigned short*)(sc + SELS_BOUND);
  sp.count = (unsigned*)(sc + SELS_COUNT);
  sp.cand_label = (unsigned*)(sc + SELS_LABEL);
  sp.cand_key = (unsigned short*)(sc + SELS_KEY);
  // pass 1: the sampled tiles, one group of them per workgroup
  sp.tile_step = step;
  sp.n_visit = (tiles + step - 1) / step;
  const int groups = sp.n_visit < SEL_GROUPS ? sp.n_visit : SEL_GROUPS;
  fp8_forward_select_kernel<0><<<groups, NT, SEL_LDS, stream>>>(sp);
  topk_bound_kernel<<<BP, TOPK_GROUPS, 0, stream>>>(sp.gmax, groups, k, batch, (unsigned short*)(sc + SELS_BOUND), sp.count, status);
  // pass 2: every tile
  sp.tile_step = 1;
  sp.n_visit = tiles;
  fp8_forward_select_kernel<1><<<tiles < 2 * di.cus ? tiles : 2 * di.cus, NT, SEL_LDS, stream>>>(sp);
  topk_pick_kernel<<<batch, TOPK_LIST, 0, stream>>>(sp.cand_label, sp.cand_key, sp.count, k, (unsigned short*)out_val_bf16, out_idx,
                                                    idx_int64 ? 1 : 0, status);
  return launch_status();
}

int xmc_dropout_quantize(const void* x, int x_type, int rows, int cols, float p, unsigned long long seed, void* out_e4m3,
                         void* stream_) {
  if (!x || !out_e4m3) return XMC_ERR_NULL;
  if (x_type != 0 && x_type != 1) return XMC_ERR_MODE;
  if (rows <= 0 || cols <= 0 || cols % 4 != 0 || !(p >= 0.f) || !(p < 1.f)) return XMC_ERR_SHAPE;
  if ((long long)rows * cols > 0x7FFFFFFFll) return XMC_ERR_RANGE;   // the random offsets are 32-bit element indices
  if (((uintptr_t)x & (x_type == 0 ? 7 : 3)) != 0 || ((uintptr_t)out_e4m3 & 3) != 0) return XMC_ERR_ALIGN;
  DeviceInfo di = device_info();
  if (di.ok != 1) return XMC_ERR_DEVICE;
  const long long n4 = (long long)rows * cols / 4;
  dropout_quantize_kernel<<<(unsigned)((n4 + 255) / 256), 256, 0, (hipStream_t)stream_>>>(x, x_type, n4, cols, p, (unsigned)(seed & 0xFFFFFFFFull),
                                                                                        (unsigned)(seed >> 32), (unsigned*)out_e4m3);
  return launch_status();
}

int xmc_debug_spin_limit(int limit) {
  return g_spin_limit.exchange(limit < 0 ? QSPIN_LIMIT : limit, std::memory_order_relaxed);
}

int xmc_profile_events(void* start_event, void* stop_event) {
  g_prof_start = (hipEvent_t)start_event;
  g_prof_stop = (hipEvent_t)stop_event;
  return XMC_OK;
}

size_t xmc_tiled_workspace_bytes(int num_chunks, int rows_per_chunk, int max_batch) {
  return xmc_tiled_workspace_bytes_ex(num_chunks, rows_per_chunk, max_batch, D);
}

size_t xmc_tiled_workspace_bytes_ex(int num_chunks, int rows_per_chunk, int max_batch, int features) {
  if (features != D && features != 1024) return 0;
  if (num_chunks <= 0 || num_chunks > MAX_CHUNKS || rows_per_chunk <= 0 || max_batch <= 0 || max_batch > T_HALVES * BP) return 0;
  const size_t rows_pad = ((size_t)rows_per_chunk + TL - 1) / TL * TL;
  const size_t tiles = (size_t)num_chunks * (rows_pad / TL);
  const size_t halves = (size_t)tiled_halves(max_batch), pairs = (halves + 1) / 2;
  const size_t rows_buf = (size_t)tiled_group(num_chunks, rows_per_chunk) * rows_pad;   // rows of one launch
  // per batch half G in both orientations; tile_ptr per pair of halves (padded to 64 entries); two loss shares per tile
  return tiled_layout((int)halves, features).g + halves * 2 * rows_buf * BP * 2 + pairs * ((tiles + 1 + 63) / 64 * 64 * 4) + (tiles * 8 + 255) / 256 * 256;
}

int xmc_tiled_step(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, int rows_last_chunk, int weight_type,
                   const void* x_bf16, int batch, int features, const int32_t* labels_coo, int nnz, float lr,
                   const uint32_t* seeds, int round_mode, int quantize_x, int saturate, void* kahan, int kahan_type,
                   int num_head, void* grad_x_bf16, float* grad_x_f32, float* loss_out, void* workspace,
                   size_t workspace_bytes, void* stream_) {
  return xmc_tiled_step_ex(chunk_ptrs, num_chunks, rows_per_chunk, rows_last_chunk, weight_type, x_bf16, batch, features, labels_coo,
                           nnz, lr, seeds, round_mode, quantize_x, saturate, kahan, kahan_type, num_head, 0.0f, 0.0f, 0ull,
                           grad_x_bf16, grad_x_f32, loss_out, workspace, workspace_bytes, stream_);
}

}  // extern "C"

// xmc_tiled_step_ex for DD features (768 or 1024)
template <int DD>
static int tiled_step_t(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, int rows_last_chunk, int weight_type,
                        const void* x_bf16, int batch, const int32_t* labels_coo, int nnz, float lr,
                        const uint32_t* seeds, int round_mode, int quantize_x, int saturate, void* kahan, int kahan_type,
                        int num_head, float weight_decay, float dropout_p, unsigned long long dropout_seed, void* grad_x_bf16,
                        float* grad_x_f32, float* loss_out, void* workspace, size_t workspace_bytes, void* stream_) {
  if (!chunk_ptrs || !x_bf16 || !workspace || !grad_x_bf16 || (nnz > 0 && !labels_coo)) return XMC_ERR_NULL;
  if (kahan_type < 0 || kahan_type > 2 || (kahan_type != 0 && (weight_type != W_E4M3 || !kahan))) return XMC_ERR_MODE;
  if (kahan_type != 0 && (num_head < 0 || num_head > rows_per_chunk || !aligned16(kahan))) return XMC_ERR_SHAPE;
  if (kahan_type == 0) num_head = 0;
  if (batch <= 0 || batch > T_HALVES * BP) return XMC_ERR_SHAPE;
  if (rows_per_chunk <= 0 || rows_last_chunk <= 0 || rows_last_chunk > rows_per_chunk) return XMC_ERR_SHAPE;
  if (num_chunks <= 0 || num_chunks > MAX_CHUNKS) return XMC_ERR_RANGE;
  // a sort key keeps 24 bits for the label: larger label spaces are taken in segments of whole chunks, each with its own
  // sorted list of the positives that fall into it and labels counted from the segment's first
  if (rows_per_chunk >= (1 << 24) - 1 || (long long)num_chunks * rows_per_chunk > 0x7FFFFFFFLL) return XMC_ERR_RANGE;
  if (nnz < 0 || nnz > MAX_POS) return XMC_ERR_RANGE;
  if (weight_type != W_E4M3 && weight_type != W_BF16) return XMC_ERR_MODE;
  if (round_mode != XMC_ROUND_RTN && round_mode != XMC_ROUND_SR_PHILOX && round_mode != XMC_ROUND_SR_FAST) return XMC_ERR_MODE;
  if (round_mode != XMC_ROUND_RTN && !seeds) return XMC_ERR_NULL;
  if (!(weight_decay >= 0.f) || !(dropout_p >= 0.f) || !(dropout_p < 1.f)) return XMC_ERR_SHAPE;
  if (kahan_type != 0 && (weight_decay != 0.f || dropout_p != 0.f)) return XMC_ERR_MODE;   // the head-Kahan layer has neither
  const DropoutParams dp = {dropout_p, 1.0f - dropout_p, (unsigned)(dropout_seed & 0xFFFFFFFFull), (unsigned)(dropout_seed >> 32)};
  const float wd = weight_decay;
  for (int c = 0; c < num_chunks; c++) {
    if (!chunk_ptrs[c]) return XMC_ERR_NULL;
    if (!aligned16(chunk_ptrs[c])) return XMC_ERR_ALIGN;
  }
  if (!aligned16(x_bf16) || ((uintptr_t)workspace & 255) != 0 || ((uintptr_t)labels_coo & 7) != 0) return XMC_ERR_ALIGN;
  if (workspace_bytes < xmc_tiled_workspace_bytes_ex(num_chunks, rows_per_chunk, batch, DD)) return XMC_ERR_WORKSPACE;
  DeviceInfo di = device_info();
  if (di.ok != 1) return XMC_ERR_DEVICE;
  hipStream_t stream = (hipStream_t)stream_;
  unsigned char* ws = (unsigned char*)workspace;

  const int rows_pad = (rows_per_chunk + TL - 1) / TL * TL;
  const int tiles_per_chunk = rows_pad / TL;
  const int num_tiles = num_chunks * tiles_per_chunk;
  const int halves = tiled_halves(batch), pairs = (halves + 1) / 2;   // halves beyond the batch are zero rows of X
  // Several chunks per launch where they lie one behind the other in memory (the bf16 layer's views of one tensor) and
  // the compensated head is not in play; the buffers are sized for that many rows either way.
  const int group_max = tiled_group(num_chunks, rows_per_chunk);
  int group = kahan_type != 0 ? 1 : group_max;
  for (int c = 0; c + 1 < num_chunks && group > 1; c++)
    if ((const unsigned char*)chunk_ptrs[c + 1] != (const unsigned char*)chunk_ptrs[c] + (size_t)rows_per_chunk * DD * (weight_type == W_BF16 ? 2 : 1))
      group = 1;
  const size_t rows_buf = (size_t)group_max * rows_pad;               // rows the G buffers hold
  const TiledLayout lay = tiled_layout(halves, DD);
  unsigned short* xb = (unsigned short*)(ws + lay.xb);
  unsigned short* xT = (unsigned short*)(ws + lay.xt);
  unsigned* keys = (unsigned*)(ws + lay.keys);
  float* gx_total = (float*)(ws + lay.gx);
  floatx4* partial = (floatx4*)(ws + lay.part);
  const size_t g_half = 2 * rows_buf * BP;    // elements of one half's G and G^T
  unsigned short* glb = (unsigned short*)(ws + lay.g);
  unsigned short* gbl = glb + rows_buf * BP;
  int* tile_ptr = (int*)(glb + halves * g_half);
  const size_t tp_stride = (size_t)(num_tiles + 1 + 63) / 64 * 64;   // entries of one pair's tile_ptr
  float* loss_part = (float*)(tile_ptr + pairs * tp_stride);         // one share per sub-tile of 32 rows
  int n_pad = 0;
  if (nnz > 0) { n_pad = 64; while (n_pad < nnz) n_pad <<= 1; }

  // chunks per segment of the label space: a multiple of the launch group, fewer than 2^24 - 1 labels
  int seg_chunks = ((1 << 24) - 2) / rows_per_chunk / group * group;
  if (seg_chunks < group) return XMC_ERR_RANGE;
  // true-FP8 arithmetic with two or four batch halves: FP8 matrix products, the logits of a pair of halves in one pass
  const bool fp8_logits = weight_type == W_E4M3 && quantize_x && halves >= 2 && !loss_out;
  // e4m3 weights, two batch halves, no compensated head: the feature-split update kernel (X^T in registers)
  const bool split_update = weight_type == W_E4M3 && halves == 2 && kahan_type == 0 && DD == D;
  tiled_prep_x_kernel<DD><<<(halves * BP * DD + 255) / 256, 256, 0, stream>>>((const unsigned short*)x_bf16, batch, halves, quantize_x,
                                                                        fp8_logits ? 1 : 0, split_update ? 1 : 0, xb, xT, gx_total,
                                                                        loss_part, loss_out ? 2 * num_tiles : 0, dp);
  for (int c = 0; c < num_chunks; c += group) {
    const int seg0 = c / seg_chunks * seg_chunks;   // first chunk of the segment
    if (c == seg0) {
      // the segment's positives of every 256 batch rows as their own sorted list (the key keeps eight bits for the row),
      // and the first key of each of its tiles
      const int seg_n = seg0 + seg_chunks <= num_chunks ? seg_chunks : num_chunks - seg0;
      for (int pr = 0; pr < pairs; pr++) {
        if (n_pad > 0)
          quad_sort_kernel<<<n_pad / 64, 256, (size_t)(n_pad + 256) * 4, stream>>>(labels_coo, nnz, n_pad, batch, 256 * pr,
                                                                                seg0 * rows_per_chunk, seg_n * rows_per_chunk,
                                                                                keys + (size_t)pr * MAX_POS, nullptr);
        tile_ptr_kernel<<<(seg_n * tiles_per_chunk + 1 + 255) / 256, 256, 0, stream>>>(
            keys + (size_t)pr * MAX_POS, n_pad, rows_per_chunk, tiles_per_chunk, seg_n * tiles_per_chunk,
            tile_ptr + pr * tp_stride + seg0 * tiles_per_chunk);
      }
    }
    void* w = chunk_ptrs[c];
    const int nch = c + group <= num_chunks ? group : num_chunks - c;                       // chunks of this launch
    const int rows = (nch - 1) * rows_per_chunk + (c + nch == num_chunks ? rows_last_chunk : rows_per_chunk);
    const int rp = (rows + TL - 1) / TL * TL;           // padded rows of this launch (the G buffers use the stride rows_buf)
    const int tiles = rp / TL;
    const unsigned label0 = (unsigned)c * (unsigned)rows_per_chunk;                  // global: the fast rounding's random words
    const unsigned label0_seg = (unsigned)(c - seg0) * (unsigned)rows_per_chunk;     // within the segment: the sorted keys
    TiledSeeds sd;
    for (int k = 0; k < T_GROUP; k++)
      sd.s[k] = seeds && k < nch ? (round_mode == XMC_ROUND_SR_FAST ? fast_seed(seeds[c + k]) : seeds[c + k]) : 0u;
    const int nh = c == 0 ? num_head : 0;   // the compensated head lives in chunk 0 (chunked_head_kahan_fp8xmc_clf.py:127)
    // label ranges of the grad_X kernel: T_SPLITS slots shared by the launch's chunks, none across a chunk boundary
    const int cs = nch > 1 ? rows_per_chunk : rp;       // rows of a chunk as the kernels see them
    const int spc_max = T_SPLITS / nch;
    int range = (cs + spc_max - 1) / spc_max;
    range = (range + TL - 1) / TL * TL;
    const int spc = (cs + range - 1) / range;            // slots (and at most ranges) per chunk
    const int splits = nch * spc;
    float* lp = loss_part + 2 * c * tiles_per_chunk;
    for (int hh = 0; fp8_logits && hh < halves; hh += 2) {
      const int nsub = 2 * tiles, lgrid = nsub < di.cus ? nsub : di.cus;
      tiled_logits_fp8_kernel<DD><<<lgrid, 512, TlgGeom<W_E4M3, DD>::LDS, stream>>>(
          w, rows, nsub, (const unsigned char*)xb + (size_t)hh * BP * DD, keys + (size_t)(hh >> 1) * MAX_POS,
          tile_ptr + (hh >> 1) * tp_stride + c * tiles_per_chunk, label0_seg, glb + hh * g_half, gbl + hh * g_half, g_half);
    }
    for (int hh = 0; !fp8_logits && hh < halves; hh++) {
      unsigned short* gl = glb + hh * g_half;
      unsigned short* gb = gbl + hh * g_half;
      const unsigned short* xh = xb + (size_t)hh * BP * DD;
      const unsigned* kh = keys + (size_t)(hh >> 1) * MAX_POS;                       // this half's pair: its keys,
      const int* tp = tile_ptr + (hh >> 1) * tp_stride + c * tiles_per_chunk;       // its tile_ptr,
      const unsigned brow0 = (unsigned)((hh & 1) * BP);                             // the half's first row within the pair
      const int pbatch = batch - 256 * (hh >> 1);                                   // and the batch rows the pair has
      const int nsub = 2 * tiles;                                   // sub-tiles of 32 label rows
      const int lgrid = nsub < di.cus ? nsub : di.cus;              // persistent: one workgroup per compute unit
      if (weight_type == W_BF16) {
        if (loss_out) tiled_logits_kernel<W_BF16, true, DD><<<lgrid, 512, TlgGeom<W_BF16, DD>::LDS, stream>>>(w, rows, nsub, xh, kh, tp, label0_seg, gl, gb, pbatch, brow0, lp);
        else tiled_logits_kernel<W_BF16, false, DD><<<lgrid, 512, TlgGeom<W_BF16, DD>::LDS, stream>>>(w, rows, nsub, xh, kh, tp, label0_seg, gl, gb, pbatch, brow0, lp);
      } else {
        if (loss_out) tiled_logits_kernel<W_E4M3, true, DD><<<lgrid, 512, TlgGeom<W_E4M3, DD>::LDS, stream>>>(w, rows, nsub, xh, kh, tp, label0_seg, gl, gb, pbatch, brow0, lp);
        else tiled_logits_kernel<W_E4M3, false, DD><<<lgrid, 512, TlgGeom<W_E4M3, DD>::LDS, stream>>>(w, rows, nsub, xh, kh, tp, label0_seg, gl, gb, pbatch, brow0, lp);
      }
    }
    // grad_X of the launch's chunks: one pass over W per pair of batch halves, then the fixed-order sums per half
    const size_t part_half = (size_t)T_SPLITS * 4 * (8 * (DD / 256)) * 256;   // floatx4 elements of one half's partials
    const int ggrid = 4 * ((splits + 7) / 8 * 8);
    for (int h0 = 0; h0 < halves; h0 += 2) {
      const unsigned short* gsrc = gbl + h0 * g_half;
      floatx4* pdst = partial + h0 * part_half;
      if (weight_type == W_BF16) {
        if (halves == 1) tiled_gradx_kernel<W_BF16, 1, DD><<<ggrid, 512, TgxGeom<W_BF16, 1, DD>::LDS, stream>>>(w, rows, (int)rows_buf, rp, range, cs, spc, gsrc, g_half, pdst, part_half);
        else tiled_gradx_kernel<W_BF16, 2, DD><<<ggrid, 512, TgxGeom<W_BF16, 2, DD>::LDS, stream>>>(w, rows, (int)rows_buf, rp, range, cs, spc, gsrc, g_half, pdst, part_half);
      } else {
        if (halves == 1) tiled_gradx_kernel<W_E4M3, 1, DD><<<ggrid, 512, TgxGeom<W_E4M3, 1, DD>::LDS, stream>>>(w, rows, (int)rows_buf, rp, range, cs, spc, gsrc, g_half, pdst, part_half);
        else tiled_gradx_kernel<W_E4M3, 2, DD><<<ggrid, 512, TgxGeom<W_E4M3, 2, DD>::LDS, stream>>>(w, rows, (int)rows_buf, rp, range, cs, spc, gsrc, g_half, pdst, part_half);
      }
    }
    const int nsub_u = tup_threads(halves) / 256;    // tiles a workgroup of the update kernel works on at a time
    const int ugroups = (tiles + TUP_TILES * nsub_u - 1) / (TUP_TILES * nsub_u);   // rounded up to eight: see the kernel's index map
    const int ugrid = tred_waves(DD) * halves / (tup_threads(halves) / 64) + ((DD / 64) / tup_csteps(halves, DD)) * ((ugroups + 7) / 8 * 8);
#define XMC_LAUNCH_UPDATE_K(WTYPE, RMODE, HV, KH)                                                                               \
  tiled_update_kernel<WTYPE, RMODE, HV, KH, DD><<<ugrid, tup_threads(HV), (size_t)tup_lds_bytes(HV, DD), stream>>>(                           \
      w, rows, tiles, glb, g_half, xT, lr, wd, sd, cs, saturate, kahan, kahan_type, nh, label0, partial, part_half, nch, spc, range, rp,  \
      weight_type == W_BF16 ? 1 : 0, gx_total)
#define XMC_LAUNCH_UPDATE_H(WTYPE, RMODE, KH)                                                                                  \
  do {                                                                                                                         \
    if (halves == 1) XMC_LAUNCH_UPDATE_K(WTYPE, RMODE, 1, KH);                                                                 \
    else if (halves == 2) XMC_LAUNCH_UPDATE_K(WTYPE, RMODE, 2, KH);                                                            \
    else XMC_LAUNCH_UPDATE_K(WTYPE, RMODE, 4, KH);                                                                             \
  } while (0)
    const bool with_head = kahan_type != 0 && nh > 0;   // only chunk 0 of the head-Kahan layer
    if (split_update) {
      int streams = (tiles + 7) / 8 * 8;
      streams = streams < 128 ? streams : 128;           // two workgroups per compute unit, four per stream
      const int grid2 = tred_waves(D) * 2 / 4 + 4 * streams;
#define XMC_LAUNCH_UPDATE2(RMODE)                                                                                              \
  tiled_update2_kernel<RMODE><<<grid2, 256, 2 * TU2_GBUF, stream>>>(w, rows, tiles, glb, g_half, (const bf16x8*)xT, lr, wd, sd, cs, saturate, \
                                                                    label0, partial, part_half, nch, spc, range, rp, gx_total)
      if (round_mode == XMC_ROUND_RTN) XMC_LAUNCH_UPDATE2(ROUND_RTN);
      else if (round_mode == XMC_ROUND_SR_FAST) XMC_LAUNCH_UPDATE2(ROUND_SR_FAST);
      else XMC_LAUNCH_UPDATE2(ROUND_SR_PHILOX);
#undef XMC_LAUNCH_UPDATE2
    } else if (weight_type == W_BF16) {
      if (round_mode == XMC_ROUND_RTN) XMC_LAUNCH_UPDATE_H(W_BF16, ROUND_RTN, false);
      else if (round_mode == XMC_ROUND_SR_FAST) XMC_LAUNCH_UPDATE_H(W_BF16, ROUND_SR_FAST, false);
      else XMC_LAUNCH_UPDATE_H(W_BF16, ROUND_SR_PHILOX, false);
    } else if (with_head) {
      if (round_mode == XMC_ROUND_RTN) XMC_LAUNCH_UPDATE_H(W_E4M3, ROUND_RTN, true);
      else if (round_mode == XMC_ROUND_SR_FAST) XMC_LAUNCH_UPDATE_H(W_E4M3, ROUND_SR_FAST, true);
      else XMC_LAUNCH_UPDATE_H(W_E4M3, ROUND_SR_PHILOX, true);
    } else {
      if (round_mode == XMC_ROUND_RTN) XMC_LAUNCH_UPDATE_H(W_E4M3, ROUND_RTN, false);
      else if (round_mode == XMC_ROUND_SR_FAST) XMC_LAUNCH_UPDATE_H(W_E4M3, ROUND_SR_FAST, false);
      else XMC_LAUNCH_UPDATE_H(W_E4M3, ROUND_SR_PHILOX, false);
    }
#undef XMC_LAUNCH_UPDATE_H
#undef XMC_LAUNCH_UPDATE_K
  }
  tiled_finalize_kernel<DD><<<(batch * DD + 255) / 256, 256, 0, stream>>>(gx_total, batch, (unsigned short*)grad_x_bf16, grad_x_f32, dp);
  if (loss_out) tiled_loss_kernel<<<1, 256, 0, stream>>>(loss_part, 2 * num_tiles, loss_out);
  return launch_status();
}

extern "C" {

int xmc_tiled_step_ex(void* const* chunk_ptrs, int num_chunks, int rows_per_chunk, int rows_last_chunk, int weight_type,
                      const void* x_bf16, int batch, int features, const int32_t* labels_coo, int nnz, float lr,
                      const uint32_t* seeds, int round_mode, int quantize_x, int saturate, void* kahan, int kahan_type,
                      int num_head, float weight_decay, float dropout_p, unsigned long long dropout_seed, void* grad_x_bf16,
                      float* grad_x_f32, float* loss_out, void* workspace, size_t workspace_bytes, void* stream_) {
  if (features == D)
    return tiled_step_t<D>(chunk_ptrs, num_chunks, rows_per_chunk, rows_last_chunk, weight_type, x_bf16, batch, labels_coo, nnz, lr, seeds,
                           round_mode, quantize_x, saturate, kahan, kahan_type, num_head, weight_decay, dropout_p, dropout_seed,
                           grad_x_bf16, grad_x_f32, loss_out, workspace, workspace_bytes, stream_);
  if (features == 1024)
    return tiled_step_t<1024>(chunk_ptrs, num_chunks, rows_per_chunk, rows_last_chunk, weight_type, x_bf16, batch, labels_coo, nnz, lr,
                              seeds, round_mode, quantize_x, saturate, kahan, kahan_type, num_head, weight_decay, dropout_p,
                              dropout_seed, grad_x_bf16, grad_x_f32, loss_out, workspace, workspace_bytes, stream_);
  return XMC_ERR_SHAPE;
}

int xmc_copy_probe(void* dst, const void* src, size_t bytes, void* stream_) {
  if (!dst || !src) return XMC_ERR_NULL;
  if (!aligned16(dst) || !aligned16(src) || bytes % 16 != 0) return XMC_ERR_ALIGN;
  if (bytes == 0) return XMC_OK;
  copy_probe_kernel<<<2048, 256, 0, (hipStream_t)stream_>>>((const uint4*)src, (uint4*)dst, bytes / 16);
  return launch_status();
}

int xmc_step_error_word(const void* workspace, int num_chunks, int rows_per_chunk, void* stream_) {
  (void)num_chunks; (void)rows_per_chunk;
  if (!workspace) return XMC_ERR_NULL;
  int word = 0;
  if (hipMemcpyAsync(&word, (const unsigned char*)workspace + xmc_step_error_offset(), 4, hipMemcpyDeviceToHost,
                     (hipStream_t)stream_) != hipSuccess) return XMC_ERR_LAUNCH;
  if (hipStreamSynchronize((hipStream_t)stream_) != hipSuccess) return XMC_ERR_LAUNCH;
  return word;
}

size_t xmc_step_error_offset(void) { return WS_FLAGS + (size_t)QF_ERR * 4; }

size_t xmc_step_sticky_error_offset(void) { return WS_FLAGS + (size_t)QF_STICKY * 4; }

int xmc_step_workgroups(void) {
  DeviceInfo di = device_info();
  if (di.ok != 1) return XMC_ERR_DEVICE;
  return (di.cus < MAX_WG ? di.cus : MAX_WG) / 32 * 32;
}

int xmc_step_xcc_ids(const void* workspace, int32_t* ids_host, int count, void* stream_) {
  if (!workspace || !ids_host) return XMC_ERR_NULL;
  if (count <= 0 || count > MAX_WG) return XMC_ERR_RANGE;
  if (hipMemcpyAsync(ids_host, (const unsigned char*)workspace + WS_FLAGS + (size_t)QF_XCC * 4, (size_t)count * 4,
                     hipMemcpyDeviceToHost, (hipStream_t)stream_) != hipSuccess) return XMC_ERR_LAUNCH;
  if (hipStreamSynchronize((hipStream_t)stream_) != hipSuccess) return XMC_ERR_LAUNCH;
  return XMC_OK;
}

int xmc_quad_placement_check(const int32_t* xcc_ids_host, int num_workgroups) {
  if (!xcc_ids_host) return XMC_ERR_NULL;
  if (num_workgroups < 32 || num_workgroups > MAX_WG || num_workgroups % 32 != 0) return XMC_ERR_RANGE;
  int bad = 0;
  for (int q = 0; q < num_workgroups / 4; q++) bad += quad_xcc_mismatch(xcc_ids_host, q) ? 1 : 0;
  return bad;
}

}  // extern "C"
