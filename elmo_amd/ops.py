"""Tensor-level wrappers over the C ABI.  torch supplies device memory and the current stream only."""
import ctypes

import torch

from . import _lib

FEATURES = 768
MAX_BATCH = 128          # fused step
MAX_BATCH_TILED = 512    # three-kernel step: up to four halves of 128 rows


def _stream_ptr():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _chunk_array(chunks):
    arr = (ctypes.c_void_p * len(chunks))()
    rows = chunks[0].shape[0]
    for i, c in enumerate(chunks):
        assert c.is_cuda and c.is_contiguous(), "weight chunks must be contiguous device tensors"
        assert c.dtype in (torch.float8_e4m3fn, torch.uint8) and c.shape == (rows, FEATURES), \
            "weight chunks must be equal-sized [rows, 768] e4m3fn tensors"
        arr[i] = c.data_ptr()
    return arr, rows


def workspace_bytes(num_chunks, rows_per_chunk):
    n = _lib.load().xmc_workspace_bytes(num_chunks, rows_per_chunk)
    if n == 0:
        raise _lib.XmcError("unsupported chunk geometry")
    return n


def alloc_workspace(num_chunks, rows_per_chunk, device):
    ws = torch.empty(workspace_bytes(num_chunks, rows_per_chunk), dtype=torch.uint8, device=device)
    # the sticky error word is only ever OR-ed into by the kernels: it starts at zero
    off = step_sticky_error_offset()
    ws[off:off + 4].zero_()
    return ws


def fp8_step(chunks, x, labels, lr, seeds=None, round_mode="rtn", scale_w=1.0, scale_x=1.0, workspace=None,
             grad_out=None, want_f32=False, weight_decay=0.0, dropout_p=0.0, dropout_seed=0):
    """One fused training step (reference: chunked_fp8xmc_clf.py:81-123).  Updates `chunks` in place and returns
    grad_input (bf16 [B, 768]) or (grad_input, grad_x_fp32) when want_f32.  weight_decay, dropout_p, dropout_seed: the
    additions of xmc_fp8_step_ex (decay inside the update, dropout of the embedding inside the step); zero = the
    reference's step."""
    lib = _lib.load()
    assert x.is_cuda and x.dtype == torch.bfloat16 and x.is_contiguous() and x.dim() == 2
    assert labels.is_cuda and labels.dtype == torch.int32 and labels.is_contiguous()
    assert labels.dim() == 2 and labels.shape[1] == 2
    batch, feat = x.shape
    arr, rows = _chunk_array(chunks)
    nc = len(chunks)
    if workspace is None:
        workspace = alloc_workspace(nc, rows, x.device)
    if grad_out is None:
        grad_out = torch.empty(batch, feat, dtype=torch.bfloat16, device=x.device)
    gf = torch.empty(batch, feat, dtype=torch.float32, device=x.device) if want_f32 else None
    sarr = None
    if seeds is not None:
        sarr = (ctypes.c_uint32 * nc)(*[int(s) & 0xFFFFFFFF for s in seeds])
    if weight_decay == 0.0 and dropout_p == 0.0:
        st = lib.xmc_fp8_step(arr, nc, rows, x.data_ptr(), batch, feat, labels.data_ptr() if labels.numel() else None,
                              labels.shape[0], float(lr), sarr, _lib.ROUND_MODES[round_mode], float(scale_w),
                              float(scale_x), grad_out.data_ptr(), gf.data_ptr() if gf is not None else None,
                              workspace.data_ptr(), workspace.numel(), _stream_ptr())
    else:
        st = lib.xmc_fp8_step_ex(arr, nc, rows, x.data_ptr(), batch, feat, labels.data_ptr() if labels.numel() else None,
                                 labels.shape[0], float(lr), sarr, _lib.ROUND_MODES[round_mode], float(scale_w),
                                 float(scale_x), float(weight_decay), float(dropout_p), int(dropout_seed) & 0xFFFFFFFFFFFFFFFF,
                                 grad_out.data_ptr(), gf.data_ptr() if gf is not None else None,
                                 workspace.data_ptr(), workspace.numel(), _stream_ptr())
    _lib.check(st, "xmc_fp8_step")
    return (grad_out, gf) if want_f32 else grad_out


def fp8_kahan_step(chunks, kahan, num_head, x, labels, lr, seeds=None, round_mode="rtn", workspace=None, grad_out=None,
                   want_f32=False):
    """One fused step of the head-Kahan layer (reference: chunked_head_kahan_fp8xmc_clf.py:95-133): as fp8_step, and the
    first num_head rows of chunk 0 are updated with the compensation buffer `kahan` ([num_head, 768] bf16 or
    float8_e5m2, updated in place)."""
    lib = _lib.load()
    assert x.is_cuda and x.dtype == torch.bfloat16 and x.is_contiguous() and x.dim() == 2
    assert labels.is_cuda and labels.dtype == torch.int32 and labels.is_contiguous()
    assert labels.dim() == 2 and labels.shape[1] == 2
    batch, feat = x.shape
    arr, rows = _chunk_array(chunks)
    nc = len(chunks)
    assert kahan.is_cuda and kahan.is_contiguous() and kahan.shape == (num_head, FEATURES)
    assert kahan.dtype in (torch.bfloat16, torch.float8_e5m2) and 0 < num_head <= rows
    if workspace is None:
        workspace = alloc_workspace(nc, rows, x.device)
    if grad_out is None:
        grad_out = torch.empty(batch, feat, dtype=torch.bfloat16, device=x.device)
    gf = torch.empty(batch, feat, dtype=torch.float32, device=x.device) if want_f32 else None
    sarr = None
    if seeds is not None:
        sarr = (ctypes.c_uint32 * nc)(*[int(s) & 0xFFFFFFFF for s in seeds])
    st = lib.xmc_fp8_kahan_step(arr, nc, rows, x.data_ptr(), batch, feat, labels.data_ptr() if labels.numel() else None,
                                labels.shape[0], float(lr), sarr, _lib.ROUND_MODES[round_mode], kahan.data_ptr(),
                                1 if kahan.dtype == torch.bfloat16 else 2, int(num_head), grad_out.data_ptr(),
                                gf.data_ptr() if gf is not None else None, workspace.data_ptr(), workspace.numel(),
                                _stream_ptr())
    _lib.check(st, "xmc_fp8_kahan_step")
    return (grad_out, gf) if want_f32 else grad_out


def fp8_forward(chunks, x, num_labels, scale_w=1.0, scale_x=1.0, workspace=None):
    """Inference logits [B, num_labels] bf16 (reference: chunked_fp8xmc_clf.py:45-60).  Any batch size: rows are
    processed in slices of at most 128, the last one padded to a multiple of 16."""
    lib = _lib.load()
    assert x.is_cuda and x.dim() == 2 and x.shape[1] == FEATURES
    xb = x.to(torch.bfloat16).contiguous()      # exact for e4m3 input
    arr, rows = _chunk_array(chunks)
    nc = len(chunks)
    if workspace is None:
        workspace = alloc_workspace(nc, rows, x.device)
    total = xb.shape[0]
    # like the reference, which returns outlogit[:, :num_labels] of the concatenated chunk outputs, the result is a
    # view of a [B, num_chunks * rows] buffer: rows start on 32-byte boundaries, which the kernel's stores want
    stride = nc * rows
    out = torch.empty(total, stride, dtype=torch.bfloat16, device=x.device)
    for lo in range(0, total, MAX_BATCH):
        hi = min(lo + MAX_BATCH, total)
        n = hi - lo
        npad = (n + 15) // 16 * 16
        xs = xb[lo:hi]
        if npad != n:
            xs = torch.cat([xs, torch.zeros(npad - n, FEATURES, dtype=xb.dtype, device=xb.device)])
            tmp = torch.empty(npad, stride, dtype=torch.bfloat16, device=x.device)
        else:
            tmp = out[lo:hi]
        st = lib.xmc_fp8_forward(arr, nc, rows, xs.data_ptr(), npad, FEATURES, float(scale_w), float(scale_x),
                                 tmp.data_ptr(), stride, num_labels, workspace.data_ptr(), workspace.numel(),
                                 _stream_ptr())
        _lib.check(st, "xmc_fp8_forward")
        if npad != n:
            out[lo:hi, :num_labels] = tmp[:n, :num_labels]
    return out[:, :num_labels]


TOPK_MAX = 128


def topk_scratch_bytes(rows_per_chunk):
    """Size of the scratch buffer fp8_forward_topk works in (the logits of one chunk and the running lists)."""
    n = _lib.load().xmc_topk_scratch_bytes(rows_per_chunk)
    assert n > 0, "rows_per_chunk must be a positive multiple of 16"
    return n


def topk_fused_scratch_bytes():
    return _lib.load().xmc_topk_fused_scratch_bytes()


def fp8_forward_topk(chunks, x, num_labels, k, scale_w=1.0, scale_x=1.0, workspace=None, scratch=None, fused=True,
                     fused_scratch=None, defer_check=False):
    """values, indices = top-k of the inference logits per row (what evaluate.py:158-159 computes as
    xfc_forward(embed).topk(k)), without the dense [B, num_labels] matrix.  values bf16 [B, k] descending, indices int64
    [B, k]; equal values are ordered by ascending label id.

    fused=True takes the two-pass kernels (selection inside the logits kernel, < 1 MB of scratch) where the label count
    allows and reads their status word back: a call that reports an overflowing candidate list (massive ties) is
    repeated on the general path, as are shapes the fused path does not take.  defer_check=True skips that read-back
    (no synchronisation) and returns (values, indices, status) with status an int32 device tensor, one word per slice
    of 128 rows, that the caller has to find zero before using the result."""
    lib = _lib.load()
    assert x.is_cuda and x.dim() == 2 and x.shape[1] == FEATURES
    assert 0 < k <= TOPK_MAX and k <= num_labels, "k must be between 1 and 128"
    xb = x.to(torch.bfloat16).contiguous()      # exact for e4m3 input
    arr, rows = _chunk_array(chunks)
    nc = len(chunks)
    if workspace is None:
        workspace = alloc_workspace(nc, rows, x.device)
    total = xb.shape[0]
    vals = torch.empty(total, k, dtype=torch.bfloat16, device=x.device)
    idx = torch.empty(total, k, dtype=torch.int64, device=x.device)
    nslices = (total + MAX_BATCH - 1) // MAX_BATCH
    status = torch.empty(nslices, dtype=torch.int32, device=x.device)      # every word is written below
    for si, lo in enumerate(range(0, total, MAX_BATCH)):
        hi = min(lo + MAX_BATCH, total)
        n = hi - lo
        npad = (n + 15) // 16 * 16
        xs = xb[lo:hi]
        if npad != n:
            # rows that pad the batch to a multiple of 16 repeat the last row (rows of zeros would tie on every label
            # and overflow the two-pass path's candidate lists); their results are dropped below
            xs = torch.cat([xs, xs[-1:].expand(npad - n, FEATURES)])
            tv = torch.empty(npad, k, dtype=torch.bfloat16, device=x.device)
        else:
            tv = vals[lo:hi]                                               # written in place
        done = False
        if fused:
            need = lib.xmc_topk_fused_scratch_bytes()
            if fused_scratch is None or fused_scratch.numel() < need:
                fused_scratch = torch.empty(need, dtype=torch.uint8, device=x.device)
            ti = idx[lo:hi] if npad == n else torch.empty(npad, k, dtype=torch.int64, device=x.device)
            st = lib.xmc_fp8_forward_topk_fused(arr, nc, rows, xs.data_ptr(), npad, FEATURES, float(scale_w), float(scale_x),
                                                int(num_labels), int(k), tv.data_ptr(), ti.data_ptr(), 1, workspace.data_ptr(),
                                                workspace.numel(), fused_scratch.data_ptr(), fused_scratch.numel(),
                                                status[si:].data_ptr(), _stream_ptr())
            if st != _lib.XMC_ERR_RANGE:
                _lib.check(st, "xmc_fp8_forward_topk_fused")
                done = defer_check or int(status[si].item()) == 0
                if done and npad != n:
                    idx[lo:hi] = ti[:n]
        if not done:
            need = lib.xmc_topk_scratch_bytes(rows)
            if scratch is None or scratch.numel() < need:
                scratch = torch.empty(need, dtype=torch.uint8, device=x.device)
            ti = torch.empty(npad, k, dtype=torch.int32, device=x.device)
            st = lib.xmc_fp8_forward_topk(arr, nc, rows, xs.data_ptr(), npad, FEATURES, float(scale_w), float(scale_x),
                                          int(num_labels), int(k), tv.data_ptr(), ti.data_ptr(), workspace.data_ptr(),
                                          workspace.numel(), scratch.data_ptr(), scratch.numel(), _stream_ptr())
            _lib.check(st, "xmc_fp8_forward_topk")
            status[si] = 0
            idx[lo:hi] = ti[:n]
        if npad != n:
            vals[lo:hi] = tv[:n]
    if defer_check:
        return vals, idx, status
    return vals, idx


def dropout_quantize(x, p, seed):
    """e4m3 tensor of dropout(x) with Triton's random stream: the reference's prototype of dropout inside the FP8 GEMM's
    operand load (tma_gemm.py:7-13,34-38) as one pass over the embedding.  x: [M, K] bf16 or float8_e4m3fn, contiguous,
    K a multiple of 4; element (m, k) is kept when tl.rand(seed, m * K + k) > p and scaled by 1 / (1 - p)."""
    lib = _lib.load()
    assert x.is_cuda and x.dim() == 2 and x.is_contiguous()
    assert x.dtype in (torch.bfloat16, torch.float8_e4m3fn)
    out = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=x.device)
    st = lib.xmc_dropout_quantize(x.data_ptr(), 0 if x.dtype == torch.bfloat16 else 1, x.shape[0], x.shape[1], float(p),
                                  int(seed), out.data_ptr(), _stream_ptr())
    _lib.check(st, "xmc_dropout_quantize")
    return out


WEIGHT_TYPES = {"e4m3": 0, "bf16": 1}


TILED_FEATURES = (768, 1024)   # input widths of the three-kernel path


def tiled_workspace_bytes(num_chunks, rows_per_chunk, max_batch=MAX_BATCH, features=FEATURES):
    n = _lib.load().xmc_tiled_workspace_bytes_ex(num_chunks, rows_per_chunk, max_batch, features)
    if n == 0:
        raise _lib.XmcError("unsupported chunk geometry")
    return n


def alloc_tiled_workspace(num_chunks, rows_per_chunk, device, max_batch=MAX_BATCH, features=FEATURES):
    return torch.empty(tiled_workspace_bytes(num_chunks, rows_per_chunk, max_batch, features), dtype=torch.uint8,
                       device=device)


def tiled_step(chunk_views, rows_per_chunk, weight_type, x, labels, lr, seeds=None, round_mode="rtn", workspace=None,
               grad_out=None, want_f32=False, quantize_x=False, saturate=False, kahan=None, num_head=0, loss_out=None,
               weight_decay=0.0, dropout_p=0.0, dropout_seed=0):
    """One training step of the bf16 layer (chunked.py:76-133) or of the simulated-FP8 mode of the FP8 layer
    (chunked_fp8xmc_clf.py:98-99,110,115-116), three kernels per chunk.  `chunk_views` are contiguous [rows, d]
    tensors with d = 768 or 1024 (views of one weight tensor, or the FP8 layer's chunk parameters): all have rows_per_chunk rows except the
    last, which may be shorter.  Updated in place; returns grad_input (bf16) or (grad_input, grad_x_fp32).
    e4m3 weights: quantize_x / saturate select the true-FP8 arithmetic (logits from e4m3(X), saturating cast) instead of
    the simulated one; `kahan` ([num_head, d] bf16 or float8_e5m2, updated in place) turns on the head-Kahan update of
    the first num_head rows of chunk 0 (chunked_head_kahan_fp8xmc_clf.py:127-131).  `loss_out` (a float32 device tensor
    with one element) receives the summed binary cross entropy of the step's logits (what chunked.py:57-72 is written
    to compute).  weight_decay, dropout_p, dropout_seed: as in fp8_step."""
    lib = _lib.load()
    assert x.is_cuda and x.dtype == torch.bfloat16 and x.is_contiguous() and x.dim() == 2
    feats = x.shape[1]
    assert feats in TILED_FEATURES, "the three-kernel path is built for 768 and 1024 input features"
    ktype = 0
    if kahan is not None:
        assert weight_type == "e4m3" and kahan.is_cuda and kahan.is_contiguous() and kahan.shape == (num_head, feats)
        assert kahan.dtype in (torch.bfloat16, torch.float8_e5m2) and 0 < num_head <= rows_per_chunk
        ktype = 1 if kahan.dtype == torch.bfloat16 else 2
    assert labels.is_cuda and labels.dtype == torch.int32 and labels.is_contiguous()
    assert labels.dim() == 2 and labels.shape[1] == 2
    assert round_mode in ("rtn", "sr_philox", "sr_fast"), \
        "the tiled path rounds to nearest, with the reference's Philox recipe or with the fast hardware mode"
    wdt = (torch.bfloat16,) if weight_type == "bf16" else (torch.float8_e4m3fn, torch.uint8)
    nc = len(chunk_views)
    arr = (ctypes.c_void_p * nc)()
    for i, c in enumerate(chunk_views):
        assert c.is_cuda and c.is_contiguous() and c.dtype in wdt and c.dim() == 2 and c.shape[1] == feats
        assert c.shape[0] == rows_per_chunk or (i == nc - 1 and 0 < c.shape[0] <= rows_per_chunk)
        arr[i] = c.data_ptr()
    batch = x.shape[0]
    assert 0 < batch <= MAX_BATCH_TILED, "batch must be at most 512"
    if workspace is None or workspace.numel() < tiled_workspace_bytes(nc, rows_per_chunk, batch, feats):
        workspace = alloc_tiled_workspace(nc, rows_per_chunk, x.device, batch, feats)
    if grad_out is None:
        grad_out = torch.empty(batch, feats, dtype=torch.bfloat16, device=x.device)
    gf = torch.empty(batch, feats, dtype=torch.float32, device=x.device) if want_f32 else None
    sarr = None
    if seeds is not None:
        sarr = (ctypes.c_uint32 * nc)(*[int(s) & 0xFFFFFFFF for s in seeds])
    if loss_out is not None:
        assert loss_out.is_cuda and loss_out.dtype == torch.float32 and loss_out.numel() == 1
    st = lib.xmc_tiled_step_ex(arr, nc, rows_per_chunk, chunk_views[-1].shape[0], WEIGHT_TYPES[weight_type], x.data_ptr(),
                            batch, feats, labels.data_ptr() if labels.numel() else None, labels.shape[0], float(lr),
                            sarr, _lib.ROUND_MODES[round_mode], int(bool(quantize_x)), int(bool(saturate)),
                            kahan.data_ptr() if kahan is not None else None, ktype, int(num_head), float(weight_decay),
                            float(dropout_p), int(dropout_seed) & 0xFFFFFFFFFFFFFFFF, grad_out.data_ptr(),
                            gf.data_ptr() if gf is not None else None,
                            loss_out.data_ptr() if loss_out is not None else None, workspace.data_ptr(), workspace.numel(),
                            _stream_ptr())
    _lib.check(st, "xmc_tiled_step")
    return (grad_out, gf) if want_f32 else grad_out


def debug_spin_limit(limit):
    """Test aid: polls of a partner's counter before a workgroup of the fused step gives up (negative: the default);
    returns the previous value."""
    return int(_lib.load().xmc_debug_spin_limit(int(limit)))


def step_error_offset():
    """Byte offset of the fused step's error word (int32) inside its workspace."""
    return int(_lib.load().xmc_step_error_offset())


def step_sticky_error_offset():
    """Byte offset of the sticky error word (int32): the error words of all fused steps since it was last zeroed."""
    return int(_lib.load().xmc_step_sticky_error_offset())


def step_error_word(workspace, num_chunks, rows_per_chunk):
    return _lib.load().xmc_step_error_word(workspace.data_ptr(), num_chunks, rows_per_chunk, _stream_ptr())
