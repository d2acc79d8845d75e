"""Closed-form numpy restatement of one classifier step.  Test infrastructure only.

Follows (reference file:line)
  FP8 / simulated-FP8 layer  src/xmc_classifiers/chunked_fp8xmc_clf.py:15-43 (state), :81-126 (step)
  bf16 layer                 src/xmc_classifiers/chunked.py:17-46 (state), :76-133 (step)
  grad_X kernel              src/triton_kernels/matmul_kernel.py:204-239, :342-353
  fused update kernels       src/triton_kernels/fuse_kernel.py:63-131 (true FP8 / bf16), :134-199 (simulated FP8)
  elementwise SGD kernel     src/triton_kernels/stochastic_rounding_kernel.py:65-99

All GEMM accumulations are carried in float64 and rounded once to fp32: the reference accumulates in
fp32 in an unspecified order, so its result lies within a few fp32 ulps of this one.
Weights are passed as e4m3fn codes (uint8) or bf16 values held in fp32; X as bf16 values held in fp32.
"""
import numpy as np

from . import codecs as C


def fp8_padded_labels(num_labels, num_chunks):
    """chunked_fp8xmc_clf.py:26 -- always adds between 1 and 16*nc rows."""
    return num_labels + 16 * num_chunks - num_labels % (16 * num_chunks)


def sigmoid_f32(z):
    z = z.astype(np.float64)
    return (1.0 / (1.0 + np.exp(-z))).astype(np.float32)


def _positives_mask(labels, n_rows_batch, lo, hi):
    """Dense {0,1} mask [hi-lo, B] of the positives that fall in label range [lo, hi) -- set semantics
    (chunked_fp8xmc_clf.py:108 is a non-accumulating index_put)."""
    m = np.zeros((hi - lo, n_rows_batch), dtype=bool)
    if len(labels):
        rows = labels[:, 0].astype(np.int64)
        cols = labels[:, 1].astype(np.int64)
        sel = (cols >= lo) & (cols < hi)
        m[cols[sel] - lo, rows[sel]] = True
    return m


def _grad_from_logits(z_f32, posmask):
    """bf16 logits -> bf16 sigmoid -> minus one at positives (chunked_fp8xmc_clf.py:107-108)."""
    z = C.bf16_round(z_f32)
    s = C.bf16_round(sigmoid_f32(z))
    g = np.where(posmask, C.bf16_round(s - np.float32(1.0)), s).astype(np.float32)
    return z, g


def fp8_step(w_codes, x_bf16, labels, lr, *, seeds=None, sr_mode="rtn", simulated=False,
             scale_w=1.0, scale_x=1.0, rand_fn=None, return_parts=False, weight_decay=0.0, dropout_p=0.0, dropout_seed=0):
    """One step of the FP8 layer.

    w_codes : list of uint8 arrays [L_c, d] (e4m3fn codes), one per chunk (equal L_c)
    x_bf16  : fp32 array [B, d] holding bf16 values
    labels  : int array [Nb, 2] (row-in-batch, global label id in the padded index space)
    sr_mode : "rtn"        W' = e4m3_satfinite(T)                      (this build's parity mode)
              "reference"  W' = e4m3_satfinite(SR20(T; philox(seed_c, l*d+k)))   (fuse_kernel.py:102-113)
              "exact"      W' = true SR of T onto the e4m3 grid with rand_fn(chunk, offsets) -> uint32
    simulated: chunked_fp8xmc_clf.py:98-99,110,115-116 -- bf16 logits from un-quantised X, update via the
              bf16 temporary, torch cast back (NaN above 464).
    scale_w, scale_x: per-tensor scales (the reference fixes both at 1.0, :101-102): true weight =
              scale_w * code value, Xq = e4m3(X / scale_x).
    weight_decay, dropout_p, dropout_seed: this build's additions to the step (xmc_fp8_step_ex), not in the reference's
              FP8 layer: T = W - lr (A + weight_decay W) with the decayed gradient formed first, in fp32; the step runs
              on X' = codecs.dropout_bf16(X) and returns the gradient in front of the dropout.
    Returns (new_codes list, gx_fp32 [B,d], grad_input bf16-valued fp32 [B,d]).
    """
    x = np.ascontiguousarray(x_bf16, dtype=np.float32)
    keep = None
    if dropout_p > 0:
        x, keep = C.dropout_bf16(x, dropout_p, dropout_seed)
    B, d = x.shape
    nc = len(w_codes)
    Lc = w_codes[0].shape[0]
    lr32 = np.float32(lr)
    if simulated:
        xl = x.astype(np.float64)                                   # bf16 X, not quantised (:99)
    else:
        xq = C.e4m3_decode(C.e4m3_encode(x / np.float32(scale_x), saturate=True))   # (:101)
        xl = xq.astype(np.float64)
    x64 = x.astype(np.float64)
    gx = np.zeros((B, d), dtype=np.float64)
    new_codes, parts = [], []
    zscale = np.float32(scale_w) * (np.float32(1.0) if simulated else np.float32(scale_x))
    for c in range(nc):
        w = C.e4m3_decode(w_codes[c])                               # exact widening
        w64 = w.astype(np.float64)
        z = ((w64 @ xl.T).astype(np.float32) * zscale).astype(np.float32)            # [L_c, B]
        pos = _positives_mask(labels, B, c * Lc, (c + 1) * Lc)
        zb, g = _grad_from_logits(z, pos)
        g64 = g.astype(np.float64)
        gx += (g64.T @ w64) * float(scale_w)                        # pre-update W (:110-112)
        a = (g64 @ x64).astype(np.float32)                          # un-quantised bf16 X (:118)
        # fuse_kernel.py:102-105; evaluated with a single rounding (fused multiply-add): whether the compiled
        # kernel contracts `w - lr*acc` is unspecified and the two differ by at most one fp32 ulp
        lr_eff = np.float32(lr32 / np.float32(scale_w))
        if weight_decay:    # decayed gradient A + (wd * scale_w) * code: one fused multiply-add in fp32
            wd_eff = np.float32(np.float32(weight_decay) * np.float32(scale_w))
            a = (float(wd_eff) * w64 + a.astype(np.float64)).astype(np.float32)
        t = (w64 - float(lr_eff) * a.astype(np.float64)).astype(np.float32)
        offs = (np.arange(Lc, dtype=np.int64)[:, None] * d + np.arange(d, dtype=np.int64)[None, :])
        if sr_mode == "rtn":
            codes = C.e4m3_encode(t, saturate=not simulated)
        elif sr_mode == "reference":
            v = C.sr_add_mask(t, C.tl_randint(seeds[c], offs), 20)
            # simulated: value parked in bf16 (exact) then torch cast (:116); true FP8: satfinite cast
            codes = C.e4m3_encode(v, saturate=not simulated)
        elif sr_mode == "exact":
            codes = C.sr_e4m3_exact(t, rand_fn(c, offs))
        else:
            raise ValueError(sr_mode)
        new_codes.append(codes)
        if return_parts:
            parts.append(dict(z=zb, g=g, a=a, t=t))
    gx32 = gx.astype(np.float32)
    if keep is not None:
        gx32 = C.dropout_backward(gx32, keep, dropout_p)
    out = (new_codes, gx32, C.bf16_round(gx32))
    return out + (parts,) if return_parts else out


def fp8_kahan_step(w_codes, kahan, x_bf16, labels, lr, num_head, *, kahan_type="bf16", seeds=None, sr_mode="rtn",
                   rand_fn=None):
    """One step of the head-Kahan FP8 layer (chunked_head_kahan_fp8xmc_clf.py:95-133; fuse_kernel.py:202-262), true FP8.

    Logits, G and grad_X exactly as fp8_step.  Update of chunk 0 (:127-131): rows [0, num_head) carry a compensation
    buffer `kahan` [num_head, d] (bf16 values or e5m2 codes):
        w  = (f32(W) + f32(k)) - lr*A          (two fp32 roundings, the second one fused)
        Wq = e4m3_sat(SR20(w))  or e4m3_sat(w) in "rtn" mode
        k' = cast( ((f32(k) + f32(W)) - f32(Wq)) - lr*A )
    with random offsets row*d + col; the remaining rows of chunk 0 are updated by a call on the sliced tensors, so
    their offsets restart at zero: (row - num_head)*d + col.  Other chunks as in fp8_step.
    sr_mode "exact" (this build's fast mode, not in the reference): exact stochastic rounding on the e4m3 grid with the
    words rand_fn(chunk, row_in_chunk * d + col), rows counted from the chunk's start everywhere.
    Returns (new_codes list, new_kahan, gx_fp32, grad_input)."""
    x = np.ascontiguousarray(x_bf16, dtype=np.float32)
    B, d = x.shape
    nc, Lc = len(w_codes), w_codes[0].shape[0]
    assert 0 <= num_head <= Lc
    lr64 = float(np.float32(lr))
    xq64 = C.e4m3_decode(C.e4m3_encode(x, saturate=True)).astype(np.float64)
    x64 = x.astype(np.float64)
    gx = np.zeros((B, d), dtype=np.float64)
    k_old = (C.e5m2_decode(kahan) if kahan_type == "e5m2" else np.asarray(kahan, dtype=np.float32)).astype(np.float32)
    new_codes, new_kahan = [], None

    def rnd(t, seed, offs, c=0, row0=0):
        if sr_mode == "rtn":
            return C.e4m3_encode(t, saturate=True)
        if sr_mode == "exact":
            return C.sr_e4m3_exact(t, rand_fn(c, offs + row0 * d))
        return C.e4m3_encode(C.sr_add_mask(t, C.tl_randint(seed, offs), 20), saturate=True)

    for c in range(nc):
        w = C.e4m3_decode(w_codes[c])
        w64 = w.astype(np.float64)
        z = (w64 @ xq64.T).astype(np.float32)
        pos = _positives_mask(labels, B, c * Lc, (c + 1) * Lc)
        _, g = _grad_from_logits(z, pos)
        g64 = g.astype(np.float64)
        gx += g64.T @ w64
        a = (g64 @ x64).astype(np.float32)
        seed = None if seeds is None else seeds[c]
        codes = np.empty_like(w_codes[c])
        cols = np.arange(d, dtype=np.int64)[None, :]
        lo = num_head if c == 0 else 0
        if c == 0 and num_head > 0:
            ah, wh = a[:num_head].astype(np.float64), w[:num_head]
            s = (wh + k_old).astype(np.float32)                                     # weights + kahan
            t = (s.astype(np.float64) - lr64 * ah).astype(np.float32)               # - lr*acc
            offs = np.arange(num_head, dtype=np.int64)[:, None] * d + cols
            codes[:num_head] = rnd(t, seed, offs, c, 0)
            wq = C.e4m3_decode(codes[:num_head])
            u = ((k_old + wh).astype(np.float32) - wq).astype(np.float32)           # kahan + old - new
            kn = (u.astype(np.float64) - lr64 * ah).astype(np.float32)              # - lr*acc
            new_kahan = C.e5m2_encode(kn, saturate=True) if kahan_type == "e5m2" else C.bf16_round(kn)
        t = (w64[lo:] - lr64 * a[lo:].astype(np.float64)).astype(np.float32)
        offs = np.arange(Lc - lo, dtype=np.int64)[:, None] * d + cols
        codes[lo:] = rnd(t, seed, offs, c, lo)
        new_codes.append(codes)
    gx32 = gx.astype(np.float32)
    return new_codes, new_kahan, gx32, C.bf16_round(gx32)


def fp8_forward(w_codes, x_any, num_labels, *, simulated=False, scale_w=1.0, scale_x=1.0):
    """Inference logits [B, num_labels] (bf16-valued fp32): chunked_fp8xmc_clf.py:45-60.  The caller passes X
    already cast to e4m3 (evaluate.py:155-156); here X is re-quantised, which is idempotent."""
    x = np.ascontiguousarray(x_any, dtype=np.float32)
    xq = C.e4m3_decode(C.e4m3_encode(x / np.float32(scale_x), saturate=True)).astype(np.float64)
    outs = []
    for wc in w_codes:
        z = (xq @ C.e4m3_decode(wc).astype(np.float64).T).astype(np.float32)
        z = (z * (np.float32(scale_w) * np.float32(scale_x))).astype(np.float32)
        outs.append(C.bf16_round(z))
    return np.concatenate(outs, axis=1)[:, :num_labels]


def topk_of_logits(logits_bf16, k):
    """What evaluate.py:158-159,235-236 take from the dense logits of xfc_forward: the k largest per row, descending.
    Ties are ordered by ascending label id (torch.topk leaves their order open).  NaN orders above every number, as in
    torch.  Returns (values [B,k], indices [B,k] int64)."""
    z = np.asarray(logits_bf16, dtype=np.float32)
    key = np.where(np.isnan(z), np.float32(np.inf), z)
    idx = np.arange(z.shape[1])
    out_v = np.empty((z.shape[0], k), dtype=np.float32)
    out_i = np.empty((z.shape[0], k), dtype=np.int64)
    for b in range(z.shape[0]):
        order = np.lexsort((idx, -key[b]))[:k]       # primary: value descending, secondary: label ascending
        out_v[b] = z[b, order]
        out_i[b] = order
    return out_v, out_i


def bf16_step(w_bf16, x_bf16, labels, lr, num_chunks, *, seeds=None, sr_mode="rtn", return_parts=False,
              return_loss=False, weight_decay=0.0, dropout_p=0.0, dropout_seed=0):
    """One step of the bf16 layer (chunked.py:85-131), weights bf16.

    w_bf16 : fp32 array [L, d] holding bf16 values (single tensor, chunk views of ceil(L/nc) rows, last short)
    sr_mode: "rtn"        W' = bf16(f32(W) - lr*f32(A))
             "reference"  W' = SR16(f32(W) - f32(A)*lr; philox(seed_c, flat idx in chunk))  (stochastic_rounding_kernel.py:80-89)
             "fast"       the same T rounded by sr_bf16_fast with the counter-hash words of the FP8 fast mode (not in the reference)
    The bf16 path of the reference ignores its weight-decay argument (:91-99): weight_decay = 0 is the reference.  With
    this build's additions (xmc_tiled_step_ex): T = W - lr (bf16(A) + weight_decay W), the decayed gradient formed first
    in fp32; dropout as in fp8_step.
    Returns (new_w [L,d] bf16-valued fp32, gx_fp32 [B,d], grad_input bf16-valued fp32[, loss with return_loss]).
    """
    w_all = np.ascontiguousarray(w_bf16, dtype=np.float32)
    x = np.ascontiguousarray(x_bf16, dtype=np.float32)
    keep = None
    if dropout_p > 0:
        x, keep = C.dropout_bf16(x, dropout_p, dropout_seed)
    B, d = x.shape
    L = w_all.shape[0]
    cs = (L + num_chunks - 1) // num_chunks
    lr32 = np.float32(lr)
    x64 = x.astype(np.float64)
    gx = np.zeros((B, d), dtype=np.float32)
    new_w = w_all.copy()
    parts = []
    loss = 0.0
    for c in range(num_chunks):
        lo, hi = c * cs, min((c + 1) * cs, L)
        if lo >= hi:
            continue
        w = w_all[lo:hi]
        w64 = w.astype(np.float64)
        z = (x64 @ w64.T).astype(np.float32)                        # [B, L_c]  (:101)
        pos = _positives_mask(labels, B, lo, hi).T
        zb, g = _grad_from_logits(z, pos)                           # (:112-113)
        loss += bce_loss_sum(zb, pos)
        g64 = g.astype(np.float64)
        gx = gx + C.bf16_round((g64 @ w64).astype(np.float32))      # partial rounded to bf16 (:116)
        a = C.bf16_round((g64.T @ x64).astype(np.float32))          # materialised bf16 grad (:119)
        if weight_decay:
            a = (float(np.float32(weight_decay)) * w64 + a.astype(np.float64)).astype(np.float32)
        if sr_mode == "rtn":
            t = (w64 - float(lr32) * a.astype(np.float64)).astype(np.float32)   # single rounding (fma)
            nw = C.bf16_round(t)
        elif sr_mode == "reference":
            t = (w64 - a.astype(np.float64) * float(lr32)).astype(np.float32)   # stochastic_rounding_kernel.py:81 (fma)
            offs = np.arange((hi - lo) * d, dtype=np.int64).reshape(hi - lo, d)
            nw = C.sr_bf16_reference(t, seeds[c], offs)
        elif sr_mode == "fast":
            # this build's own mode: hardware stochastic rounding fed with the counter-hash words of the FP8 fast mode
            t = (w64 - a.astype(np.float64) * float(lr32)).astype(np.float32)
            grow = np.arange(lo, hi, dtype=np.int64)[:, None] + np.zeros((1, d), dtype=np.int64)
            cols = np.zeros((hi - lo, 1), dtype=np.int64) + np.arange(d, dtype=np.int64)[None, :]
            nw = C.sr_bf16_fast(t, C.fast_sr_words(seeds[c], grow, cols, d))
        else:
            raise ValueError(sr_mode)
        new_w[lo:hi] = nw
        if return_parts:
            parts.append(dict(z=zb, g=g, a=a, t=t))
    if keep is not None:
        gx = C.dropout_backward(gx, keep, dropout_p)
    out = (new_w, gx, C.bf16_round(gx))
    if return_loss:
        out = out + (loss,)
    return out + (parts,) if return_parts else out


def dense_step(w, x, labels, lr, wd, num_chunks, dtype="float32"):
    """One step of the fp32 / fp16 branch of the `chunked` layer (chunked.py:85-124): everything in the weight's type,
    weight decay folded into the gradient, plain SGD.
        Z = cast(X W_c^T); S = cast(sigmoid(Z)); G = S, cast(S - 1) at positives (set semantics)        :101-113
        gX += f32(cast(G W_c))                                                                         :116
        A = cast(G^T X); A = cast(A + wd*W_c); W_c = cast(W_c - lr*A)                                  :119-124
    cast = round to the weight's type (float32: the float64 sums rounded once; float16: rounded to half).  wd and lr
    enter as Python floats (torch's alpha): the elementwise results are computed in fp32 and rounded once.
    Returns (new_w, gx_fp32, grad_input in the weight's type, held in fp32)."""
    assert dtype in ("float32", "float16")
    cast = (lambda a: np.asarray(a, dtype=np.float64).astype(np.float32)) if dtype == "float32" else \
           (lambda a: np.asarray(a, dtype=np.float64).astype(np.float16).astype(np.float32))
    w_all = cast(w)
    xc = cast(x)
    B, d = xc.shape
    L = w_all.shape[0]
    cs = (L + num_chunks - 1) // num_chunks
    x64 = xc.astype(np.float64)
    gx = np.zeros((B, d), dtype=np.float32)
    new_w = w_all.copy()
    for c in range(num_chunks):
        lo, hi = c * cs, min((c + 1) * cs, L)
        if lo >= hi:
            continue
        w64 = w_all[lo:hi].astype(np.float64)
        z = cast(x64 @ w64.T)
        pos = _positives_mask(labels, B, lo, hi).T
        s = cast(1.0 / (1.0 + np.exp(-z.astype(np.float64))))
        g = np.where(pos, cast(s.astype(np.float64) - 1.0), s).astype(np.float32)
        g64 = g.astype(np.float64)
        gx = (gx + cast(g64 @ w64)).astype(np.float32)
        a = cast(g64.T @ x64)
        # torch's add_(other, alpha): self + alpha*other evaluated in fp32 and rounded to the tensor's type
        a = cast((a.astype(np.float32) + np.float32(wd) * w_all[lo:hi]).astype(np.float32))
        new_w[lo:hi] = cast((w_all[lo:hi] + np.float32(-lr) * a).astype(np.float32))
    return new_w, gx, cast(gx)


def bce_loss_sum(z_bf16, posmask):
    """Summed binary cross entropy with logits, the quantity chunked.py:57-72 is written to return when it is handed
    the logits: sum(max(z,0)) - sum(z at positives) + sum(log(1 + exp(-|z|))).  float64; z are the bf16 logits."""
    z = np.asarray(z_bf16, dtype=np.float64)
    return float(np.maximum(z, 0.0).sum() - z[np.asarray(posmask, dtype=bool)].sum() + np.log1p(np.exp(-np.abs(z))).sum())


def bf16_forward(w_bf16, x_bf16):
    """chunked.py:48-53: one matmul, bf16 out."""
    z = (np.asarray(x_bf16, np.float64) @ np.asarray(w_bf16, np.float64).T).astype(np.float32)
    return C.bf16_round(z)


def scalar_fp8_step_tiny(w_codes, x_bf16, labels, lr, scale_w=1.0, scale_x=1.0, simulated=False):
    """Brute-force scalar loops (pure Python floats = float64) for tiny inputs; RTN mode, one chunk.
    Independent of the vectorised code above except for the scalar codecs.
    simulated (chunked_fp8xmc_clf.py:98-99,110,115-116): the logits take X as it is (bf16, not quantised to e4m3) and
    the final cast is torch's (no saturation: NaN above 464); everything else is the same arithmetic."""
    L, d = w_codes.shape
    B = x_bf16.shape[0]
    dec = [float(v) for v in C.E4M3_TABLE]
    w = [[dec[int(w_codes[l, k])] for k in range(d)] for l in range(L)]
    if simulated:
        assert scale_w == 1.0 and scale_x == 1.0
        xq = [[float(x_bf16[b, k]) for k in range(d)] for b in range(B)]
    else:
        xq = [[dec[int(C.e4m3_encode(np.float32(x_bf16[b, k]) / np.float32(scale_x)))] for k in range(d)] for b in range(B)]
    posset = {(int(r), int(c)) for r, c in labels}
    g = [[0.0] * B for _ in range(L)]
    zs = np.float32(scale_w) * np.float32(scale_x)
    for l in range(L):
        for b in range(B):
            acc = 0.0
            for k in range(d):
                acc += w[l][k] * xq[b][k]
            z = float(C.bf16_round(np.float32(np.float32(acc) * zs)))
            s = float(C.bf16_round(np.float32(1.0 / (1.0 + np.exp(-z)))))
            if (b, l) in posset:
                s = float(C.bf16_round(np.float32(np.float32(s) - np.float32(1.0))))
            g[l][b] = s
    gx = np.zeros((B, d), dtype=np.float32)
    for b in range(B):
        for k in range(d):
            acc = 0.0
            for l in range(L):
                acc += g[l][b] * w[l][k]
            gx[b, k] = np.float32(acc * float(scale_w))
    new = np.zeros((L, d), dtype=np.uint8)
    for l in range(L):
        for k in range(d):
            acc = 0.0
            for b in range(B):
                acc += g[l][b] * float(x_bf16[b, k])
            t = np.float32(w[l][k] - float(np.float32(np.float32(lr) / np.float32(scale_w))) * float(np.float32(acc)))
            new[l, k] = C.e4m3_encode(t, saturate=not simulated)
    return new, gx
