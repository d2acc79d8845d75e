"""Inference logits of the FP8 layer (reference: chunked_fp8xmc_clf.py:45-60) against the oracle: bf16 logits
within 1 ulp, padding rows dropped, any batch size."""
import numpy as np
import pytest

import helpers as H
from elmo_amd import synth
from oracle import codecs as C
from oracle import step as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("nc,rows,batch,num_labels", [(2, 64, 16, 100), (3, 208, 32, 600), (2, 1040, 5, 2065), (1, 4096, 130, 4000)])
def test_forward_parity(gpu, nc, rows, batch, num_labels):
    import torch
    from elmo_amd import ops
    case = H.make_case(nc, rows, max(batch, 16) // 16 * 16 if batch % 16 == 0 else 16, 51)
    x = __import__("elmo_amd.synth", fromlist=["make_x"]).make_x(batch, 768, 52)
    chunks, _, _ = H.to_device_case(case, gpu)
    xd = torch.from_numpy(x).to(gpu).to(torch.bfloat16)
    # the evaluator hands over X already cast to e4m3 (evaluate.py:155-156); both forms must give the same logits
    out_bf = ops.fp8_forward(chunks, xd, num_labels).float().cpu().numpy()
    out_f8 = ops.fp8_forward(chunks, xd.to(torch.float8_e4m3fn), num_labels).float().cpu().numpy()
    assert out_bf.shape == (batch, num_labels)
    assert np.array_equal(out_bf, out_f8)
    ref = O.fp8_forward(case["chunks"], x, num_labels)
    H.assert_bf16_close(out_bf, ref)
    top_ref = np.argsort(-ref, axis=1)[:, :5]
    top_got = np.argsort(-out_bf, axis=1)[:, :5]
    assert np.mean(top_ref == top_got) > 0.95


def test_forward_scales(gpu):
    import torch
    from elmo_amd import ops
    case = H.make_case(2, 128, 16, 53, w_scale=2.0 ** -5)
    chunks, xd, _ = H.to_device_case(case, gpu)
    out = ops.fp8_forward(chunks, xd, 256, scale_w=2.0 ** -5, scale_x=0.25).float().cpu().numpy()
    ref = O.fp8_forward(case["chunks"], case["x"], 256, scale_w=2.0 ** -5, scale_x=0.25)
    H.assert_bf16_close(out, ref)


@pytest.mark.parametrize("nc,rows,batch,num_labels,k", [
    (1, 64, 16, 64, 5),             # a single tile, k small
    (3, 2048, 48, 6000, 100),       # padding rows of the last chunk dropped
    (2, 1024, 20, 2048, 128),       # batch padded to 32, largest k
    (4, 4096, 128, 16000, 100),     # full batch
    (2, 64, 16, 70, 70),            # k equal to the number of labels
    (3, 16384, 32, 49000, 100),     # one group above 32,768 labels: two workgroups and two lists per batch row
    (5, 16384, 16, 81920, 7),       # the same, k small, nothing dropped
])
@pytest.mark.parametrize("fused", [False, True])
def test_topk_forward(gpu, nc, rows, batch, num_labels, k, fused):
    """Top-k without the dense logits - the chunk-wise path, and the two-pass path where the label count admits it (the
    op falls back by itself where it does not) - against the dense logits of the same library (bit-equal values, ids that point at them, the
    documented order among ties) and against the oracle's top-k of the oracle's logits."""
    import torch
    from elmo_amd import ops
    case = H.make_case(nc, rows, batch, 70 + nc, std=0.5)
    chunks, x, _ = H.to_device_case(case, gpu)
    dense = ops.fp8_forward(chunks, x, num_labels).float().cpu().numpy()
    vals, idx = ops.fp8_forward_topk(chunks, x, num_labels, k, fused=fused)
    assert vals.shape == (batch, k) and idx.shape == (batch, k) and idx.dtype == torch.int64
    v, i = vals.float().cpu().numpy(), idx.cpu().numpy()
    want_v, want_i = O.topk_of_logits(dense, k)
    assert np.array_equal(v, want_v)
    assert np.array_equal(i, want_i)
    assert i.min() >= 0 and i.max() < num_labels
    # the oracle end to end: same values wherever its logits equal the library's
    ref = O.fp8_forward(case["chunks"], case["x"], num_labels)
    rv, ri = O.topk_of_logits(ref, k)
    assert H.bf16_ulp_distance(v, rv).max() <= 1          # the logits themselves agree to one bf16 ulp
    assert (i == ri).mean() > 0.8                         # a one-ulp difference can reorder near-ties


def test_topk_with_repeated_values(gpu):
    """Weights with few distinct values give logits with many exact ties across chunk boundaries."""
    import torch
    from elmo_amd import ops
    rng = np.random.default_rng(3)
    codes = rng.choice(np.array([0x30, 0xB0, 0x38, 0x00], dtype=np.uint8), size=(4096, 768))
    codes[1000:3000] = codes[0:2000]                                   # identical rows in both chunks
    case = dict(x=synth.make_x(16, 768, 5), chunks=[codes[:2048].copy(), codes[2048:].copy()], labels=np.zeros((0, 2), np.int32))
    chunks, x, _ = H.to_device_case(case, gpu)
    dense = ops.fp8_forward(chunks, x, 4096).float().cpu().numpy()
    vals, idx = ops.fp8_forward_topk(chunks, x, 4096, 100)
    want_v, want_i = O.topk_of_logits(dense, 100)
    assert np.array_equal(vals.float().cpu().numpy(), want_v) and np.array_equal(idx.cpu().numpy(), want_i)


@pytest.mark.gpu
@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("k,nc", [(100, 2), (7, 2), (100, 3), (7, 3)])
def test_topk_when_most_logits_tie(gpu, k, nc, fused):
    """Nearly all rows of W are one and the same row: more logits reach the running bound than the selection keeps in
    fast memory, and the k-th value is a tie of thousands that the label id has to break - with three chunks across
    the two lists of a batch row, which the last kernel merges."""
    from elmo_amd import ops
    rng = np.random.default_rng(11)
    rows = 16384
    base = rng.choice(np.array([0x30, 0xB0, 0x38, 0x28], dtype=np.uint8), size=768)
    codes = np.tile(base, (nc * rows, 1))
    odd = rng.choice(nc * rows, size=60, replace=False)                # a few rows that differ, above or below the rest
    codes[odd] = rng.choice(np.array([0x30, 0xB0, 0x38, 0x28], dtype=np.uint8), size=(60, 768))
    case = dict(x=synth.make_x(24, 768, 6), chunks=[codes[c * rows:(c + 1) * rows].copy() for c in range(nc)],
                labels=np.zeros((0, 2), np.int32))
    chunks, x, _ = H.to_device_case(case, gpu)
    num_labels = nc * rows - 5
    dense = ops.fp8_forward(chunks, x, num_labels).float().cpu().numpy()
    vals, idx = ops.fp8_forward_topk(chunks, x, num_labels, k, fused=fused)
    want_v, want_i = O.topk_of_logits(dense, k)
    assert np.array_equal(vals.float().cpu().numpy(), want_v) and np.array_equal(idx.cpu().numpy(), want_i)
    if fused:
        # the two-pass path by itself reports that a candidate list overflowed (the op above then repeated the call)
        _, _, status = ops.fp8_forward_topk(chunks, x, num_labels, k, fused=True, defer_check=True)
        assert int(status[0]) & 1


@pytest.mark.parametrize("fused", [False, True])
def test_topk_at_the_shipped_670k_geometry(gpu, fused):
    """amazontitles670k.yaml ships num_chunks: 2, i.e. chunks of 335,056 rows: larger than one selection segment, so each
    chunk is taken in three pieces.  Against torch.topk of the library's own dense logits (values bit-equal; ids point at
    those values and agree wherever the value is unique in its row)."""
    import torch
    from elmo_amd import ops
    L, nc, k, batch = 670091, 2, 100, 16
    rows = (L + 16 * nc - L % (16 * nc)) // nc
    assert rows == 335056 and rows > (1 << 18)
    gen = torch.Generator(device=gpu).manual_seed(12)
    chunks = [(torch.randn(rows, 768, generator=gen, device=gpu) * 0.3).to(torch.float8_e4m3fn) for _ in range(nc)]
    x = torch.from_numpy(synth.make_x(batch, 768, 13)).to(gpu).to(torch.bfloat16)
    dense = ops.fp8_forward(chunks, x, L)
    if fused:
        vals, idx, status = ops.fp8_forward_topk(chunks, x, L, k, fused=True, defer_check=True)
        assert int(status[0]) == 0                 # the two-pass path produced this result itself
    else:
        vals, idx = ops.fp8_forward_topk(chunks, x, L, k, fused=False)
    tv, ti = torch.topk(dense.float(), k, dim=1)
    assert torch.equal(vals.float(), tv)
    assert torch.equal(dense.float().gather(1, idx), tv) and int(idx.max()) < L and int(idx.min()) >= 0
    # the documented order among equal values: ascending label id
    v, i = vals.float().cpu().numpy(), idx.cpu().numpy()
    tie = v[:, 1:] == v[:, :-1]
    assert np.all(i[:, 1:][tie] > i[:, :-1][tie])
    uniq = np.ones_like(v, dtype=bool); uniq[:, 1:] &= ~tie; uniq[:, :-1] &= ~tie
    assert np.array_equal(i[uniq], ti.cpu().numpy()[uniq])
    # labels from both chunks and from all three pieces of a chunk appear
    assert (i >= rows).any() and (i < rows).any()


@pytest.mark.parametrize("k,batch,num_labels", [(100, 128, 262144 - 7), (5, 50, 200000), (128, 16, 140000), (1, 16, 70000)])
def test_two_pass_topk_equals_the_chunkwise_one(gpu, k, batch, num_labels):
    """The two selections through the C ABI on the same weights: bit-equal values, equal label ids (both order equal
    values by ascending label id), status word zero, and the sampled first pass at every stride (k = 1 and 5 visit one
    tile in 16, k = 100 and 128 one in 4)."""
    import torch
    from elmo_amd import ops
    nc = 4
    rows = (num_labels + 16 * nc - num_labels % (16 * nc)) // nc
    gen = torch.Generator(device=gpu).manual_seed(100 + k)
    chunks = [(torch.randn(rows, 768, generator=gen, device=gpu) * 0.4).to(torch.float8_e4m3fn) for _ in range(nc)]
    x = torch.from_numpy(synth.make_x(batch, 768, 14)).to(gpu).to(torch.bfloat16)
    v0, i0 = ops.fp8_forward_topk(chunks, x, num_labels, k, fused=False)
    v1, i1, status = ops.fp8_forward_topk(chunks, x, num_labels, k, fused=True, defer_check=True)
    assert int(status.abs().sum()) == 0
    assert torch.equal(v0.view(torch.int16), v1.view(torch.int16)) and torch.equal(i0, i1)
    # a second call on the same scratch-free path gives the same again (counts and status are reset by the call)
    v2, i2, status = ops.fp8_forward_topk(chunks, x, num_labels, k, fused=True, defer_check=True)
    assert int(status.abs().sum()) == 0 and torch.equal(v1.view(torch.int16), v2.view(torch.int16)) and torch.equal(i1, i2)


def test_two_pass_topk_with_heads_first_and_nan(gpu):
    """Labels sorted by frequency put the large logits into the first rows: the first pass samples tiles across the
    whole range, so its bound stays useful (status zero).  Two weight rows hold a NaN code (0x7F, 0xFF): their logits
    are NaN, which orders above every number as in torch.topk, whatever its sign, the smaller label first."""
    import torch
    from elmo_amd import ops
    L, nc, k, batch = 160000, 2, 100, 32
    rows = L // nc
    gen = torch.Generator(device=gpu).manual_seed(21)
    scale = torch.linspace(1.5, 0.05, L, device=gpu).unsqueeze(1)       # head labels first
    w = torch.randn(L, 768, generator=gen, device=gpu) * scale
    w8 = w.to(torch.float8_e4m3fn)
    raw = w8.view(torch.uint8)
    raw[1234, 5] = 0x7F
    raw[150001, 700] = 0xFF
    chunks = [w8[c * rows:(c + 1) * rows].contiguous() for c in range(nc)]
    x = torch.from_numpy(synth.make_x(batch, 768, 15)).to(gpu).to(torch.bfloat16)
    dense = ops.fp8_forward(chunks, x, L).float()
    assert torch.isnan(dense[:, 1234]).all() and torch.isnan(dense[:, 150001]).all()
    for fused in (True, False):
        if fused:
            vals, idx, status = ops.fp8_forward_topk(chunks, x, L, k, fused=True, defer_check=True)
            assert int(status[0]) == 0
        else:
            vals, idx = ops.fp8_forward_topk(chunks, x, L, k, fused=False)
        v = vals.float()
        assert torch.isnan(v[:, :2]).all() and not torch.isnan(v[:, 2:]).any()
        assert torch.equal(idx[:, 0], torch.full_like(idx[:, 0], 1234)) and torch.equal(idx[:, 1], torch.full_like(idx[:, 1], 150001))
        finite = dense.clone()
        finite[:, 1234] = -float("inf"); finite[:, 150001] = -float("inf")
        tv, _ = torch.topk(finite, k - 2, dim=1)
        assert torch.equal(v[:, 2:], tv) and torch.equal(dense.gather(1, idx[:, 2:]), tv)


@pytest.mark.parametrize("rows,cols,p,seed,as_e4m3", [(128, 768, 0.1, 40, False), (16, 768, 0.7, 123456789012, False),
                                                       (33, 1024, 0.3, 7, True), (128, 768, 0.0, 1, True)])
def test_dropout_quantize_matches_the_oracle(gpu, rows, cols, p, seed, as_e4m3):
    """Dropout fused with the e4m3 cast (the reference's prototype, tma_gemm.py:7-13,34-38) against the oracle: bit-equal
    codes for bf16 and e4m3 input, a 64-bit seed, p = 0."""
    import torch
    from elmo_amd import ops
    rng = np.random.default_rng(seed % 1000)
    x = C.bf16_round(rng.standard_normal((rows, cols)).astype(np.float32) * 4.0)
    x[0, :8] = [500.0, -500.0, 448.0, 0.0, -0.0, 2.0 ** -9, 2.0 ** -10, 300.0]     # saturation, zeros, the smallest codes
    xd = torch.from_numpy(x).to(gpu).to(torch.bfloat16)
    if as_e4m3:
        xd = xd.clamp(-448, 448).to(torch.float8_e4m3fn)         # torch's own cast turns 500 into NaN
        x = xd.float().cpu().numpy()
    out = ops.dropout_quantize(xd, p, seed)
    assert out.dtype == torch.float8_e4m3fn and out.shape == (rows, cols)
    want = C.dropout_quantize(x, p, seed)
    got = out.view(torch.uint8).cpu().numpy()
    assert np.array_equal(got, want)
