"""Parity of the three-kernel path (bf16 layer and simulated-FP8 mode, through the C ABI) against the CPU oracle.

Tolerances: round-to-nearest weights within 1 grid step (e4m3 step; bf16: one ulp of the operands of the update, see
check_bf16_weights) of the oracle with all but a small fraction identical (the fp32 accumulators differ by summation order only); the reference's stochastic-rounding recipe
bit-identical wherever the fp32 value T it rounds is, i.e. for all but the same small fraction; grad_X accumulator
within 1e-3 of its largest entry, grad_input its round-to-nearest bf16 image."""
import numpy as np
import pytest

import helpers as H
from elmo_amd import synth
from oracle import codecs as C
from oracle import step as O

pytestmark = pytest.mark.gpu


def bf16_case(L, batch, seed, pos_mean=5.0):
    x = synth.make_x(batch, 768, seed)
    w = C.bf16_round(synth.make_weights_np(L, 768, seed, 0.02))
    labels = synth.make_labels(batch, L, pos_mean, 1.0, seed).astype(np.int32)
    return x, w, labels


def run_bf16(x, w, labels, nc, device, mode, seeds, lr=0.05):
    import torch
    from elmo_amd import ops
    L = w.shape[0]
    cs = (L + nc - 1) // nc
    wt = torch.from_numpy(C.bf16_bits(w).view(np.int16)).to(device).view(torch.bfloat16)
    views = [wt[c * cs:min((c + 1) * cs, L)] for c in range(nc) if c * cs < L]
    xt = torch.from_numpy(C.bf16_bits(x).view(np.int16)).to(device).view(torch.bfloat16)
    lab = torch.from_numpy(labels).to(device).contiguous()
    g, gf = ops.tiled_step(views, cs, "bf16", xt, lab, lr, seeds=seeds, round_mode=mode, want_f32=True)
    return wt.float().cpu().numpy(), gf.cpu().numpy(), g.float().cpu().numpy()


def check_bf16_weights(new, ref_w, w0, x=None, lr=0.05):
    """Updated bf16 weights: identical except where the bf16 rounding of grad_W (chunked.py:119) or of the result flipped
    because the fp32 sums were taken in another order.  Such a flip moves the weight by one bf16 ulp of lr*A or of the
    result (the first can cause the second); each is bounded by 2^-7 (|w_old| + |w_new|), which also covers results next
    to zero after cancellation.  A flip of one bf16 entry of G itself (one ulp of a sigmoid, at most 2^-8) moves a whole
    row of grad_W by that times |x|: an absolute floor of lr * 2^-8 * max|x|, twice over."""
    tol = 1.5 * 2.0 ** -7 * (np.abs(w0) + np.abs(ref_w)) + 1e-30
    if x is not None:
        tol = tol + 2.0 * lr * 2.0 ** -8 * np.abs(x).max()
    assert np.all(np.abs(new - ref_w) <= tol), float(np.max(np.abs(new - ref_w) / tol))
    assert (new != ref_w).mean() < 2e-3, (new != ref_w).mean()


def check_gx(gf, gb, ref_gx, tol=1e-3):
    scale = np.abs(ref_gx).max()
    assert np.abs(gf - ref_gx).max() <= tol * scale
    assert np.array_equal(C.bf16_bits(gb), C.bf16_bits(C.bf16_round(gf)))


@pytest.mark.parametrize("L,nc,batch,seed", [
    (64, 1, 16, 31),            # a single tile
    (1000, 3, 24, 32),          # ragged chunks (334, 334, 332), batch not a multiple of 16
    (5000, 2, 128, 33),         # full batch
    (20011, 4, 64, 34),         # prime label count
    (3000, 2, 200, 35),         # two batch halves, the second one short
    (1500, 3, 256, 36),         # two full halves
    (2000, 2, 300, 37),         # three halves (run as four, the last one empty), positives on rows past 256
    (1300, 3, 512, 38),         # the largest batch: four halves, the batch the reference's chunked configs ship
])
def test_bf16_layer_rtn_parity(gpu, L, nc, batch, seed):
    x, w, labels = bf16_case(L, batch, seed)
    new, gf, gb = run_bf16(x, w, labels, nc, gpu, "rtn", None)
    ref_w, ref_gx, _ = O.bf16_step(w, x, labels, 0.05, nc, sr_mode="rtn")
    check_bf16_weights(new, ref_w, w, x)
    # the per-chunk partial is rounded to bf16 before it is accumulated (chunked.py:116): a flip of that rounding moves
    # an entry by one bf16 ulp of the partial, hence the looser bound
    check_gx(gf, gb, ref_gx, tol=4e-3)


@pytest.mark.parametrize("wd,p", [(0.05, 0.0), (0.0, 0.3), (0.02, 0.1)])
def test_weight_decay_and_fused_dropout_on_the_three_kernel_path(gpu, wd, p):
    """bf16 layer: T = W - lr (bf16(A) + wd W) and dropout of X in the preparation kernel; simulated-FP8 mode: the same
    with the fp32 gradient.  Against the oracle, whose treatment of both is pinned by closed forms on the CPU."""
    import torch
    from elmo_amd import ops
    L, nc, batch, lr, dseed = 3000, 3, 40, 0.5, 0x1357_9BDF_2468
    x, w, labels = bf16_case(L, batch, 39)
    cs = (L + nc - 1) // nc
    wt = torch.from_numpy(C.bf16_bits(w).view(np.int16)).to(gpu).view(torch.bfloat16)
    views = [wt[c * cs:min((c + 1) * cs, L)] for c in range(nc)]
    xt = torch.from_numpy(C.bf16_bits(x).view(np.int16)).to(gpu).view(torch.bfloat16)
    lab = torch.from_numpy(labels).to(gpu).contiguous()
    g, gf = ops.tiled_step(views, cs, "bf16", xt, lab, lr, want_f32=True, weight_decay=wd, dropout_p=p, dropout_seed=dseed)
    ref_w, ref_gx, _ = O.bf16_step(w, x, labels, lr, nc, weight_decay=wd, dropout_p=p, dropout_seed=dseed)
    plain_w = O.bf16_step(w, x, labels, lr, nc)[0]
    assert (plain_w != ref_w).mean() > 0.02
    check_bf16_weights(wt.float().cpu().numpy(), ref_w, w, x, lr=lr)
    check_gx(gf.cpu().numpy(), g.float().cpu().numpy(), ref_gx, tol=4e-3)
    if p > 0:       # dropped elements have an exactly zero gradient
        keep = C.dropout_bf16(x, p, dseed)[1]
        assert np.all(gf.cpu().numpy()[~keep] == 0) and np.any(gf.cpu().numpy()[keep] != 0)
    # simulated FP8
    case = H.make_case(3, 1008, 48, 64)
    chunks, xs, labs = H.to_device_case(case, gpu)
    g, gf = ops.tiled_step(chunks, chunks[0].shape[0], "e4m3", xs, labs, lr, want_f32=True, weight_decay=wd, dropout_p=p,
                           dropout_seed=dseed)
    ref_codes, ref_gx, _ = O.fp8_step(case["chunks"], case["x"], case["labels"], lr, simulated=True, weight_decay=wd,
                                      dropout_p=p, dropout_seed=dseed)
    d = np.concatenate([H.e4m3_ulp_distance(a, b).ravel() for a, b in zip(H.chunks_to_numpy(chunks), ref_codes)])
    assert d.max() <= 1 and (d != 0).mean() < 2e-3
    check_gx(gf.cpu().numpy(), g.float().cpu().numpy(), ref_gx)
    # the head-Kahan layer takes neither option
    kah = torch.zeros(64, 768, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(Exception):
        ops.tiled_step(chunks, chunks[0].shape[0], "e4m3", xs, labs, lr, quantize_x=True, saturate=True, kahan=kah,
                       num_head=64, weight_decay=0.01)


def test_bf16_layer_reference_stochastic_rounding(gpu):
    L, nc, batch = 3000, 3, 32
    x, w, labels = bf16_case(L, batch, 41)
    seeds = [12345, 999999, 7]
    new, gf, gb = run_bf16(x, w, labels, nc, gpu, "sr_philox", seeds)
    ref_w, ref_gx, _ = O.bf16_step(w, x, labels, 0.05, nc, seeds=seeds, sr_mode="reference")
    check_bf16_weights(new, ref_w, w, x)
    # stochastic rounding really happened: differs from round-to-nearest in a sizeable share of the weights
    rtn_w, _, _ = O.bf16_step(w, x, labels, 0.05, nc, sr_mode="rtn")
    assert (new != rtn_w).mean() > 0.2
    # a different seed gives a different result
    new2, _, _ = run_bf16(x, w, labels, nc, gpu, "sr_philox", [1, 2, 3])
    assert (new2 != new).mean() > 0.1


def test_loss_of_a_ragged_case_with_large_logits(gpu):
    """Loss fused into the logits kernel: ragged chunks, batch not a multiple of 16, weights large enough that the
    logits leave the linear range of the softplus; padded batch rows and rows past the chunk must not count."""
    import torch
    from elmo_amd import ops
    L, nc, batch = 1000, 3, 24
    w = C.bf16_round(synth.make_weights_np(L, 768, 41, 2.0))
    x = synth.make_x(batch, 768, 41)
    labels = synth.make_labels(batch, L, 6.0, 1.0, 41)
    wt = torch.from_numpy(C.bf16_bits(w).view(np.int16)).to(gpu).view(torch.bfloat16)
    xt = torch.from_numpy(C.bf16_bits(x).view(np.int16)).to(gpu).view(torch.bfloat16)
    lt = torch.from_numpy(labels).to(gpu)
    cs = (L + nc - 1) // nc
    views = [wt[c * cs:min((c + 1) * cs, L)] for c in range(nc)]
    loss = torch.zeros(1, dtype=torch.float32, device=gpu)
    ops.tiled_step(views, cs, "bf16", xt, lt, 0.0, round_mode="rtn", loss_out=loss)
    _, _, _, ref_loss = O.bf16_step(w, x, labels, 0.0, nc, sr_mode="rtn", return_loss=True)
    assert abs(loss.item() - ref_loss) <= 1e-4 * abs(ref_loss), (loss.item(), ref_loss)
    # a second call gives the same bits (fixed summation order)
    loss2 = torch.zeros(1, dtype=torch.float32, device=gpu)
    ops.tiled_step(views, cs, "bf16", xt, lt, 0.0, round_mode="rtn", loss_out=loss2)
    assert loss.item() == loss2.item()


def test_bf16_layer_duplicates_and_no_positives(gpu):
    x, w, labels = bf16_case(640, 16, 51)
    dup = np.array([[0, 5], [0, 5], [3, 639], [3, 639], [15, 0]], dtype=np.int32)
    new, gf, gb = run_bf16(x, w, dup, 2, gpu, "rtn", None)
    ref_w, ref_gx, _ = O.bf16_step(w, x, dup, 0.05, 2, sr_mode="rtn")
    check_bf16_weights(new, ref_w, w, x)
    check_gx(gf, gb, ref_gx, tol=4e-3)
    none = np.zeros((0, 2), dtype=np.int32)
    new, gf, gb = run_bf16(x, w, none, 2, gpu, "rtn", None)
    ref_w, ref_gx, _ = O.bf16_step(w, x, none, 0.05, 2, sr_mode="rtn")
    check_bf16_weights(new, ref_w, w, x)
    check_gx(gf, gb, ref_gx, tol=4e-3)


def test_bf16_layer_many_positives_over_four_halves(gpu):
    """30,000 positives (close to the 32,768 a step accepts) spread over 512 batch rows, i.e. over both sorted lists, with
    pairs on the first and last row of every half; entries outside the batch are ignored."""
    L, nc, batch = 2048, 2, 512
    x, w, _ = bf16_case(L, batch, 39)
    rng = np.random.default_rng(40)
    flat = rng.choice(batch * L, size=30000, replace=False)
    labels = np.stack([flat // L, flat % L], axis=1).astype(np.int32)
    edge = np.array([[r, c] for r in (0, 127, 128, 255, 256, 383, 384, 511) for c in (0, L - 1, 1023, 1024)], dtype=np.int32)
    labels = np.concatenate([labels, edge])
    bogus = np.array([[512, 3], [-1, 3], [700, 9], [3, L], [3, -1]], dtype=np.int32)
    mixed = np.concatenate([labels, bogus])
    mixed = mixed[rng.permutation(len(mixed))]
    new, gf, gb = run_bf16(x, w, mixed, nc, gpu, "rtn", None)
    ref_w, ref_gx, _ = O.bf16_step(w, x, labels, 0.05, nc, sr_mode="rtn")
    check_bf16_weights(new, ref_w, w, x)
    check_gx(gf, gb, ref_gx, tol=4e-3)


def run_sim(case, device, mode, seeds, lr=0.05):
    from elmo_amd import ops
    chunks, x, labels = H.to_device_case(case, device)
    g, gf = ops.tiled_step(chunks, chunks[0].shape[0], "e4m3", x, labels, lr, seeds=seeds, round_mode=mode, want_f32=True)
    return H.chunks_to_numpy(chunks), gf.cpu().numpy(), g.float().cpu().numpy()


@pytest.mark.parametrize("nc,rows,batch,seed", [(1, 64, 16, 61), (3, 208, 32, 62), (2, 4096, 128, 63)])
def test_simulated_fp8_rtn_parity(gpu, nc, rows, batch, seed):
    case = H.make_case(nc, rows, batch, seed)
    new, gf, gb = run_sim(case, gpu, "rtn", None)
    ref_codes, ref_gx, _ = O.fp8_step(case["chunks"], case["x"], case["labels"], 0.05, sr_mode="rtn", simulated=True)
    mism = total = 0
    for a, b in zip(new, ref_codes):
        d = H.e4m3_ulp_distance(a, b)
        assert d.max() <= 1
        mism += int((d != 0).sum()); total += d.size
    assert mism / total < 2e-3
    check_gx(gf, gb, ref_gx)


def test_simulated_fp8_differs_from_true_fp8_logits(gpu):
    """The simulated mode takes its logits from the un-quantised X (chunked_fp8xmc_clf.py:99): its grad_X must match the
    simulated oracle and not the true-FP8 one."""
    case = H.make_case(2, 1024, 32, 64)
    _, gf, _ = run_sim(case, gpu, "rtn", None)
    _, gx_sim, _ = O.fp8_step(case["chunks"], case["x"], case["labels"], 0.05, sr_mode="rtn", simulated=True)
    _, gx_true, _ = O.fp8_step(case["chunks"], case["x"], case["labels"], 0.05, sr_mode="rtn", simulated=False)
    assert np.abs(gf - gx_sim).max() < 0.2 * np.abs(gx_true - gx_sim).max()


def test_simulated_fp8_reference_stochastic_rounding_and_overflow(gpu):
    case = H.make_case(2, 512, 32, 65)
    seeds = [424242, 17]
    new, gf, gb = run_sim(case, gpu, "sr_philox", seeds)
    ref_codes, ref_gx, _ = O.fp8_step(case["chunks"], case["x"], case["labels"], 0.05, seeds=seeds, sr_mode="reference",
                                      simulated=True)
    mism = total = 0
    for a, b in zip(new, ref_codes):
        d = H.e4m3_ulp_distance(a, b)
        assert d.max() <= 1
        mism += int((d != 0).sum()); total += d.size
    assert mism / total < 2e-3
    # the cast back to e4m3 does not saturate (torch semantics, :116): a weight pushed beyond 464 becomes NaN
    big = H.make_case(1, 64, 16, 66)
    big["chunks"][0][:] = 0x7E                     # +448 everywhere
    big["labels"] = np.array([[b, l] for b in range(16) for l in range(8)], dtype=np.int32)
    new, _, _ = run_sim(big, gpu, "rtn", None, lr=2000.0)
    ref_codes, _, _ = O.fp8_step(big["chunks"], big["x"], big["labels"], 2000.0, sr_mode="rtn", simulated=True)
    assert np.array_equal(new[0] & 0x7F == 0x7F, ref_codes[0] & 0x7F == 0x7F) and (new[0] & 0x7F == 0x7F).any()


def test_chunked_module_contract(gpu):
    import torch
    from test_host_cpu import make_cfg
    from xmc_classifiers.chunked import XMCBCECHUNKEDLayer
    cfg = make_cfg("cuda:0", 1000, 3, rounding="rtn")
    cfg.model.xmc.dtype = "bfloat16"
    torch.manual_seed(0)
    xfc = XMCBCECHUNKEDLayer(cfg)
    assert xfc.xfc_weight.shape == (1000, 768) and xfc.xfc_weight.dtype == torch.bfloat16 and xfc.chunk_size == 334
    assert list(xfc.state_dict().keys()) == []            # a plain tensor attribute, as in the reference
    enc = torch.nn.Linear(768, 768, bias=False).to(gpu).to(torch.bfloat16)
    tokens = torch.randn(24, 768, device=gpu, dtype=torch.bfloat16)
    labels = torch.tensor([[0, 3], [0, 999], [5, 17], [23, 500], [23, 500]], dtype=torch.int32, device=gpu)
    w0 = xfc.xfc_weight.float().cpu().numpy()
    ptr = xfc.xfc_weight.data_ptr()
    out = enc(tokens)
    loss = xfc.xfc_forward_backward(out, labels, [0.05], skip_loss=True)
    assert loss == 0 and xfc.iteration == 1 and xfc.xfc_weight.data_ptr() == ptr
    g = xfc.grad_input
    assert g.shape == (24, 768) and g.dtype == torch.bfloat16
    ref_w, ref_gx, _ = O.bf16_step(w0, out.detach().float().cpu().numpy(), labels.cpu().numpy(), 0.05, 3, sr_mode="rtn")
    check_bf16_weights(xfc.xfc_weight.float().cpu().numpy(), ref_w, w0, out.detach().float().cpu().numpy())
    out.backward(g[0:24, :])
    assert enc.weight.grad is not None
    logits = xfc.xfc_forward(tokens)
    assert logits.shape == (24, 1000)
    # skip_loss=False: the summed binary cross entropy of the step's logits (what chunked.py:57-72 is written to return)
    w1 = xfc.xfc_weight.float().cpu().numpy()
    out2 = enc(tokens)
    loss = xfc.xfc_forward_backward(out2, labels, [0.05], skip_loss=False)
    _, _, _, ref_loss = O.bf16_step(w1, out2.detach().float().cpu().numpy(), labels.cpu().numpy(), 0.05, 3, sr_mode="rtn",
                                    return_loss=True)
    assert isinstance(loss, float) and abs(loss - ref_loss) <= 1e-4 * abs(ref_loss), (loss, ref_loss)
    with pytest.raises(AssertionError):      # no such weight type in the reference's dtype_map either
        cfg2 = make_cfg("cuda:0", 1000, 3)
        cfg2.model.xmc.dtype = "float8"
        XMCBCECHUNKEDLayer(cfg2)


def test_fp8_module_simulated_mode(gpu):
    import torch
    from test_host_cpu import make_cfg
    from xmc_classifiers.chunked_fp8xmc_clf import Fp8XMCBCEChunkedLayer
    torch.manual_seed(0)
    xfc = Fp8XMCBCEChunkedLayer(make_cfg("cuda:0", 1000, 2, simulated=True, rounding="rtn"))
    tokens = torch.randn(32, 768, device=gpu, dtype=torch.bfloat16) * 0.05
    labels = torch.tensor([[0, 3], [31, 999]], dtype=torch.int32, device=gpu)
    before = [w.view(torch.uint8).cpu().numpy().copy() for w in xfc.xfc_weight]
    assert xfc.xfc_forward_backward(tokens, labels, [0.05]) == 0
    ref_codes, ref_gx, _ = O.fp8_step(before, tokens.float().cpu().numpy(), labels.cpu().numpy(), 0.05, sr_mode="rtn",
                                      simulated=True)
    for w, r in zip(xfc.xfc_weight, ref_codes):
        d = H.e4m3_ulp_distance(w.view(torch.uint8).cpu().numpy(), r)
        assert d.max() <= 1 and (d != 0).mean() < 2e-3
    assert xfc.grad_input.shape == (32, 768)


def run_kahan(case, k0, ktype, nh, device, mode, seeds, lr=0.05, path="tiled"):
    import torch
    from elmo_amd import ops
    chunks, x, labels = H.to_device_case(case, device)
    if ktype == "e5m2":
        kt = torch.from_numpy(k0.copy()).to(device).view(torch.float8_e5m2)
    else:
        kt = torch.from_numpy(C.bf16_bits(k0).view(np.int16)).to(device).view(torch.bfloat16)
    if path == "fused":
        ws = ops.alloc_workspace(len(chunks), chunks[0].shape[0], device)
        g, gf = ops.fp8_kahan_step(chunks, kt, nh, x, labels, lr, seeds=seeds, round_mode=mode, want_f32=True, workspace=ws)
        assert ops.step_error_word(ws, len(chunks), chunks[0].shape[0]) == 0
    else:
        g, gf = ops.tiled_step(chunks, chunks[0].shape[0], "e4m3", x, labels, lr, seeds=seeds, round_mode=mode, want_f32=True,
                               quantize_x=True, saturate=True, kahan=kt, num_head=nh)
    kn = kt.view(torch.uint8).cpu().numpy() if ktype == "e5m2" else kt.float().cpu().numpy()
    return H.chunks_to_numpy(chunks), kn, gf.cpu().numpy(), g.float().cpu().numpy()


@pytest.mark.parametrize("path,shape", [("tiled", (2, 512, 32, 208)), ("fused", (2, 512, 32, 208)),
                                        ("fused", (3, 8192, 128, 8192)), ("fused", (1, 4096, 48, 4001)),
                                        ("fused", (1, 2048, 32, 2048))])
@pytest.mark.parametrize("ktype,mode", [("bf16", "rtn"), ("bf16", "sr_philox"), ("e5m2", "rtn"), ("bf16", "sr_fast"),
                                        ("e5m2", "sr_fast")])
def test_head_kahan_parity(gpu, ktype, mode, path, shape):
    """True-FP8 arithmetic with the compensated head (fuse_kernel.py:202-262) on the three-kernel path and on the fused
    one (xmc_fp8_kahan_step): a head that ends inside a tile, one that is the whole first chunk with more tiles than
    quads, a single chunk whose last rows lie behind the head, and a layer that is all head (no second launch)."""
    nc, rows, batch, nh = shape
    case = H.make_case(nc, rows, batch, 81)
    rng = np.random.default_rng(2)
    if ktype == "e5m2":
        k0 = C.e5m2_encode(rng.standard_normal((nh, 768)).astype(np.float32) * 1e-3)
    else:
        k0 = C.bf16_round(rng.standard_normal((nh, 768)).astype(np.float32) * 1e-3)
    seeds = [31337, 5] if mode != "rtn" else None
    seeds = None if seeds is None else (seeds + [77, 78])[:nc]
    new, kn, gf, gb = run_kahan(case, k0, ktype, nh, gpu, mode, seeds, path=path)

    def rand_fn(c, offs):      # the fast mode's words, by global label row
        return C.fast_sr_words(seeds[c], c * rows + offs // 768, offs % 768)

    ref_codes, ref_k, ref_gx, _ = O.fp8_kahan_step(case["chunks"], k0, case["x"], case["labels"], 0.05, nh, kahan_type=ktype,
                                                   seeds=seeds, rand_fn=rand_fn,
                                                   sr_mode={"rtn": "rtn", "sr_philox": "reference", "sr_fast": "exact"}[mode])
    mism = total = 0
    for a, b in zip(new, ref_codes):
        d = H.e4m3_ulp_distance(a, b)
        assert d.max() <= 1
        mism += int((d != 0).sum()); total += d.size
    assert mism / total < 2e-3
    check_gx(gf, gb, ref_gx)
    # the buffer: identical wherever the weight is (it holds what that rounding dropped); elsewhere it differs by the
    # weight's grid step, so that weight + buffer still agree
    same = new[0][:nh] == ref_codes[0][:nh]
    kf = C.e5m2_decode(kn) if ktype == "e5m2" else kn
    rf = C.e5m2_decode(ref_k) if ktype == "e5m2" else ref_k
    # (one grid step where the fp32 values in front of the cast differ in their last bits: a quarter of the value for
    # e5m2, whose subnormal step is 2^-16)
    tol = (2.0 ** -2 if ktype == "e5m2" else 2.0 ** -7) * np.abs(rf) + (2.0 ** -16 if ktype == "e5m2" else 1e-7)
    assert np.all(np.abs(kf - rf)[same] <= tol[same])
    tot_g = C.e4m3_decode(new[0][:nh]).astype(np.float64) + kf
    tot_r = C.e4m3_decode(ref_codes[0][:nh]).astype(np.float64) + rf
    assert np.abs(tot_g - tot_r).max() <= (2.0 ** -2 if ktype == "e5m2" else 2.0 ** -6) * np.abs(rf).max() + 1e-6


def test_true_fp8_on_the_tiled_path_matches_the_fused_oracle(gpu):
    """quantize_x + saturate turn the three-kernel path into the arithmetic of the fused kernel (no buffer)."""
    from elmo_amd import ops
    case = H.make_case(2, 1024, 32, 82)
    chunks, x, labels = H.to_device_case(case, gpu)
    g, gf = ops.tiled_step(chunks, 1024, "e4m3", x, labels, 0.05, round_mode="rtn", want_f32=True, quantize_x=True,
                           saturate=True)
    ref_codes, ref_gx, _ = O.fp8_step(case["chunks"], case["x"], case["labels"], 0.05, sr_mode="rtn")
    for a, b in zip(H.chunks_to_numpy(chunks), ref_codes):
        d = H.e4m3_ulp_distance(a, b)
        assert d.max() <= 1 and (d != 0).mean() < 2e-3
    check_gx(gf.cpu().numpy(), g.float().cpu().numpy(), ref_gx)


def test_true_fp8_with_a_batch_of_256(gpu):
    """Batches above 128 rows run on the three-kernel path in two halves: logits and grad_X per half, grad_W over both."""
    import torch
    from elmo_amd import ops
    case = H.make_case(2, 1024, 256, 61, pos_mean=4.0, extra_labels=[[255, 2047], [128, 0], [127, 0], [200, 1000], [200, 1000]])
    chunks, x, labels = H.to_device_case(case, gpu)
    g, gf = ops.tiled_step(chunks, 1024, "e4m3", x, labels, 0.05, round_mode="rtn", want_f32=True, quantize_x=True, saturate=True)
    ref_codes, ref_gx, _ = O.fp8_step(case["chunks"], case["x"], case["labels"], 0.05, sr_mode="rtn")
    new = H.chunks_to_numpy(chunks)
    mism = total = 0
    for a, b in zip(new, ref_codes):
        d = H.e4m3_ulp_distance(a, b)
        assert d.max() <= 1
        mism += int((d != 0).sum()); total += d.size
    assert mism / total < 2e-3
    assert gf.shape == (256, 768)
    assert np.abs(gf.cpu().numpy() - ref_gx).max() <= 1e-3 * np.abs(ref_gx).max()

    # the module routes such a batch there by itself
    from test_host_cpu import make_cfg
    from xmc_classifiers.chunked_fp8xmc_clf import Fp8XMCBCEChunkedLayer
    cfg = make_cfg("cuda:0", 2000, 2, rounding="rtn")
    cfg.data.batch_size = 256
    torch.manual_seed(3)
    xfc = Fp8XMCBCEChunkedLayer(cfg)
    w0 = [w.data.view(torch.uint8).cpu().numpy() for w in xfc.xfc_weight]
    emb = torch.from_numpy(C.bf16_bits(synth.make_x(256, 768, 62)).view(np.int16)).to(gpu).view(torch.bfloat16)
    lab = torch.from_numpy(synth.make_labels(256, 2000, 4.0, 1.0, 62)).to(gpu)
    assert xfc.xfc_forward_backward(emb, lab, [0.05]) == 0
    ref_codes, ref_gx, ref_gi = O.fp8_step(w0, emb.float().cpu().numpy(), lab.cpu().numpy(), 0.05, sr_mode="rtn")
    for wt, b in zip(xfc.xfc_weight, ref_codes):
        assert H.e4m3_ulp_distance(wt.data.view(torch.uint8).cpu().numpy(), b).max() <= 1
    assert xfc.grad_input.shape == (256, 768)
    H.assert_bf16_close(xfc.grad_input.float().cpu().numpy(), ref_gi)


def test_true_fp8_fast_rounding_on_the_three_kernel_path(gpu):
    """sr_fast with e4m3 weights: the same random words as the fused kernel (one hash per four weights of a global row),
    so the result equals the oracle's exact stochastic rounding fed with those words, and - with at most 128 batch rows -
    the fused kernel's own output except where the two paths' fp32 sums differ."""
    from elmo_amd import ops
    nc, rows = 2, 272
    case = H.make_case(nc, rows, 160, 64, pos_mean=4.0)
    seeds = [31337, 4242]

    def rand_fn(c, offs):
        r, k = offs // 768, offs % 768
        return C.fast_sr_words(seeds[c], c * rows + r, k)

    chunks, x, labels = H.to_device_case(case, gpu)
    ops.tiled_step(chunks, rows, "e4m3", x, labels, 0.05, seeds=seeds, round_mode="sr_fast", quantize_x=True, saturate=True)
    ref, _, _ = O.fp8_step(case["chunks"], case["x"], case["labels"], 0.05, sr_mode="exact", rand_fn=rand_fn)
    total = mism = 0
    for a, b in zip(H.chunks_to_numpy(chunks), ref):
        d = H.e4m3_ulp_distance(a, b)
        assert d.max() <= 1
        mism += int((d != 0).sum()); total += d.size
    assert mism / total < 2e-3, (mism, total)
    # an unknown mode is refused before anything is launched
    w = torch_bf16_weights(gpu, 64)
    with pytest.raises(AssertionError):
        ops.tiled_step([w], 64, "bf16", x[:16], labels[:0], 0.05, seeds=[1], round_mode="sr_exact")

    case = H.make_case(nc, rows, 64, 65)
    c1, x1, l1 = H.to_device_case(case, gpu)
    c2, _, _ = H.to_device_case(case, gpu)
    ops.tiled_step(c1, rows, "e4m3", x1, l1, 0.05, seeds=seeds, round_mode="sr_fast", quantize_x=True, saturate=True)
    ops.fp8_step(c2, x1, l1, 0.05, seeds=seeds, round_mode="sr_fast")
    diff = sum(int((a != b).sum()) for a, b in zip(H.chunks_to_numpy(c1), H.chunks_to_numpy(c2)))
    assert diff / (nc * rows * 768) < 2e-3


def torch_bf16_weights(device, rows):
    import torch
    return torch.zeros(rows, 768, dtype=torch.bfloat16, device=device)


def test_head_kahan_module(gpu):
    import types
    import torch
    from test_host_cpu import make_cfg
    from xmc_classifiers.chunked_head_kahan_fp8xmc_clf import Fp8XMCBCEChunkedHeadKahanLayer
    cfg = make_cfg("cuda:0", 1000, 2, rounding="rtn")
    cfg.training.FP8 = types.SimpleNamespace(using_head_kahan=True, fp8_head_kahan=False, head_ratio=0.2)
    torch.manual_seed(0)
    xfc = Fp8XMCBCEChunkedHeadKahanLayer(cfg)
    assert xfc.num_labels == 1024 and xfc.num_head == 204 and xfc.head_kahan.shape == (204, 768)
    assert xfc.head_kahan.dtype == torch.bfloat16 and sorted(xfc.state_dict().keys()) == ["xfc_weight.0", "xfc_weight.1"]
    tokens = torch.randn(32, 768, device=gpu, dtype=torch.bfloat16) * 0.05
    labels = torch.tensor([[0, 3], [31, 999], [4, 100]], dtype=torch.int32, device=gpu)
    before = [w.view(torch.uint8).cpu().numpy().copy() for w in xfc.xfc_weight]
    assert xfc.xfc_forward_backward(tokens, labels, [0.05]) == 0 and xfc.iteration == 1
    ref_codes, ref_k, _, _ = O.fp8_kahan_step(before, np.zeros((204, 768), np.float32), tokens.float().cpu().numpy(),
                                              labels.cpu().numpy(), 0.05, 204, sr_mode="rtn")
    for w, r in zip(xfc.xfc_weight, ref_codes):
        d = H.e4m3_ulp_distance(w.view(torch.uint8).cpu().numpy(), r)
        assert d.max() <= 1 and (d != 0).mean() < 2e-3
    assert float(xfc.head_kahan.float().abs().max()) > 0            # the buffer picked up the rounding residue
    assert xfc.xfc_forward(tokens).shape == (32, 1000)
    # a batch that is not a multiple of 16 takes the three-kernel path: same arithmetic, same oracle
    before = [w.view(torch.uint8).cpu().numpy().copy() for w in xfc.xfc_weight]
    k_before = xfc.head_kahan.float().cpu().numpy().copy()
    lab24 = torch.tensor([[0, 3], [23, 999], [4, 100]], dtype=torch.int32, device=gpu)
    assert xfc.xfc_forward_backward(tokens[:24], lab24, [0.05]) == 0
    ref_codes, ref_k, _, _ = O.fp8_kahan_step(before, k_before, tokens[:24].float().cpu().numpy(), lab24.cpu().numpy(), 0.05,
                                              204, sr_mode="rtn")
    for w, r in zip(xfc.xfc_weight, ref_codes):
        d = H.e4m3_ulp_distance(w.view(torch.uint8).cpu().numpy(), r)
        assert d.max() <= 1 and (d != 0).mean() < 2e-3
    cfg2 = make_cfg("cuda:0", 1000, 2)
    cfg2.training.FP8 = types.SimpleNamespace(using_head_kahan=False, fp8_head_kahan=False, head_ratio=0.2)
    plain = Fp8XMCBCEChunkedHeadKahanLayer(cfg2)                      # no buffer: the fused kernel
    assert plain.xfc_forward_backward(tokens, labels, [0.05]) == 0 and not hasattr(plain, "head_kahan")


def test_tiled_step_replays_in_a_captured_graph(gpu):
    """The three-kernel path launches kernels only (no memset, no allocation, no synchronisation), so a caller may record
    it into a graph: three replays, with eager work and synchronisations between them, give bit for bit what three eager
    steps give (bf16 layer, round-to-nearest, ragged chunks, batch in two halves)."""
    import torch
    from elmo_amd import ops
    x, w, labels = bf16_case(3000, 200, 36)
    L, nc = w.shape[0], 2
    cs = (L + nc - 1) // nc
    wt = torch.from_numpy(C.bf16_bits(w).view(np.int16)).to(gpu).view(torch.bfloat16)
    start = wt.clone()
    views = [wt[c * cs:min((c + 1) * cs, L)] for c in range(nc)]
    xt = torch.from_numpy(C.bf16_bits(x).view(np.int16)).to(gpu).view(torch.bfloat16)
    lab = torch.from_numpy(labels).to(gpu).contiguous()
    ws = ops.alloc_tiled_workspace(nc, cs, gpu, 200)
    gout = torch.empty(200, 768, dtype=torch.bfloat16, device=gpu)
    eager = []
    for _ in range(3):
        ops.tiled_step(views, cs, "bf16", xt, lab, 0.05, round_mode="rtn", workspace=ws, grad_out=gout)
        eager.append((wt.view(torch.int16).clone(), gout.view(torch.int16).clone()))
    wt.copy_(start)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.tiled_step(views, cs, "bf16", xt, lab, 0.05, round_mode="rtn", workspace=ws, grad_out=gout)
    assert torch.equal(wt.view(torch.int16), start.view(torch.int16))      # the capture ran nothing
    for k in range(3):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(wt.view(torch.int16), eager[k][0]), f"weights differ after replay {k}"
        assert torch.equal(gout.view(torch.int16), eager[k][1]), f"grad_input differs after replay {k}"
        scratch = torch.randn(1 << 20, device=gpu).sum().item()      # unrelated eager work between the replays
        assert scratch == scratch


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_chunked_module_fp32_fp16_branch_with_weight_decay(gpu, dtype):
    """chunked.py:122-124: fp32 / fp16 weights take the plain SGD branch with weight decay, at any batch size (here 300,
    more than the kernels' 256).  Against the oracle's restatement, which is held to torch CPU operations."""
    import torch
    from test_host_cpu import make_cfg
    from xmc_classifiers.chunked import XMCBCECHUNKEDLayer
    L, nc, B, lr, wd = 1000, 3, 300, 0.05, 0.5
    cfg = make_cfg("cuda:0", L, nc)
    cfg.model.xmc.dtype = dtype
    cfg.training.xmc.wd = wd
    cfg.training.precision.mode = "purefp" if dtype == "float32" else "custom"
    cfg.data.batch_size = B
    torch.manual_seed(3)
    xfc = XMCBCECHUNKEDLayer(cfg)
    tdt = torch.float32 if dtype == "float32" else torch.float16
    assert xfc._dtype == tdt and xfc.xfc_weight.dtype == tdt and xfc.xfc_weight.shape == (L, 768)
    w0 = xfc.xfc_weight.float().cpu().numpy().copy()
    x = synth.make_x(B, 768, 8)
    labels = synth.make_labels(B, L, 3.0, 1.0, 8)
    xd = torch.from_numpy(x).to(gpu).to(torch.bfloat16)                  # the encoder hands over bf16; the layer casts (:89-90)
    ld = torch.from_numpy(labels).to(gpu)
    loss = xfc.xfc_forward_backward(xd, ld, [lr])
    assert loss == 0 and xfc.iteration == 1 and xfc.grad_input.dtype == tdt and xfc.grad_input.shape == (B, 768)
    new, gx, gi = O.dense_step(w0, x, labels, lr, wd, nc, dtype)
    got = xfc.xfc_weight.float().cpu().numpy()
    ulp = 2.0 ** -23 if dtype == "float32" else 2.0 ** -10
    assert np.all(np.abs(new - got) <= 8 * ulp * np.maximum(np.abs(new), np.abs(w0).max()))
    assert np.abs(xfc.grad_input.float().cpu().numpy() - gi).max() <= (1e-4 if dtype == "float32" else 4e-3) * np.abs(gi).max()
    # weight decay reached the update
    nowd, _, _ = O.dense_step(w0, x, labels, lr, 0.0, nc, dtype)
    assert np.abs(nowd - got).max() > 10 * ulp * np.abs(got).max()


@pytest.mark.gpu
def test_true_fp8_arithmetic_at_batch_512(gpu):
    """The FP8 layer at the batch its shipped 670K configuration uses twice over (512 rows, four halves on the three-kernel
    path): logits from e4m3(X), saturating cast, round to nearest - against the true-FP8 oracle."""
    from elmo_amd import ops
    case = H.make_case(2, 1024, 512, 64, pos_mean=4.0)
    chunks, x, labels = H.to_device_case(case, gpu)
    g, gf = ops.tiled_step(chunks, 1024, "e4m3", x, labels, 0.05, round_mode="rtn", want_f32=True, quantize_x=True, saturate=True)
    ref_codes, ref_gx, _ = O.fp8_step(case["chunks"], case["x"], case["labels"], 0.05, sr_mode="rtn")
    new = H.chunks_to_numpy(chunks)
    for a, b in zip(new, ref_codes):
        d = H.e4m3_ulp_distance(a, b)
        assert d.max() <= 1 and (d != 0).mean() < 5e-3
    check_gx(gf.cpu().numpy(), g.float().cpu().numpy(), ref_gx)


@pytest.mark.parametrize("L,nc,batch,mode", [
    (4096, 4, 32, "rtn"),             # four chunks of 1,024 rows in one launch
    (4093, 4, 48, "rtn"),             # the last chunk three rows short
    (10240, 10, 16, "sr_philox"),     # ten chunks: launches of eight and two; a seed per chunk
    (2048, 2, 200, "sr_philox"),      # two batch halves
    (64 * 1200, 2, 16, "rtn"),        # chunks above the row budget of a launch stay one per launch
])
def test_bf16_layer_with_several_chunks_per_launch(gpu, L, nc, batch, mode):
    """Chunks that are a multiple of 64 rows long and lie one behind the other in memory (the bf16 layer's views) are taken
    several per launch: same results as the oracle's chunk-by-chunk step - per-chunk seeds and random offsets, the
    per-chunk bf16 rounding of grad_X."""
    x, w, labels = bf16_case(L, batch, 300 + nc)
    seeds = [1000 + 7 * c for c in range(nc)] if mode != "rtn" else None
    new, gf, gb = run_bf16(x, w, labels, nc, gpu, mode, seeds)
    ref_w, ref_gx, _ = O.bf16_step(w, x, labels, 0.05, nc, seeds=seeds, sr_mode="rtn" if mode == "rtn" else "reference")
    check_bf16_weights(new, ref_w, w, x)
    check_gx(gf, gb, ref_gx, tol=4e-3)
    if mode != "rtn":
        # a seed that belongs to another chunk would show: the same step with the seeds rotated differs in every chunk
        new2, _, _ = run_bf16(x, w, labels, nc, gpu, mode, seeds[1:] + seeds[:1])
        cs = (L + nc - 1) // nc
        for c in range(nc):
            assert (new2[c * cs:(c + 1) * cs] != new[c * cs:(c + 1) * cs]).mean() > 0.1


@pytest.mark.parametrize("mode,quant", [("sr_philox", False), ("sr_fast", True), ("rtn", False)])
def test_e4m3_chunks_in_one_allocation_take_one_launch(gpu, mode, quant):
    """e4m3 chunks that are views of one tensor (1,024 rows each) against the same chunks as separate tensors, which run one
    per launch: bit-equal weights and grad_X bits (the partial sums keep their order within a chunk; across chunks the
    fp32 totals are added in the same order)."""
    import torch
    from elmo_amd import ops
    nc, rows, batch = 3, 1024, 256 if quant else 64
    case = H.make_case(nc, rows, batch, 77)
    chunks, x, labels = H.to_device_case(case, gpu)
    whole = torch.cat(chunks).contiguous()
    views = [whole[c * rows:(c + 1) * rows] for c in range(nc)]
    seeds = [5, 6, 7]
    kw = dict(seeds=None if mode == "rtn" else seeds, round_mode=mode, want_f32=True, quantize_x=quant, saturate=quant)
    g1, gf1 = ops.tiled_step(views, rows, "e4m3", x, labels, 0.05, **kw)
    g0, gf0 = ops.tiled_step(chunks, rows, "e4m3", x, labels, 0.05, **kw)
    assert torch.equal(torch.cat(chunks).view(torch.uint8), whole.view(torch.uint8))
    assert torch.equal(g0.view(torch.int16), g1.view(torch.int16))
    assert torch.allclose(gf0, gf1, rtol=0, atol=1e-6 * float(gf0.abs().max()))


def test_bf16_layer_fast_stochastic_rounding(gpu):
    """The bf16 layer with this build's fast mode (hardware conversion to bf16, counter-hash words): equal to the oracle
    wherever the fp32 value it rounds is (as for the Philox recipe), different from round-to-nearest, seed-dependent,
    and unbiased: over more than a million weights the mean error against the exact update is below 1e-3 of the mean
    |delta w| (round-to-nearest of such small updates is not)."""
    L, nc, batch = 2048, 2, 64
    x, w, labels = bf16_case(L, batch, 43, pos_mean=20.0)
    seeds = [4242, 77]
    new, gf, gb = run_bf16(x, w, labels, nc, gpu, "sr_fast", seeds, lr=0.5)
    ref_w, ref_gx, _ = O.bf16_step(w, x, labels, 0.5, nc, seeds=seeds, sr_mode="fast")
    check_bf16_weights(new, ref_w, w, x, lr=0.5)
    check_gx(gf, gb, ref_gx, tol=4e-3)
    rtn_w, _, _ = O.bf16_step(w, x, labels, 0.5, nc, sr_mode="rtn")
    assert (new != rtn_w).mean() > 0.2
    new2, _, _ = run_bf16(x, w, labels, nc, gpu, "sr_fast", [1, 2], lr=0.5)
    assert (new2 != new).mean() > 0.1
    # unbiasedness against the exact (fp64) update t = w - lr * bf16(A)
    parts = O.bf16_step(w, x, labels, 0.5, nc, sr_mode="rtn", return_parts=True)[-1]
    t = np.concatenate([p["t"] for p in parts]).astype(np.float64)
    assert t.size > 10 ** 6
    dw = np.abs(t - w).mean()
    assert abs((new.astype(np.float64) - t).mean()) <= 1e-3 * dw


def test_chunked_module_with_the_fast_rounding(gpu):
    """XMCBCECHUNKEDLayer with training.xmc.rounding = "sr_fast": the step equals the oracle's with the seeds the module
    drew from the global CPU generator (one per chunk, as the reference draws them, chunked.py:126)."""
    import torch
    from test_host_cpu import make_cfg
    from xmc_classifiers.chunked import XMCBCECHUNKEDLayer
    cfg = make_cfg("cuda:0", 1000, 3, rounding="sr_fast")
    cfg.model.xmc.dtype = "bfloat16"
    torch.manual_seed(3)
    xfc = XMCBCECHUNKEDLayer(cfg)
    emb = torch.randn(32, 768, device=gpu, dtype=torch.bfloat16)
    labels = torch.tensor([[0, 3], [1, 999], [5, 17], [31, 500]], dtype=torch.int32, device=gpu)
    w0 = xfc.xfc_weight.float().cpu().numpy()
    torch.manual_seed(11)
    seeds = [torch.randint(0, 1000000, (1,)).item() for _ in range(3)]
    torch.manual_seed(11)
    xfc.xfc_forward_backward(emb, labels, [0.5], skip_loss=True)
    x_np = emb.float().cpu().numpy()
    ref_w, _, _ = O.bf16_step(w0, x_np, labels.cpu().numpy(), 0.5, 3, seeds=seeds, sr_mode="fast")
    check_bf16_weights(xfc.xfc_weight.float().cpu().numpy(), ref_w, w0, x_np, lr=0.5)
    rtn_w, _, _ = O.bf16_step(w0, x_np, labels.cpu().numpy(), 0.5, 3, sr_mode="rtn")
    assert (xfc.xfc_weight.float().cpu().numpy() != rtn_w).mean() > 0.1
