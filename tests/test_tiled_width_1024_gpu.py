"""The three-kernel path at 1024 input features (the width of the reference's large encoders; 768 is covered by
test_tiled_gpu.py): bf16 layer, simulated-FP8 mode, true-FP8 arithmetic and the head-Kahan update, through the C ABI,
against the CPU oracle, which is written for any width.  Tolerances as in test_tiled_gpu.py."""
import numpy as np
import pytest

import helpers as H
from elmo_amd import synth
from oracle import codecs as C
from oracle import step as O
from test_tiled_gpu import check_bf16_weights, check_gx

pytestmark = pytest.mark.gpu

FEATS = 1024


def bf16_case(L, batch, seed, pos_mean=5.0):
    x = synth.make_x(batch, FEATS, seed)
    w = C.bf16_round(synth.make_weights_np(L, FEATS, seed, 0.02))
    labels = synth.make_labels(batch, L, pos_mean, 1.0, seed).astype(np.int32)
    return x, w, labels


def run_bf16(x, w, labels, nc, device, mode, seeds, lr=0.05, **kw):
    import torch
    from elmo_amd import ops
    L = w.shape[0]
    cs = (L + nc - 1) // nc
    wt = torch.from_numpy(C.bf16_bits(w).view(np.int16)).to(device).view(torch.bfloat16)
    views = [wt[c * cs:min((c + 1) * cs, L)] for c in range(nc) if c * cs < L]
    xt = torch.from_numpy(C.bf16_bits(x).view(np.int16)).to(device).view(torch.bfloat16)
    lab = torch.from_numpy(labels).to(device).contiguous()
    g, gf = ops.tiled_step(views, cs, "bf16", xt, lab, lr, seeds=seeds, round_mode=mode, want_f32=True, **kw)
    assert g.shape == (x.shape[0], FEATS)
    return wt.float().cpu().numpy(), gf.cpu().numpy(), g.float().cpu().numpy()


def code_mismatch(new, ref):
    mism = total = 0
    for a, b in zip(new, ref):
        d = H.e4m3_ulp_distance(a, b)
        assert d.max() <= 1
        mism += int((d != 0).sum()); total += d.size
    return mism / total


@pytest.mark.parametrize("L,nc,batch,seed", [
    (64, 1, 16, 131),           # a single tile
    (1000, 3, 24, 132),         # ragged chunks, batch not a multiple of 16
    (20011, 4, 128, 133),       # prime label count, full first half
    (3000, 2, 200, 134),        # two batch halves, the second one short
    (1300, 3, 512, 135),        # four halves
])
def test_bf16_layer_rtn_parity(gpu, L, nc, batch, seed):
    x, w, labels = bf16_case(L, batch, seed)
    new, gf, gb = run_bf16(x, w, labels, nc, gpu, "rtn", None)
    ref_w, ref_gx, _ = O.bf16_step(w, x, labels, 0.05, nc, sr_mode="rtn")
    check_bf16_weights(new, ref_w, w, x)
    check_gx(gf, gb, ref_gx, tol=4e-3)


def test_bf16_layer_stochastic_rounding_decay_dropout_and_loss(gpu):
    import torch
    from elmo_amd import ops
    L, nc, batch = 3000, 3, 40
    x, w, labels = bf16_case(L, batch, 141)
    seeds = [12345, 999999, 7]
    # the reference's recipe: the Philox offset of a weight is row * 1024 + column
    new, gf, gb = run_bf16(x, w, labels, nc, gpu, "sr_philox", seeds)
    ref_w, ref_gx, _ = O.bf16_step(w, x, labels, 0.05, nc, seeds=seeds, sr_mode="reference")
    check_bf16_weights(new, ref_w, w, x)
    rtn_w, _, _ = O.bf16_step(w, x, labels, 0.05, nc, sr_mode="rtn")
    assert (new != rtn_w).mean() > 0.2
    # the fast mode: one hash per four weights of a row, index = row * 256 + column / 4
    new, gf, gb = run_bf16(x, w, labels, nc, gpu, "sr_fast", seeds)
    ref_w, _, _ = O.bf16_step(w, x, labels, 0.05, nc, seeds=seeds, sr_mode="fast")
    check_bf16_weights(new, ref_w, w, x)
    assert (new != rtn_w).mean() > 0.2
    # weight decay and dropout of X (offset of an element: row * 1024 + column)
    dseed = 0x1357_9BDF_2468
    new, gf, gb = run_bf16(x, w, labels, nc, gpu, "rtn", None, lr=0.5, weight_decay=0.02, dropout_p=0.1, dropout_seed=dseed)
    ref_w, ref_gx, _ = O.bf16_step(w, x, labels, 0.5, nc, weight_decay=0.02, dropout_p=0.1, dropout_seed=dseed)
    check_bf16_weights(new, ref_w, w, x, lr=0.5)
    check_gx(gf, gb, ref_gx, tol=4e-3)
    keep = C.dropout_bf16(x, 0.1, dseed)[1]
    assert np.all(gf[~keep] == 0) and np.any(gf[keep] != 0)
    # loss fused into the logits kernel
    w2 = C.bf16_round(synth.make_weights_np(L, FEATS, 142, 1.0))
    wt = torch.from_numpy(C.bf16_bits(w2).view(np.int16)).to(gpu).view(torch.bfloat16)
    xt = torch.from_numpy(C.bf16_bits(x).view(np.int16)).to(gpu).view(torch.bfloat16)
    cs = L // nc
    loss = torch.zeros(1, dtype=torch.float32, device=gpu)
    ops.tiled_step([wt[c * cs:(c + 1) * cs] for c in range(nc)], cs, "bf16", xt, torch.from_numpy(labels).to(gpu), 0.0,
                   round_mode="rtn", loss_out=loss)
    ref_loss = O.bf16_step(w2, x, labels, 0.0, nc, sr_mode="rtn", return_loss=True)[3]
    assert abs(loss.item() - ref_loss) <= 1e-4 * abs(ref_loss), (loss.item(), ref_loss)


@pytest.mark.parametrize("nc,rows,batch,seed", [(1, 64, 16, 161), (3, 208, 32, 162), (2, 4096, 128, 163), (2, 1024, 256, 164)])
def test_simulated_fp8_parity(gpu, nc, rows, batch, seed):
    from elmo_amd import ops
    case = H.make_case(nc, rows, batch, seed, features=FEATS)
    chunks, x, labels = H.to_device_case(case, gpu)
    g, gf = ops.tiled_step(chunks, rows, "e4m3", x, labels, 0.05, round_mode="rtn", want_f32=True)
    ref_codes, ref_gx, _ = O.fp8_step(case["chunks"], case["x"], case["labels"], 0.05, sr_mode="rtn", simulated=True)
    assert code_mismatch(H.chunks_to_numpy(chunks), ref_codes) < 2e-3
    check_gx(gf.cpu().numpy(), g.float().cpu().numpy(), ref_gx)
    # the reference's stochastic rounding
    seeds = [424242 + c for c in range(nc)]
    chunks, x, labels = H.to_device_case(case, gpu)
    ops.tiled_step(chunks, rows, "e4m3", x, labels, 0.05, seeds=seeds, round_mode="sr_philox")
    ref_codes, _, _ = O.fp8_step(case["chunks"], case["x"], case["labels"], 0.05, seeds=seeds, sr_mode="reference",
                                 simulated=True)
    assert code_mismatch(H.chunks_to_numpy(chunks), ref_codes) < 2e-3


@pytest.mark.parametrize("batch", [32, 256, 512])
def test_true_fp8_arithmetic(gpu, batch):
    """quantize_x + saturate: logits from e4m3(X), saturating cast of the updated weights; round to nearest and the fast
    stochastic rounding (index of a group of four weights: global row * 256 + column / 4)."""
    from elmo_amd import ops
    nc, rows = 2, 1008
    case = H.make_case(nc, rows, batch, 171, pos_mean=4.0, features=FEATS)
    chunks, x, labels = H.to_device_case(case, gpu)
    g, gf = ops.tiled_step(chunks, rows, "e4m3", x, labels, 0.05, round_mode="rtn", want_f32=True, quantize_x=True,
                           saturate=True)
    ref_codes, ref_gx, _ = O.fp8_step(case["chunks"], case["x"], case["labels"], 0.05, sr_mode="rtn")
    assert code_mismatch(H.chunks_to_numpy(chunks), ref_codes) < 2e-3
    check_gx(gf.cpu().numpy(), g.float().cpu().numpy(), ref_gx)
    seeds = [31337, 4242]

    def rand_fn(c, offs):
        r, k = offs // FEATS, offs % FEATS
        return C.fast_sr_words(seeds[c], c * rows + r, k, FEATS)

    chunks, x, labels = H.to_device_case(case, gpu)
    ops.tiled_step(chunks, rows, "e4m3", x, labels, 0.05, seeds=seeds, round_mode="sr_fast", quantize_x=True, saturate=True)
    ref, _, _ = O.fp8_step(case["chunks"], case["x"], case["labels"], 0.05, sr_mode="exact", rand_fn=rand_fn)
    assert code_mismatch(H.chunks_to_numpy(chunks), ref) < 2e-3


@pytest.mark.parametrize("ktype,mode", [("bf16", "rtn"), ("bf16", "sr_philox"), ("e5m2", "rtn")])
def test_head_kahan(gpu, ktype, mode):
    import torch
    from elmo_amd import ops
    nc, rows, batch, nh = 2, 512, 32, 208
    case = H.make_case(nc, rows, batch, 181, features=FEATS)
    rng = np.random.default_rng(2)
    k0 = rng.standard_normal((nh, FEATS)).astype(np.float32) * 1e-3
    k0 = C.e5m2_encode(k0) if ktype == "e5m2" else C.bf16_round(k0)
    seeds = [77, 88] if mode != "rtn" else None
    chunks, x, labels = H.to_device_case(case, gpu)
    if ktype == "e5m2":
        kt = torch.from_numpy(k0.copy()).to(gpu).view(torch.float8_e5m2)
    else:
        kt = torch.from_numpy(C.bf16_bits(k0).view(np.int16)).to(gpu).view(torch.bfloat16)
    g, gf = ops.tiled_step(chunks, rows, "e4m3", x, labels, 0.05, seeds=seeds, round_mode=mode, want_f32=True,
                           quantize_x=True, saturate=True, kahan=kt, num_head=nh)
    ref_codes, ref_k, ref_gx, _ = O.fp8_kahan_step(case["chunks"], k0, case["x"], case["labels"], 0.05, nh, kahan_type=ktype,
                                                   seeds=seeds, sr_mode={"rtn": "rtn", "sr_philox": "reference"}[mode])
    new = H.chunks_to_numpy(chunks)
    assert code_mismatch(new, ref_codes) < 4e-3
    check_gx(gf.cpu().numpy(), g.float().cpu().numpy(), ref_gx)
    # weight + compensation term, the quantity the buffer exists to preserve
    if ktype == "e5m2":
        kn, rf = C.e5m2_decode(kt.view(torch.uint8).cpu().numpy()), C.e5m2_decode(ref_k)
    else:
        kn, rf = kt.float().cpu().numpy(), ref_k
    tot_g = C.e4m3_decode(new[0][:nh]).astype(np.float64) + kn
    tot_r = C.e4m3_decode(ref_codes[0][:nh]).astype(np.float64) + rf
    assert np.abs(tot_g - tot_r).max() <= (2.0 ** -2 if ktype == "e5m2" else 2.0 ** -6) * np.abs(rf).max() + 2.0 ** -16


def test_unsupported_widths_are_refused(gpu):
    import torch
    from elmo_amd import _lib, ops
    for feats in (64, 512, 896, 2048):
        w = torch.zeros(64, feats, dtype=torch.bfloat16, device=gpu)
        x = torch.zeros(16, feats, dtype=torch.bfloat16, device=gpu)
        lab = torch.zeros(0, 2, dtype=torch.int32, device=gpu)
        with pytest.raises(AssertionError):
            ops.tiled_step([w], 64, "bf16", x, lab, 0.05)
        assert _lib.load().xmc_tiled_workspace_bytes_ex(1, 64, 16, feats) == 0


def test_chunked_module_at_1024(gpu):
    """XMCBCECHUNKEDLayer with input_features = 1024: two steps against the oracle, inference through the BLAS."""
    import torch
    from test_host_cpu import make_cfg
    from xmc_classifiers.chunked import XMCBCECHUNKEDLayer
    cfg = make_cfg("cuda:0", 3000, 3, rounding="rtn")
    cfg.model.xmc.dtype = "bfloat16"
    cfg.model.xmc.input_features = FEATS
    cfg.data.batch_size = 48
    torch.manual_seed(5)
    xfc = XMCBCECHUNKEDLayer(cfg)
    assert xfc.xfc_weight.shape == (3000, FEATS)
    w = xfc.xfc_weight.float().cpu().numpy()
    for it in range(2):
        x = synth.make_x(48, FEATS, 190 + it)
        labels = synth.make_labels(48, 3000, 5.0, 1.0, 190 + it).astype(np.int32)
        emb = torch.from_numpy(C.bf16_bits(x).view(np.int16)).to(gpu).view(torch.bfloat16)
        assert xfc.xfc_forward_backward(emb, torch.from_numpy(labels).to(gpu), [0.05]) == 0
        ref_w, ref_gx, ref_gi = O.bf16_step(w, x, labels, 0.05, 3, sr_mode="rtn")
        check_bf16_weights(xfc.xfc_weight.float().cpu().numpy(), ref_w, w, x)
        assert xfc.grad_input.shape == (48, FEATS)
        H.assert_bf16_close(xfc.grad_input.float().cpu().numpy(), ref_gi, floor_rel=4e-3)
        w = xfc.xfc_weight.float().cpu().numpy()
    logits = xfc.xfc_forward(emb)
    assert logits.shape == (48, 3000)


def test_fp8_modules_at_1024(gpu):
    """Fp8XMCBCEChunkedLayer and the head-Kahan layer with input_features = 1024: the step runs on the three-kernel path
    with the true-FP8 arithmetic (oracle: fp8_step / fp8_kahan_step), inference through a library GEMM per chunk on the
    exactly widened operands (oracle: fp8_forward, whose products are the same and whose fp32 sums differ in order)."""
    import types
    import torch
    from test_host_cpu import make_cfg
    from xmc_classifiers.chunked_fp8xmc_clf import Fp8XMCBCEChunkedLayer
    from xmc_classifiers.chunked_head_kahan_fp8xmc_clf import Fp8XMCBCEChunkedHeadKahanLayer
    cfg = make_cfg("cuda:0", 2000, 2, rounding="rtn")
    cfg.model.xmc.input_features = FEATS
    torch.manual_seed(7)
    xfc = Fp8XMCBCEChunkedLayer(cfg)
    assert [tuple(w.shape) for w in xfc.xfc_weight] == [(1008, FEATS)] * 2 and xfc._dtype == torch.float8_e4m3fn
    x = synth.make_x(48, FEATS, 201)
    labels = synth.make_labels(48, 2000, 5.0, 1.0, 201).astype(np.int32)
    emb = torch.from_numpy(C.bf16_bits(x).view(np.int16)).to(gpu).view(torch.bfloat16)
    w0 = [w.data.view(torch.uint8).cpu().numpy().copy() for w in xfc.xfc_weight]
    assert xfc.xfc_forward_backward(emb, torch.from_numpy(labels).to(gpu), [0.05]) == 0 and xfc.iteration == 1
    ref_codes, ref_gx, ref_gi = O.fp8_step(w0, x, labels, 0.05, sr_mode="rtn")
    assert code_mismatch([w.data.view(torch.uint8).cpu().numpy() for w in xfc.xfc_weight], ref_codes) < 2e-3
    assert xfc.grad_input.shape == (48, FEATS) and xfc.grad_input.dtype == torch.bfloat16
    H.assert_bf16_close(xfc.grad_input.float().cpu().numpy(), ref_gi)
    assert xfc.last_step_error() == 0
    xfc.check_steps()
    # inference: as the evaluator calls it (embedding cast to the layer's type first), dense and top-k
    w1 = [w.data.view(torch.uint8).cpu().numpy() for w in xfc.xfc_weight]
    logits = xfc.xfc_forward(emb.to(xfc._dtype))
    ref = O.fp8_forward(w1, x, 2000)
    assert logits.shape == (48, 2000) and logits.dtype == torch.bfloat16
    H.assert_bf16_close(logits.float().cpu().numpy(), ref)
    vals, idx = xfc.xfc_forward_topk(emb.to(xfc._dtype), 10)
    tv, ti = logits.topk(10)
    assert torch.equal(vals, tv) and torch.equal(idx, ti)
    # the default rounding of this width is the fast stochastic one, on the same path
    cfg_sr = make_cfg("cuda:0", 2000, 2)
    cfg_sr.model.xmc.input_features = FEATS
    xfc_sr = Fp8XMCBCEChunkedLayer(cfg_sr)
    assert xfc_sr.rounding == "sr_fast" and xfc_sr.xfc_forward_backward(emb, torch.from_numpy(labels).to(gpu), [0.05]) == 0

    # head-Kahan layer
    cfgk = make_cfg("cuda:0", 1000, 2, rounding="rtn")
    cfgk.model.xmc.input_features = FEATS
    cfgk.training.FP8 = types.SimpleNamespace(using_head_kahan=True, fp8_head_kahan=False, head_ratio=0.2)
    torch.manual_seed(8)
    xk = Fp8XMCBCEChunkedHeadKahanLayer(cfgk)
    assert xk.num_labels == 1024 and xk.num_head == 204 and xk.head_kahan.shape == (204, FEATS)
    tokens = emb[:32]
    lab = torch.tensor([[0, 3], [31, 999], [4, 100]], dtype=torch.int32, device=gpu)
    before = [w.view(torch.uint8).cpu().numpy().copy() for w in xk.xfc_weight]
    assert xk.xfc_forward_backward(tokens, lab, [0.05]) == 0
    ref_codes, ref_k, _, _ = O.fp8_kahan_step(before, np.zeros((204, FEATS), np.float32), x[:32], lab.cpu().numpy(), 0.05, 204,
                                              sr_mode="rtn")
    assert code_mismatch([w.view(torch.uint8).cpu().numpy() for w in xk.xfc_weight], ref_codes) < 2e-3
    assert float(xk.head_kahan.float().abs().max()) > 0
    assert xk.xfc_forward(tokens.to(xk._dtype)).shape == (32, 1000)
