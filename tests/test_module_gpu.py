"""The drop-in classifier module driven exactly as the reference's training loop and evaluator drive it
(src/runner.py:139-157, src/evaluate.py:153-159), with a stub encoder in place of the transformer."""
import io

import numpy as np
import pytest

import helpers as H
from test_host_cpu import make_cfg
from oracle import codecs as C
from oracle import step as O

pytestmark = pytest.mark.gpu


def build(gpu, num_labels=1000, num_chunks=2, **extra):
    import torch
    from xmc_classifiers.chunked_fp8xmc_clf import Fp8XMCBCEChunkedLayer
    torch.manual_seed(0)
    return Fp8XMCBCEChunkedLayer(make_cfg("cuda:0", num_labels, num_chunks, **extra))


def test_construction_matches_reference_layout(gpu):
    import torch
    xfc = build(gpu, 1000, 2)
    assert xfc.num_labels == 1000 + 32 - 1000 % 32 == 1024 and xfc.num_labels_i == 512      # padding rule
    assert xfc._dtype == torch.float8_e4m3fn and len(xfc.xfc_weight) == 2
    assert all(w.dtype == torch.float8_e4m3fn and w.shape == (512, 768) and not w.requires_grad and w.is_cuda
               for w in xfc.xfc_weight)
    assert sorted(xfc.state_dict().keys()) == ["xfc_weight.0", "xfc_weight.1"]
    # xavier-uniform bound sqrt(6 / (L_pad + d)) before the cast: every code decodes inside it (plus rounding)
    bound = np.sqrt(6.0 / (1024 + 768))
    w = C.e4m3_decode(xfc.xfc_weight[0].view(torch.uint8).cpu().numpy())
    assert np.abs(w).max() <= bound * 1.07 and np.abs(w).max() > bound * 0.8
    xfc2 = build(gpu, 1024, 2)
    assert xfc2.num_labels == 1056                     # already aligned: a full extra group of 16 * num_chunks


def test_training_call_contract(gpu):
    import torch
    xfc = build(gpu, 1000, 2, rounding="rtn")
    assert xfc.last_step_error() == 0                   # nothing has run yet
    enc = torch.nn.Linear(768, 768, bias=False).to(gpu).to(torch.bfloat16)
    torch.manual_seed(1)
    tokens = torch.randn(32, 768, device=gpu, dtype=torch.bfloat16)
    labels = torch.tensor([[0, 3], [0, 999], [5, 17], [31, 500], [31, 500]], dtype=torch.int32, device=gpu)
    ptrs = [w.data_ptr() for w in xfc.xfc_weight]
    before = [w.view(torch.uint8).clone() for w in xfc.xfc_weight]

    out = enc(tokens)                                   # has grad_fn
    out_copy = out.detach().clone()
    grad_fn = out.grad_fn
    loss = xfc.xfc_forward_backward(out, labels, [0.05], skip_loss=True)
    assert loss == 0 and xfc.iteration == 1
    assert xfc.last_step_error() == 0                   # no workgroup gave up waiting
    assert torch.equal(out.detach().view(torch.int16), out_copy.view(torch.int16)) and out.grad_fn is grad_fn
    g = xfc.grad_input
    assert g.shape == (32, 768) and g.dtype == out.dtype and g.is_cuda
    g[0:32, :].div_(2)                                  # runner.py:155 (gradient accumulation)
    out.backward(g[0:32, :])                            # runner.py:157
    expect = (g.float().t() @ tokens.float())           # closed form of the stub's weight gradient
    assert torch.allclose(enc.weight.grad.float(), expect, rtol=2e-2, atol=2e-2 * expect.abs().max().item())
    # weights were updated in place
    assert [w.data_ptr() for w in xfc.xfc_weight] == ptrs
    assert any(not torch.equal(a, w.view(torch.uint8)) for a, w in zip(before, xfc.xfc_weight))
    # parity of this exact call with the oracle
    chunks_np = [b.cpu().numpy() for b in before]
    x_np = out_copy.float().cpu().numpy()
    ref_codes, ref_gx, ref_gb = O.fp8_step(chunks_np, x_np, labels.cpu().numpy(), 0.05, sr_mode="rtn")
    for w, r in zip(xfc.xfc_weight, ref_codes):
        assert H.e4m3_ulp_distance(w.view(torch.uint8).cpu().numpy(), r).max() <= 1
    assert np.abs(g.float().cpu().numpy() * 2 - ref_gb).max() <= 2e-2 * np.abs(ref_gb).max()


def test_module_options_for_weight_decay_and_fused_dropout(gpu):
    """training.xmc.fp8_weight_decay and training.xmc.fused_dropout (absent: the reference's behaviour, checked by every
    other test of this file): the step equals the oracle's with the same options and the seed the module drew from the
    global CPU generator after the chunk seeds; in eval mode no dropout is applied."""
    import torch
    xfc = build(gpu, 1000, 2, rounding="rtn", fp8_weight_decay=0.2, fused_dropout=0.25)
    before = [w.view(torch.uint8).cpu().numpy().copy() for w in xfc.xfc_weight]
    torch.manual_seed(3)
    x = (0.05 * torch.randn(32, 768, device=gpu)).to(torch.bfloat16)
    labels = torch.tensor([[0, 3], [0, 999], [5, 17], [31, 500]], dtype=torch.int32, device=gpu)
    torch.manual_seed(77)
    xfc.train()
    xfc.xfc_forward_backward(x, labels, [0.5])
    torch.manual_seed(77)
    for _ in range(2):
        torch.randint(0, 1000000, (1,)).item()
    dseed = torch.randint(0, 2 ** 62, (1,)).item()
    ref_codes, ref_gx, ref_gb = O.fp8_step(before, x.float().cpu().numpy(), labels.cpu().numpy(), 0.5, weight_decay=0.2,
                                           dropout_p=0.25, dropout_seed=dseed)
    for w, r in zip(xfc.xfc_weight, ref_codes):
        d = H.e4m3_ulp_distance(w.view(torch.uint8).cpu().numpy(), r)
        assert d.max() <= 1 and (d != 0).mean() < 2e-3
    g = xfc.grad_input.float().cpu().numpy()
    assert np.array_equal(g == 0, ref_gb == 0)                     # the same mask
    assert np.abs(g - ref_gb).max() <= 2e-2 * np.abs(ref_gb).max()
    xfc.eval()
    mid = [w.view(torch.uint8).cpu().numpy().copy() for w in xfc.xfc_weight]
    xfc.xfc_forward_backward(x, labels, [0.5])
    ref_codes = O.fp8_step(mid, x.float().cpu().numpy(), labels.cpu().numpy(), 0.5, weight_decay=0.2)[0]
    for w, r in zip(xfc.xfc_weight, ref_codes):
        assert H.e4m3_ulp_distance(w.view(torch.uint8).cpu().numpy(), r).max() <= 1
    assert xfc.last_step_error() == 0


def test_default_rounding_draws_seeds_from_the_global_cpu_generator(gpu):
    import torch
    xfc = build(gpu, 500, 3)
    assert xfc.rounding == "sr_fast"
    x = torch.randn(16, 768, device=gpu).to(torch.bfloat16)
    labels = torch.zeros((0, 2), dtype=torch.int32, device=gpu)
    torch.manual_seed(123)
    expected_next = None
    xfc.xfc_forward_backward(x, labels, [0.05])
    after = torch.randint(0, 1000000, (1,)).item()
    torch.manual_seed(123)
    for _ in range(3):                                   # one draw per chunk, as chunked_fp8xmc_clf.py:113
        torch.randint(0, 1000000, (1,)).item()
    assert torch.randint(0, 1000000, (1,)).item() == after


def test_evaluator_contract_and_checkpoint_roundtrip(gpu):
    import torch
    xfc = build(gpu, 1000, 2)
    torch.manual_seed(2)
    embed = torch.randn(40, 768, device=gpu).to(torch.bfloat16)
    logits = xfc.xfc_forward(embed.to(xfc._dtype))       # evaluate.py:155-158
    assert logits.shape == (40, 1000) and logits.dtype == torch.bfloat16
    vals, idx = torch.topk(logits, k=5)                  # evaluate.py:159
    chunks_np = [w.view(torch.uint8).cpu().numpy() for w in xfc.xfc_weight]
    ref = O.fp8_forward(chunks_np, embed.float().cpu().numpy(), 1000)
    H.assert_bf16_close(logits.float().cpu().numpy(), ref)
    ref_top = np.argsort(-ref, axis=1, kind="stable")[:, :5]
    assert np.mean(np.sort(ref_top, axis=1) == np.sort(idx.cpu().numpy(), axis=1)) > 0.97
    # the same top-k without the dense logits: values equal, ids equal wherever the library routine's choice is unique
    tv, ti = xfc.xfc_forward_topk(embed.to(xfc._dtype), 5)
    assert torch.equal(tv, vals)
    assert torch.equal(logits.gather(1, ti), vals) and ti.dtype == torch.int64
    same = ti == idx
    assert same.float().mean() > 0.9
    # runner.py:246 pickles xfc.xfc_weight with torch.save; :257 assigns it back
    buf = io.BytesIO()
    torch.save({"xfc_weight": xfc.xfc_weight, "model": xfc.state_dict()}, buf)
    buf.seek(0)
    ck = torch.load(buf, weights_only=False)
    for a, b in zip(ck["xfc_weight"], xfc.xfc_weight):
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    xfc.load_state_dict(ck["model"])


def test_error_convention(gpu):
    import torch
    xfc = build(gpu, 1000, 2)
    labels = torch.zeros((0, 2), dtype=torch.int32, device=gpu)
    with pytest.raises(AssertionError):
        xfc.xfc_forward_backward(torch.randn(17, 768, device=gpu).to(torch.bfloat16), labels, [0.05])
    with pytest.raises(AssertionError):
        xfc.xfc_forward_backward(torch.randn(16, 512, device=gpu).to(torch.bfloat16), labels, [0.05])
    with pytest.raises(AssertionError):
        xfc.xfc_forward_backward(torch.randn(16, 768).to(torch.bfloat16), labels, [0.05])
    with pytest.raises(AssertionError):      # the simulated mode has no fast stochastic rounding and no scales
        build(gpu, 1000, 2, simulated=True, rounding="sr_fast")
    with pytest.raises(AssertionError):
        build(gpu, 1000, 2, simulated=True, scale_w=0.5)


def test_simulated_mode_forward_uses_the_unquantised_embedding(gpu):
    """chunked_fp8xmc_clf.py:51-52: in simulated-FP8 mode the inference logits are matmul(embed.bf16, W.bf16) - the
    embedding is NOT quantised to e4m3 there (the true-FP8 branch :53-56 quantises it).  Checked against the closed form
    on the CPU (exact products of bf16 x e4m3 values summed in float64, rounded to bf16) for a bf16 embedding, and
    against the true-FP8 layer for an embedding the evaluator has already cast to e4m3 (evaluate.py:155-156)."""
    import torch
    xfc = build(gpu, 1000, 2, simulated=True)
    xfc8 = build(gpu, 1000, 2)
    for a, b in zip(xfc8.xfc_weight, xfc.xfc_weight):
        a.data.copy_(b.data)
    torch.manual_seed(4)
    embed = torch.randn(24, 768, device=gpu).to(torch.bfloat16)
    logits = xfc.xfc_forward(embed)
    assert logits.shape == (24, 1000) and logits.dtype == torch.bfloat16
    w = np.concatenate([C.e4m3_decode(p.view(torch.uint8).cpu().numpy()) for p in xfc.xfc_weight])[:1000]
    x = embed.float().cpu().numpy()
    exact = x.astype(np.float64) @ w.astype(np.float64).T
    H.assert_bf16_close(logits.float().cpu().numpy(), C.bf16_round(exact.astype(np.float32)))
    # the quantised product differs visibly: the two modes must not be confused
    q = xfc8.xfc_forward(embed).float().cpu().numpy()
    assert np.abs(q - exact).max() > 4 * np.abs(logits.float().cpu().numpy() - exact).max()
    # an embedding that is already e4m3 gives the same logits in both modes, up to the summation order of the GEMM
    e8 = embed.to(torch.float8_e4m3fn)
    H.assert_bf16_close(xfc.xfc_forward(e8).float().cpu().numpy(), xfc8.xfc_forward(e8).float().cpu().numpy())
    tv, ti = xfc.xfc_forward_topk(embed, 5)
    assert torch.equal(tv, logits.topk(5).values) and torch.equal(logits.gather(1, ti), tv)


def test_module_reports_a_failed_step_without_synchronising(gpu):
    """The last kernel of every fused step ORs the step's error word into a sticky word of the workspace, and the module
    sends that word to pinned host memory behind every step; a later call raises once a non-zero copy has arrived.  The
    failure is staged from the host (the step's error word is overwritten on the stream between the step kernel and
    nothing else: here the sticky word itself, as the step's last kernel would have left it), every kernel runs
    normally.  Further steps are enqueued behind the failed one without any synchronisation before the check: their
    clean error words must not hide the failure."""
    import torch
    xfc = build(gpu, 1000, 2, rounding="rtn")
    x = torch.randn(16, 768, device=gpu).to(torch.bfloat16)
    labels = torch.zeros((0, 2), dtype=torch.int32, device=gpu)
    xfc.xfc_forward_backward(x, labels, [0.05])
    torch.cuda.synchronize()
    xfc._check_previous_steps()                          # a clean step: nothing raised
    assert int(xfc._err_host.sum()) == 0 and int(xfc._err_dev.item()) == 0
    xfc._err_dev.fill_(2)                                # as if the placement check of a step had failed
    raised = 0
    for _ in range(8):                                   # clean steps behind it, no synchronisation: one of these calls
        try:                                             # (whichever finds a copy of the word arrived) reports it
            xfc.xfc_forward_backward(x, labels, [0.05])
        except RuntimeError as e:
            assert "XCD" in str(e)
            raised += 1
    assert raised == 1                                   # reported once: the word was cleared, later steps run
    assert xfc.last_step_error() == 0                    # the last step itself was clean (synchronises)
    xfc.check_steps()
    # the end-of-run check finds a failure of the very last step
    xfc.xfc_forward_backward(x, labels, [0.05])
    xfc._err_dev.fill_(1)
    with pytest.raises(RuntimeError, match="gave up"):
        xfc.check_steps()
    xfc.check_steps()


def test_step_kernels_keep_the_sticky_error_word(gpu):
    """Through the C ABI: a step's error word lands in the sticky word, which later steps do not clear."""
    import torch
    import ctypes
    from elmo_amd import ops, _lib
    dev = gpu
    chunks = [torch.zeros(64, 768, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)]
    x = torch.zeros(16, 768, dtype=torch.bfloat16, device=dev)
    labels = torch.zeros((0, 2), dtype=torch.int32, device=dev)
    ws = ops.alloc_workspace(1, 64, dev)
    soff, eoff = ops.step_sticky_error_offset(), ops.step_error_offset()
    sticky = ws[soff:soff + 4].view(torch.int32)
    assert int(sticky.item()) == 0
    ops.fp8_step(chunks, x, labels, 0.05, round_mode="rtn", workspace=ws)
    assert int(sticky.item()) == 0 and ops.step_error_word(ws, 1, 64) == 0
    sticky.fill_(4)                                      # a bit no kernel sets: must survive the following steps
    ops.fp8_step(chunks, x, labels, 0.05, round_mode="rtn", workspace=ws)
    ops.fp8_step(chunks, x, labels, 0.05, round_mode="rtn", workspace=ws)
    assert int(sticky.item()) == 4 and ops.step_error_word(ws, 1, 64) == 0


def test_give_up_path_of_the_fused_step(gpu):
    """The bounded waits of the fused step, forced to expire from the host (a polling limit of 0: a wait that is not
    satisfied at once gives up).  Every kernel must still exit normally; the step's error word and the sticky word
    carry bit 0; and no weight may be updated from missing data: a member's quarter of a row either keeps its old codes or
    holds the oracle's update, because a workgroup that gives up finishes the tile whose G is complete and stops before the next.
    The next step with the default limit is clean again, and the module turns the sticky word into an exception."""
    import torch
    from elmo_amd import ops
    from test_host_cpu import make_cfg
    from xmc_classifiers.chunked_fp8xmc_clf import Fp8XMCBCEChunkedLayer
    nc, rows, batch = 3, 16384, 64            # 768 tiles: twelve per quad, enough for the members to drift apart
    case = H.make_case(nc, rows, batch, 301)
    chunks, x, labels = H.to_device_case(case, gpu)
    ws = ops.alloc_workspace(nc, rows, gpu)
    soff = ops.step_sticky_error_offset()
    sticky = ws[soff:soff + 4].view(torch.int32)
    ref_codes, _, _ = O.fp8_step(case["chunks"], case["x"], case["labels"], 0.05, sr_mode="rtn")
    prev = ops.debug_spin_limit(0)
    try:
        gave_up = False
        for attempt in range(8):              # whether a wait finds its counter at once depends on timing
            for c, old in zip(chunks, case["chunks"]):
                c.view(torch.uint8).copy_(torch.from_numpy(old))
            ops.fp8_step(chunks, x, labels, 0.05, round_mode="rtn", workspace=ws)
            torch.cuda.synchronize()          # the kernels ran to their end
            word = ops.step_error_word(ws, nc, rows)
            assert word in (0, 1)
            new = H.chunks_to_numpy(chunks)
            updated = total = 0
            for a, old, ref in zip(new, case["chunks"], ref_codes):
                # the unit of the update is a member's feature quarter of a row (the members of a quad stop at
                # different tiles)
                same_old = (a == old).reshape(-1, 4, 192).all(axis=2)
                good = (H.e4m3_ulp_distance(a, ref) <= 1).reshape(-1, 4, 192).all(axis=2)
                assert np.all(same_old | good), "a row segment was updated from incomplete data"
                updated += int((~same_old).sum()); total += same_old.size
            if word == 1:
                gave_up = True
                assert int(sticky.item()) & 1
                assert updated < total        # the step stopped early
                break
        assert gave_up, "no wait expired in eight steps with a polling limit of 0"
    finally:
        assert ops.debug_spin_limit(prev) == 0
    # the default limit again: a clean, complete step; the sticky word keeps the earlier failure until the caller clears it
    for c, old in zip(chunks, case["chunks"]):
        c.view(torch.uint8).copy_(torch.from_numpy(old))
    ops.fp8_step(chunks, x, labels, 0.05, round_mode="rtn", workspace=ws)
    assert ops.step_error_word(ws, nc, rows) == 0 and int(sticky.item()) & 1
    for a, ref in zip(H.chunks_to_numpy(chunks), ref_codes):
        assert H.e4m3_ulp_distance(a, ref).max() <= 1
    # the module raises for such a step
    cfg = make_cfg("cuda:0", 3 * 16384 - 48, 3, rounding="rtn")
    cfg.data.batch_size = batch
    xfc = Fp8XMCBCEChunkedLayer(cfg)
    prev = ops.debug_spin_limit(0)
    try:
        raised = False
        for attempt in range(8):
            try:
                xfc.xfc_forward_backward(x, labels, [0.05])
                xfc.check_steps()
            except RuntimeError as e:
                raised = "gave up waiting" in str(e)
                break
        assert raised
    finally:
        ops.debug_spin_limit(prev)
    xfc.xfc_forward_backward(x, labels, [0.05])
    xfc.check_steps()
