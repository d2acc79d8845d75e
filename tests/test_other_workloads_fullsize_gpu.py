"""The other benchmark workloads at their full sizes, through properties that do not need the whole oracle where the
whole oracle would take minutes: sampled label rows against the oracle after a real round-to-nearest step (the update
of a row depends only on that row, X and the positives), lr = 0 leaves every weight unchanged, grad_X against library
GEMMs.  The bf16 workload is small enough for the whole oracle.  Tolerances as in the small-size parity tests."""
import numpy as np
import pytest

import helpers as H
from elmo_amd import synth
from oracle import codecs as C
from oracle import step as O

pytestmark = pytest.mark.gpu


def make_fp8_workload(name, device):
    import torch
    cfg = synth.CONFIGS[name]
    nc = cfg.num_chunks
    rows = O.fp8_padded_labels(cfg.num_labels, nc) // nc
    gen = torch.Generator(device=device).manual_seed(cfg.seed)
    chunks = [(torch.randn(rows, 768, generator=gen, device=device) * 0.02).to(torch.float8_e4m3fn) for _ in range(nc)]
    x_np = synth.make_x(cfg.batch, 768, cfg.seed)
    labels_np = synth.make_labels(cfg.batch, cfg.num_labels, cfg.pos_mean, cfg.zipf_s, cfg.seed)
    x = torch.from_numpy(x_np).to(device).to(torch.bfloat16)
    labels = torch.from_numpy(labels_np).to(device)
    return cfg, nc, rows, chunks, x, labels, x_np, labels_np


def sample_rows(labels_np, nc, rows, seed):
    """Rows around tile and chunk boundaries, the labels that have positives, and random ones."""
    rng = np.random.default_rng(seed)
    pos_rows = np.unique(labels_np[:, 1])
    edges = [rows - 1, rows, rows + 1, 2 * rows - 1, (nc - 1) * rows, nc * rows - 1]
    return np.unique(np.concatenate([np.arange(0, 130), pos_rows[:300], edges, rng.integers(0, nc * rows, 400)]))


def check_sampled_rows(chunks, rows, sample, before, x_np, labels_np, lr, **oracle_kw):
    import torch
    w_old = np.stack([before[int(r)] for r in sample])
    remap = {int(r): i for i, r in enumerate(sample)}
    lab = np.array([(b, remap[int(l)]) for b, l in labels_np if int(l) in remap], dtype=np.int32).reshape(-1, 2)
    ref_codes, _, _ = O.fp8_step([w_old], x_np, lab, lr, sr_mode="rtn", **oracle_kw)
    got = np.stack([chunks[r // rows][r % rows].view(torch.uint8).cpu().numpy() for r in sample])
    d = H.e4m3_ulp_distance(got, ref_codes[0])
    assert d.max() <= 1 and np.mean(d != 0) < 2e-3, (int(d.max()), float(np.mean(d != 0)))
    assert np.mean(got != w_old) > 0.3                       # the step really changed the weights


def snapshot(chunks, rows, sample):
    import torch
    return {int(r): chunks[r // rows][r % rows].view(torch.uint8).cpu().numpy().copy() for r in sample}


def test_fused_step_at_2m8_labels(gpu):
    """2,812,281 labels in 22 chunks, batch 128, about 4,600 positives: the fused kernel."""
    import torch
    from elmo_amd import ops
    cfg, nc, rows, chunks, x, labels, x_np, labels_np = make_fp8_workload("cfg4_fp8_3m", gpu)
    sample = sample_rows(labels_np, nc, rows, 1)
    before = snapshot(chunks, rows, sample)
    ws = ops.alloc_workspace(nc, rows, gpu)
    ops.fp8_step(chunks, x, labels, 0.05, round_mode="rtn", workspace=ws)
    assert ops.step_error_word(ws, nc, rows) == 0
    check_sampled_rows(chunks, rows, sample, before, x_np, labels_np, 0.05)
    del chunks, ws
    torch.cuda.empty_cache()


def test_three_kernel_path_at_8m6_labels_and_a_batch_of_256(gpu):
    """8,600,000 labels in 33 chunks, batch 256 in two halves, true-FP8 arithmetic on the three-kernel path: lr = 0 is
    the identity, grad_X equals library GEMMs over all chunks, sampled rows equal the oracle after a real step."""
    import torch
    from elmo_amd import ops
    cfg, nc, rows, chunks, x, labels, x_np, labels_np = make_fp8_workload("cfg5_fp8_8m6", gpu)
    assert cfg.batch == 256
    ws = ops.alloc_tiled_workspace(nc, rows, gpu, cfg.batch)
    probe = [0, nc // 2, nc - 1]
    keep = {c: chunks[c].view(torch.uint8).clone() for c in probe}
    g, gf = ops.tiled_step(chunks, rows, "e4m3", x, labels, 0.0, round_mode="rtn", workspace=ws, want_f32=True,
                           quantize_x=True, saturate=True)
    for c in probe:
        a, b = keep[c], chunks[c].view(torch.uint8)
        assert bool(((a == b) | (((a | b) & 0x7F) == 0)).all())          # +0 and -0 are the same weight
    xq = x.to(torch.float8_e4m3fn).float()
    ref = torch.zeros(cfg.batch, 768, device=gpu, dtype=torch.float64)
    lab = labels.long()
    for c, wc in enumerate(chunks):
        w = wc.float()
        s = torch.sigmoid((w @ xq.t()).to(torch.bfloat16).float()).to(torch.bfloat16)
        sel = (lab[:, 1] >= c * rows) & (lab[:, 1] < (c + 1) * rows)
        s[lab[sel, 1] - c * rows, lab[sel, 0]] -= 1.0
        ref += (s.float().t() @ w).double()
        del w, s
    ref = ref.float()
    scale = ref.abs().max().item()
    assert (gf - ref).abs().max().item() <= 2e-3 * scale
    assert torch.equal(g.view(torch.int16), gf.to(torch.bfloat16).view(torch.int16))
    sample = sample_rows(labels_np, nc, rows, 2)
    before = snapshot(chunks, rows, sample)
    ops.tiled_step(chunks, rows, "e4m3", x, labels, 0.05, round_mode="rtn", workspace=ws, quantize_x=True, saturate=True)
    check_sampled_rows(chunks, rows, sample, before, x_np, labels_np, 0.05)
    del chunks, ws, keep
    torch.cuda.empty_cache()


def test_simulated_fp8_at_500k_labels(gpu):
    """500,000 labels in 8 chunks, batch 128, simulated FP8 (bf16 arithmetic on e4m3 weights, torch cast)."""
    import torch
    from elmo_amd import ops
    cfg, nc, rows, chunks, x, labels, x_np, labels_np = make_fp8_workload("cfg3_simfp8_500k", gpu)
    sample = sample_rows(labels_np, nc, rows, 3)
    before = snapshot(chunks, rows, sample)
    ops.tiled_step(chunks, rows, "e4m3", x, labels, 0.05, round_mode="rtn")
    check_sampled_rows(chunks, rows, sample, before, x_np, labels_np, 0.05, simulated=True)
    del chunks
    torch.cuda.empty_cache()


def test_bf16_layer_at_131k_labels_against_the_whole_oracle(gpu):
    """131,072 labels in 8 chunks of 16,384 rows, batch 32, bf16 weights: small enough for the whole oracle."""
    from test_tiled_gpu import check_bf16_weights, check_gx, run_bf16
    cfg = synth.CONFIGS["cfg1_bf16_131k"]
    x = synth.make_x(cfg.batch, 768, cfg.seed)
    w = C.bf16_round(synth.make_weights_np(cfg.num_labels, 768, cfg.seed, 0.02))
    labels = synth.make_labels(cfg.batch, cfg.num_labels, cfg.pos_mean, cfg.zipf_s, cfg.seed).astype(np.int32)
    new, gf, gb = run_bf16(x, w, labels, cfg.num_chunks, gpu, "rtn", None)
    ref_w, ref_gx, _ = O.bf16_step(w, x, labels, 0.05, cfg.num_chunks, sr_mode="rtn")
    check_bf16_weights(new, ref_w, w, x)
    check_gx(gf, gb, ref_gx)


def test_label_space_above_2_24_on_the_three_kernel_path(gpu):
    """16,785,408 labels (64 chunks of 262,272 rows, 12.9 GB of e4m3 weights), batch 32, true-FP8 arithmetic: the positives
    are sorted in two segments of the label space (63 chunks + 1).  Positives on both sides of the segment boundary, at
    label 2^24 and beyond and on the last label; lr = 0 is the identity, grad_X equals library GEMMs over all chunks,
    sampled rows (among them every row with a positive) equal the oracle after a real step."""
    import torch
    from elmo_amd import ops
    nc, rows, batch = 64, 262272, 32
    L = nc * rows
    assert L >= 1 << 24
    gen = torch.Generator(device=gpu).manual_seed(9)
    chunks = [(torch.randn(rows, 768, generator=gen, device=gpu) * 0.02).to(torch.float8_e4m3fn) for _ in range(nc)]
    x_np = synth.make_x(batch, 768, 9)
    base = synth.make_labels(batch, L, 6.0, 1.0, 9)
    special = np.array([(0, 63 * rows - 1), (1, 63 * rows), (2, (1 << 24) - 1), (3, 1 << 24), (4, (1 << 24) + 1234), (5, L - 1),
                        (31, L - 64), (7, 1 << 24), (7, 62 * rows + 5)], dtype=base.dtype)
    labels_np = np.concatenate([base, special])
    x = torch.from_numpy(x_np).to(gpu).to(torch.bfloat16)
    labels = torch.from_numpy(labels_np).to(gpu)
    ws = ops.alloc_tiled_workspace(nc, rows, gpu, batch)
    probe = [0, 62, 63]
    keep = {c: chunks[c].view(torch.uint8).clone() for c in probe}
    g, gf = ops.tiled_step(chunks, rows, "e4m3", x, labels, 0.0, round_mode="rtn", workspace=ws, want_f32=True,
                           quantize_x=True, saturate=True)
    for c in probe:
        a, b = keep[c], chunks[c].view(torch.uint8)
        assert bool(((a == b) | (((a | b) & 0x7F) == 0)).all())
    xq = x.to(torch.float8_e4m3fn).float()
    ref = torch.zeros(batch, 768, device=gpu, dtype=torch.float64)
    lab = labels.long()
    for c, wc in enumerate(chunks):
        w = wc.float()
        s = torch.sigmoid((w @ xq.t()).to(torch.bfloat16).float()).to(torch.bfloat16)
        sel = (lab[:, 1] >= c * rows) & (lab[:, 1] < (c + 1) * rows)
        s[lab[sel, 1] - c * rows, lab[sel, 0]] -= 1.0
        ref += (s.float().t() @ w).double()
        del w, s
    ref = ref.float()
    assert (gf - ref).abs().max().item() <= 2e-3 * ref.abs().max().item()
    sample = np.unique(np.concatenate([sample_rows(labels_np, nc, rows, 4), special[:, 1],
                                       np.arange(63 * rows - 70, 63 * rows + 70), np.arange((1 << 24) - 70, (1 << 24) + 70)]))
    before = snapshot(chunks, rows, sample)
    ops.tiled_step(chunks, rows, "e4m3", x, labels, 0.05, seeds=list(range(nc)), round_mode="rtn", workspace=ws, quantize_x=True,
                   saturate=True)
    check_sampled_rows(chunks, rows, sample, before, x_np, labels_np, 0.05)
    # inference over the same label space: dense logits (columns around 2^24 and the last ones against a library GEMM on
    # those rows) and the top-10 without the dense logits
    x16 = x[:16].contiguous()
    out = ops.fp8_forward(chunks, x16, L - 5)
    assert out.shape == (16, L - 5)
    cols = np.unique(np.concatenate([np.arange((1 << 24) - 40, (1 << 24) + 40), np.arange(L - 45, L - 5), np.arange(0, 40),
                                     np.arange(63 * rows - 20, 63 * rows + 20)]))
    wsel = torch.stack([chunks[int(c) // rows][int(c) % rows] for c in cols]).float()
    ref_z = (x16.to(torch.float8_e4m3fn).float() @ wsel.t()).to(torch.bfloat16)
    got_z = out[:, torch.from_numpy(cols).to(gpu)]
    H.assert_bf16_close(got_z.float().cpu().numpy(), ref_z.float().cpu().numpy())
    vals, idx = ops.fp8_forward_topk(chunks, x16, L - 5, 10)
    tv, ti = out.float().topk(10, dim=1)
    assert torch.equal(vals.float(), tv)
    unique = (tv[:, 1:-1] != tv[:, :-2]) & (tv[:, 1:-1] != tv[:, 2:])       # bf16 logits tie often: compare the untied entries
    assert torch.equal(idx[:, 1:-1][unique], ti[:, 1:-1][unique]) and int(unique.sum()) > 40
    assert int(idx.max()) < L - 5
    del chunks, ws, keep, out
    torch.cuda.empty_cache()
