"""The headline workload at its full size (670 091 labels, 11 chunks, batch 128), checked through properties that
do not need the whole oracle: sampled label rows against the oracle (the update of a row depends only on that
row, X and the positives), lr = 0 leaves every weight byte unchanged, grad_X against an fp32 library GEMM,
positives change exactly the rows they name, and the inference logits and their top-100 against library routines."""
import numpy as np
import pytest

import helpers as H
from elmo_amd import synth
from oracle import codecs as C
from oracle import step as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def big(gpu):
    import torch
    cfg = synth.CONFIGS["cfg2_fp8_670k"]
    nc = cfg.num_chunks
    L_pad = O.fp8_padded_labels(cfg.num_labels, nc)
    rows = L_pad // nc
    gen = torch.Generator(device=gpu).manual_seed(cfg.seed)
    chunks = [(torch.randn(rows, 768, generator=gen, device=gpu) * 0.02).to(torch.float8_e4m3fn) for _ in range(nc)]
    x_np = synth.make_x(cfg.batch, 768, cfg.seed)
    labels_np = synth.make_labels(cfg.batch, cfg.num_labels, cfg.pos_mean, cfg.zipf_s, cfg.seed)
    x = torch.from_numpy(x_np).to(gpu).to(torch.bfloat16)
    labels = torch.from_numpy(labels_np).to(gpu)
    return dict(cfg=cfg, nc=nc, rows=rows, chunks=chunks, x=x, labels=labels, x_np=x_np, labels_np=labels_np)


def test_inference_topk_at_full_size(gpu, big):
    """670 091 labels: the dense logits against an fp32 library GEMM on sampled columns, and the top-100 merged group by
    group (two chunks per group here, the last group a single short chunk) against torch.topk of the dense logits:
    identical values, ids that point at them, all below the label count."""
    import torch
    from elmo_amd import ops
    cfg = big["cfg"]
    dense = ops.fp8_forward(big["chunks"], big["x"], cfg.num_labels)
    assert dense.shape == (128, cfg.num_labels)
    xq = big["x"].to(torch.float8_e4m3fn).float()
    for c in (0, 5, big["nc"] - 1):
        n = min(big["rows"], cfg.num_labels - c * big["rows"])
        ref = (xq @ big["chunks"][c].float().t())[:, :n]
        got = dense[:, c * big["rows"]:c * big["rows"] + n].float()
        assert (got - ref).abs().max().item() <= 2.0 ** -7 * ref.abs().max().item()     # one bf16 rounding of the logit
    vals, idx = ops.fp8_forward_topk(big["chunks"], big["x"], cfg.num_labels, 100)
    want = torch.topk(dense, 100, dim=1)
    assert torch.equal(vals.view(torch.int16), want.values.contiguous().view(torch.int16))
    assert int(idx.min()) >= 0 and int(idx.max()) < cfg.num_labels
    assert torch.equal(torch.gather(dense, 1, idx).view(torch.int16), vals.view(torch.int16))
    assert bool((idx.sort(dim=1).values[:, 1:] != idx.sort(dim=1).values[:, :-1]).all())   # no label twice


def test_lr_zero_is_identity_and_gradx_matches_library_gemm(gpu, big):
    import torch
    from elmo_amd import ops
    before = [c.view(torch.uint8).clone() for c in big["chunks"]]
    ws = ops.alloc_workspace(big["nc"], big["rows"], gpu)
    g, gf = ops.fp8_step(big["chunks"], big["x"], big["labels"], 0.0, round_mode="rtn", workspace=ws, want_f32=True)
    assert ops.step_error_word(ws, big["nc"], big["rows"]) == 0
    for a, c in zip(before, big["chunks"]):
        b = c.view(torch.uint8)
        same = (a == b) | (((a | b) & 0x7F) == 0)          # +0 and -0 are the same weight
        assert bool(same.all())
    # grad_X = G^T W with G from bf16 logits of the FP8-quantised X: fp32 library GEMMs on the same device
    xq = big["x"].to(torch.float8_e4m3fn).float()
    ref = torch.zeros(128, 768, device=gpu, dtype=torch.float64)
    lab = big["labels"].long()
    for c, wc in enumerate(big["chunks"]):
        w = wc.float()
        z = (w @ xq.t()).to(torch.bfloat16).float()
        s = torch.sigmoid(z).to(torch.bfloat16)
        sel = (lab[:, 1] >= c * big["rows"]) & (lab[:, 1] < (c + 1) * big["rows"])
        s[lab[sel, 1] - c * big["rows"], lab[sel, 0]] -= 1.0
        ref += (s.double().t() @ w.double())
    ref = ref.float()
    scale = ref.abs().max().item()
    assert (gf - ref).abs().max().item() <= 1e-2 * scale
    assert (gf - ref).abs().max().item() <= 2e-3 * scale
    assert torch.equal(g.view(torch.int16), gf.to(torch.bfloat16).view(torch.int16))


def test_sampled_rows_match_oracle_after_a_real_step(gpu, big):
    import torch
    from elmo_amd import ops
    nc, rows = big["nc"], big["rows"]
    rng = np.random.default_rng(0)
    # rows around tile and chunk boundaries, the head labels (where the positives are), and random ones
    pos_rows = np.unique(big["labels_np"][:, 1])
    sample = np.unique(np.concatenate([np.arange(0, 130), pos_rows[:200], [rows - 1, rows, rows + 1, 2 * rows - 1, nc * rows - 1],
                                       rng.integers(0, nc * rows, 400)]))
    before = {int(r): big["chunks"][r // rows][r % rows].view(torch.uint8).cpu().numpy().copy() for r in sample}
    ws = ops.alloc_workspace(nc, rows, gpu)
    ops.fp8_step(big["chunks"], big["x"], big["labels"], 0.05, round_mode="rtn", workspace=ws)
    assert ops.step_error_word(ws, nc, rows) == 0
    w_old = np.stack([before[int(r)] for r in sample])
    # oracle on the sampled rows only: remap the positives that name a sampled row
    remap = {int(r): i for i, r in enumerate(sample)}
    lab = np.array([(b, remap[int(l)]) for b, l in big["labels_np"] if int(l) in remap], dtype=np.int32).reshape(-1, 2)
    ref_codes, _, _ = O.fp8_step([w_old], big["x_np"], lab, 0.05, sr_mode="rtn")
    got = np.stack([big["chunks"][r // rows][r % rows].view(torch.uint8).cpu().numpy() for r in sample])
    d = H.e4m3_ulp_distance(got, ref_codes[0])
    assert d.max() <= 1 and np.mean(d != 0) < 2e-3
    assert np.mean(got != w_old) > 0.3                       # the step really changed the weights


def test_sampled_rows_match_exact_stochastic_rounding_after_a_real_sr_fast_step(gpu, big):
    """The headline's own rounding mode at full size: after a real `sr_fast` step over all 670 K labels, sampled rows
    (tile and chunk boundaries, labels with positives, random ones) equal the oracle's exact stochastic rounding fed with
    the same counter-hash words (global row, column, hashed per-chunk seed), up to the one-grid-step differences the fp32
    summation order of grad_W causes."""
    import torch
    from elmo_amd import ops
    nc, rows = big["nc"], big["rows"]
    rng = np.random.default_rng(1)
    pos_rows = np.unique(big["labels_np"][:, 1])
    sample = np.unique(np.concatenate([np.arange(0, 70), pos_rows[:150], [rows - 1, rows, rows + 63, rows + 64, 5 * rows - 1, nc * rows - 1],
                                       rng.integers(0, nc * rows, 300)]))
    seeds = [1000 + 17 * c for c in range(nc)]
    before = np.stack([big["chunks"][r // rows][r % rows].view(torch.uint8).cpu().numpy().copy() for r in sample])
    ws = ops.alloc_workspace(nc, rows, gpu)
    ops.fp8_step(big["chunks"], big["x"], big["labels"], 0.05, seeds=seeds, round_mode="sr_fast", workspace=ws)
    assert ops.step_error_word(ws, nc, rows) == 0
    remap = {int(r): i for i, r in enumerate(sample)}
    lab = np.array([(b, remap[int(l)]) for b, l in big["labels_np"] if int(l) in remap], dtype=np.int32).reshape(-1, 2)

    def rand_fn(c, offs):          # the oracle sees one chunk made of the sampled rows: map its offsets back
        r, k = offs // 768, offs % 768
        grow = sample[r]
        out = np.zeros(offs.shape, dtype=np.uint32)
        for ch in np.unique(grow // rows):           # the seed is per chunk
            sel = grow // rows == ch
            out[sel] = C.fast_sr_words(seeds[int(ch)], grow[sel], k[sel])
        return out

    ref_codes, _, _ = O.fp8_step([before], big["x_np"], lab, 0.05, sr_mode="exact", rand_fn=rand_fn)
    got = np.stack([big["chunks"][r // rows][r % rows].view(torch.uint8).cpu().numpy() for r in sample])
    d = H.e4m3_ulp_distance(got, ref_codes[0])
    assert d.max() <= 1 and np.mean(d != 0) < 2e-3
    assert np.mean(got != before) > 0.3


def test_batch_256_at_the_chunk_size_of_the_largest_workload(gpu):
    """True FP8 with 256 batch rows on chunks of 262,144 rows (the chunk size of the 8.6 M-label workload, four chunks
    here): the one-pass FP8 logits, the eight-wavefront grad_X and the feature-split update at their real launch shapes.
    lr = 0 leaves the weights alone; after a real step sampled rows equal the oracle's; grad_X equals fp64 library
    GEMMs on the same device."""
    import torch
    from elmo_amd import ops
    nc, rows, batch, L = 4, 262144, 256, 4 * 262144 - 37
    gen = torch.Generator(device=gpu).manual_seed(5)
    chunks = [(torch.randn(rows, 768, generator=gen, device=gpu) * 0.02).to(torch.float8_e4m3fn) for _ in range(nc)]
    x_np = synth.make_x(batch, 768, 5)
    labels_np = synth.make_labels(batch, L, 8.0, 1.1, 5)
    x = torch.from_numpy(x_np).to(gpu).to(torch.bfloat16)
    labels = torch.from_numpy(labels_np).to(gpu)
    ws = ops.alloc_tiled_workspace(nc, rows, gpu, batch)
    kw = dict(round_mode="rtn", workspace=ws, quantize_x=True, saturate=True, want_f32=True)
    before = [c.view(torch.uint8).clone() for c in chunks]
    g, gf = ops.tiled_step(chunks, rows, "e4m3", x, labels, 0.0, **kw)
    for a, c in zip(before, chunks):
        b = c.view(torch.uint8)
        assert bool(((a == b) | (((a | b) & 0x7F) == 0)).all())
    xq = x.to(torch.float8_e4m3fn).float()
    ref = torch.zeros(batch, 768, device=gpu, dtype=torch.float64)
    lab = labels.long()
    for c, wc in enumerate(chunks):
        w = wc.float()
        z = (w @ xq.t()).to(torch.bfloat16).float()
        s = torch.sigmoid(z).to(torch.bfloat16)
        sel = (lab[:, 1] >= c * rows) & (lab[:, 1] < (c + 1) * rows)
        s[lab[sel, 1] - c * rows, lab[sel, 0]] -= 1.0
        ref += (s.double().t() @ w.double())
        del w, z, s
    ref = ref.float()
    assert (gf - ref).abs().max().item() <= 2e-3 * ref.abs().max().item()
    assert torch.equal(g.view(torch.int16), gf.to(torch.bfloat16).view(torch.int16))
    # a real step: sampled rows (tile and chunk boundaries, the head labels, random ones) against the oracle
    rng = np.random.default_rng(1)
    pos_rows = np.unique(labels_np[:, 1])
    sample = np.unique(np.concatenate([np.arange(0, 130), pos_rows[:300], [rows - 1, rows, rows + 1, 3 * rows - 1, 3 * rows, nc * rows - 1],
                                       rng.integers(0, nc * rows, 500)]))
    w_old = np.stack([chunks[r // rows][r % rows].view(torch.uint8).cpu().numpy().copy() for r in sample])
    ops.tiled_step(chunks, rows, "e4m3", x, labels, 0.05, **kw)
    remap = {int(r): i for i, r in enumerate(sample)}
    lab_s = np.array([(b, remap[int(l)]) for b, l in labels_np if int(l) in remap], dtype=np.int32).reshape(-1, 2)
    ref_codes, _, _ = O.fp8_step([w_old], x_np, lab_s, 0.05, sr_mode="rtn")
    got = np.stack([chunks[r // rows][r % rows].view(torch.uint8).cpu().numpy() for r in sample])
    d = H.e4m3_ulp_distance(got, ref_codes[0])
    assert d.max() <= 1 and np.mean(d != 0) < 2e-3
    assert np.mean(got != w_old) > 0.3
