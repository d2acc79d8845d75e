"""Stochastic-rounding modes of the fused step on the GPU.

sr_philox  the reference bit recipe (Philox word per element, add 20 bits, mask, cast): compared code-for-code
           with the oracle's "reference" mode on the same seeds; the only admissible differences come from the
           fp32 summation order of grad_W and are at most one grid step.
sr_fast    true stochastic rounding by the hardware converter: compared code-for-code with the oracle's exact
           SR fed with the same counter-hash words, and checked for unbiasedness over > 10^6 updated weights
           (mean error <= 1e-3 * mean |delta w|).
"""
import numpy as np
import pytest

import helpers as H
from oracle import codecs as C
from oracle import step as O

pytestmark = pytest.mark.gpu


def run(case, device, mode, seeds, lr=0.05):
    from elmo_amd import ops
    chunks, x, labels = H.to_device_case(case, device)
    ws = ops.alloc_workspace(len(chunks), chunks[0].shape[0], device)
    ops.fp8_step(chunks, x, labels, lr, seeds=seeds, round_mode=mode, workspace=ws)
    assert ops.step_error_word(ws, len(chunks), chunks[0].shape[0]) == 0
    return H.chunks_to_numpy(chunks)


def test_sr_philox_matches_reference_recipe(gpu):
    case = H.make_case(3, 208, 32, 41)
    seeds = [123456, 7, 999999]
    new = run(case, gpu, "sr_philox", seeds)
    ref, _, _ = O.fp8_step(case["chunks"], case["x"], case["labels"], 0.05, seeds=seeds, sr_mode="reference")
    total = mism = 0
    for a, b in zip(new, ref):
        d = H.e4m3_ulp_distance(a, b)
        assert d.max() <= 1
        mism += int((d != 0).sum()); total += d.size
    assert mism / total < 1e-3, (mism, total)
    # a different seed gives a different rounding pattern; the same seed reproduces it bit for bit
    again = run(case, gpu, "sr_philox", seeds)
    other = run(case, gpu, "sr_philox", [1, 2, 3])
    assert all(np.array_equal(a, b) for a, b in zip(new, again))
    assert any(not np.array_equal(a, b) for a, b in zip(new, other))


def test_sr_fast_matches_exact_stochastic_rounding_with_the_same_words(gpu):
    nc, rows = 2, 272
    case = H.make_case(nc, rows, 32, 42)
    seeds = [31337, 4242]

    def rand_fn(c, offs):
        r, k = offs // 768, offs % 768
        return C.fast_sr_words(seeds[c], c * rows + r, k)

    new = run(case, gpu, "sr_fast", seeds)
    ref, _, _ = O.fp8_step(case["chunks"], case["x"], case["labels"], 0.05, sr_mode="exact", rand_fn=rand_fn)
    total = mism = 0
    for a, b in zip(new, ref):
        d = H.e4m3_ulp_distance(a, b)
        assert d.max() <= 1
        mism += int((d != 0).sum()); total += d.size
    assert mism / total < 1e-3, (mism, total)


def test_sr_fast_is_unbiased_over_a_million_weights(gpu):
    nc, rows = 2, 768                       # 2 * 768 * 768 = 1.18e6 updated weights
    case = H.make_case(nc, rows, 64, 43, std=0.02)
    _, _, _, parts = O.fp8_step(case["chunks"], case["x"], case["labels"], 0.05, return_parts=True)
    t = np.concatenate([p["t"] for p in parts]).astype(np.float64)            # exact (fp32) update targets
    w_old = C.e4m3_decode(np.concatenate(case["chunks"])).astype(np.float64)
    dw = np.abs(t - w_old).mean()
    errs = []
    for seed in (1, 2, 3):
        new = C.e4m3_decode(np.concatenate(run(case, gpu, "sr_fast", [seed, seed + 100]))).astype(np.float64)
        errs.append((new - t).mean())
        # every result is one of the two grid neighbours of its target
        assert np.all(np.abs(new - t) <= np.maximum(np.abs(t) * 2.0 ** -3, 2.0 ** -9) * 1.0001)
    mean_err = float(np.mean(errs))
    assert abs(mean_err) <= 1e-3 * dw, (mean_err, dw)
    # round-to-nearest of the same targets is NOT what we got (the rounding really is stochastic) ...
    rtn = C.e4m3_decode(np.concatenate(run(case, gpu, "rtn", None))).astype(np.float64)
    assert np.mean(rtn != new) > 0.2
    # ... and below 2^-6, where the reference recipe rounds to nearest, the hardware mode stays unbiased
    sub = np.abs(t) < 2.0 ** -6
    assert sub.mean() > 0.3
    assert abs((new - t)[sub].mean()) <= 2e-3 * np.abs(t - w_old)[sub].mean()


def test_saturation_at_448(gpu):
    import torch
    from elmo_amd import ops
    # weights at +-448 pushed outwards by a huge learning rate must stay at +-448 in every mode (no NaN)
    x = np.zeros((16, 768), dtype=np.float32); x[:, :] = 1.0 / 32
    codes = np.full((64, 768), 0x7E, dtype=np.uint8); codes[1::2] = 0xFE
    labels = np.array([(b, l) for b in range(16) for l in range(0, 64, 2)], dtype=np.int32)   # positives on even rows
    for mode in ("rtn", "sr_philox", "sr_fast"):
        case = dict(x=x, chunks=[codes.copy()], labels=labels)
        chunks, xd, lab = H.to_device_case(case, gpu)
        ops.fp8_step(chunks, xd, lab, 1.0e4, seeds=[5], round_mode=mode)
        out = chunks[0].view(torch.uint8).cpu().numpy()
        assert np.all(out[0::2] == 0x7E) and np.all(out[1::2] == 0xFE), mode
