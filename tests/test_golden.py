"""The committed fixtures of tests/golden/ (made by tests/golden/make_fixtures.py): published known answers for the
random generator and the number formats, and seeded tiny steps.  CPU tests hold the oracle to them bit for bit; the GPU
tests hold the HIP paths to the same vectors with the tolerances of the parity tests (updated weights within one grid
step and all but 0.5 % identical - tiny cases have few weights - grad_X within 1e-3 of the largest entry)."""
import os

import numpy as np
import pytest

import helpers as H
from oracle import codecs as C
from oracle import step as O

FIX = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fixtures.npz"))


def _fp8_inputs():
    x = C.bf16_from_bits(FIX["fp8_x_bits"])
    codes = FIX["fp8_codes"]
    chunks = [codes[:32].copy(), codes[32:].copy()]
    return x, chunks, FIX["fp8_labels"], float(FIX["fp8_lr"]), FIX["fp8_seeds"]


def test_philox_known_answers():
    for ctr, key, out in zip(FIX["philox_ctr"], FIX["philox_key"], FIX["philox_out"]):
        got = C.philox4x32(*[np.uint32(v) for v in ctr], np.uint32(key[0]), np.uint32(key[1]))
        assert [int(np.asarray(g).reshape(-1)[0]) for g in got] == [int(v) for v in out]
    assert np.array_equal(C.tl_randint(1024, np.arange(4)), FIX["tl_randint_seed1024"])


def test_number_format_tables():
    codes = np.arange(256, dtype=np.uint8)
    for table, dec in ((FIX["e4m3_table"], C.e4m3_decode), (FIX["e5m2_table"], C.e5m2_decode)):
        got = dec(codes)
        assert np.array_equal(np.isnan(got), np.isnan(table))
        ok = ~np.isnan(table)
        assert np.array_equal(got[ok], table[ok])


def test_oracle_reproduces_the_fp8_step_vectors():
    x, chunks, labels, lr, seeds = _fp8_inputs()
    new, gx, gi = O.fp8_step(chunks, x, labels, lr, sr_mode="rtn")
    assert np.array_equal(np.concatenate(new), FIX["fp8_rtn_codes"])
    assert np.array_equal(gx, FIX["fp8_gx_f32"])
    assert np.array_equal(C.bf16_bits(gi), FIX["fp8_grad_input_bits"])
    new, _, _ = O.fp8_step(chunks, x, labels, lr, seeds=seeds, sr_mode="reference")
    assert np.array_equal(np.concatenate(new), FIX["fp8_sr_reference_codes"])
    new, gx, _ = O.fp8_step(chunks, x, labels, lr, sr_mode="rtn", simulated=True)
    assert np.array_equal(np.concatenate(new), FIX["fp8_sim_rtn_codes"])
    assert np.array_equal(gx, FIX["fp8_sim_gx_f32"])


def test_oracle_reproduces_the_bf16_step_vectors():
    x = C.bf16_from_bits(FIX["bf16_x_bits"])
    w = C.bf16_from_bits(FIX["bf16_w_bits"])
    nw, gx, _ = O.bf16_step(w, x, FIX["bf16_labels"], 0.05, 2, sr_mode="rtn")
    assert np.array_equal(C.bf16_bits(nw), FIX["bf16_rtn_w_bits"])
    assert np.array_equal(gx, FIX["bf16_gx_f32"])


def _check_codes(got, want, max_frac=5e-3):
    d = H.e4m3_ulp_distance(got, want)
    assert d.max() <= 1
    assert (d != 0).mean() < max_frac, (d != 0).mean()


@pytest.mark.gpu
def test_fused_step_against_the_vectors(gpu):
    import torch
    from elmo_amd import ops
    x, chunks, labels, lr, seeds = _fp8_inputs()
    case = dict(x=x, chunks=chunks, labels=labels)
    dchunks, dx, dlabels = H.to_device_case(case, gpu)
    g, gf = ops.fp8_step(dchunks, dx, dlabels, lr, round_mode="rtn", want_f32=True)
    _check_codes(np.concatenate(H.chunks_to_numpy(dchunks)), FIX["fp8_rtn_codes"])
    ref = FIX["fp8_gx_f32"]
    assert np.abs(gf.cpu().numpy() - ref).max() <= 1e-3 * np.abs(ref).max()
    # reference stochastic rounding: the same random word per element, so again at most one grid step where the
    # fp32 sum differs in its last bits
    dchunks, dx, dlabels = H.to_device_case(case, gpu)
    ops.fp8_step(dchunks, dx, dlabels, lr, seeds=seeds, round_mode="sr_philox")
    _check_codes(np.concatenate(H.chunks_to_numpy(dchunks)), FIX["fp8_sr_reference_codes"], max_frac=2e-2)
    torch.cuda.synchronize()


@pytest.mark.gpu
def test_tiled_paths_against_the_vectors(gpu):
    import torch
    from elmo_amd import ops
    x, chunks, labels, lr, seeds = _fp8_inputs()
    dchunks, dx, dlabels = H.to_device_case(dict(x=x, chunks=chunks, labels=labels), gpu)
    g, gf = ops.tiled_step(dchunks, 32, "e4m3", dx, dlabels, lr, round_mode="rtn", want_f32=True)
    _check_codes(np.concatenate(H.chunks_to_numpy(dchunks)), FIX["fp8_sim_rtn_codes"])
    ref = FIX["fp8_sim_gx_f32"]
    assert np.abs(gf.cpu().numpy() - ref).max() <= 1e-3 * np.abs(ref).max()

    xb = C.bf16_from_bits(FIX["bf16_x_bits"])
    w0 = C.bf16_from_bits(FIX["bf16_w_bits"])
    wt = torch.from_numpy(FIX["bf16_w_bits"].view(np.int16)).to(gpu).view(torch.bfloat16)
    dxb = torch.from_numpy(FIX["bf16_x_bits"].view(np.int16)).to(gpu).view(torch.bfloat16)
    dl = torch.from_numpy(FIX["bf16_labels"]).to(gpu)
    g, gf = ops.tiled_step([wt[:35], wt[35:]], 35, "bf16", dxb, dl, 0.05, round_mode="rtn", want_f32=True)
    new = wt.float().cpu().numpy()
    ref_w = C.bf16_from_bits(FIX["bf16_rtn_w_bits"])
    tol = 1.5 * 2.0 ** -7 * (np.abs(w0) + np.abs(ref_w)) + 2.0 * 0.05 * 2.0 ** -8 * np.abs(xb).max()
    assert np.all(np.abs(new - ref_w) <= tol)
    assert (new != ref_w).mean() < 5e-3
    ref = FIX["bf16_gx_f32"]
    assert np.abs(gf.cpu().numpy() - ref).max() <= 4e-3 * np.abs(ref).max()   # one bf16 ulp of a chunk's partial
