"""Writes tests/golden/fixtures.npz: small input/output vectors for the classifier step.

Two kinds of vectors:
  * known answers that exist outside this repository: the three Random123 Philox-4x32-10 vectors and the first four
    words of Triton's tl.randint for seed 1024 (the generator behind fuse_kernel.py:12,30 and
    stochastic_rounding_kernel.py:12,22 of the reference), and the e4m3fn / e5m2 decode tables of the torch CPU library;
  * regression vectors of this build's CPU oracle for seeded tiny steps (FP8 layer in RTN and reference-SR mode, bf16
    layer in RTN mode).  The reference ships no golden vectors for this path, so these pin the oracle against drift
    and give the GPU tests a fixed target; they were NOT produced by running the reference.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from elmo_amd import synth  # noqa: E402
from oracle import codecs as C  # noqa: E402
from oracle import step as O  # noqa: E402


def main():
    out = {}
    # Random123 kat_vectors: counter, key -> output
    out["philox_ctr"] = np.array([[0, 0, 0, 0], [0xFFFFFFFF] * 4, [0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344]], dtype=np.uint32)
    out["philox_key"] = np.array([[0, 0], [0xFFFFFFFF, 0xFFFFFFFF], [0xA4093822, 0x299F31D0]], dtype=np.uint32)
    out["philox_out"] = np.array([[0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8],
                                  [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD],
                                  [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]], dtype=np.uint32)
    out["tl_randint_seed1024"] = np.array([3876201247, 854061192, 798737492, 713463838], dtype=np.uint32)
    codes = torch.arange(256, dtype=torch.uint8)
    out["e4m3_table"] = codes.view(torch.float8_e4m3fn).float().numpy()
    out["e5m2_table"] = codes.view(torch.float8_e5m2).float().numpy()

    # tiny FP8 step: 2 chunks x 32 rows, batch 16, a duplicated positive and one in the last row
    nc, rows, batch, seed = 2, 32, 16, 21
    L = nc * rows
    x = synth.make_x(batch, 768, seed)
    w = synth.make_weights_np(L, 768, seed, 0.02)
    wc = C.e4m3_encode(w, saturate=True)
    labels = np.concatenate([synth.make_labels(batch, L, 3.0, 1.0, seed), np.array([[2, 5], [2, 5], [15, L - 1]], dtype=np.int32)])
    chunks = [wc[c * rows:(c + 1) * rows].copy() for c in range(nc)]
    seeds = np.array([1024, 77], dtype=np.uint32)
    out["fp8_x_bits"] = C.bf16_bits(x)
    out["fp8_codes"] = wc
    out["fp8_labels"] = labels.astype(np.int32)
    out["fp8_seeds"] = seeds
    out["fp8_lr"] = np.float32(0.05)
    new_rtn, gx, gi = O.fp8_step(chunks, x, labels, 0.05, sr_mode="rtn")
    out["fp8_rtn_codes"] = np.concatenate(new_rtn)
    out["fp8_gx_f32"] = gx
    out["fp8_grad_input_bits"] = C.bf16_bits(gi)
    new_sr, _, _ = O.fp8_step(chunks, x, labels, 0.05, seeds=seeds, sr_mode="reference")
    out["fp8_sr_reference_codes"] = np.concatenate(new_sr)
    new_sim, gx_sim, _ = O.fp8_step(chunks, x, labels, 0.05, sr_mode="rtn", simulated=True)
    out["fp8_sim_rtn_codes"] = np.concatenate(new_sim)
    out["fp8_sim_gx_f32"] = gx_sim

    # tiny bf16 step: 70 labels in 2 chunks (35 + 35), batch 8
    Lb, ncb, bb, seedb = 70, 2, 8, 22
    xb = synth.make_x(bb, 768, seedb)
    wb = C.bf16_round(synth.make_weights_np(Lb, 768, seedb, 0.02))
    lb = synth.make_labels(bb, Lb, 3.0, 1.0, seedb)
    out["bf16_x_bits"] = C.bf16_bits(xb)
    out["bf16_w_bits"] = C.bf16_bits(wb)
    out["bf16_labels"] = lb.astype(np.int32)
    nw, gxb, gib = O.bf16_step(wb, xb, lb, 0.05, ncb, sr_mode="rtn")
    out["bf16_rtn_w_bits"] = C.bf16_bits(nw)
    out["bf16_gx_f32"] = gxb
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "fixtures.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
