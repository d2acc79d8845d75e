"""Shared helpers of the parity tests: build seeded cases, run the HIP path through the C ABI wrappers, run the
oracle on the same inputs, and measure distances in units in the last place."""
import numpy as np

from elmo_amd import synth
from oracle import codecs as C
from oracle import step as O


def make_case(num_chunks, rows_per_chunk, batch, seed, pos_mean=5.0, zipf_s=1.0, std=0.02, extra_labels=None,
              w_scale=1.0, features=768):
    L = num_chunks * rows_per_chunk
    x = synth.make_x(batch, features, seed)
    w = synth.make_weights_np(L, features, seed, std) / np.float32(w_scale)
    codes = C.e4m3_encode(w, saturate=True)
    labels = synth.make_labels(batch, L, pos_mean, zipf_s, seed)
    if extra_labels is not None:
        labels = np.concatenate([labels, np.asarray(extra_labels, dtype=np.int32).reshape(-1, 2)], axis=0)
    chunks = [codes[c * rows_per_chunk:(c + 1) * rows_per_chunk].copy() for c in range(num_chunks)]
    return dict(x=x, chunks=chunks, labels=labels.astype(np.int32), L=L)


def e4m3_ulp_distance(a_codes, b_codes):
    """Distance in grid steps between e4m3 codes (sign-magnitude -> signed integer line)."""
    def lin(c):
        c = c.astype(np.int32)
        mag = c & 0x7F
        return np.where(c & 0x80, -mag, mag)
    return np.abs(lin(a_codes) - lin(b_codes))


def bf16_ulp_distance(a_f32, b_f32):
    def lin(v):
        b = C.bf16_bits(v).astype(np.int32)
        mag = b & 0x7FFF
        return np.where(b & 0x8000, -mag, mag)
    return np.abs(lin(a_f32) - lin(b_f32))


def to_device_case(case, device):
    import torch
    chunks = [torch.from_numpy(c).to(device).view(torch.float8_e4m3fn) for c in case["chunks"]]
    x = torch.from_numpy(C.bf16_bits(case["x"]).view(np.int16)).to(device).view(torch.bfloat16)
    labels = torch.from_numpy(case["labels"]).to(device).contiguous()
    return chunks, x, labels


def chunks_to_numpy(chunks):
    import torch
    return [c.view(torch.uint8).cpu().numpy() for c in chunks]


def bf16_tensor_to_f32_numpy(t):
    import torch
    return t.float().cpu().numpy()


def assert_bf16_close(got, ref, floor_rel=5e-5, min_equal=0.99):
    """bf16 values agree to 1 ulp, except next to zero where cancellation in the fp32 accumulator dominates: there
    the difference must stay below floor_rel * max|ref|.  Most entries must be identical."""
    got = np.asarray(got, dtype=np.float32)
    ref = np.asarray(ref, dtype=np.float32)
    ulp = np.abs(ref) * 2.0 ** -7
    tol = np.maximum(ulp, floor_rel * np.abs(ref).max())
    assert np.all(np.abs(got - ref) <= tol), float(np.max(np.abs(got - ref) / tol))
    assert np.mean(got == ref) >= min_equal, float(np.mean(got == ref))
