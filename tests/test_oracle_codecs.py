"""Pins the oracle's number formats and random bits (CPU only).

Every check here is against something other than the oracle's own formula: torch's CPU casts, the published
Random123 known-answer vectors for Philox-4x32-10, exhaustive enumeration of the random field, and the
reference's own second (pure-torch) statement of the stochastic-rounding recipe (src/utils.py:143-156,178-191).
"""
import numpy as np
import pytest
import torch

from oracle import codecs as C


def test_e4m3_decode_all_codes_match_torch():
    codes = np.arange(256, dtype=np.uint8)
    ours = C.e4m3_decode(codes)
    theirs = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.isnan(ours), np.isnan(theirs))
    ok = ~np.isnan(ours)
    assert np.array_equal(ours[ok], theirs[ok])
    assert np.isnan(ours[0x7F]) and np.isnan(ours[0xFF]) and ours[0x7E] == 448.0 and ours[0x01] == 2.0 ** -9


def _boundary_sweep():
    vals = C.E4M3_TABLE[:0x7F].astype(np.float64)          # all finite non-negative grid points
    mids = (vals[:-1] + vals[1:]) / 2
    pts = np.concatenate([vals, mids, np.nextafter(mids.astype(np.float32), np.float32(0)).astype(np.float64),
                          np.nextafter(mids.astype(np.float32), np.float32(1e9)).astype(np.float64),
                          [448.0, 449.0, 460.0, 463.99, 464.0, 2.0 ** -10, 0.00098, 0.0009, 1e-10, 0.0]])
    rng = np.random.default_rng(0)
    pts = np.concatenate([pts, rng.uniform(0, 500, 20000), rng.uniform(0, 0.05, 20000),
                          np.exp(rng.uniform(np.log(1e-6), np.log(448), 20000))])
    pts = np.concatenate([pts, -pts]).astype(np.float32)
    return pts


def test_e4m3_encode_matches_torch_cast_where_torch_is_finite():
    x = _boundary_sweep()
    ours = C.e4m3_encode(x, saturate=False)
    theirs = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    # torch maps out-of-range to NaN (0x7f / 0xff); compare sign-insensitively for NaN
    nan_o = (ours & 0x7F) == 0x7F
    nan_t = (theirs & 0x7F) == 0x7F
    assert np.array_equal(nan_o, nan_t)
    assert np.array_equal(ours[~nan_o], theirs[~nan_t])


def test_e4m3_encode_overflow_edges():
    x = np.array([448, 449, 464, 464.001, 465, 480, 1e30, np.inf, -465, -np.inf], dtype=np.float32)
    sat = C.e4m3_decode(C.e4m3_encode(x, saturate=True))
    assert np.array_equal(sat, np.array([448, 448, 448, 448, 448, 448, 448, 448, -448, -448], dtype=np.float32))
    uns = C.e4m3_encode(x, saturate=False)
    assert list(uns[:3]) == [0x7E, 0x7E, 0x7E] and all((uns[3:] & 0x7F) == 0x7F)
    # ties to even on the subnormal lattice and in a normal binade
    t = np.array([2.0 ** -10, 3 * 2.0 ** -10, 1.0625, 1.1875], dtype=np.float32)
    assert np.array_equal(C.e4m3_decode(C.e4m3_encode(t)), np.array([0.0, 2 * 2.0 ** -9, 1.0, 1.25], dtype=np.float32))
    assert np.isnan(C.e4m3_decode(C.e4m3_encode(np.array([np.nan], dtype=np.float32))))[0]


def test_bf16_round_matches_torch():
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(100000).astype(np.float32) * 3,
                        np.array([1.00390625, 1.01171875, 1.0039063, 3e38, 3.4e38, 1e-40, -1.00390625, 0.0], np.float32)])
    # exact ties: bf16 grid point + half an ulp
    base = (rng.standard_normal(5000).astype(np.float32).view(np.uint32) & 0xFFFF0000) | 0x8000
    x = np.concatenate([x, base.astype(np.uint32).view(np.float32)])
    ours = C.bf16_round(x)
    theirs = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    assert np.array_equal(ours.view(np.uint32), theirs.view(np.uint32))


PHILOX_KATS = [
    ((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
    ((0xffffffff,) * 4, (0xffffffff, 0xffffffff), (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
    ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
     (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
]


@pytest.mark.parametrize("ctr,key,out", PHILOX_KATS)
def test_philox_random123_known_answers(ctr, key, out):
    got = C.philox4x32(*[np.array([c], dtype=np.uint64) for c in ctr], key[0], key[1])
    assert tuple(int(g[0]) for g in got) == out


def test_tl_randint_recorded_words():
    # words produced by Triton's tl.randint(seed=1024, offsets 0..3) (library routine run through the interpreter, values recorded beforehand)
    assert list(C.tl_randint(1024, np.arange(4))) == [3876201247, 854061192, 798737492, 713463838]


def test_tl_rand_matches_the_triton_library():
    """The uniform fp32 of tl.rand against vectors the Triton library in this image produced through its interpreter
    (tests/golden/make_triton_rand.py): bit-equal, three seeds and offset ranges."""
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "triton_rand.json")) as f:
        cases = json.load(f)["cases"]
    assert len(cases) == 3
    for key, want in cases.items():
        seed, start = (int(v) for v in key.split(":"))
        got = C.tl_rand(seed, np.arange(start, start + len(want))).view(np.uint32)
        assert np.array_equal(got, np.array(want, dtype=np.uint32)), key


def test_dropout_quantize_against_torch_and_its_invariants():
    """The oracle's dropout + e4m3 cast: kept entries equal torch's CPU cast of x / (1 - p) (a different implementation of
    the cast), dropped ones are zero, the kept fraction is 1 - p, p = 0 is the plain cast, and the mask depends on
    (seed, flat offset) only."""
    rng = np.random.default_rng(5)
    x = C.bf16_round(rng.standard_normal((64, 768)).astype(np.float32) * 3.0)
    p, seed = 0.3, 40
    codes = C.dropout_quantize(x, p, seed)
    keep = C.tl_rand(seed, np.arange(64 * 768).reshape(64, 768)) > np.float32(p)
    want = (torch.from_numpy(x) / (1.0 - torch.tensor(p, dtype=torch.float32))).clamp(-448, 448).to(torch.float8_e4m3fn)
    want = want.view(torch.uint8).numpy()
    assert np.array_equal(codes[keep], want[keep]) and np.all(codes[~keep] == 0)
    assert abs(keep.mean() - 0.7) < 0.01
    plain = torch.from_numpy(x).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(C.dropout_quantize(x, 0.0, seed), plain)
    # rows 8..15 taken alone draw the words of flat offsets 0.. again: the mask of rows 0..7, not of rows 8..15
    alone = C.tl_rand(seed, np.arange(8 * 768).reshape(8, 768)) > np.float32(p)
    assert np.array_equal(alone, keep[:8]) and not np.array_equal(alone, keep[8:16])


@pytest.mark.parametrize("k,value", [(20, 1.03125), (20, -0.3), (20, 3.3e-3), (16, 1.00390625 * 1.3), (16, -7.77)])
def test_sr_recipe_probability_equals_dropped_fraction_exhaustively(k, value):
    t = np.full(1 << k, value, dtype=np.float32)
    r = np.arange(1 << k, dtype=np.uint64)
    out = C.sr_add_mask(t, r, k)
    lo = (t.view(np.uint32)[0] & ~np.uint32((1 << k) - 1))
    lo_f = np.array([lo], dtype=np.uint32).view(np.float32)[0]
    hi_f = np.array([lo + (1 << k)], dtype=np.uint32).view(np.float32)[0]
    assert set(np.unique(out)) <= {lo_f, hi_f}                      # floor or ceil in magnitude
    frac = int(t.view(np.uint32)[0] & np.uint32((1 << k) - 1))
    assert int((out == hi_f).sum()) == frac                         # exactly frac of the 2^k random values round up
    mean = out.astype(np.float64).mean()
    assert abs(mean - float(np.float32(value))) <= abs(hi_f - lo_f) * 2.0 ** -k * 1.01   # unbiased up to one grid step / 2^k


def test_sr_recipe_matches_reference_torch_statement():
    # src/utils.py:143-156: result = (int32 bits + rand20) & -1048576 ; :178-191 with 16 bits for bf16
    g = torch.Generator().manual_seed(0)
    p = torch.randn(200000, generator=g) * 0.05
    r20 = torch.randint(0, 1 << 20, p.shape, generator=g, dtype=torch.int32)
    ref = (r20 + p.view(torch.int32)).bitwise_and(-1048576).view(torch.float32).numpy()
    assert np.array_equal(C.sr_add_mask(p.numpy(), r20.numpy().astype(np.uint32), 20).view(np.uint32), ref.view(np.uint32))
    r16 = torch.randint(0, 1 << 16, p.shape, generator=g, dtype=torch.int32)
    ref16 = (r16 + p.view(torch.int32)).bitwise_and(-65536).view(torch.float32).numpy()
    assert np.array_equal(C.sr_add_mask(p.numpy(), r16.numpy().astype(np.uint32), 16).view(np.uint32), ref16.view(np.uint32))


def test_sr_exact_is_unbiased_everywhere_and_saturates():
    rng = np.random.default_rng(3)
    for value in [1.03125, 0.3777, 0.0043945, 0.00097656, 2.1e-4, -0.0123, 447.0]:
        t = np.full(1 << 20, value, dtype=np.float32)
        r = (np.arange(1 << 20, dtype=np.uint64) << np.uint64(12)) | rng.integers(0, 4096, 1 << 20).astype(np.uint64)
        dec = C.e4m3_decode(C.sr_e4m3_exact(t, r)).astype(np.float64)
        assert len(np.unique(dec)) <= 2
        grid = 2.0 ** -9 if abs(value) < 2.0 ** -6 else 2.0 ** (np.floor(np.log2(abs(value))) - 3)
        assert abs(dec.mean() - float(np.float32(value))) <= grid * 2.0 ** -19
    big = np.array([460.0, 1000.0, -1e9], dtype=np.float32)
    assert np.array_equal(C.e4m3_decode(C.sr_e4m3_exact(big, np.array([0xFFFFFFFF] * 3, dtype=np.uint64))),
                          np.array([448.0, 448.0, -448.0], dtype=np.float32))
    # the reference recipe, by contrast, is biased below 2^-6: its final cast rounds to nearest (fuse_kernel.py:29-36)
    t = np.full(1 << 20, 0.00097656 * 0.5, dtype=np.float32)
    ref = C.e4m3_decode(C.e4m3_encode(C.sr_add_mask(t, np.arange(1 << 20, dtype=np.uint64), 20))).astype(np.float64)
    assert abs(ref.mean() - float(t[0])) > 1e-4


def test_sr_exact_agrees_with_hardware_converter_observations():
    # (value, random word, code) triples read back from v_cvt_sr_fp8_f32 on an MI355X
    obs = [(1.03125, 0xBFFFFFFF, 0x38), (1.03125, 0xC0000000, 0x39), (1.09375, 0x3FFFFFFF, 0x38), (1.09375, 0x40000000, 0x39),
           (-1.03125, 0xC0000000, 0xB9), (0.00439453125, 0xBFFFFFFF, 0x02), (0.00439453125, 0xC0000000, 0x03),
           (0.0009765625, 0x7FFFFFFF, 0x00), (0.0009765625, 0x80000000, 0x01), (0.01611328125, 0xC0000000, 0x09),
           (447.0, 0x000FFFFF, 0x7D), (447.0, 0x3FFFFFFF, 0x7E), (1.0, 0xFFFFFFFF, 0x38)]
    for v, r, code in obs:
        got = int(C.sr_e4m3_exact(np.array([v], dtype=np.float32), np.array([r], dtype=np.uint64))[0])
        assert got == code, (v, hex(r), hex(got), hex(code))


def test_e5m2_codec_matches_torch():
    """e5m2 codes decode as the top byte of an IEEE half; the encoder equals torch's cast wherever torch stays finite and
    saturates at 57344 where the compiled kernels do."""
    codes = np.arange(256, dtype=np.uint8)
    ref = torch.from_numpy(codes).view(torch.float8_e5m2).float().numpy()
    got = C.e5m2_decode(codes)
    assert np.array_equal(np.isnan(ref), np.isnan(got)) and np.array_equal(ref[~np.isnan(ref)], got[~np.isnan(got)])
    rng = np.random.default_rng(5)
    x = np.concatenate([rng.standard_normal(100000).astype(np.float32) * np.float32(10.0) ** rng.integers(-7, 5, 100000),
                        np.array([0.0, -0.0, 2.0 ** -16, 2.0 ** -17, 3 * 2.0 ** -17, 57344.0, 61439.0, 1.25, 1.375, 1.125],
                                 dtype=np.float32)]).astype(np.float32)
    t = torch.from_numpy(x).to(torch.float8_e5m2)
    ref_codes = t.view(torch.uint8).numpy()
    finite = np.isfinite(t.float().numpy())
    assert np.array_equal(C.e5m2_encode(x, saturate=False)[finite], ref_codes[finite])
    assert np.array_equal(C.e5m2_encode(x, saturate=False), ref_codes)                  # overflow -> inf as torch
    big = np.array([61440.0, 1e6, np.inf, -1e9], dtype=np.float32)
    assert np.array_equal(C.e5m2_decode(C.e5m2_encode(big, saturate=True)), np.array([57344.0, 57344.0, 57344.0, -57344.0], np.float32))


def test_fast_rounding_words_look_uniform_and_independent():
    """The random words of the fast rounding mode (this build's own definition: one hash per four weights, the first
    weight takes it as it is, the others multiples of it): the top bits, which the converter uses, are uniform for every
    position in the group, and neighbouring weights, rows and seeds are uncorrelated."""
    rows = np.arange(4096, dtype=np.int64)[:, None]
    cols = np.arange(768, dtype=np.int64)[None, :]
    w = C.fast_sr_words(12345, np.broadcast_to(rows, (4096, 768)), np.broadcast_to(cols, (4096, 768)))
    u = (w >> np.uint32(12)).astype(np.float64) / float(1 << 20)        # the 20 bits above the discarded ones
    n = u.size
    for pos in range(4):                                                # every position of the group of four
        v = u[:, pos::4]
        assert abs(v.mean() - 0.5) < 4.0 / np.sqrt(12 * v.size)
        hist = np.bincount((v * 16).astype(np.int64).ravel(), minlength=16)
        assert np.abs(hist / v.size - 1 / 16).max() < 5.0 * np.sqrt((1 / 16) * (15 / 16) / v.size)
    def corr(a, b):
        return float(np.corrcoef(a.ravel(), b.ravel())[0, 1])
    lim = 5.0 / np.sqrt(n / 4)
    assert abs(corr(u[:, 0::4], u[:, 1::4])) < lim and abs(corr(u[:, 0::4], u[:, 3::4])) < lim      # within a group
    assert abs(corr(u[:, 1::4], u[:, 2::4])) < lim
    assert abs(corr(u[:, :-4], u[:, 4:])) < 5.0 / np.sqrt(n) and abs(corr(u[:-1], u[1:])) < 5.0 / np.sqrt(n)   # next group, next row
    w2 = C.fast_sr_words(12346, np.broadcast_to(rows, (4096, 768)), np.broadcast_to(cols, (4096, 768)))
    u2 = (w2 >> np.uint32(12)).astype(np.float64) / float(1 << 20)
    assert abs(corr(u, u2)) < 5.0 / np.sqrt(n)                                                      # next seed


@pytest.mark.parametrize("value", [1.00390625 * 1.3, -7.77, 3.3e-5, 1.0])
def test_sr_bf16_fast_probability_equals_dropped_fraction_exhaustively(value):
    """The fast mode's rounding to bf16 over all 2^16 values of the upper half of the random word (the lower half must not
    matter): floor or ceil in magnitude, ceil exactly `dropped bits` times out of 2^16, a bf16 value unchanged."""
    t = np.full(1 << 16, value, dtype=np.float32)
    hi = np.arange(1 << 16, dtype=np.uint64) << np.uint64(16)
    out = C.sr_bf16_fast(t, hi | np.uint64(0xABCD))
    assert np.array_equal(out, C.sr_bf16_fast(t, hi))
    bits = int(t.view(np.uint32)[0])
    lo_f = np.array([bits & 0xFFFF0000], dtype=np.uint32).view(np.float32)[0]
    hi_f = np.array([(bits & 0xFFFF0000) + 0x10000], dtype=np.uint32).view(np.float32)[0]
    assert set(np.unique(out)) <= {lo_f, hi_f}
    assert int((out == hi_f).sum()) == (bits & 0xFFFF) or (bits & 0xFFFF) == 0
    # the reference's recipe with the same 16 bits in the low half gives the same values (it adds the LOW 16 bits)
    assert np.array_equal(out, C.sr_add_mask(t, hi >> np.uint64(16), 16))
