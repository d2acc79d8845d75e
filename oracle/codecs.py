"""Number formats and random bits used by the step (numpy, CPU).  Test infrastructure only.

Follows
  src/triton_kernels/fuse_kernel.py:10-44             stochastic_rounding_to_{bf16,fp8,fakefp8}
  src/triton_kernels/stochastic_rounding_kernel.py:10-28
  src/utils.py:132-194                                 pure-torch statement of the same bit recipe
  triton.language.random (philox, randint)             third-party, shipped with torch 2.6.0 (Triton 3.2):
                                                       Philox-4x32-10 as published by Salmon et al. (Random123)
"""
import numpy as np

E4M3_MAX = 448.0


# --------------------------------------------------------------------------- bf16
def bf16_round(x):
    """Round fp32 values to the nearest bf16 (ties to even); result is fp32 holding bf16 values."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    bias = 0x7FFF + ((u >> 16) & 1)
    r = ((u + bias) & 0xFFFF0000).astype(np.uint32)
    nan = np.isnan(x)
    if nan.any():
        r = np.where(nan, (x.view(np.uint32) | 0x00400000) & 0xFFFF0000, r).astype(np.uint32)
    return r.view(np.float32).reshape(x.shape)


def bf16_bits(x):
    """bf16 values (fp32 container) -> uint16 bit patterns."""
    return (np.ascontiguousarray(x, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)


def bf16_from_bits(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# --------------------------------------------------------------------------- e4m3fn (OCP FP8)
def _e4m3_table():
    codes = np.arange(256, dtype=np.int64)
    s = codes >> 7
    e = (codes >> 3) & 15
    m = codes & 7
    v = np.where(e == 0, m * 2.0 ** -9, (1.0 + m / 8.0) * 2.0 ** (e - 7.0))
    v = np.where((e == 15) & (m == 7), np.nan, v)
    return np.where(s == 1, -v, v).astype(np.float32)


E4M3_TABLE = _e4m3_table()


def e4m3_decode(codes):
    """uint8 e4m3fn codes -> fp32 (exact).  1-4-3, bias 7, no inf, 0x7f/0xff = NaN."""
    return E4M3_TABLE[np.asarray(codes, dtype=np.uint8)]


def e4m3_encode(x, saturate=True):
    """fp32 -> e4m3fn code, round to nearest even.

    saturate=True  : |x| > 448 (including inf) -> +-448, the "satfinite" conversion the compiled
                     Triton kernels use (fuse_kernel.py:35 `.to(tl.float8e4nv)`).
    saturate=False : torch.Tensor.to(torch.float8_e4m3fn) semantics: values that round above 448
                     (|x| > 464) become NaN (chunked_fp8xmc_clf.py:116, simulated-FP8 write-back).
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    a = np.abs(x).astype(np.float64)
    sign = (x.view(np.uint32) >> 31).astype(np.uint8) << 7
    nan = np.isnan(x)
    a = np.where(nan, 0.0, a)
    if saturate:
        a = np.minimum(a, E4M3_MAX)
    over = a > 464.0
    a = np.where(over, 0.0, a)
    # exponent of the binade, clamped to the subnormal lattice
    _, ex = np.frexp(a)                      # a = f * 2**ex, f in [0.5, 1)
    e = np.maximum(ex - 1, -6)               # floor(log2 a), >= -6
    quantum = np.ldexp(1.0, e - 3)
    q = np.rint(a / quantum)                 # half-to-even, exact scaling
    val = q * quantum                        # representable (may have carried into next binade)
    _, ex2 = np.frexp(val)
    e2 = ex2 - 1
    is_sub = (val < 2.0 ** -6)
    exp_field = np.where(is_sub, 0, e2 + 7).astype(np.int64)
    man = np.where(is_sub, val * 512.0, (val / np.ldexp(1.0, e2) - 1.0) * 8.0)
    man = np.where(val == 0, 0, man).astype(np.int64)
    code = (exp_field << 3 | man).astype(np.uint8)
    code = np.where(val == 0, 0, code).astype(np.uint8)
    code = np.where(over | nan, 0x7F, code).astype(np.uint8)
    return (code | sign).astype(np.uint8).reshape(x.shape)


# --------------------------------------------------------------------------- e5m2 (OCP FP8, the Kahan buffer option)
def e5m2_decode(codes):
    """uint8 e5m2 codes -> fp32 (exact): the top byte of an IEEE half."""
    c = np.asarray(codes, dtype=np.uint8).astype(np.uint16) << np.uint16(8)
    return c.view(np.float16).astype(np.float32)


def e5m2_encode(x, saturate=True):
    """fp32 -> e5m2 code, round to nearest even (1-5-2, bias 15, max normal 57344, subnormal step 2^-16).
    saturate=True: finite overflow and inf -> +-57344 (the satfinite conversion of the compiled kernels,
    fuse_kernel.py:255); saturate=False: torch.Tensor.to(torch.float8_e5m2) semantics (overflow -> inf)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    a = np.abs(x).astype(np.float64)
    sign = ((x.view(np.uint32) >> 31).astype(np.uint8) << 7).astype(np.uint8)
    nan = np.isnan(x)
    a = np.where(nan, 0.0, a)
    if saturate:
        a = np.minimum(a, 57344.0)
    _, ex = np.frexp(a)
    e = np.maximum(ex - 1, -14)
    quantum = np.ldexp(1.0, e - 2)
    val = np.rint(a / quantum) * quantum
    over = val > 57344.0
    _, ex2 = np.frexp(np.where(over, 1.0, val))
    e2 = ex2 - 1
    is_sub = val < 2.0 ** -14
    exp_field = np.where(is_sub, 0, e2 + 15).astype(np.int64)
    man = np.where(is_sub, val * 65536.0, (val / np.ldexp(1.0, e2) - 1.0) * 4.0)
    man = np.where(val == 0, 0, man).astype(np.int64)
    code = ((exp_field << 2) | man).astype(np.uint8)
    code = np.where(val == 0, 0, code).astype(np.uint8)
    code = np.where(over, 0x7C, code).astype(np.uint8)          # inf
    code = np.where(nan, 0x7F, code).astype(np.uint8)
    return (code | sign).astype(np.uint8).reshape(x.shape)


# --------------------------------------------------------------------------- Philox-4x32-10
_PH_M0 = np.uint64(0xD2511F53)
_PH_M1 = np.uint64(0xCD9E8D57)
_PH_W0 = 0x9E3779B9
_PH_W1 = 0xBB67AE85


def philox4x32(c0, c1, c2, c3, k0, k1, rounds=10):
    """Vectorised Philox-4x32; all inputs broadcastable uint32 arrays; returns 4 uint32 arrays."""
    c0, c1, c2, c3 = [np.asarray(c, dtype=np.uint64) & 0xFFFFFFFF for c in (c0, c1, c2, c3)]
    c0, c1, c2, c3 = np.broadcast_arrays(c0, c1, c2, c3)
    k0 = int(k0) & 0xFFFFFFFF
    k1 = int(k1) & 0xFFFFFFFF
    for _ in range(rounds):
        p0 = _PH_M0 * c0
        p1 = _PH_M1 * c2
        hi0, lo0 = p0 >> np.uint64(32), p0 & np.uint64(0xFFFFFFFF)
        hi1, lo1 = p1 >> np.uint64(32), p1 & np.uint64(0xFFFFFFFF)
        c0, c1, c2, c3 = hi1 ^ c1 ^ np.uint64(k0), lo1, hi0 ^ c3 ^ np.uint64(k1), lo0
        k0 = (k0 + _PH_W0) & 0xFFFFFFFF
        k1 = (k1 + _PH_W1) & 0xFFFFFFFF
    return tuple(c.astype(np.uint32) for c in (c0, c1, c2, c3))


def tl_randint(seed, offsets):
    """First Philox word for counter (offset,0,0,0), key (seed_lo, seed_hi): what `tl.randint(seed, offs)`
    returns for int32 offsets (fuse_kernel.py:12,30; offsets are the element's flat index, fuse_kernel.py:107)."""
    seed = int(seed) & 0xFFFFFFFFFFFFFFFF
    offs = np.asarray(offsets).astype(np.int64) & 0xFFFFFFFF
    z = np.zeros_like(offs)
    return philox4x32(offs, z, z, z, seed & 0xFFFFFFFF, seed >> 32)[0]


def tl_rand(seed, offsets):
    """`tl.rand(seed, offs)`: the first Philox word as a uniform fp32 in [0, 1) - the word reinterpreted as int32,
    negative values mapped to -x - 1, converted to fp32 (nearest even) and multiplied by 4.6566127342e-10 in fp32
    (Triton language/random.py, uint_to_uniform_float; what the reference's dropout prototype compares with p,
    tma_gemm.py:8-10).  Pinned by vectors from the Triton library's interpreter in tests/golden/triton_rand.json."""
    x = tl_randint(seed, offsets).view(np.int32).astype(np.int64)
    x = np.where(x < 0, -x - 1, x)
    return (x.astype(np.float32) * np.float32(4.6566127342e-10)).astype(np.float32)


def dropout_quantize(x, p, seed, row_stride=None):
    """e4m3 codes of dropout(x): element (m, k) is kept when tl_rand(seed, m * row_stride + k) > p and then scaled by
    1 / (1 - p) in fp32, else zero; cast to e4m3 (nearest even, saturating) - `_dropout` of tma_gemm.py:7-13 applied
    to the whole operand (the prototype calls it per tile with these offsets, tma_gemm.py:34-38).  x: fp32 array [M, K]
    of bf16 or e4m3 values."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    m, k = x.shape
    stride = k if row_stride is None else int(row_stride)
    offs = (np.arange(m, dtype=np.int64)[:, None] * stride + np.arange(k, dtype=np.int64)[None, :])
    keep = tl_rand(seed, offs) > np.float32(p)
    scaled = (x / (np.float32(1.0) - np.float32(p))).astype(np.float32)
    return e4m3_encode(np.where(keep, scaled, np.float32(0.0)), saturate=True)


def dropout_bf16(x, p, seed):
    """The dropped-out embedding of the steps' fused dropout, in the layer's type: element (b, k) of the bf16-valued fp32
    array x [B, K] is kept when tl_rand(seed, b * K + k) > p; X' = bf16(keep ? x / (1 - p) : 0) with the division in
    fp32.  Returns (X' as bf16-valued fp32, keep mask).  Not in the reference's step (its training loop applies
    nn.Dropout before the layer, model.py:135,165; the prototype of the fusion is tma_gemm.py:7-13)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    m, k = x.shape
    offs = (np.arange(m, dtype=np.int64)[:, None] * k + np.arange(k, dtype=np.int64)[None, :])
    keep = tl_rand(seed, offs) > np.float32(p)
    scaled = (x / (np.float32(1.0) - np.float32(p))).astype(np.float32)
    return bf16_round(np.where(keep, scaled, np.float32(0.0)).astype(np.float32)), keep


def dropout_backward(g, keep, p):
    """Gradient in front of the dropout: g * keep / (1 - p), the division in fp32."""
    g = np.ascontiguousarray(g, dtype=np.float32)
    return np.where(keep, (g / (np.float32(1.0) - np.float32(p))).astype(np.float32), np.float32(0.0)).astype(np.float32)


# --------------------------------------------------------------------------- stochastic rounding
def sr_add_mask(t, rand, k):
    """The reference bit recipe: add the low k random bits to the fp32 bit pattern, clear the low k bits.
    k = 20 for e4m3 (fuse_kernel.py:29-36), 16 for bf16 (fuse_kernel.py:10-16).  Returns fp32."""
    t = np.ascontiguousarray(t, dtype=np.float32)
    mask = np.uint64((1 << k) - 1)
    u = t.view(np.uint32).astype(np.uint64)
    u = (u + (np.asarray(rand).astype(np.uint64) & mask)) & np.uint64(0xFFFFFFFF)
    u = (u & ~mask).astype(np.uint32)
    return u.view(np.float32).reshape(t.shape)


def sr_e4m3_reference(t, seed, offsets):
    """fp32 -> e4m3 code as stochastic_rounding_to_fp8 does: SR20 bit recipe then RTNE/satfinite cast."""
    return e4m3_encode(sr_add_mask(t, tl_randint(seed, offsets), 20), saturate=True)


def sr_bf16_reference(t, seed, offsets):
    """fp32 -> bf16 value as stochastic_rounding_to_bf16 does (the final cast is exact)."""
    return sr_add_mask(t, tl_randint(seed, offsets), 16)


def sr_e4m3_exact(t, rand32):
    """True stochastic rounding of fp32 onto the e4m3fn grid (normal AND subnormal range), saturating
    at +-448: round |t| up with probability equal to the dropped fraction, using the top 20 bits of
    rand32.  Not part of the reference; it is the definition of this build's fast SR mode."""
    t = np.ascontiguousarray(t, dtype=np.float32)
    a = np.minimum(np.abs(t), np.float32(E4M3_MAX)).astype(np.float64)
    r20 = (np.asarray(rand32).astype(np.uint64) >> np.uint64(12)).astype(np.float64)
    _, ex = np.frexp(a)
    quantum = np.ldexp(1.0, np.maximum(ex - 1, -6) - 3)     # grid spacing at |t| (2^-9 below 2^-6)
    y = a / quantum                                         # exact
    lo = np.floor(y)
    up = (y - lo) * 1048576.0 + r20 >= 1048576.0            # exact in float64
    v = np.minimum((lo + up) * quantum, E4M3_MAX).astype(np.float32)
    return e4m3_encode(np.copysign(v, t), saturate=True)


def sr_bf16_fast(t, rand32):
    """fp32 -> bf16 value as the hardware converter of this build's fast mode rounds (v_cvt_sr_bf16_f32): the upper 16 bits
    of the random word are added to the fp32 bit pattern and the lower 16 bits dropped - round up with probability equal
    to the dropped fraction.  Not part of the reference (whose recipe adds the low 16 bits of a Philox word, sr_add_mask)."""
    t = np.ascontiguousarray(t, dtype=np.float32)
    u = t.view(np.uint32).astype(np.uint64) + (np.asarray(rand32).astype(np.uint64) >> np.uint64(16))
    u = (u & np.uint64(0xFFFF0000)).astype(np.uint32)
    return u.view(np.float32).reshape(t.shape)


# --------------------------------------------------------------------------- this build's fast SR random words
def fast_sr_words(seed, global_rows, cols, features=768):
    """Random word per weight of the fast stochastic-rounding mode (not part of the reference): one 32-bit mix per
    group of 4 consecutive weights of a row, idx = global_row * (features/4) + col/4; the first weight takes the mix
    itself, the other three its products with odd constants; the seed is mixed first.  Restates
    fast_seed/fast_mix/fast_word of elmo_amd/csrc/xmc_common.h."""
    M = np.uint64(0xFFFFFFFF)
    idx = (np.asarray(global_rows, dtype=np.uint64) * np.uint64(features // 4) + (np.asarray(cols, dtype=np.uint64) >> np.uint64(2))) & M
    sd = int(seed) & 0xFFFFFFFF            # fast_seed: the caller's seed through a full 32-bit mixer
    sd ^= sd >> 16; sd = (sd * 0x7FEB352D) & 0xFFFFFFFF; sd ^= sd >> 15; sd = (sd * 0x846CA68B) & 0xFFFFFFFF; sd ^= sd >> 16
    h = (idx * np.uint64(0x9E3779B1) + np.uint64(sd)) & M
    h ^= h >> np.uint64(16)
    h = (h * np.uint64(0x85EBCA77)) & M
    h ^= h >> np.uint64(15)
    k = np.array([1, 0x27D4EB2F, 0x165667B1, 0x9E3779B1], dtype=np.uint64)[np.asarray(cols, dtype=np.int64) & 3]
    return ((h * k) & M).astype(np.uint32)
