"""CPU restatement of the ELMO extreme-classifier training step.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory: it is the checker used by the tests, by the smoke run and by the
CPU-baseline leg of the benchmark, never the thing measured or shipped.

Modules
  codecs      e4m3fn / bf16 codecs, Philox-4x32-10, stochastic-rounding bit recipes
  step        closed-form numpy restatement of the three step variants
  torch_port  line-by-line PyTorch-CPU port of the bf16 chunked layer (CPU baseline)

Pinning status (each item is exercised in tests/test_oracle_*.py):
  e4m3fn decode/encode   pinned: torch CPU casts (all 256 codes, rounding-boundary sweep,
                         448/464/465 edge, subnormal lattice)
  bf16 rounding          pinned: torch CPU cast on a boundary sweep
  Philox-4x32-10         pinned: Random123 known-answer vectors and the four tl.randint
                         words recorded for seed 1024
  SR bit recipe          pinned: exhaustive enumeration of all 2^k random values
                         (probability of rounding up == dropped fraction), floor/ceil
                         membership, and the reference's second, pure-torch statement
                         of the same recipe
  step (fp8/sim/bf16)    pinned: brute-force scalar loops on tiny inputs, chunking
                         invariance, duplicate-positive set semantics, and the
                         independent torch_port restatement
The reference holds no golden vectors or asserting tests for this path, so nothing
beyond the above exists to pin against.
"""
