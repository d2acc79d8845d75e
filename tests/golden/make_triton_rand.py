"""Writes tests/golden/triton_rand.json: tl.rand(seed, offsets) of the Triton library in this image, run through its
CPU interpreter (TRITON_INTERPRET=1), as fp32 bit patterns.  tl.rand is what the reference's dropout prototype draws
its keep mask from (src/triton_kernels/tma_gemm.py:8-13); this pins the oracle's restatement of the uint32 -> uniform
float conversion (the Philox words themselves are pinned by the Random123 vectors).  Library code only: nothing of the
reference is imported or run."""
import json
import os
os.environ["TRITON_INTERPRET"] = "1"
import numpy as np
import torch
import triton
import triton.language as tl


@triton.jit
def _rand(out_ptr, seed, n, BLOCK: tl.constexpr):
    offs = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    r = tl.rand(seed, offs)
    tl.store(out_ptr + offs, r, mask=offs < n)


def main():
    cases = {}
    for seed, start in [(40, 0), (1024, 0), (7, 98304)]:
        n = 64
        out = torch.zeros(start + n, dtype=torch.float32)
        _rand[((start + n + 63) // 64,)](out, seed, start + n, BLOCK=64)
        cases[f"{seed}:{start}"] = [int(v) for v in out[start:].numpy().view(np.uint32)]
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "triton_rand.json")
    with open(path, "w") as f:
        json.dump({"triton": triton.__version__, "cases": cases}, f)
    print("wrote", path)


if __name__ == "__main__":
    main()
