"""PyTorch-CPU port of the reference's bf16 chunked layer step.  Test infrastructure only.

It mirrors src/xmc_classifiers/chunked.py:85-131 operation by operation with torch CPU ops (bf16 matmuls
with fp32 accumulation, in-place sigmoid, non-accumulating index_put), with the Triton `_sgd` update
(src/triton_kernels/stochastic_rounding_kernel.py:65-99) replaced by its round-to-nearest form
`bf16(f32(W) - lr*f32(A))`.  It serves two purposes: an independent cross-check of oracle.step.bf16_step and
the timed CPU baseline reported beside the GPU number.
"""
import torch


@torch.no_grad()
def bf16_chunked_step(weight, embed, labels, lr, num_chunks):
    """weight: bf16 [L,d] (updated in place); embed: bf16 [B,d]; labels: int32 [Nb,2].  Returns grad_input bf16."""
    rows, cols = labels[:, 0].long(), labels[:, 1].long()
    L, d = weight.shape
    bsz = embed.shape[0]
    chunk = (L + num_chunks - 1) // num_chunks
    grad_input = torch.zeros(bsz, d, dtype=torch.float32)
    for c in range(num_chunks):
        lo, hi = c * chunk, min((c + 1) * chunk, L)
        if lo >= hi:
            continue
        w = weight[lo:hi]
        out = torch.matmul(embed, w.t())                      # :101
        mask = (cols >= lo) & (cols < hi)                     # :103-105
        r, cc = rows[mask], cols[mask] - lo
        torch.sigmoid(out, out=out)                           # :112
        out[r, cc] -= 1.0                                     # :113
        grad_input += torch.matmul(out, w)                    # :116
        wgrad = out.t().mm(embed)                             # :119
        w.copy_((w.float() - lr * wgrad.float()).to(torch.bfloat16))   # RTN form of :126-127
    return grad_input.to(torch.bfloat16)
