"""bf16 chunked extreme-classifier layer on the MI355X kernels.

Mirror of the reference's XMCBCECHUNKEDLayer (src/xmc_classifiers/chunked.py): same constructor argument, methods
(`xfc_forward`, `xfc_forward_backward`), attributes (`xfc_weight` - ONE [num_labels, 768] tensor, a plain attribute and
not a Parameter, as there - `grad_input`, `_dtype`, `num_labels`, `num_chunks`, `chunk_size`, `iteration`, `loss`) and
error convention.  The reference's per-chunk sequence (matmul, sigmoid, index_put, matmul, mm, sgd_update with
stochastic rounding; chunked.py:97-127) is one call into the C ABI, three kernels per chunk.

The bf16 weight type - the one the reference's stochastic-rounding kernel serves (chunked.py:125-127) - runs on the
gfx950 kernels.  As in the reference's bf16 path, weight decay and momentum are not applied there
(stochastic_rounding_kernel.py:91-99 ignores wd; momentum_buff is allocated but never used).

fp32 / fp16 weights (precision mode 'purefp', model.xmc.dtype float16/float32) take the reference's other branch
(chunked.py:97-124), which has no custom kernel in the reference either: library GEMMs (torch.matmul -> hipBLASLt on the
GPU) and elementwise torch operations in the weight's type, with weight decay: A += wd*W; W += -lr*A.  It is restated
here operation by operation, on the GPU, for any batch size; momentum stays unused as in the reference.

Optional, not in the reference: training.xmc.rounding = "sr_philox" (default: the reference's Philox recipe) | "rtn" |
"sr_fast" (the hardware's stochastic conversion to bf16 with a counter hash: unbiased, not the reference's random stream,
and not bound by the 48 vector instructions per weight of the Philox recipe).
"""
import torch
from torch import nn

from .. import ops

dtype_map = {'float16': torch.float16, 'bfloat16': torch.bfloat16, 'float32': torch.float32,
             'float8': torch.float8_e4m3fn}


def _opt(node, name, default):
    try:
        v = getattr(node, name)
    except Exception:
        return default
    return default if v is None else v


class XMCBCECHUNKEDLayer(nn.Module):
    '''
    Custom XMC layer fused with BCE Loss.
    Vanilla XMC Layer with Chunked updates (bf16 weights on this build).
    '''

    def __init__(self, cfg):
        super(XMCBCECHUNKEDLayer, self).__init__()
        self.cfg = cfg
        self.device = torch.device(cfg.environment.device)
        # same precedence as the reference (chunked.py:21-23)
        self._dtype = dtype_map[cfg.model.xmc.dtype]
        self._dtype = torch.float32 if cfg.training.precision.mode in ['purefp'] else self._dtype
        self._dtype = dtype_map[cfg.training.precision.purelp_dtype] if cfg.training.precision.mode in ['purelp'] else self._dtype
        assert self._dtype in (torch.bfloat16, torch.float32, torch.float16), f"unsupported weight type {self._dtype}"
        assert self.device.type == "cuda", "XMCBCECHUNKEDLayer needs a GPU device: there is no CPU path"
        features = cfg.model.xmc.input_features
        assert features in ops.TILED_FEATURES or self._dtype != torch.bfloat16, \
            f"the gfx950 kernels of the bf16 layer are built for {ops.TILED_FEATURES} input features"
        self.features = features

        num_labels = cfg.data.num_labels
        self.num_labels = num_labels
        self.num_chunks = self.cfg.model.xmc.num_chunks
        self.chunk_size = (num_labels + self.num_chunks - 1) // self.num_chunks

        self.xfc_weight = torch.empty(self.num_labels, features, dtype=self._dtype).to(self.device)
        nn.init.normal_(self.xfc_weight, mean=0.0, std=0.02)

        if _opt(cfg.training.xmc, "momentum", 0) != 0:   # allocated and never used, as in the reference (:38-39)
            self.momentum_buff = torch.zeros(self.num_labels, features, dtype=self._dtype, device=self.device)

        self.rounding = _opt(cfg.training.xmc, "rounding", "sr_philox")
        assert self.rounding in ("sr_philox", "rtn", "sr_fast")
        self.wd = float(_opt(cfg.training.xmc, "wd", 0.0))      # used by the fp32 / fp16 branch only (chunked.py:123)
        self.grad_input = torch.zeros(cfg.data.batch_size, features, dtype=self._dtype, device=self.device)
        self.dummy = torch.zeros(1, dtype=self._dtype, device=self.device)
        self.loss = torch.tensor(0.0, device=self.device)
        self.iteration = 0
        self._workspace = None
        if self._dtype == torch.bfloat16:
            self._workspace = ops.alloc_tiled_workspace(self.num_chunks, self.chunk_size, self.device,
                                                        min(max(int(cfg.data.batch_size), ops.MAX_BATCH), ops.MAX_BATCH_TILED),
                                                        features)

    def _chunks(self):
        w = self.xfc_weight
        assert w.is_contiguous() and w.dtype == self._dtype and w.shape == (self.num_labels, self.features)
        views = []
        for c in range(self.num_chunks):
            lo, hi = c * self.chunk_size, min((c + 1) * self.chunk_size, self.num_labels)
            if lo < hi:
                views.append(w[lo:hi])
        return views

    @torch.no_grad()
    def xfc_forward(self, embed):
        '''
        Mainly used during inference (chunked.py:48-53): one bf16 matmul through the GPU BLAS, as in the reference.
        '''
        return torch.matmul(embed, self.xfc_weight.t())

    @torch.no_grad()
    def _compute_loss(self, outlogit, rows, cols):
        '''
        BCE-with-logits summed over a dense logit block (chunked.py:55-72).
        '''
        z = outlogit.float()
        loss = z.clamp(min=0.0).sum() - z[rows, cols].sum() + torch.log1p(torch.exp(-z.abs())).sum()
        return loss.item()

    @torch.no_grad()
    def xfc_forward_backward(self, embed, labels, xmc_lr, skip_loss=True):
        '''
        Computes activation gradients for the XMC layer fused with BCE Loss and applies the SGD update.
        Args:
            embed: Encoder or bottleneck layer output, [B, 768] or [B, 1024], B <= 512 (any value; bf16 weights).
            labels: Positive labels in sparse format (row,col). shape = (Nb,2).
            xmc_lr: list of learning rates, only [0] is used.
            skip_loss: Whether to skip the loss calculation.  When False the summed binary cross entropy of the step's
                       logits is computed inside the logits kernel and returned (one host synchronisation).  This is
                       the value the reference's _compute_loss is written to return (chunked.py:57-72); the reference
                       itself passes the weight chunk where the logits belong (chunked.py:109).
        '''
        assert embed.is_cuda and embed.dim() == 2 and embed.shape[1] == self.features
        assert labels.is_cuda and labels.dim() == 2 and labels.shape[1] == 2
        if self._dtype != torch.bfloat16:
            return self._dense_step(embed.detach(), labels, xmc_lr, skip_loss)
        assert embed.shape[0] <= ops.MAX_BATCH_TILED, "batch must be at most 512"
        x = embed.detach()
        if x.dtype != self._dtype:
            x = x.to(self._dtype)
        x = x.contiguous()
        lab = labels if labels.dtype == torch.int32 else labels.to(torch.int32)
        lab = lab.contiguous()
        loss = 0
        views = self._chunks()
        # one seed per chunk from the global CPU generator, as the reference draws them (chunked.py:126)
        seeds = [torch.randint(0, 1000000, (1,)).item() for _ in range(len(views))]
        loss_out = None if skip_loss else torch.zeros(1, dtype=torch.float32, device=x.device)
        self.grad_input = ops.tiled_step(views, self.chunk_size, "bf16", x, lab, xmc_lr[0], seeds=seeds,
                                         round_mode=self.rounding, workspace=self._workspace, loss_out=loss_out)
        self.iteration += 1
        if loss_out is not None:
            loss = loss_out.item()
        return loss

    def _dense_step(self, embed, labels, xmc_lr, skip_loss):
        """fp32 / fp16 weights: chunked.py:85-124 operation by operation (library GEMMs and elementwise operations in the
        weight's type; grad_input accumulated in fp32; weight decay folded into the gradient before the update)."""
        rows, cols = labels[:, 0].long(), labels[:, 1].long()
        loss = 0
        bsz = embed.shape[0]
        if embed.dtype != self._dtype:
            embed = embed.to(self._dtype)                                          # :89-90
        grad_input = torch.zeros(bsz, self.features, dtype=torch.float32, device=self.device)   # :93
        for chunk_idx in range(self.num_chunks):
            start_idx = chunk_idx * self.chunk_size
            end_idx = min(start_idx + self.chunk_size, self.num_labels)
            if start_idx >= end_idx:
                continue
            weight_chunk = self.xfc_weight[start_idx:end_idx, :]
            outlogit_chunk = torch.matmul(embed, weight_chunk.t())                 # :101
            mask = (cols >= start_idx) & (cols < end_idx)                          # :103-105
            rows_chunk, cols_chunk = rows[mask], cols[mask] - start_idx
            if not skip_loss:
                # the summed binary cross entropy of the chunk's logits: what _compute_loss is written to return (the
                # reference hands it the weight chunk instead of the logits, chunked.py:109)
                loss += self._compute_loss(outlogit_chunk, rows_chunk, cols_chunk)
            torch.sigmoid(outlogit_chunk, out=outlogit_chunk)                      # :112
            outlogit_chunk[rows_chunk, cols_chunk] -= 1.0                          # :113 (set semantics)
            grad_input += torch.matmul(outlogit_chunk, weight_chunk)               # :116
            xfc_weight_grad = outlogit_chunk.t().mm(embed)                         # :119
            xfc_weight_grad.add_(weight_chunk, alpha=self.wd)                      # :123
            weight_chunk.add_(xfc_weight_grad, alpha=-xmc_lr[0])                   # :124
        self.grad_input = grad_input.to(self._dtype)                               # :130
        self.iteration += 1
        return loss
