"""bf16 chunked extreme-classifier layer on the MI355X kernels.

Mirror of the reference's XMCBCECHUNKEDLayer (src/xmc_classifiers/chunked.py): same constructor argument, methods
(`xfc_forward`, `xfc_forward_backward`), attributes (`xfc_weight` - ONE [num_labels, 768] tensor, a plain attribute and
not a Parameter, as there - `grad_input`, `_dtype`, `num_labels`, `num_chunks`, `chunk_size`, `iteration`, `loss`) and
error convention.  The reference's per-chunk sequence (matmul, sigmoid, index_put, matmul, mm, sgd_update with
stochastic rounding; chunked.py:97-127) is one call into the C ABI, three kernels per chunk.

Only the bf16 weight type - the one the reference's stochastic-rounding kernel serves (chunked.py:125-127) - runs on
the gfx950 kernels; fp32 / fp16 weights (precision modes 'purefp', float16) are refused with an AssertionError rather
than routed through PyTorch.  As in the reference's bf16 path, weight decay and momentum are not applied
(stochastic_rounding_kernel.py:91-99 ignores wd; momentum_buff is allocated but never used).

Optional, not in the reference: training.xmc.rounding = "sr_philox" (default: the reference's Philox recipe) | "rtn".
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
        assert self._dtype == torch.bfloat16, \
            f"XMCBCECHUNKEDLayer on gfx950 supports bf16 weights only (got {self._dtype}); there is no PyTorch fallback"
        assert self.device.type == "cuda", "XMCBCECHUNKEDLayer needs a GPU device: there is no CPU path"
        features = cfg.model.xmc.input_features
        assert features == ops.FEATURES, f"the gfx950 kernels are built for {ops.FEATURES} input features"

        num_labels = cfg.data.num_labels
        self.num_labels = num_labels
        self.num_chunks = self.cfg.model.xmc.num_chunks
        self.chunk_size = (num_labels + self.num_chunks - 1) // self.num_chunks

        self.xfc_weight = torch.empty(self.num_labels, features, dtype=self._dtype).to(self.device)
        nn.init.normal_(self.xfc_weight, mean=0.0, std=0.02)

        if _opt(cfg.training.xmc, "momentum", 0) != 0:   # allocated and never used, as in the reference (:38-39)
            self.momentum_buff = torch.zeros(self.num_labels, features, dtype=self._dtype, device=self.device)

        self.rounding = _opt(cfg.training.xmc, "rounding", "sr_philox")
        assert self.rounding in ("sr_philox", "rtn")
        self.grad_input = torch.zeros(cfg.data.batch_size, features, dtype=self._dtype, device=self.device)
        self.dummy = torch.zeros(1, dtype=self._dtype, device=self.device)
        self.loss = torch.tensor(0.0, device=self.device)
        self.iteration = 0
        self._workspace = ops.alloc_tiled_workspace(self.num_chunks, self.chunk_size, self.device,
                                                    min(max(int(cfg.data.batch_size), ops.MAX_BATCH), ops.MAX_BATCH_TILED))

    def _chunks(self):
        w = self.xfc_weight
        assert w.is_contiguous() and w.dtype == torch.bfloat16 and w.shape == (self.num_labels, ops.FEATURES)
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
            embed: Encoder or bottleneck layer output, [B, 768], B <= 256 (any value).
            labels: Positive labels in sparse format (row,col). shape = (Nb,2).
            xmc_lr: list of learning rates, only [0] is used.
            skip_loss: Whether to skip the loss calculation.  When False the summed binary cross entropy of the step's
                       logits is computed inside the logits kernel and returned (one host synchronisation).  This is
                       the value the reference's _compute_loss is written to return (chunked.py:57-72); the reference
                       itself passes the weight chunk where the logits belong (chunked.py:109).
        '''
        assert embed.is_cuda and embed.dim() == 2 and embed.shape[1] == ops.FEATURES
        assert embed.shape[0] <= ops.MAX_BATCH_TILED, "batch must be at most 256"
        assert labels.is_cuda and labels.dim() == 2 and labels.shape[1] == 2
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
