"""FP8 chunked extreme-classifier layer with Kahan-compensated head labels, on the MI355X kernels.

Mirror of the reference's Fp8XMCBCEChunkedHeadKahanLayer (src/xmc_classifiers/chunked_head_kahan_fp8xmc_clf.py): same
constructor argument, methods, attributes (`xfc_weight` ParameterList of e4m3fn chunks, `head_kahan` [num_head, 768] in
bf16 or float8_e5m2, `num_head`, `grad_input`, `_dtype`, `iteration`) and configuration fields
(training.FP8.using_head_kahan, training.FP8.fp8_head_kahan, training.FP8.head_ratio, training.xmc.simulated_fp8).

Without the compensation buffer (using_head_kahan false) and without simulated FP8 the step is the fused kernel of
Fp8XMCBCEChunkedLayer.  With the buffer the step is the fused kernel as well (ops.fp8_kahan_step: the tiles that hold
head rows run first, in a variant of the kernel that carries the Kahan recurrence of fuse_kernel.py:202-262 for the
first num_head rows of chunk 0; the other tiles follow in the plain kernel) whenever the batch is a multiple of 16;
any other batch runs on the three-kernel path in the same true-FP8 arithmetic (logits from e4m3(X), saturating cast).
As in the reference, simulated FP8 takes precedence over the compensation (:122-124).

Optional, not in the reference: training.xmc.rounding ("sr_philox" default with simulated FP8, else "sr_fast"; "rtn").
"""
import torch
from torch import nn

from .. import ops
from .chunked_fp8xmc_clf import _opt

dtype_map = {'float16': torch.float16, 'bfloat16': torch.bfloat16, 'float32': torch.float32,
             'float8': torch.float8_e4m3fn}


class Fp8XMCBCEChunkedHeadKahanLayer(nn.Module):
    '''
    Chunked FP8 XMC classifier
    '''

    def __init__(self, cfg):
        super(Fp8XMCBCEChunkedHeadKahanLayer, self).__init__()
        self.cfg = cfg
        self.device = torch.device(cfg.environment.device)
        self._dtype = torch.float8_e4m3fn
        self.fake_fp8_matmul = cfg.training.xmc.simulated_fp8
        self.using_head_kahan = cfg.training.FP8.using_head_kahan
        self.num_chunks = self.cfg.model.xmc.num_chunks
        self.num_labels = cfg.data.num_labels + 16 * self.num_chunks - cfg.data.num_labels % (16 * self.num_chunks)
        self.num_labels_i = self.num_labels // self.num_chunks
        assert self.num_labels_i % 16 == 0
        features = cfg.model.xmc.input_features
        assert features in ops.TILED_FEATURES, f"the gfx950 kernels are built for {ops.TILED_FEATURES} input features"
        self.features = features
        # 768 features: fused step and inference kernel; 1,024: three-kernel path (same arithmetic) and a library GEMM per
        # chunk on the exactly widened operands for inference, as the reference does (:64-67)
        self._other_width = features != ops.FEATURES
        assert self.device.type == "cuda", "Fp8XMCBCEChunkedHeadKahanLayer needs a GPU device: there is no CPU path"

        xfc_weight = torch.empty(self.num_labels, features, dtype=torch.float32)
        nn.init.xavier_uniform_(xfc_weight)
        self.xfc_weight = nn.ParameterList([
            nn.Parameter(xfc_weight[i * self.num_labels_i:(i + 1) * self.num_labels_i].to(torch.float8_e4m3fn)
                         .to(self.device).contiguous(), requires_grad=False)
            for i in range(self.num_chunks)])
        del xfc_weight
        n_labels = 0
        for i in range(self.num_chunks):
            n_labels += self.xfc_weight[i].shape[0]
            assert self.xfc_weight[i].shape[0] == self.num_labels_i
        assert n_labels == self.num_labels

        if self.using_head_kahan:
            self.fp8_head_kahan = cfg.training.FP8.fp8_head_kahan
            self.num_head = int(cfg.training.FP8.head_ratio * self.num_labels)
            kdt = torch.float8_e5m2 if self.fp8_head_kahan else torch.bfloat16
            self.head_kahan = torch.zeros(self.num_head, features, dtype=kdt, device=self.device)
            assert 0 < self.num_head <= self.num_labels_i
        self._tiled = bool(self.fake_fp8_matmul or self.using_head_kahan or self._other_width)
        self.rounding = _opt(cfg.training.xmc, "rounding", "sr_philox" if self.fake_fp8_matmul else "sr_fast")
        assert self.rounding in (("sr_philox", "rtn") if self.fake_fp8_matmul else ("sr_fast", "sr_philox", "rtn"))
        self.block_size = 16
        self.loss = torch.tensor(0.0, device=self.device)
        self.iteration = 0
        self.grad_input = None
        self._workspace = None if self._other_width else ops.alloc_workspace(self.num_chunks, self.num_labels_i, self.device)
        self._tiled_workspace = (ops.alloc_tiled_workspace(self.num_chunks, self.num_labels_i, self.device, ops.MAX_BATCH,
                                                           features) if self._tiled else None)

    def _chunks(self):
        return [w.data for w in self.xfc_weight]

    @torch.no_grad()
    def xfc_forward(self, embed):
        '''
        Mainly used during inference: logits [B, cfg.data.num_labels] in bf16 (padding rows dropped, :71).
        '''
        assert embed.is_cuda and embed.dim() == 2
        if self.fake_fp8_matmul:
            # simulated FP8 (:62-63): a bf16 GEMM per chunk on the embedding as it comes, not quantised to e4m3
            x = embed.to(torch.bfloat16)
            outs = [torch.matmul(x, w.data.to(torch.bfloat16).t()) for w in self.xfc_weight]
            return torch.cat(outs, dim=1)[:, :self.cfg.data.num_labels]
        if self._other_width:
            # e4m3 operands widened exactly to bf16, fp32 sums: only their order differs from an FP8 GEMM
            xq = embed.to(torch.float8_e4m3fn).to(torch.bfloat16)
            outs = [torch.matmul(xq, w.data.to(torch.bfloat16).t()) for w in self.xfc_weight]
            return torch.cat(outs, dim=1)[:, :self.cfg.data.num_labels]
        return ops.fp8_forward(self._chunks(), embed, self.cfg.data.num_labels, 1.0, 1.0, self._workspace)

    @torch.no_grad()
    def _compute_loss(self, outlogit, rows, cols):
        z = outlogit.float()
        loss = z.clamp(min=0.0).sum() - z[rows, cols].sum() + torch.log1p(torch.exp(-z.abs())).sum()
        return loss.item()

    @torch.no_grad()
    def xfc_forward_backward(self, embed, labels, xmc_lr, skip_loss=True):
        '''
        Computes activation gradients for the XMC layer fused with BCE Loss and applies the SGD update.
        Args as Fp8XMCBCEChunkedLayer.xfc_forward_backward; skip_loss is ignored as in the reference; returns 0.
        '''
        assert embed.is_cuda and embed.dim() == 2 and embed.shape[1] == self.features
        assert embed.shape[0] <= ops.MAX_BATCH and (self._tiled or embed.shape[0] % 16 == 0), \
            "batch must be a multiple of 16 and at most 128 (the reference data loader uses drop_last)"
        assert labels.is_cuda and labels.dim() == 2 and labels.shape[1] == 2
        x = embed.detach()
        if x.dtype != torch.bfloat16:
            x = x.to(torch.bfloat16)
        x = x.contiguous()
        lab = labels if labels.dtype == torch.int32 else labels.to(torch.int32)
        lab = lab.contiguous()
        loss = 0
        seeds = [torch.randint(0, 1000000, (1,)).item() for _ in range(self.num_chunks)]      # :120
        if self.fake_fp8_matmul:
            self.grad_input = ops.tiled_step(self._chunks(), self.num_labels_i, "e4m3", x, lab, xmc_lr[0], seeds=seeds,
                                             round_mode=self.rounding, workspace=self._tiled_workspace)
        elif self.using_head_kahan and embed.shape[0] % 16 == 0 and not self._other_width:
            self.grad_input = ops.fp8_kahan_step(self._chunks(), self.head_kahan, self.num_head, x, lab, xmc_lr[0],
                                                 seeds=seeds, round_mode=self.rounding, workspace=self._workspace)
        elif self.using_head_kahan:
            self.grad_input = ops.tiled_step(self._chunks(), self.num_labels_i, "e4m3", x, lab, xmc_lr[0], seeds=seeds,
                                             round_mode=self.rounding, workspace=self._tiled_workspace, quantize_x=True,
                                             saturate=True, kahan=self.head_kahan, num_head=self.num_head)
        elif self._other_width:
            self.grad_input = ops.tiled_step(self._chunks(), self.num_labels_i, "e4m3", x, lab, xmc_lr[0], seeds=seeds,
                                             round_mode=self.rounding, workspace=self._tiled_workspace, quantize_x=True,
                                             saturate=True)
        else:
            self.grad_input = ops.fp8_step(self._chunks(), x, lab, xmc_lr[0], seeds=seeds, round_mode=self.rounding,
                                           workspace=self._workspace)
        self.iteration += 1
        return loss

    def filter_non_local_inds(self, rows, cols, start, end):
        mask = (cols >= start) & (cols < end)
        return rows[mask], cols[mask] - start
