"""FP8 chunked extreme-classifier layer on the MI355X kernels.

Mirror of the reference's Fp8XMCBCEChunkedLayer (src/xmc_classifiers/chunked_fp8xmc_clf.py): same constructor
argument, methods (`xfc_forward`, `xfc_forward_backward`, `filter_non_local_inds`), attributes (`xfc_weight`
ParameterList of e4m3fn chunks, `grad_input`, `_dtype`, `num_labels`, `num_labels_i`, `iteration`, `loss`) and
error convention (AssertionError for shape / layout / device problems), so src/model.py and src/runner.py can
use it unchanged.  The per-chunk Python loop of the reference is replaced by ONE call into the C ABI that
covers all chunks; there is no CPU or PyTorch fallback.

Configuration read (attribute style, OmegaConf not required):
  environment.device, data.num_labels, model.xmc.num_chunks, model.xmc.input_features,
  training.xmc.simulated_fp8
Optional, not in the reference (all default to the reference's behaviour):
  training.xmc.rounding   "sr_fast" (default) | "sr_philox" | "rtn"
        sr_philox reproduces the reference's bit recipe (Philox word per element, fuse_kernel.py:29-36);
        sr_fast rounds stochastically with the hardware converter and a counter hash: unbiased on the whole
        e4m3 grid (subnormals included), not bit-identical to the reference's random stream
  training.xmc.scale_w, training.xmc.scale_x   per-tensor scales (reference: 1.0, 1.0)
  training.xmc.fp8_weight_decay   decay inside the FP8 update, T = W - lr (A + wd W) (reference: none, 0.0)
  training.xmc.fused_dropout      dropout probability of the embedding applied inside the step while the module is in
        training mode, in place of an nn.Dropout in front of the layer (model.py:135,165); grad_input is then the
        gradient in front of that dropout (reference: none, 0.0).  The mask's seed is drawn from the global CPU generator
        after the chunk seeds.
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


class Fp8XMCBCEChunkedLayer(nn.Module):
    '''
    Chunked FP8 XMC classifier
    '''

    def __init__(self, cfg):
        super(Fp8XMCBCEChunkedLayer, self).__init__()
        self.cfg = cfg
        self.device = torch.device(cfg.environment.device)
        self._dtype = torch.float8_e4m3fn
        self.fake_fp8_matmul = cfg.training.xmc.simulated_fp8
        self.num_chunks = self.cfg.model.xmc.num_chunks
        # reference padding rule (chunked_fp8xmc_clf.py:26): always adds between 1 and 16*num_chunks rows
        self.num_labels = cfg.data.num_labels + 16 * self.num_chunks - cfg.data.num_labels % (16 * self.num_chunks)
        self.num_labels_i = self.num_labels // self.num_chunks
        assert self.num_labels_i % 16 == 0
        features = cfg.model.xmc.input_features
        assert features in ops.TILED_FEATURES, f"the gfx950 kernels are built for {ops.TILED_FEATURES} input features"
        assert self.device.type == "cuda", "Fp8XMCBCEChunkedLayer needs a GPU device: there is no CPU path"
        self.features = features
        # The fused step and the inference kernels are built for 768 features.  A layer of 1,024 trains on the
        # three-kernel path (same arithmetic, rounding modes and random words) and takes its inference logits from a
        # library GEMM per chunk on the exactly widened operands, as the reference does (:52-55).
        self._other_width = features != ops.FEATURES

        # same initialisation as the reference (:29-32): xavier-uniform on the padded fp32 matrix, cast per chunk
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

        # simulated FP8 (:98-99,115-116) runs on the three-kernel path, which rounds with the reference's recipe
        self.rounding = _opt(cfg.training.xmc, "rounding", "sr_philox" if self.fake_fp8_matmul else "sr_fast")
        assert self.rounding in (("sr_philox", "rtn") if self.fake_fp8_matmul else ("sr_fast", "sr_philox", "rtn"))
        self.scale_w = float(_opt(cfg.training.xmc, "scale_w", 1.0))
        self.scale_x = float(_opt(cfg.training.xmc, "scale_x", 1.0))
        self.weight_decay = float(_opt(cfg.training.xmc, "fp8_weight_decay", 0.0))
        self.fused_dropout = float(_opt(cfg.training.xmc, "fused_dropout", 0.0))
        assert self.weight_decay >= 0.0 and 0.0 <= self.fused_dropout < 1.0
        self.block_size = 16
        self.loss = torch.tensor(0.0, device=self.device)
        self.iteration = 0
        self.grad_input = None
        # all scratch memory of the step comes from the torch allocator (so that max_memory_allocated sees it)
        self._workspace = (None if self._other_width else
                           ops.alloc_workspace(self.num_chunks, self.num_labels_i, self.device))
        self._tiled_workspace = None
        self._fused_ran = False      # the error word in the workspace is defined once a fused step has run
        # After every fused step the workspace's sticky error word (the error words of all steps since it was last
        # zeroed, OR-ed together by the kernels) is copied to pinned host memory on the step's stream, without waiting;
        # later calls look at the copies that have arrived (see _check_previous_steps).  A ring of slots, so that a copy
        # still in flight is never overwritten by the next one.
        off = ops.step_sticky_error_offset()
        self._err_dev = None if self._other_width else self._workspace[off:off + 4].view(torch.int32)
        self._err_slots = 4
        self._err_host = torch.zeros(self._err_slots, dtype=torch.int32).pin_memory()
        self._err_events = [None] * self._err_slots
        self._err_next = 0
        # batches of more than 128 rows (up to 512) also run on the three-kernel path, with the true-FP8 arithmetic
        self._max_batch = int(_opt(cfg.data, "batch_size", ops.MAX_BATCH))
        if self.fake_fp8_matmul:
            assert self.scale_w == 1.0 and self.scale_x == 1.0, "simulated FP8 has no per-tensor scales"
        # the fused kernel's sort keys hold 24 bits of label: larger label spaces run on the three-kernel path, which sorts
        # the positives per segment of the label space
        self._wide = self.num_labels >= (1 << 24) - 1
        if self._other_width:
            assert self.scale_w == 1.0 and self.scale_x == 1.0, "per-tensor scales belong to the fused step (768 features)"
        if self.fake_fp8_matmul or self._max_batch > ops.MAX_BATCH or self._wide or self._other_width:
            self._tiled_workspace = ops.alloc_tiled_workspace(self.num_chunks, self.num_labels_i, self.device,
                                                              min(max(self._max_batch, ops.MAX_BATCH), ops.MAX_BATCH_TILED),
                                                              features)

    def _chunks(self):
        return [w.data for w in self.xfc_weight]

    def _simulated_logits(self, embed):
        # simulated FP8 (:51-52): matmul(embed.bf16, W.bf16) per chunk with the embedding as it comes - NOT quantised
        # to e4m3, unlike the true-FP8 branch (:53-56).  (The evaluator casts the embedding to e4m3 itself before the
        # call, evaluate.py:155-156; such an input is widened exactly.)  A library bf16 GEMM per chunk, as in the
        # reference; this debugging mode has no kernel of its own here.
        x = embed.to(torch.bfloat16)
        outs = [torch.matmul(x, w.data.to(torch.bfloat16).t()) for w in self.xfc_weight]
        return torch.cat(outs, dim=1)[:, :self.cfg.data.num_labels]

    def _widened_logits(self, embed):
        # true-FP8 logits (:53-56) for a width the inference kernel is not built for: Z = W_i e4m3(X)^T per chunk through
        # the library's bf16 GEMM.  Both operands are e4m3 values, which bf16 holds exactly, and the products are summed
        # in fp32, so only the order of the fp32 sums differs from an FP8 GEMM.
        xq = embed.to(torch.float8_e4m3fn).to(torch.bfloat16)
        outs = [torch.matmul(xq, w.data.to(torch.bfloat16).t()) for w in self.xfc_weight]
        return torch.cat(outs, dim=1)[:, :self.cfg.data.num_labels]

    @torch.no_grad()
    def xfc_forward(self, embed):
        '''
        Mainly used during inference: logits [B, cfg.data.num_labels] in bf16 (padding rows dropped).
        '''
        assert embed.is_cuda and embed.dim() == 2
        if self.fake_fp8_matmul:
            return self._simulated_logits(embed)
        if self._other_width:
            return self._widened_logits(embed)
        return ops.fp8_forward(self._chunks(), embed, self.cfg.data.num_labels, self.scale_w, self.scale_x,
                               self._workspace)

    @torch.no_grad()
    def xfc_forward_topk(self, embed, k):
        '''
        values, indices = xfc_forward(embed).topk(k) (what evaluate.py:158-159,235-236 compute) without the dense
        [B, num_labels] logits: the top-k is merged chunk by chunk.  Not in the reference; k <= 128.
        '''
        assert embed.is_cuda and embed.dim() == 2
        if self.fake_fp8_matmul or self._other_width:
            vals, idx = (self._simulated_logits(embed) if self.fake_fp8_matmul else self._widened_logits(embed)).topk(k)
            return vals, idx
        return ops.fp8_forward_topk(self._chunks(), embed, self.cfg.data.num_labels, k, self.scale_w, self.scale_x,
                                    self._workspace)

    @torch.no_grad()
    def _compute_loss(self, outlogit, rows, cols):
        '''
        BCE-with-logits summed over a dense logit block (reference :62-78; never reached in training because
        the training loop always passes skip_loss=True).
        '''
        z = outlogit.float()
        loss = z.clamp(min=0.0).sum() - z[rows, cols].sum() + torch.log1p(torch.exp(-z.abs())).sum()
        return loss.item()

    @torch.no_grad()
    def xfc_forward_backward(self, embed, labels, xmc_lr, skip_loss=True):
        '''
        Computes activation gradients for the XMC layer fused with BCE Loss and applies the SGD update.
        Args:
            embed: Encoder or bottleneck layer output, bf16 [B, 768] or [B, 1024], B a multiple of 16 and <= 512 (the
                   fused kernel takes up to 128 rows of 768 features, everything else runs on the three-kernel path).
            labels: Positive labels in sparse format, int32 [Nb, 2] = (row in batch, label id).
            xmc_lr: list of learning rates, only [0] is used.
            skip_loss: ignored, as in the reference's FP8 layer; the return value is 0.
        '''
        assert embed.is_cuda and embed.dim() == 2 and embed.shape[1] == self.features
        assert embed.shape[0] <= ops.MAX_BATCH_TILED and (self.fake_fp8_matmul or embed.shape[0] % 16 == 0), \
            "batch must be a multiple of 16 and at most 512 (the reference data loader uses drop_last)"
        assert labels.is_cuda and labels.dim() == 2 and labels.shape[1] == 2
        x = embed.detach()
        if x.dtype != torch.bfloat16:
            x = x.to(torch.bfloat16)
        x = x.contiguous()
        lab = labels if labels.dtype == torch.int32 else labels.to(torch.int32)
        lab = lab.contiguous()
        loss = 0
        # one seed per chunk from the global CPU generator, exactly as the reference draws them (:113)
        seeds = [torch.randint(0, 1000000, (1,)).item() for _ in range(self.num_chunks)]
        extra = dict(weight_decay=self.weight_decay)
        if self.fused_dropout > 0.0 and self.training:
            extra.update(dropout_p=self.fused_dropout, dropout_seed=torch.randint(0, 2 ** 62, (1,)).item())
        if self.fake_fp8_matmul:
            self.grad_input = ops.tiled_step(self._chunks(), self.num_labels_i, "e4m3", x, lab, xmc_lr[0], seeds=seeds,
                                             round_mode=self.rounding, workspace=self._tiled_workspace, **extra)
        elif embed.shape[0] > ops.MAX_BATCH or self._wide or self._other_width:
            # the fused kernel holds 128 batch rows; larger batches take the three-kernel path with the same arithmetic
            # (logits from e4m3(X), saturating cast) and the same rounding modes and random words
            assert self.scale_w == 1.0 and self.scale_x == 1.0, "per-tensor scales need a batch of at most 128 rows of 768 features"
            self.grad_input = ops.tiled_step(self._chunks(), self.num_labels_i, "e4m3", x, lab, xmc_lr[0], seeds=seeds,
                                             round_mode=self.rounding, workspace=self._tiled_workspace, quantize_x=True,
                                             saturate=True, **extra)
        else:
            self._check_previous_steps()
            self.grad_input = ops.fp8_step(self._chunks(), x, lab, xmc_lr[0], seeds=seeds, round_mode=self.rounding,
                                           scale_w=self.scale_w, scale_x=self.scale_x, workspace=self._workspace, **extra)
            self._fused_ran = True
            # the sticky error word follows the step on the stream into pinned host memory; nobody waits for it here
            slot = self._err_next
            if self._err_events[slot] is not None:
                self._err_events[slot].synchronize()      # that copy was enqueued four steps ago
                self._raise_on_error(int(self._err_host[slot]))
            self._err_host[slot:slot + 1].copy_(self._err_dev, non_blocking=True)
            ev = torch.cuda.Event()
            ev.record()
            self._err_events[slot] = ev
            self._err_next = (slot + 1) % self._err_slots
        self.iteration += 1
        return loss

    def _raise_on_error(self, word):
        if word != 0:
            self._err_dev.zero_()                 # on the stream, behind every step enqueued so far
            self._err_host.zero_()
            self._err_events = [None] * self._err_slots
            raise RuntimeError(
                f"a fused classifier step failed (error word {word}): "
                + ("a workgroup gave up waiting for its partners (another stream kept the device busy?); " if word & 1 else "")
                + ("the workgroups of a quad were not placed on one XCD; " if word & 2 else "")
                + "the weights and grad_input of that step are incomplete")

    def _check_previous_steps(self):
        """Raises if a fused step reported a failure and a copy of the sticky error word taken behind it has reached the
        host.  Never waits: a copy that is still on its way is looked at by a later call.  The word is sticky, so a
        failure is not lost when later, clean steps have run in between."""
        for slot in range(self._err_slots):
            ev = self._err_events[slot]
            if ev is not None and ev.query():
                self._err_events[slot] = None
                self._raise_on_error(int(self._err_host[slot]))

    def check_steps(self):
        """Waits for the steps enqueued so far and raises if any of them failed (the end of a run, a checkpoint).  Not
        part of the reference's interface."""
        if self._fused_ran:
            torch.cuda.current_stream().synchronize()
            self._raise_on_error(int(self._err_dev.item()))

    def last_step_error(self):
        """Error word of the last fused step (0 = fine; non-zero = a workgroup gave up waiting for its partners, e.g.
        because another stream kept the device busy, and that step's results are invalid).  Synchronises the stream.
        Not part of the reference's interface."""
        if not self._fused_ran:
            return 0
        return ops.step_error_word(self._workspace, self.num_chunks, self.xfc_weight[0].shape[0])

    def filter_non_local_inds(self, rows, cols, start, end):
        mask = (cols >= start) & (cols < end)
        return rows[mask], cols[mask] - start
