"""Loss wrappers with the reference's signatures (`forward(input, target, model=None)`,
pfeife/loss.py:4-70).

`CrossEntropyLoss` / `HFCrossEntropyLoss` are the mean-reduced cross entropy of
nn.CrossEntropyLoss computed by the pf_cross_entropy_fwd/bwd kernels when the
logits live on the GPU; `SumLoss` uses pf_sum_fwd.  The wrappers are ordinary
autograd nodes, so user code keeps calling `loss.backward()`.
"""
import torch
import torch.nn as nn


def _kernels_for(t):
    if t.device.type != "cuda":
        raise RuntimeError("pfeife_amd.loss: the HIP loss kernels need GPU tensors (got %s)" % t.device)
    from .hip import HipKernels

    k = getattr(_kernels_for, "_k", None)
    if k is None:
        k = _kernels_for._k = HipKernels(t.device.index)
    return k


_scratch = {}


def _scratch_buffer(name, shape, dtype, device):
    """Per-shape work buffers of the loss kernels, allocated once: every micro-batch's loss is
    evaluated on the same stream in turn, and each buffer's last reader (the backward kernel, or the
    copy of the gradient into the stage's own buffer) is enqueued before the next micro-batch's
    writer, so a training loop makes no allocator call and no fill here."""
    key = (name, tuple(shape), dtype, str(device))
    t = _scratch.get(key)
    if t is None:
        if len(_scratch) > 64:
            _scratch.clear()
        t = _scratch[key] = torch.empty(shape, dtype=dtype, device=device)
    return t


class _CrossEntropyFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, target, ignore_index):
        k = _kernels_for(logits)
        logits = logits.contiguous()
        target = target.contiguous()
        rows, classes = logits.shape
        row_loss = _scratch_buffer("row_loss", (rows,), torch.float32, logits.device)
        # saved for backward: per call, a second loss may be evaluated before the first one's backward
        row_lse = torch.empty(rows, dtype=torch.float32, device=logits.device)
        loss = torch.empty(2, dtype=torch.float32, device=logits.device)   # {mean loss, 1 / counted rows}
        k.run("cross_entropy_fwd", logits, target, row_loss, row_lse, loss, rows, classes, ignore_index)
        ctx.save_for_backward(logits, target, row_lse, loss)
        ctx.ignore_index = ignore_index
        return loss[0]      # a view of this call's own result pair: no copy kernel

    @staticmethod
    def backward(ctx, grad_out):
        logits, target, row_lse, loss = ctx.saved_tensors
        k = _kernels_for(logits)
        rows, classes = logits.shape
        dlogits = _scratch_buffer("dlogits", logits.shape, logits.dtype, logits.device)
        g = grad_out.detach()
        if g.dtype != torch.float32 or not g.is_contiguous():
            g = g.to(torch.float32).contiguous()
        k.run("cross_entropy_bwd", logits, target, row_lse, g, loss, dlogits, rows, classes, ctx.ignore_index)
        return dlogits, None, None


class _SumFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        k = _kernels_for(x)
        xc = x.contiguous()
        partial = torch.empty(k.reduce_workspace(xc.numel()), dtype=torch.float32, device=x.device)
        out = torch.empty(1, dtype=torch.float32, device=x.device)
        k.run("sum_fwd", xc, partial, out, xc.numel())
        ctx.shape, ctx.dtype = x.shape, x.dtype
        return out[0].to(x.dtype)

    @staticmethod
    def backward(ctx, grad_out):
        return grad_out.to(ctx.dtype).expand(ctx.shape)


def cross_entropy(logits, target, ignore_index=-100):
    """Mean cross entropy over [rows, classes] logits and int64 targets (HIP kernels)."""
    return _CrossEntropyFn.apply(logits, target, ignore_index)


class LossWrapper(nn.Module):
    def forward(self, input, target, model=None):
        return _SumFn.apply(input)


class SumLoss(LossWrapper):
    def forward(self, input, target, model=None):
        if isinstance(input, (tuple, list)):
            input = input[0]
        return _SumFn.apply(input)


class MaskedLMOutputLoss(LossWrapper):
    def forward(self, input, target, model=None):
        if input.loss is not None:
            return input.loss
        return _SumFn.apply(input.logits)


class RescaleLoss(LossWrapper):
    def __init__(self, loss_fn, scale=1.0):
        super().__init__()
        self.loss_fn = loss_fn
        self.scale = scale

    def forward(self, input, target, model=None):
        return self.loss_fn(input, target, model) * self.scale


class NormalizeLoss(LossWrapper):
    """Rescales the loss by powers of two until 1/2 <= |loss| <= 1 (host-synchronising)."""

    def __init__(self, loss_fn):
        super().__init__()
        self.loss_fn = loss_fn

    def forward(self, input, target, model=None):
        loss = self.loss_fn(input, target, model)
        if loss.item() == 0:
            return loss
        while abs(loss.item()) < 1:
            loss = loss * 2
        while abs(loss.item()) > 1:
            loss = loss / 2
        return loss


class CrossEntropyLoss(LossWrapper):
    def __init__(self, num_labels=10):
        super().__init__()
        self.num_labels = num_labels

    def forward(self, input, target, model=None):
        return cross_entropy(input.view(-1, self.num_labels), target)


class HFCrossEntropyLoss(LossWrapper):
    def __init__(self, num_labels=10):
        super().__init__()
        self.num_labels = num_labels

    def forward(self, input, target, model=None):
        return cross_entropy(input.logits.view(-1, self.num_labels), target)
