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


class _CrossEntropyFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, target, ignore_index):
        k = _kernels_for(logits)
        logits = logits.contiguous()
        target = target.contiguous()
        rows, classes = logits.shape
        row_loss = torch.empty(rows, dtype=torch.float32, device=logits.device)
        row_lse = torch.empty(rows, dtype=torch.float32, device=logits.device)
        loss = torch.empty(2, dtype=torch.float32, device=logits.device)
        k.run("cross_entropy_fwd", logits, target, row_loss, row_lse, loss, rows, classes, ignore_index)
        ctx.save_for_backward(logits, target, row_lse, loss)
        ctx.ignore_index = ignore_index
        return loss[0].clone()

    @staticmethod
    def backward(ctx, grad_out):
        logits, target, row_lse, loss = ctx.saved_tensors
        k = _kernels_for(logits)
        rows, classes = logits.shape
        dlogits = torch.empty_like(logits)
        g = grad_out.detach().to(torch.float32).contiguous()
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
