"""Cross-entropy over the vocabulary axis of the LM's logits (the reference harness applies
nn.CrossEntropyLoss() to outputs.view(-1, vocab_size), test_transformer.py:195-197, which under autograd is a
cast, a log-softmax, a gather, a mean and their backward) in three kernels: per-row loss and statistics, the
reduction over the rows, and the gradient.  Statistics are fp32; the gradient is rounded to the logits' dtype once,
like the cast's backward.  Everything runs in the HIP library: CPU tensors and other dtypes raise."""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import ops


class _RowLossFn(torch.autograd.Function):
    """reduction 'none': fp32 [rows]."""

    @staticmethod
    def forward(ctx, logits, target, ignore_index):
        loss, stats = ops.softmax_xent_fwd(logits, target, ignore_index)
        ctx.save_for_backward(logits, target, stats)
        return loss

    @staticmethod
    def backward(ctx, dloss):
        logits, target, stats = ctx.saved_tensors
        dloss = dloss.float()
        if dloss.dim() == 1 and dloss.shape[0] > 1 and dloss.stride(0) not in (0, 1):
            dloss = dloss.contiguous()
        return ops.softmax_xent_bwd(logits, target, stats, dloss), None, None


class _ReducedLossFn(torch.autograd.Function):
    """reduction 'sum' or 'mean' (over the rows whose target is not the ignore index): an fp32 scalar."""

    @staticmethod
    def forward(ctx, logits, target, ignore_index, mean):
        rows, stats = ops.softmax_xent_fwd(logits, target, ignore_index)
        loss, scale = ops.softmax_xent_reduce(rows, target, ignore_index, mean)
        ctx.save_for_backward(logits, target, stats, scale)
        return loss

    @staticmethod
    def backward(ctx, dloss):
        logits, target, stats, scale = ctx.saved_tensors
        return ops.softmax_xent_bwd(logits, target, stats, dloss.float().reshape(1), scale=scale), None, None, None


def cross_entropy(logits: torch.Tensor, target: torch.Tensor, ignore_index: int = -100,
                  reduction: str = "mean") -> torch.Tensor:
    """F.cross_entropy(logits.float(), target) for logits [rows, classes] and class-index targets [rows].

    Rows whose target is `ignore_index` have zero loss and zero gradient, and "mean" divides by the number of the
    other rows, as torch does.  A target outside [0, classes) that is not the ignore index is an error: torch
    asserts on the device; here that row's loss is NaN (so is any reduction that includes it), without a
    synchronisation."""
    if reduction not in ("mean", "sum", "none"):
        raise ValueError(f"cross_entropy: unknown reduction {reduction!r}")
    if logits.dim() != 2 or target.dim() != 1 or target.shape[0] != logits.shape[0]:
        raise ValueError("cross_entropy: logits must be [rows, classes] and target [rows]")
    ignore_index = -100 if ignore_index is None else int(ignore_index)
    if target.dtype != torch.int64:
        if target.is_floating_point():
            raise ValueError("cross_entropy: class-probability targets are not supported, pass class indices")
        target = target.long()
    target = target.contiguous()
    if reduction == "none":
        return _RowLossFn.apply(logits, target, ignore_index)
    return _ReducedLossFn.apply(logits, target, ignore_index, reduction == "mean")


class CrossEntropyLoss(nn.Module):
    """nn.CrossEntropyLoss() for [rows, classes] logits and class-index targets."""

    def __init__(self, ignore_index: int = -100, reduction: str = "mean"):
        super().__init__()
        self.ignore_index = ignore_index
        self.reduction = reduction

    def forward(self, logits: torch.Tensor, target: torch.Tensor) -> torch.Tensor:
        return cross_entropy(logits, target, self.ignore_index, self.reduction)
