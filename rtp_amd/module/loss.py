"""Cross-entropy over the vocabulary axis of the LM's logits in two kernels (the reference harness applies
nn.CrossEntropyLoss() to outputs.view(-1, vocab_size), test_transformer.py:195-197, which under autograd is a
cast, a log-softmax, a gather, a mean and their backward).  Statistics are fp32; the gradient is rounded to the
logits' dtype once, like the cast's backward."""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops


class _RowLossFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, target):
        loss, stats = ops.softmax_xent_fwd(logits, target)
        ctx.save_for_backward(logits, target, stats)
        return loss

    @staticmethod
    def backward(ctx, dloss):
        logits, target, stats = ctx.saved_tensors
        return ops.softmax_xent_bwd(logits, target, stats, dloss), None


def cross_entropy(logits: torch.Tensor, target: torch.Tensor, ignore_index: Optional[int] = None,
                  reduction: str = "mean") -> torch.Tensor:
    """F.cross_entropy(logits.float(), target) for logits [rows, classes] and class-index targets [rows].

    Rows whose target is `ignore_index` (or any index outside [0, classes)) have zero loss and zero gradient;
    "mean" divides by the number of rows, or by the number of rows not ignored when `ignore_index` is given.
    Inputs the kernels do not take (odd class counts, other dtypes, CPU tensors) go through torch."""
    if reduction not in ("mean", "sum", "none"):
        raise ValueError(f"cross_entropy: unknown reduction {reduction!r}")
    if logits.dim() != 2 or target.dim() != 1 or target.shape[0] != logits.shape[0]:
        raise ValueError("cross_entropy: logits must be [rows, classes] and target [rows]")
    if target.dtype != torch.int64 or not ops.softmax_xent_supported(logits):
        return F.cross_entropy(logits.float(), target, reduction=reduction,
                               ignore_index=-100 if ignore_index is None else ignore_index)
    rows = _RowLossFn.apply(logits, target.contiguous())
    if reduction == "none":
        return rows
    if reduction == "sum":
        return rows.sum()
    if ignore_index is None:
        return rows.mean()
    return rows.sum() / (target != ignore_index).sum()


class CrossEntropyLoss(nn.Module):
    """nn.CrossEntropyLoss() for [rows, classes] logits and class-index targets."""

    def __init__(self, ignore_index: Optional[int] = None, reduction: str = "mean"):
        super().__init__()
        self.ignore_index = ignore_index
        self.reduction = reduction

    def forward(self, logits: torch.Tensor, target: torch.Tensor) -> torch.Tensor:
        return cross_entropy(logits, target, self.ignore_index, self.reduction)
