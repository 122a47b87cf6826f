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
        ctx.ignore_index = ignore_index
        return loss

    @staticmethod
    def backward(ctx, dloss):
        logits, target, stats = ctx.saved_tensors
        dloss = dloss.float()
        if dloss.dim() == 1 and dloss.shape[0] > 1 and dloss.stride(0) not in (0, 1):
            dloss = dloss.contiguous()
        return ops.softmax_xent_bwd(logits, target, stats, dloss, ignore_index=ctx.ignore_index), None, None


class _ReducedLossFn(torch.autograd.Function):
    """reduction 'sum' or 'mean' (over the rows whose target is not the ignore index): an fp32 scalar."""

    @staticmethod
    def forward(ctx, logits, target, ignore_index, mean):
        rows, stats = ops.softmax_xent_fwd(logits, target, ignore_index)
        loss, scale = ops.softmax_xent_reduce(rows, target, ignore_index, mean)
        ctx.save_for_backward(logits, target, stats, scale)
        ctx.ignore_index = ignore_index
        return loss

    @staticmethod
    def backward(ctx, dloss):
        logits, target, stats, scale = ctx.saved_tensors
        return ops.softmax_xent_bwd(logits, target, stats, dloss.float().reshape(1), scale=scale,
                                    ignore_index=ctx.ignore_index), None, None, None


class _LinearCrossEntropyFn(torch.autograd.Function):
    """cross_entropy(layer(x), target) for a rotated column-parallel layer, the logits never stored: the forward
    product leaves softmax statistics, the backward runs the product once more and writes the logits' gradient,
    which then takes the layer's ordinary backward."""

    @staticmethod
    def forward(ctx, x, anchor, layer, target, ignore_index, mean):
        from ..ring import Rotation, ring_order
        from .utils import as_rows
        store = layer._store
        n_s, k = layer.output_size_per_partition, layer.in_features
        x2 = as_rows(x, k)
        rot = Rotation(store.home, ring_order(layer.rank, layer.world_size), group=store.stage_group)
        runs = rot.acquire(0)
        if rot.steps != 1 or len(runs) != 1:
            raise RuntimeError("linear_cross_entropy needs all shards of the layer in one run (rotation window = all)")
        b_off = n_s * k if layer.has_bias else None
        rows, stats = ops.rotated_linear_xent_fwd(x2, runs[0][0], 0, b_off, n_s, k, target, ignore_index)
        rot.release(0)
        loss, scale = ops.softmax_xent_reduce(rows, target, ignore_index, mean)
        ctx.layer, ctx.ignore_index, ctx.x_shape = layer, ignore_index, x.shape
        ctx.save_for_backward(x2, target, stats, scale)
        return loss

    @staticmethod
    def backward(ctx, dloss):
        from ..ring import Rotation, ring_order, run_wgrad
        from . import shard_ops as S
        layer = ctx.layer
        x2, target, stats, scale = ctx.saved_tensors
        store = layer._store
        n_s, k, ws = layer.output_size_per_partition, layer.in_features, layer.world_size
        b_off = n_s * k if layer.has_bias else None
        order = ring_order(layer.rank, ws, reverse=True)
        rot = Rotation(store.home, order, group=store.stage_group)
        flat = rot.acquire(0)[0][0]
        dlogits = ops.rotated_linear_xent_bwd(x2, flat, 0, b_off, n_s, k, target, ctx.ignore_index, stats,
                                              dloss.float().reshape(1), scale)
        dx = None
        if ctx.needs_input_grad[0]:
            dx = torch.empty_like(x2)
            S.col_dgrad(dlogits, flat, 0, n_s, k, dx, 0)
        rot.release(0)
        runs = store.grad_runs(order)

        def param_grads():
            for first, cnt, accumulate in runs:
                S.col_wgrad(dlogits, x2, store.grads, first, 0, n_s, k, first * n_s, cnt, accumulate, b_off=b_off,
                            store=store)
            store.grads_ready()

        run_wgrad(dlogits.device, param_grads, (dlogits, x2))
        return (dx.view(ctx.x_shape) if dx is not None else None), None, None, None, None, None


def linear_cross_entropy(x: torch.Tensor, layer, target: torch.Tensor, ignore_index: int = -100,
                         reduction: str = "mean") -> torch.Tensor:
    """cross_entropy(layer(x).view(-1, classes), target) for a ColumnParallelLinear `layer` (the LM's logits layer,
    rtp/models/transformer_lm_rtp.py:223, and the harness loss, benchmarks/rtp_benchmark.py:182) without the
    [rows, classes] logits ever reaching memory: their softmax statistics come out of the forward product's epilogue
    and their gradient out of a second run of that product in the backward pass.  Same values as the two separate
    calls (the logits are rounded to the layer's dtype before they enter the loss, as the stored ones would be).
    Needs a shard width that is a multiple of 64 columns and the rotation window that covers the whole layer."""
    if reduction not in ("mean", "sum"):
        raise ValueError("linear_cross_entropy: reduction must be 'mean' or 'sum'")
    if target.dim() != 1 or target.numel() * x.shape[-1] != x.numel():
        raise ValueError("linear_cross_entropy: target must hold one class index per row of x")
    target = (target if target.dtype == torch.int64 else target.long()).contiguous()
    return _LinearCrossEntropyFn.apply(x, layer._anchor, layer, target, int(ignore_index), reduction == "mean")


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
