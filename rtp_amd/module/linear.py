"""Rotated column- and row-parallel Linear (counterparts of rtp/module/linear.py:137-305 and :307-476).

Forward runs one rotation over the `ws` weight shards: at step i the shard (rank+i) % ws is in the
staging slot, its GEMM writes straight into its column block of the output (column-parallel; the
reference's torch.cat at linear.py:222 disappears) or accumulates into the output (row-parallel,
linear.py:389-392), while the next shard streams into the other slot.  Backward walks the shards in the
reverse order, needs each shard once more for the input gradient, and writes each shard's weight/bias
gradient straight into its home gradient row (the reference's gradient ring, collectives.py:196-200,
has nothing left to carry on one device).
"""
from __future__ import annotations

from typing import Callable, Optional

import torch
import torch.nn as nn
import torch.nn.init as init

from .. import ops
from ..ring import Rotation, ring_order, run_wgrad
from . import shard_ops as S
from .collectives import RotatedLayer, resolve_world
from .utils import affine_weight, as_rows, divide_and_check_no_remainder


class ModelParallelLinear(nn.Linear):
    """One column shard: rows [rank*N/ws, (rank+1)*N/ws) of the master weight and bias
    (rtp/module/linear.py:32-82)."""

    def __init__(self, in_features: int, out_features: int, world_size: int, rank: int, bias: bool = True,
                 device=None, dtype=None):
        self.world_size = world_size
        self.rank = rank
        self.output_size_per_partition = divide_and_check_no_remainder(out_features, world_size)
        super().__init__(in_features, self.output_size_per_partition, bias, device=device, dtype=dtype)

    def affine_weight(self, linear_layer) -> None:
        if linear_layer is not None:
            affine_weight(self.weight, linear_layer.weight, self.output_size_per_partition, 0, self.world_size,
                          self.rank)
            if self.bias is not None:
                affine_weight(self.bias, linear_layer.bias, self.output_size_per_partition, 0, self.world_size,
                              self.rank)


class ModelParallelLinear2(nn.Linear):
    """One row shard: columns [rank*K/ws, (rank+1)*K/ws) of the master weight; every shard carries
    bias/ws so that the sum over shards restores the bias (rtp/module/linear.py:84-135)."""

    def __init__(self, in_features: int, out_features: int, world_size: int, rank: int, bias: bool = True,
                 device=None, dtype=None):
        self.world_size = world_size
        self.rank = rank
        self.input_size_per_partition = divide_and_check_no_remainder(in_features, world_size)
        super().__init__(self.input_size_per_partition, out_features, bias, device=device, dtype=dtype)

    def affine_weight(self, linear_layer) -> None:
        if linear_layer is not None:
            affine_weight(self.weight, linear_layer.weight, self.input_size_per_partition, 1, self.world_size,
                          self.rank)
            if self.bias is not None:
                with torch.no_grad():
                    self.bias.data.copy_(linear_layer.bias.data)
                    self.bias.data.div_(self.world_size)


class _ColumnLinearFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, anchor, layer):
        store = layer._store
        n_s, k, ws = layer.output_size_per_partition, layer.in_features, layer.world_size
        x2 = as_rows(x, k)
        y = torch.empty(x2.shape[0], layer.out_features, dtype=x2.dtype, device=x2.device)
        b_off = n_s * k if layer.has_bias else None
        rot = Rotation(store.home, ring_order(layer.rank, ws), group=store.stage_group)
        for j in range(rot.steps):
            for flat, first, cnt in rot.acquire(j):
                S.col_fwd(x2, flat, 0, n_s, k, b_off, y, first * n_s)
            rot.release(j)
        ctx.layer = layer
        ctx.x_shape = x.shape
        ctx.save_for_backward(x2)
        return y.view(*x.shape[:-1], layer.out_features)

    @staticmethod
    def backward(ctx, dy):
        layer = ctx.layer
        (x2,) = ctx.saved_tensors
        store = layer._store
        n_s, k, ws = layer.output_size_per_partition, layer.in_features, layer.world_size
        dy2 = as_rows(dy, layer.out_features)
        need_dx = ctx.needs_input_grad[0]
        order = ring_order(layer.rank, ws, reverse=True)
        dx = None
        if need_dx:
            dx = torch.empty_like(x2)
            rot = Rotation(store.home, order, group=store.stage_group)
            acc = ops.ShardSum(dx, sum(len(w) for w in rot.windows))
            i = 0
            for j in range(rot.steps):
                for flat, first, cnt in rot.acquire(j):
                    c_out, c_in = acc.target(i)
                    S.col_dgrad(dy2, flat, 0, n_s, k, c_out, first * n_s, c_in=c_in)
                    i += 1
                rot.release(j)
        runs = store.grad_runs(order)

        def param_grads():
            for first, cnt, accumulate in runs:
                S.col_wgrad(dy2, x2, store.grads, first, 0, n_s, k, first * n_s, cnt, accumulate,
                            b_off=n_s * k if layer.has_bias else None, store=store)
            store.grads_ready()

        run_wgrad(dy2.device, param_grads, (dy2, x2))
        return (dx.view(ctx.x_shape) if need_dx else None), None, None


class _ColumnReluMlpFn(torch.autograd.Function):
    """linear2(relu(linear1(x))) over two column-parallel layers with the ReLU folded into the matrix products:
    forward in the epilogue of linear1's product, backward as a mask (h > 0) in the epilogue of linear2's
    input-gradient product.  Same values as the three separate modules."""

    @staticmethod
    def forward(ctx, x, anchor1, anchor2, lin1, lin2, residual_grad=False, keep=None):
        k1, f, n2 = lin1.in_features, lin1.out_features, lin2.out_features
        x2 = as_rows(x, k1)
        rows, dt, dev = x2.shape[0], x2.dtype, x2.device
        h = torch.empty(rows, f, dtype=dt, device=dev)
        y = torch.empty(rows, n2, dtype=dt, device=dev)
        for lin, src, dst, relu in ((lin1, x2, h, True), (lin2, h, y, False)):
            n_s, k = lin.output_size_per_partition, lin.in_features
            b_off = n_s * k if lin.has_bias else None
            rot = Rotation(lin._store.home, ring_order(lin.rank, lin.world_size), group=lin._store.stage_group)
            for j in range(rot.steps):
                for flat, first, cnt in rot.acquire(j):
                    S.col_fwd(src, flat, 0, n_s, k, b_off, dst, first * n_s, relu=relu)
                rot.release(j)
            if relu and keep is not None:
                h.mul_(keep)  # dropout on the hidden activations: 0 or 1 / (1 - p) per element
        ctx.layers = (lin1, lin2)
        ctx.x_shape = x.shape
        ctx.residual_grad = residual_grad
        ctx.keep = keep
        ctx.save_for_backward(x2, h)
        return y.view(*x.shape[:-1], n2)

    @staticmethod
    def backward(ctx, dy):
        lin1, lin2 = ctx.layers
        x2, h = ctx.saved_tensors
        dy2 = as_rows(dy, lin2.out_features)
        need_dx = ctx.needs_input_grad[0]
        dh = torch.empty_like(h)
        dx = torch.empty_like(x2) if need_dx else None
        # (layer, its output gradient, its input, its input gradient, mask applied to that input gradient)
        for lin, g, inp, dinp, gate in ((lin2, dy2, h, dh, h), (lin1, dh, x2, dx, None)):
            store = lin._store
            n_s, k = lin.output_size_per_partition, lin.in_features
            order = ring_order(lin.rank, lin.world_size, reverse=True)
            if dinp is not None:
                rot = Rotation(store.home, order, group=store.stage_group)
                steps = sum(len(w) for w in rot.windows)
                # residual_grad: y = norm(x + mlp(x)) sends x's whole gradient through here (dy + mlp'(dy))
                init = dy2 if (ctx.residual_grad and lin is lin1) else None
                acc = ops.ShardSum(dinp, steps, init=init)
                i = 0
                for j in range(rot.steps):
                    for flat, first, cnt in rot.acquire(j):
                        c_out, c_in = acc.target(i)
                        S.col_dgrad(g, flat, 0, n_s, k, c_out, first * n_s, c_in=c_in,
                                    gate=gate if i == steps - 1 else None)
                        i += 1
                    rot.release(j)
                if lin is lin2 and ctx.keep is not None:
                    dh.mul_(ctx.keep)  # h > 0 already implies a kept element; what is left is the 1 / (1 - p)
            runs = store.grad_runs(order)

            def param_grads(lin=lin, store=store, g=g, inp=inp, runs=runs, n_s=n_s, k=k):
                for first, cnt, accumulate in runs:
                    S.col_wgrad(g, inp, store.grads, first, 0, n_s, k, first * n_s, cnt, accumulate,
                                b_off=n_s * k if lin.has_bias else None, store=store)
                store.grads_ready()

            run_wgrad(g.device, param_grads, (g, inp))
        return (dx.view(ctx.x_shape) if need_dx else None), None, None, None, None, None, None


def column_relu_mlp(x: torch.Tensor, lin1: "ColumnParallelLinear", lin2: "ColumnParallelLinear",
                    residual_grad: bool = False, dropout_p: float = 0.0) -> torch.Tensor:
    """lin2(dropout(relu(lin1(x)))) with the ReLU fused into the products of the two rotated layers.  residual_grad:
    the backward returns dy + mlp'(dy), for a caller whose residual connection does not propagate x's gradient itself
    (add_layer_norm(..., x_grad_via_branch=True)).  dropout_p > 0: the hidden activations are multiplied by a keep
    mask drawn from torch's device generator (0 or 1 / (1 - p)), and so is their gradient."""
    if lin1.out_features != lin2.in_features:
        raise ValueError("column_relu_mlp: lin1.out_features must equal lin2.in_features")
    if residual_grad and lin2.out_features != lin1.in_features:
        raise ValueError("column_relu_mlp: residual_grad needs an output of the input's width")
    keep = None
    if dropout_p > 0.0:
        rows = x.numel() // x.shape[-1]
        keep = torch.empty(rows, lin1.out_features, dtype=x.dtype, device=x.device).bernoulli_(1.0 - dropout_p)
        keep.mul_(1.0 / (1.0 - dropout_p))
    return _ColumnReluMlpFn.apply(x, lin1._anchor, lin2._anchor, lin1, lin2, bool(residual_grad), keep)


class _RowLinearFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, anchor, layer):
        store = layer._store
        k_s, n, ws = layer.input_size_per_partition, layer.out_features, layer.world_size
        x2 = as_rows(x, layer.in_features)
        y = torch.empty(x2.shape[0], n, dtype=x2.dtype, device=x2.device)
        b_off = n * k_s if layer.has_bias else None
        rot = Rotation(store.home, ring_order(layer.rank, ws), group=store.stage_group)
        acc = ops.ShardSum(y, sum(len(w) for w in rot.windows))
        i = 0
        for j in range(rot.steps):
            for flat, first, cnt in rot.acquire(j):
                c_out, c_in = acc.target(i)
                S.row_fwd(x2, flat, 0, n, k_s, b_off, c_out, first * k_s, c_in=c_in)
                i += 1
            rot.release(j)
        ctx.layer = layer
        ctx.x_shape = x.shape
        ctx.save_for_backward(x2)
        return y.view(*x.shape[:-1], n)

    @staticmethod
    def backward(ctx, dy):
        layer = ctx.layer
        (x2,) = ctx.saved_tensors
        store = layer._store
        k_s, n, ws = layer.input_size_per_partition, layer.out_features, layer.world_size
        dy2 = as_rows(dy, n)
        need_dx = ctx.needs_input_grad[0]
        order = ring_order(layer.rank, ws, reverse=True)
        dx = None
        if need_dx:
            dx = torch.empty_like(x2)
            rot = Rotation(store.home, order, group=store.stage_group)
            for j in range(rot.steps):
                for flat, first, cnt in rot.acquire(j):
                    S.row_dgrad(dy2, flat, 0, n, k_s, dx, first * k_s)
                rot.release(j)
        runs = store.grad_runs(order)

        def param_grads():
            for first, cnt, accumulate in runs:
                S.row_wgrad(dy2, x2, store.grads, first, 0, n, k_s, first * k_s, cnt, accumulate,
                            b_off=n * k_s if layer.has_bias else None, store=store)
            store.grads_ready()

        run_wgrad(dy2.device, param_grads, (dy2, x2))
        return (dx.view(ctx.x_shape) if need_dx else None), None, None


class _ParallelLinearBase(RotatedLayer):
    _shard_cls = None
    _fn = None

    def __init__(self, in_features: int, out_features: int, bias: bool = True, gather_weight: bool = True,
                 init_method: Callable[[torch.Tensor], torch.Tensor] = init.xavier_normal_, stride: int = 1,
                 keep_master_weight_for_test: bool = False, device=None, dtype=None, group=None,
                 linear_layer: Optional[nn.Linear] = None) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.gather_weight = gather_weight
        self.group = group
        self.world_size, self.rank = resolve_world(group)
        self.has_bias = bias
        self.output_size_per_partition = divide_and_check_no_remainder(out_features, self.world_size) \
            if self._shard_cls is ModelParallelLinear else out_features
        self.input_size_per_partition = divide_and_check_no_remainder(in_features, self.world_size) \
            if self._shard_cls is ModelParallelLinear2 else in_features
        if linear_layer is not None and device is None:
            device = linear_layer.weight.device
        if linear_layer is not None and dtype is None:
            dtype = linear_layer.weight.dtype
        linears = []
        for s in range(self.world_size):
            shard = self._shard_cls(in_features, out_features, world_size=self.world_size, rank=s, bias=bias,
                                    device=device, dtype=dtype)
            shard.affine_weight(linear_layer)
            linears.append(shard)
        self._init_store(linears)
        self.linears = list(self.shards)
        self.linear = self.linears[self.rank]

    def forward(self, input_: torch.Tensor) -> torch.Tensor:
        return type(self)._fn.apply(input_, self._anchor, self)

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, bias={self.has_bias}, "
                f"shards={self.world_size}")


class ColumnParallelLinear(_ParallelLinearBase):
    """Y = X W^T + b with W split into `ws` row blocks (output columns); outputs of the shards are
    laid side by side.  Constructor arguments follow rtp/module/linear.py:158-171; `linear_layer`
    imports the weights of an unsharded nn.Linear."""
    _shard_cls = ModelParallelLinear
    _fn = _ColumnLinearFn


class RowParallelLinear(_ParallelLinearBase):
    """Y = sum_s X[:, s-block] W_s^T + ws * (b/ws) with W split into `ws` column blocks
    (rtp/module/linear.py:328-407)."""
    _shard_cls = ModelParallelLinear2
    _fn = _RowLinearFn
