"""Rotated out-channel-sharded 2-D convolution (counterpart of rtp/module/conv.py:17-198).

Shard s owns output channels [s*Co/ws, (s+1)*Co/ws): weight [Co/ws, Ci, kh, kw] and the bias slice (conv.py:43-47,
affine_weight along dim 0); the shards' outputs are concatenated on the channel dimension (conv.py:114).  A shard's
weight is, as stored in the flat buffer, the row-major [Co/ws, Ci*kh*kw] operand of a product over the patch matrix
of the input, and the library runs the three products of the layer as implicit GEMMs that gather the patches as they
go -- the patch matrix never exists in memory:

    y[:, shard's channels] = W_s . patches(x) + b_s       one launch per rotation window, NCHW written directly
    dW_s, db_s             = dy_s . patches(x)^T, sums    one launch per run of gradient rows
    dx                     = sum_s W_s^T . dy_s           one launch per rotation window (fp32 between windows)

groups = 1 and zero padding only.
"""
from __future__ import annotations

from typing import Optional, Union

import torch
import torch.nn as nn

from .. import ops
from ..ring import Rotation, ring_order, run_wgrad
from .collectives import RotatedLayer, resolve_world
from .utils import affine_weight, divide_and_check_no_remainder


class ModelParallelConv2d(nn.Conv2d):
    """One shard: an nn.Conv2d with out_channels / world_size output channels (rtp/module/conv.py:17-47)."""

    def __init__(self, in_channels: int, out_channels: int, kernel_size, stride=1, padding: Union[str, int] = 0,
                 dilation=1, groups: int = 1, bias: bool = True, padding_mode: str = "zeros", world_size: int = 1,
                 rank: int = 0, device=None, dtype=None) -> None:
        self.world_size, self.rank = world_size, rank
        self.output_size_per_partition = divide_and_check_no_remainder(out_channels, world_size)
        super().__init__(in_channels, self.output_size_per_partition, kernel_size, stride, padding, dilation, groups,
                         bias, padding_mode, device=device, dtype=dtype)

    def affine_weight(self, Conv2d_layer: Optional[nn.Conv2d]) -> None:
        if Conv2d_layer is None:
            return
        n = self.output_size_per_partition
        affine_weight(self.weight, Conv2d_layer.weight, n, 0, self.world_size, self.rank)
        if self.bias is not None:
            affine_weight(self.bias, Conv2d_layer.bias, n, 0, self.world_size, self.rank)


def _pair_padding(conv: nn.Conv2d):
    if isinstance(conv.padding, str):
        if conv.padding == "valid":
            return 0, 0
        total = [d * (k - 1) for d, k in zip(conv.dilation, conv.kernel_size)]
        if any(t % 2 for t in total):
            raise NotImplementedError("rotated conv: padding='same' with an odd total padding is not implemented")
        return total[0] // 2, total[1] // 2
    return tuple(conv.padding)


class _ColumnConvFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, anchor, layer):
        store = layer._store
        n_s, ws, co = layer.output_size_per_partition, layer.world_size, layer.out_channels
        geom = ops.conv_geom(x.shape, layer.kernel_size, layer.stride, layer.padding, layer.dilation)
        k = geom.c * geom.kh * geom.kw
        y = torch.empty(geom.n, co, geom.ho, geom.wo, dtype=x.dtype, device=x.device)
        b_off = n_s * k if layer.has_bias else None
        rot = Rotation(store.home, ring_order(layer.rank, ws), group=store.stage_group)
        for j in range(rot.steps):
            for flat, first, cnt in rot.acquire(j):
                ops.conv2d_fwd(x, geom, flat, 0, b_off, n_s, y, first * n_s)
            rot.release(j)
        ctx.layer, ctx.geom = layer, geom
        ctx.save_for_backward(x)
        return y

    @staticmethod
    def backward(ctx, dy):
        layer, geom = ctx.layer, ctx.geom
        (x,) = ctx.saved_tensors
        store = layer._store
        n_s, ws = layer.output_size_per_partition, layer.world_size
        k = geom.c * geom.kh * geom.kw
        order = ring_order(layer.rank, ws, reverse=True)
        dx = None
        if ctx.needs_input_grad[0]:
            dx = torch.empty(geom.n, geom.c, geom.h, geom.w, dtype=dy.dtype, device=dy.device)
            rot = Rotation(store.home, order, group=store.stage_group)
            acc = ops.ShardSum(dx, sum(len(w) for w in rot.windows))
            i = 0
            for j in range(rot.steps):
                for flat, first, cnt in rot.acquire(j):
                    c_out, c_in = acc.target(i)
                    ops.conv2d_dgrad(dy, geom, flat, 0, n_s, first * n_s, c_out, addend=c_in)
                    i += 1
                rot.release(j)
        runs = store.grad_runs(order)
        b_off = n_s * k if layer.has_bias else None

        def param_grads():
            for first, cnt, accumulate in runs:
                ops.conv2d_wgrad(dy, x, geom, store.grads[first:first + cnt], 0, b_off, n_s, first * n_s, accumulate)
            store.grads_ready()

        run_wgrad(dy.device, param_grads, (dy, x))
        return dx, None, None


class ColumnParallelConv2d(RotatedLayer):
    """Signature follows rtp/module/conv.py:50-67; `Conv2d_layer` imports the weights of an unsharded nn.Conv2d.
    groups != 1 and padding modes other than 'zeros' raise NotImplementedError."""

    def __init__(self, in_channels: int, out_channels: int, kernel_size, stride=1, padding: Union[str, int] = 0,
                 dilation=1, groups: int = 1, bias: bool = True, padding_mode: str = "zeros", device=None, dtype=None,
                 group=None, gather_output: bool = True, Conv2d_layer: Optional[nn.Conv2d] = None) -> None:
        super().__init__()
        if groups != 1 or padding_mode != "zeros":
            raise NotImplementedError("rotated conv: groups != 1 and non-zero padding modes are not implemented")
        self.in_channels, self.out_channels = in_channels, out_channels
        self.gather_output = gather_output
        self.group = group
        self.world_size, self.rank = resolve_world(group)
        self.has_bias = bias
        self.output_size_per_partition = divide_and_check_no_remainder(out_channels, self.world_size)
        if Conv2d_layer is not None and device is None:
            device = Conv2d_layer.weight.device
        if Conv2d_layer is not None and dtype is None:
            dtype = Conv2d_layer.weight.dtype
        layers = []
        for s in range(self.world_size):
            shard = ModelParallelConv2d(in_channels, out_channels, kernel_size, stride, padding, dilation, groups, bias,
                                        padding_mode, world_size=self.world_size, rank=s, device=device, dtype=dtype)
            shard.affine_weight(Conv2d_layer)
            layers.append(shard)
        proto = layers[0]
        self.kernel_size, self.stride, self.dilation = tuple(proto.kernel_size), tuple(proto.stride), tuple(proto.dilation)
        self.padding = _pair_padding(proto)
        self._init_store(layers)
        self.layers = list(self.shards)
        self.conv = self.layers[self.rank]

    def forward(self, input_: torch.Tensor) -> torch.Tensor:
        if input_.dim() != 4 or input_.shape[1] != self.in_channels:
            raise ValueError(f"ColumnParallelConv2d: expected an [N, {self.in_channels}, H, W] input, got "
                             f"{tuple(input_.shape)}")
        return _ColumnConvFn.apply(input_, self._anchor, self)

    def extra_repr(self) -> str:
        return (f"{self.in_channels}, {self.out_channels}, kernel_size={self.kernel_size}, stride={self.stride}, "
                f"padding={self.padding}, dilation={self.dilation}, bias={self.has_bias}, shards={self.world_size}")
