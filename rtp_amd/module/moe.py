"""Rotated expert-sharded MoE layer (counterpart of WeightMOELayer, rtp/module/moe.py:101-187).

Tokens are routed by the top-2 gate, moved into per-expert capacity buffers by a row gather (the
reference's dense "sec,sm->ecm" einsum), pushed through the expert FFN of each shard as that shard
rotates through the staging buffer, and combined back with the gate weights (the "sec,ecm->sm" einsum
as a two-row weighted gather).  There is no all-to-all.
"""
from __future__ import annotations

from typing import Any, Optional, Union

import torch
import torch.nn as nn
from torch import Tensor
from torch.nn import Module, ModuleList

from .. import ops
from ..ring import Rotation, ring_order
from .collectives import RotatedLayer, resolve_world


class _DispatchFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, routing):
        out = torch.empty(routing.e * routing.capacity, x.shape[1], dtype=x.dtype, device=x.device)
        ops.moe_dispatch(x, routing, out)
        ctx.routing = routing
        return out

    @staticmethod
    def backward(ctx, d_out):
        r = ctx.routing
        d_out = d_out if d_out.stride(1) == 1 else d_out.contiguous()
        dx = torch.empty(r.s, d_out.shape[1], dtype=d_out.dtype, device=d_out.device)
        ops.moe_combine(d_out, r, dx, None)
        return dx, None


class _CombineFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, y, weight, routing):
        out = torch.empty(routing.s, y.shape[1], dtype=y.dtype, device=y.device)
        w = weight.detach().float().contiguous()
        ops.moe_combine(y, routing, out, w)
        ctx.routing = routing
        ctx.save_for_backward(y, w)
        return out

    @staticmethod
    def backward(ctx, d_out):
        r = ctx.routing
        y, w = ctx.saved_tensors
        d_out = d_out if d_out.stride(1) == 1 else d_out.contiguous()
        dy = torch.empty_like(y)
        ops.moe_dispatch(d_out, r, dy, w)
        dw = ops.moe_combine_dweight(d_out, y, r)
        return dy, dw, None


class _ExpertsFn(torch.autograd.Function):
    """y[e*C:(e+1)*C] = linear2(relu(linear1(x[e*C:(e+1)*C]))) with expert shards rotated."""

    @staticmethod
    def forward(ctx, x, anchor, layer):
        store = layer._store
        ws, n_local = layer.world_size, layer.num_local_experts
        rows_per_expert = x.shape[0] // (ws * n_local)
        y = torch.empty_like(x)
        hidden = []
        order = ring_order(layer.rank, ws)
        rot = Rotation(store.home, order)
        for i, idx in enumerate(order):
            views = store.views(rot.acquire(i))
            for j in range(n_local):
                w1, b1, w2, b2 = views[4 * j:4 * j + 4]
                r0 = (idx * n_local + j) * rows_per_expert
                chunk = x[r0:r0 + rows_per_expert]
                h = torch.empty(rows_per_expert, w1.shape[0], dtype=x.dtype, device=x.device)
                ops.linear_fwd(chunk, w1, h, bias=b1, relu=True)
                ops.linear_fwd(h, w2, y[r0:r0 + rows_per_expert], bias=b2)
                hidden.append((idx, j, h))
            rot.release(i)
        ctx.layer = layer
        ctx.hidden = {(idx, j): h for idx, j, h in hidden}
        ctx.save_for_backward(x)
        return y

    @staticmethod
    def backward(ctx, dy):
        layer = ctx.layer
        (x,) = ctx.saved_tensors
        store = layer._store
        ws, n_local = layer.world_size, layer.num_local_experts
        rows_per_expert = x.shape[0] // (ws * n_local)
        dy = dy if dy.stride(1) == 1 else dy.contiguous()
        dx = torch.empty_like(x)
        order = ring_order(layer.rank, ws, reverse=True)
        rot = Rotation(store.home, order)
        for i, idx in enumerate(order):
            views = store.views(rot.acquire(i))
            grads, accumulate = store.grad_views(idx)
            for j in range(n_local):
                w1, b1, w2, b2 = views[4 * j:4 * j + 4]
                g_w1, g_b1, g_w2, g_b2 = grads[4 * j:4 * j + 4]
                r0 = (idx * n_local + j) * rows_per_expert
                h = ctx.hidden.pop((idx, j))
                dy_e = dy[r0:r0 + rows_per_expert]
                dh = torch.empty_like(h)
                ops.linear_dgrad(dy_e, w2, dh, gate=h)
                ops.linear_dgrad(dh, w1, dx[r0:r0 + rows_per_expert])
                c = (lambda g: g if accumulate else None)
                ops.linear_wgrad(dy_e, h, g_w2, c_in=c(g_w2))
                ops.colsum(dy_e, g_b2, accumulate=accumulate)
                ops.linear_wgrad(dh, x[r0:r0 + rows_per_expert], g_w1, c_in=c(g_w1))
                ops.colsum(dh, g_b1, accumulate=accumulate)
            rot.release(i)
        return dx, None, None


def _check_expert(expert: Module) -> None:
    names = [n for n, _ in expert.named_parameters()]
    if names != ["linear1.weight", "linear1.bias", "linear2.weight", "linear2.bias"]:
        raise NotImplementedError(
            "WeightMOELayer runs experts of the form linear2(relu(linear1(x))) with biases "
            f"(parameters linear1.weight/bias, linear2.weight/bias); got {names}")
    act = getattr(expert, "activation", None)
    if act is not None and not isinstance(act, nn.ReLU):
        raise NotImplementedError("WeightMOELayer experts must use ReLU")
    for name in ("dropout1", "dropout2"):
        drop = getattr(expert, name, None)
        if isinstance(drop, nn.Dropout) and drop.p > 0:
            raise NotImplementedError("WeightMOELayer experts must use dropout 0")


class WeightMOELayer(RotatedLayer):
    """Signature follows rtp/module/moe.py:102-103.  `experts` is this rank's local expert (or
    ModuleList); since one process emulates every rank, the other ranks' experts are created as copies
    of it, and `original_experts` -- the reference's weight import for the local shard -- may also be
    a list with one entry per shard to give every shard its own weights."""

    def __init__(self, gate: Module, experts: Union[Module, ModuleList], group: Optional[Any] = None, device=None,
                 dtype=None, original_experts=None) -> None:
        super().__init__()
        import copy

        self.gate = gate
        local = experts if isinstance(experts, ModuleList) else ModuleList([experts])
        for expert in local:
            _check_expert(expert)
            for p in expert.parameters():
                p.expert = True  # type: ignore
        self.group = group
        self.world_size, self.rank = resolve_world(group)
        self.num_local_experts = len(local)
        shard_lists = []
        for s in range(self.world_size):
            shard = local if s == self.rank else ModuleList([copy.deepcopy(e) for e in local])
            if device is not None or dtype is not None:
                shard = shard.to(device=device, dtype=dtype)
            src = None
            if original_experts is not None:
                src = original_experts[s] if isinstance(original_experts, (list, tuple)) else (
                    original_experts if s == self.rank else None)
            if src is not None:
                with torch.no_grad():
                    for p, q in zip(shard.parameters(), src.parameters()):
                        p.data.copy_(q.data)
            shard_lists.append(shard)
        self._init_store(shard_lists)
        self.experts_list = list(self.shards)
        self.experts = self.experts_list[self.rank]
        self.l_aux = None

    def forward(self, *input: Tensor, noise: Optional[Tensor] = None, **kwargs: Any) -> Tensor:
        assert len(input) == 1, "only single input Tensor supported"
        assert len(input[0].shape) == 3, "input Tensor must have dimensions: (s)equence, (t)oken, (m)odel"
        assert input[0].shape[0] % len(self.experts) == 0, "num tokens must be order of number of local experts"
        x = input[0]
        d_model = x.shape[2]
        reshaped = x.reshape(-1, d_model)
        if reshaped.stride(1) != 1 or (reshaped.shape[0] > 1 and reshaped.stride(0) != d_model):
            reshaped = reshaped.contiguous()
        routing, weight, l_aux = self.gate.route(reshaped, noise)
        self.l_aux = l_aux.to(x.dtype)
        dispatched = _DispatchFn.apply(reshaped, routing)
        expert_out = _ExpertsFn.apply(dispatched, self._anchor, self)
        combined = _CombineFn.apply(expert_out, weight, routing)
        return combined.reshape(x.shape)
