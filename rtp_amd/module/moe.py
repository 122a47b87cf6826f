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


_JOIN_INPUT_GRADIENTS = True  # False: autograd adds the two input gradients itself (what the tests compare with)


class _ForkFn(torch.autograd.Function):
    """The layer's tokens feed two consumers, the gate projection and the dispatch (rtp/module/moe.py:146-148), and
    autograd would add their two input gradients with a kernel of its own.  Here both consumers read an alias made by
    this function and share `box`: the dispatch's backward (which autograd runs first: it was recorded later) leaves its
    gradient in the box, the gate projection's input-gradient kernel adds it in its epilogue, and this backward passes
    that sum on.  If the order or the shapes do not allow that, the two gradients are added here."""

    @staticmethod
    def forward(ctx, x, box):
        ctx.box = box
        return x.view_as(x), x.view_as(x)

    @staticmethod
    def backward(ctx, d_gate, d_dispatch):
        box = ctx.box
        box.pop("dx", None)
        if d_gate is None or d_dispatch is None:
            return (d_dispatch if d_gate is None else d_gate), None
        if box.pop("summed", False):
            return d_gate, None
        return d_gate + d_dispatch, None


class _DispatchFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, routing, box=None):
        out = torch.empty(routing.e * routing.capacity, x.shape[1], dtype=x.dtype, device=x.device)
        ops.moe_dispatch(x, routing, out)
        ctx.routing = routing
        ctx.box = box
        return out

    @staticmethod
    def backward(ctx, d_out):
        r = ctx.routing
        d_out = d_out if d_out.stride(1) == 1 else d_out.contiguous()
        dx = torch.empty(r.s, d_out.shape[1], dtype=d_out.dtype, device=d_out.device)
        ops.moe_combine(d_out, r, dx, None)
        if ctx.box is not None:
            ctx.box["dx"] = dx
        return dx, None, None


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
    """y[e*C:(e+1)*C] = linear2(relu(linear1(x[e*C:(e+1)*C]))) for every expert e, expert shards rotated.
    The experts of a staged run are one group each of a grouped GEMM: group g reads its own capacity slab."""

    @staticmethod
    def _geom(layer, x):
        store = layer._store
        n_local = layer.num_local_experts
        c_rows = x.shape[0] // (layer.world_size * n_local)
        m_dim = x.shape[1]
        f_dim = store.shapes[0][0]
        return store, n_local, c_rows, m_dim, f_dim

    @staticmethod
    def forward(ctx, x, anchor, layer):
        store, n_local, c_rows, m_dim, f_dim = _ExpertsFn._geom(layer, x)
        es = x.element_size()
        h = torch.empty(x.shape[0], f_dim, dtype=x.dtype, device=x.device)
        y = torch.empty_like(x)
        rot = Rotation(store.home, ring_order(layer.rank, layer.world_size), group=store.stage_group)
        for j in range(rot.steps):
            for flat, first, cnt in rot.acquire(j):
                for le in range(n_local):
                    w1, b1, w2, b2 = store.offsets[4 * le:4 * le + 4]
                    r0 = (first * n_local + le) * c_rows
                    common = dict(groups=cnt, b_sg=store.numel, bias_sg=store.numel, a_kcontig=True, b_kcontig=True)
                    ops.gemm_raw(x.dtype, a=x.data_ptr() + r0 * m_dim * es, b=flat.data_ptr() + w1 * es,
                                 bias=flat.data_ptr() + b1 * es, c_out=h.data_ptr() + r0 * f_dim * es, m=c_rows,
                                 n=f_dim, k=m_dim, lda=m_dim, ldb=m_dim, ldc=f_dim, relu=True,
                                 a_sg=n_local * c_rows * m_dim, c_sg=n_local * c_rows * f_dim, **common)
                    ops.gemm_raw(x.dtype, a=h.data_ptr() + r0 * f_dim * es, b=flat.data_ptr() + w2 * es,
                                 bias=flat.data_ptr() + b2 * es, c_out=y.data_ptr() + r0 * m_dim * es, m=c_rows,
                                 n=m_dim, k=f_dim, lda=f_dim, ldb=f_dim, ldc=m_dim,
                                 a_sg=n_local * c_rows * f_dim, c_sg=n_local * c_rows * m_dim, **common)
            rot.release(j)
        ctx.layer = layer
        ctx.save_for_backward(x, h)
        return y

    @staticmethod
    def backward(ctx, dy):
        layer = ctx.layer
        x, h = ctx.saved_tensors
        store, n_local, c_rows, m_dim, f_dim = _ExpertsFn._geom(layer, x)
        es = x.element_size()
        dy = dy.contiguous()
        dh = torch.empty_like(h)
        dx = torch.empty_like(x)
        order = ring_order(layer.rank, layer.world_size, reverse=True)
        rot = Rotation(store.home, order, group=store.stage_group)
        for j in range(rot.steps):
            for flat, first, cnt in rot.acquire(j):
                for le in range(n_local):
                    w1, _, w2, _ = store.offsets[4 * le:4 * le + 4]
                    r0 = (first * n_local + le) * c_rows
                    common = dict(groups=cnt, b_sg=store.numel, a_kcontig=True, b_kcontig=False)
                    # dH = (dY W2) masked by H > 0 ; dX = dH W1
                    ops.gemm_raw(x.dtype, a=dy.data_ptr() + r0 * m_dim * es, b=flat.data_ptr() + w2 * es,
                                 c_out=dh.data_ptr() + r0 * f_dim * es, gate=h.data_ptr() + r0 * f_dim * es,
                                 ld_gate=f_dim, gate_sg=n_local * c_rows * f_dim, m=c_rows, n=f_dim, k=m_dim, lda=m_dim,
                                 ldb=f_dim, ldc=f_dim, a_sg=n_local * c_rows * m_dim, c_sg=n_local * c_rows * f_dim,
                                 **common)
                    ops.gemm_raw(x.dtype, a=dh.data_ptr() + r0 * f_dim * es, b=flat.data_ptr() + w1 * es,
                                 c_out=dx.data_ptr() + r0 * m_dim * es, m=c_rows, n=m_dim, k=f_dim, lda=f_dim,
                                 ldb=m_dim, ldc=m_dim, a_sg=n_local * c_rows * f_dim, c_sg=n_local * c_rows * m_dim,
                                 **common)
            rot.release(j)
        runs = store.grad_runs(order)  # attaches (and on first use allocates) the gradient storage
        g = store.grads
        for first, cnt, accumulate in runs:
            for le in range(n_local):
                w1, b1, w2, b2 = store.offsets[4 * le:4 * le + 4]
                r0 = (first * n_local + le) * c_rows
                base = g.data_ptr() + first * store.numel * es
                # stream_out: an expert's gradient (tens of MB per launch) is not read again before the optimiser, and
                # written with ordinary stores it evicts the launch's own operands from the caches (468 -> 338 us)
                common = dict(groups=cnt, c_sg=store.numel, cin_sg=store.numel, a_kcontig=False, b_kcontig=False,
                              stream_out=True)
                # dW2 = dY^T H ; dW1 = dH^T X  (contraction over the expert's capacity rows); the bias gradients are
                # the row sums of the first operands and come out of the same launches where the library can fuse them
                c2 = base + w2 * es
                fused2 = ops.gemm_raw(
                    x.dtype, a=dy.data_ptr() + r0 * m_dim * es, b=h.data_ptr() + r0 * f_dim * es, c_out=c2,
                    c_in=c2 if accumulate else None, ld_cin=f_dim, m=m_dim, n=f_dim, k=c_rows, lda=m_dim, ldb=f_dim,
                    ldc=f_dim, a_sg=n_local * c_rows * m_dim, b_sg=n_local * c_rows * f_dim, rowsum=base + b2 * es,
                    rowsum_sg=store.numel, rowsum_accum=accumulate, **common)
                c1 = base + w1 * es
                fused1 = ops.gemm_raw(
                    x.dtype, a=dh.data_ptr() + r0 * f_dim * es, b=x.data_ptr() + r0 * m_dim * es, c_out=c1,
                    c_in=c1 if accumulate else None, ld_cin=m_dim, m=f_dim, n=m_dim, k=c_rows, lda=f_dim, ldb=m_dim,
                    ldc=m_dim, a_sg=n_local * c_rows * f_dim, b_sg=n_local * c_rows * m_dim, rowsum=base + b1 * es,
                    rowsum_sg=store.numel, rowsum_accum=accumulate, **common)
                for s in range(first, first + cnt):  # otherwise: column sums over each expert's own rows
                    r = (s * n_local + le) * c_rows
                    if not fused2:
                        ops.colsum(dy[r:r + c_rows], g[s, b2:b2 + m_dim], accumulate=accumulate)
                    if not fused1:
                        ops.colsum(dh[r:r + c_rows], g[s, b1:b1 + f_dim], accumulate=accumulate)
        store.grads_ready()
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
        box = None
        to_gate = to_dispatch = reshaped
        if _JOIN_INPUT_GRADIENTS and reshaped.requires_grad and torch.is_grad_enabled():
            box = {}
            to_gate, to_dispatch = _ForkFn.apply(reshaped, box)
        routing, weight, l_aux = self.gate.route(to_gate, noise, box)
        self.l_aux = l_aux
        dispatched = _DispatchFn.apply(to_dispatch, routing, box)
        expert_out = _ExpertsFn.apply(dispatched, self._anchor, self)
        combined = _CombineFn.apply(expert_out, weight, routing)
        return combined.reshape(x.shape)
