"""GShard top-2 gate with a rotated, expert-sharded gate projection (counterpart of
rtp/module/top2gate.py:25-220).

The routing decisions come from the HIP routing kernels as compact per-token records; the dense
[S,E,C] combine/dispatch tensors of the reference API are materialised only when a caller asks the
gate module for them directly.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn as nn
from torch import Tensor

from .. import ops
from ..ring import Rotation, ring_order
from . import shard_ops as S
from .collectives import RotatedLayer, resolve_world
from .utils import affine_weight, as_rows, divide_and_check_no_remainder


def gumbel_rsample(shape, device: torch.device) -> Tensor:
    """Gumbel(0,1) noise for the second-expert choice (rtp/module/top2gate.py:25-32)."""
    one = torch.tensor(1.0, device=device)
    zero = torch.tensor(0.0, device=device)
    return torch.distributions.gumbel.Gumbel(zero, one).rsample(shape)


class _RouteFn(torch.autograd.Function):
    """logits[S,E] (+ noise) -> (weight[S,2], l_aux); the integer routing rides on `holder`.  l_aux comes out in
    `l_aux_dtype` (fp32, or bf16 written by the routing kernels themselves: no cast kernel)."""

    @staticmethod
    def forward(ctx, logits, noise, holder, l_aux_dtype):
        typed = l_aux_dtype if l_aux_dtype == torch.bfloat16 else None
        r = ops.top2_route(logits.float().contiguous(), noise.float().contiguous(), typed)
        holder.append(r)
        ctx.routing = r
        ctx.in_dtype = logits.dtype
        ctx.set_materialize_grads(False)  # an unused output (l_aux outside the loss) arrives as None, not as zeros
        l_aux = r.l_aux_typed if typed is not None else r.l_aux
        if l_aux.dtype != l_aux_dtype:
            l_aux = l_aux.to(l_aux_dtype)
        return r.weight, l_aux

    @staticmethod
    def backward(ctx, d_weight, d_l_aux):
        if d_weight is None and d_l_aux is None:
            return None, None, None, None
        d_logits = ops.top2_route_bwd(ctx.routing, d_weight, d_l_aux)
        return (d_logits if d_logits.dtype == ctx.in_dtype else d_logits.to(ctx.in_dtype)), None, None, None


def top2_route(logits: Tensor, noise: Optional[Tensor] = None, l_aux_dtype: Optional[torch.dtype] = None):
    """Differentiable compact routing: returns (routing, weight[S,2], l_aux); l_aux in l_aux_dtype (default fp32)."""
    if noise is None:
        noise = gumbel_rsample(logits.shape, logits.device)
    holder = []
    weight, l_aux = _RouteFn.apply(logits, noise, holder, l_aux_dtype or torch.float32)
    return holder[0], weight, l_aux


def dense_from_routing(r: ops.Routing, weight: Tensor, dtype: torch.dtype) -> Tuple[Tensor, Tensor]:
    """The reference's combine_weights[S,E,C] and dispatch_mask[S,E,C] (top2gate.py:95-103), built from
    the compact routing.  API compatibility only: the MoE layer never forms these."""
    s_idx = torch.arange(r.s, device=weight.device).repeat_interleave(2)
    e_idx = r.expert.reshape(-1).long()
    c_idx = r.slot.reshape(-1).long()
    vals = (weight * r.keep.to(weight.dtype)).reshape(-1)
    combine = torch.zeros(r.s, r.e, r.capacity, dtype=weight.dtype, device=weight.device)
    combine = combine.index_put((s_idx, e_idx, c_idx), vals, accumulate=True)
    return combine.to(dtype), combine.bool()


def top2gating(logits: Tensor, noise: Optional[Tensor] = None) -> Tuple[Tensor, Tensor, Tensor]:
    """(l_aux, combine_weights, dispatch_mask) as rtp/module/top2gate.py:43-105 returns them."""
    r, weight, l_aux = top2_route(logits, noise, logits.dtype)
    combine, dispatch = dense_from_routing(r, weight, logits.dtype)
    return l_aux, combine, dispatch


def _run_rows(flat: Tensor, e_s: int, m: int) -> Optional[Tensor]:
    """The expert rows of a run of staged gate shards as one [cnt * e_s, M] matrix: a gate shard's flat buffer is
    exactly its [e_s, M] weight, so consecutive shards are consecutive rows."""
    if flat.shape[1] != e_s * m or not flat.is_contiguous():
        return None
    return flat.view(flat.shape[0] * e_s, m)


class _GateProjectionFn(torch.autograd.Function):
    """logits[S,E] = x[S,M] @ wg^T with wg's expert rows sharded and rotated; fp32 logits.  Runs of at most 16
    experts take the streaming gate kernels (one pass over the tokens each way), others the tiled product."""

    @staticmethod
    def forward(ctx, x, anchor, layer, box=None):
        """`box` (a dict, optional): where another consumer of the same x leaves its input gradient under "dx" before
        this backward runs; the input-gradient kernel here then adds it in its epilogue and sets box["summed"], so that
        whoever joins the two paths hands this one on as their sum (see moe._ForkFn)."""
        store = layer._store
        ws, e_s = layer.world_size, layer.num_local_experts
        x2 = as_rows(x, layer.model_dim)
        ctx.box = box
        logits = torch.empty(x2.shape[0], layer.num_experts, dtype=torch.float32, device=x2.device)
        rot = Rotation(store.home, ring_order(layer.rank, ws), group=store.stage_group)
        for j in range(rot.steps):
            for flat, first, cnt in rot.acquire(j):
                rows = _run_rows(flat, e_s, layer.model_dim)
                if rows is not None and ops.gate_supported(x2, rows):
                    ops.gate_fwd(x2, rows, logits, first * e_s)
                else:
                    S.col_fwd(x2, flat, 0, e_s, layer.model_dim, None, logits, first * e_s)
            rot.release(j)
        ctx.layer = layer
        ctx.save_for_backward(x2)
        return logits

    @staticmethod
    def backward(ctx, d_logits):
        layer = ctx.layer
        (x2,) = ctx.saved_tensors
        store = layer._store
        ws, e_s = layer.world_size, layer.num_local_experts
        m = layer.model_dim
        dl32 = d_logits.float().contiguous()
        dl = None  # the tiled products take the gradient in the weights' dtype; made only if one of them runs

        def low():
            nonlocal dl
            if dl is None:
                dl = dl32.to(x2.dtype)
            return dl

        need_dx = ctx.needs_input_grad[0]
        order = ring_order(layer.rank, ws, reverse=True)
        dx = None
        if need_dx:
            dx = torch.empty_like(x2)
            rot = Rotation(store.home, order, group=store.stage_group)
            steps = sum(len(w) for w in rot.windows)
            acc = ops.ShardSum(dx, steps)
            i = 0
            for j in range(rot.steps):
                for flat, first, cnt in rot.acquire(j):
                    rows = _run_rows(flat, e_s, m)
                    if steps == 1 and rows is not None and ops.gate_supported(dx, rows):
                        other = ctx.box.pop("dx", None) if ctx.box is not None else None
                        if other is not None and (other.shape != dx.shape or other.dtype != dx.dtype or
                                                  other.stride(1) != 1):
                            ctx.box["dx"], other = other, None
                        ops.gate_dgrad(dl32, first * e_s, rows, dx, init=other)   # the only run: dx needs no summing
                        if other is not None:
                            ctx.box["summed"] = True
                    else:
                        c_out, c_in = acc.target(i)
                        S.col_dgrad(low(), flat, 0, e_s, m, c_out, first * e_s, c_in=c_in)
                    i += 1
                rot.release(j)
        for first, cnt, accumulate in store.grad_runs(order):
            rows = _run_rows(store.grads[first:first + cnt], e_s, m)
            if rows is not None and ops.gate_supported(x2, rows):
                ops.gate_wgrad(dl32, first * e_s, x2, rows, accumulate)
            else:
                S.col_wgrad(low(), x2, store.grads, first, 0, e_s, m, first * e_s, cnt, accumulate)
        store.grads_ready()
        return dx, None, None, None


class Top2Gate(RotatedLayer):
    """Unsharded gate (rtp/module/top2gate.py:109-137): forward(input[S,M]) = top2gating(wg(input)), and the master a
    WeightTop2Gate can be built from.  The projection is the rotated gate's with a single shard holding every expert
    row, so it runs on the same kernels."""

    def __init__(self, model_dim: int, num_experts: int) -> None:
        super().__init__()
        self.model_dim = model_dim
        self.num_experts = num_experts
        self.world_size, self.rank, self.num_local_experts = 1, 0, num_experts
        self._init_store([nn.Linear(model_dim, num_experts, bias=False)])
        # registered once, under the reference's name: state_dict() is exactly {"wg.weight"} (top2gate.py:124)
        wg = self.shards[0]
        del self._modules["shards"]
        self.shards = [wg]
        self.wg = wg

    def forward(self, input: Tensor, noise: Optional[Tensor] = None) -> Tuple[Tensor, Tensor, Tensor]:
        logits = _GateProjectionFn.apply(input, self._anchor, self)
        r, weight, l_aux = top2_route(logits, noise, input.dtype)
        combine, dispatch = dense_from_routing(r, weight, input.dtype)
        return l_aux, combine, dispatch


class WeightTop2Gate(RotatedLayer):
    """Signature follows rtp/module/top2gate.py:157-164.  forward(input[S,M]) returns the reference's
    (l_aux, combine_weights[S,E,C], dispatch_mask[S,E,C]); route() returns the compact form the MoE
    layer uses.  `noise` (fp32 [S,E]) may be passed to make the second choice reproducible."""

    def __init__(self, model_dim: int, num_experts: int, gate: Optional[nn.Module] = None, device=None,
                 dtype=None) -> None:
        super().__init__()
        self.model_dim = model_dim
        self.num_experts = num_experts
        self.world_size, self.rank = resolve_world(None)
        self.num_local_experts = divide_and_check_no_remainder(num_experts, self.world_size)
        if gate is not None and device is None:
            device = gate.wg.weight.device
        if gate is not None and dtype is None:
            dtype = gate.wg.weight.dtype
        wgs = []
        for s in range(self.world_size):
            wg = nn.Linear(model_dim, self.num_local_experts, bias=False, device=device, dtype=dtype)
            if gate is not None:
                affine_weight(wg.weight, gate.wg.weight, self.num_local_experts, 0, self.world_size, s)
            wgs.append(wg)
        self._init_store(wgs)
        self.wgs = list(self.shards)
        self.wg = self.wgs[self.rank]

    def logits(self, input: Tensor, box=None) -> Tensor:
        return _GateProjectionFn.apply(input, self._anchor, self, box)

    def route(self, input: Tensor, noise: Optional[Tensor] = None, box=None):
        """(routing, weight[S,2], l_aux in the input's dtype)."""
        return top2_route(self.logits(input, box), noise, input.dtype)

    def forward(self, input: Tensor, noise: Optional[Tensor] = None) -> Tuple[Tensor, Tensor, Tensor]:
        r, weight, l_aux = self.route(input, noise)
        combine, dispatch = dense_from_routing(r, weight, input.dtype)
        return l_aux, combine, dispatch
