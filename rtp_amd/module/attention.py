"""Rotated head-sharded multi-head attention (counterpart of rtp/module/attention.py:17-267 and the
multi_head_attention_forward it calls, rtp/module/functional.py:464-833 with E_div = ws).

Shard s owns heads [s*H/ws, (s+1)*H/ws): a packed in-projection [3E/ws, E] made of that head group's
Q, K and V rows, and the matching column block [E, E/ws] of the out-projection with bias/ws
(attention.py:78-104).  Per rotation step:  qkv = x W_in^T + b_in  ->  scores = q k^T (batched over
(batch, head) by strides into the packed projection, no re-layout)  ->  softmax(scale*scores + mask)
->  o = p v  ->  out += o W_o^T + b_o/ws.  The sum over shards restores the unsharded layer.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor
from torch.nn.modules.linear import NonDynamicallyQuantizableLinear
from torch.nn.parameter import Parameter

from .. import ops
from ..ring import Rotation, ring_order
from .collectives import RotatedLayer
from .utils import (affine_weight, affine_weight_attention, as_rows, attention_block_index,
                    divide_and_check_no_remainder)


class SubParallelMultiheadAttention(nn.Module):
    """Parameters of one head group (rtp/module/attention.py:17-104).  Declaration order fixes the
    flat-shard layout: in_proj_weight, in_proj_bias, out_proj.weight, out_proj.bias."""

    def __init__(self, embed_dim, num_heads, world_size, rank, dropout=0., bias=True, add_bias_kv=False,
                 add_zero_attn=False, kdim=None, vdim=None, batch_first=False, device=None, dtype=None) -> None:
        if embed_dim <= 0 or num_heads <= 0:
            raise ValueError(f"embed_dim and num_heads must be greater than 0, got embed_dim={embed_dim} and "
                             f"num_heads={num_heads} instead")
        super().__init__()
        kdim = embed_dim if kdim is None else kdim
        vdim = embed_dim if vdim is None else vdim
        if kdim != embed_dim or vdim != embed_dim or add_bias_kv or add_zero_attn:
            raise NotImplementedError("rotated attention: kdim/vdim != embed_dim, add_bias_kv and add_zero_attn "
                                      "are not implemented")
        self.embed_dim, self.kdim, self.vdim = embed_dim, kdim, vdim
        self._qkv_same_embed_dim = True
        self.num_heads = num_heads
        self.dropout = dropout
        self.batch_first = batch_first
        self.head_dim = embed_dim // num_heads
        assert self.head_dim * num_heads == embed_dim, "embed_dim must be divisible by num_heads"
        self.world_size, self.rank = world_size, rank
        self.num_heads_per_partition = divide_and_check_no_remainder(num_heads, world_size)
        self.embed_dim_per_partition = divide_and_check_no_remainder(embed_dim, world_size)
        e_s = self.embed_dim_per_partition
        kw = {"device": device, "dtype": dtype}
        self.in_proj_weight = Parameter(torch.empty((3 * e_s, embed_dim), **kw))
        self.bias = bias
        if bias:
            self.in_proj_bias = Parameter(torch.empty(3 * e_s, **kw))
        else:
            self.register_parameter("in_proj_bias", None)
        self.out_proj = NonDynamicallyQuantizableLinear(e_s, embed_dim, bias=bias, **kw)
        self.bias_k = self.bias_v = None
        self.add_zero_attn = add_zero_attn
        self._reset_parameters()

    def _reset_parameters(self) -> None:
        # The reference leaves in_proj_* as torch.empty (attention.py:57,64); give them the
        # nn.MultiheadAttention defaults instead of uninitialised memory.
        nn.init.xavier_uniform_(self.in_proj_weight)
        if self.in_proj_bias is not None:
            nn.init.constant_(self.in_proj_bias, 0.)
            nn.init.constant_(self.out_proj.bias, 0.)

    def affine_weight(self, mha) -> None:
        if mha is None:
            return
        idx = attention_block_index(self.rank, self.world_size)
        e_s = self.embed_dim_per_partition
        affine_weight_attention(self.in_proj_weight, mha.in_proj_weight, idx, e_s, 0, self.world_size, self.rank)
        if self.bias:
            affine_weight_attention(self.in_proj_bias, mha.in_proj_bias, idx, e_s, 0, self.world_size, self.rank)
        affine_weight(self.out_proj.weight, mha.out_proj.weight, e_s, 1, self.world_size, self.rank)
        if self.bias:
            with torch.no_grad():
                self.out_proj.bias.data.copy_(mha.out_proj.bias.data)
                self.out_proj.bias.data.div_(self.world_size)


def _bmm(dtype, *, a, a_off, lda, a_kc, a_s, b, b_off, ldb, b_kc, b_s, c, c_off, ldc, c_s, m, n, k, batch, zdiv,
         out_f32=False):
    esz = a.element_size()
    csz = 4 if out_f32 else esz
    ops.gemm_raw(dtype, a=a.data_ptr() + a_off * esz, b=b.data_ptr() + b_off * esz, c_out=c.data_ptr() + c_off * csz,
                 m=m, n=n, k=k, lda=lda, ldb=ldb, ldc=ldc, a_kcontig=a_kc, b_kcontig=b_kc, batch=batch, zdiv=zdiv,
                 a_s=a_s, b_s=b_s, c_s=c_s, out_f32=out_f32)


class _AttentionFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, anchor, layer, mask, causal, want_weights):
        store = layer._store
        L, N, E = x.shape
        ws, h_s, d, e_s = layer.world_size, layer.num_heads_per_partition, layer.head_dim, layer.embed_dim_per_partition
        dt = x.dtype
        x2 = as_rows(x, E)
        rows, Z = L * N, N * h_s
        scale = 1.0 / math.sqrt(d)
        out = torch.empty(rows, E, dtype=dt, device=x.device)
        acc = ops.ShardSum(out, ws)
        order = ring_order(layer.rank, ws)
        rot = Rotation(store.home, order)
        saved = {}
        weights = None
        for i, idx in enumerate(order):
            views = store.views(rot.acquire(i))
            w_in = views[0]
            b_in, w_o, b_o = (views[1], views[2], views[3]) if layer.has_bias else (None, views[1], None)
            qkv = torch.empty(rows, 3 * e_s, dtype=dt, device=x.device)
            ops.linear_fwd(x2, w_in, qkv, bias=b_in)
            scores = torch.empty(Z, L, L, dtype=torch.float32, device=x.device)
            ld = N * 3 * e_s
            _bmm(dt, a=qkv, a_off=0, lda=ld, a_kc=True, a_s=(3 * e_s, d), b=qkv, b_off=e_s, ldb=ld, b_kc=True,
                 b_s=(3 * e_s, d), c=scores, c_off=0, ldc=L, c_s=(h_s * L * L, L * L), m=L, n=L, k=d, batch=Z,
                 zdiv=h_s, out_f32=True)
            p = torch.empty(Z, L, L, dtype=dt, device=x.device)
            ops.softmax_fwd(scores, p, mask=mask, causal=causal, scale=scale)
            del scores
            o = torch.empty(rows, e_s, dtype=dt, device=x.device)
            _bmm(dt, a=p, a_off=0, lda=L, a_kc=True, a_s=(h_s * L * L, L * L), b=qkv, b_off=2 * e_s, ldb=ld,
                 b_kc=False, b_s=(3 * e_s, d), c=o, c_off=0, ldc=N * e_s, c_s=(e_s, d), m=L, n=d, k=L, batch=Z,
                 zdiv=h_s)
            c_out, c_in = acc.target(i)
            ops.linear_fwd(o, w_o, c_out, c_in=c_in, bias=b_o)
            rot.release(i)
            saved[idx] = (qkv, p, o)
            if want_weights and i == ws - 1:
                weights = p.view(N, h_s, L, L)
        ctx.layer = layer
        ctx.dims = (L, N, E)
        ctx.saved = saved
        ctx.save_for_backward(x2)
        ctx.mark_non_differentiable(*([weights] if weights is not None else []))
        y = out.view(L, N, E)
        return (y, weights) if weights is not None else (y, None)

    @staticmethod
    def backward(ctx, dout, _dweights=None):
        layer = ctx.layer
        (x2,) = ctx.saved_tensors
        store = layer._store
        L, N, E = ctx.dims
        ws, h_s, d, e_s = layer.world_size, layer.num_heads_per_partition, layer.head_dim, layer.embed_dim_per_partition
        dt = x2.dtype
        rows, Z = L * N, N * h_s
        scale = 1.0 / math.sqrt(d)
        dout2 = as_rows(dout, E)
        need_dx = ctx.needs_input_grad[0]
        dx = torch.empty_like(x2) if need_dx else None
        acc = ops.ShardSum(dx, ws) if need_dx else None
        order = ring_order(layer.rank, ws, reverse=True)
        rot = Rotation(store.home, order)
        ld = N * 3 * e_s
        for i, idx in enumerate(order):
            views = store.views(rot.acquire(i))
            w_in = views[0]
            w_o = views[2] if layer.has_bias else views[1]
            qkv, p, o = ctx.saved.pop(idx)
            grads, accumulate = store.grad_views(idx)
            if layer.has_bias:
                g_w_in, g_b_in, g_w_o, g_b_o = grads
            else:
                (g_w_in, g_w_o), g_b_in, g_b_o = grads, None, None
            # out-projection
            do = torch.empty(rows, e_s, dtype=dt, device=x2.device)
            ops.linear_dgrad(dout2, w_o, do)
            ops.linear_wgrad(dout2, o, g_w_o, c_in=g_w_o if accumulate else None)
            if g_b_o is not None:
                ops.colsum(dout2, g_b_o, accumulate=accumulate)
            # attention core
            dqkv = torch.empty(rows, 3 * e_s, dtype=dt, device=x2.device)
            dp = torch.empty(Z, L, L, dtype=torch.float32, device=x2.device)
            _bmm(dt, a=do, a_off=0, lda=N * e_s, a_kc=True, a_s=(e_s, d), b=qkv, b_off=2 * e_s, ldb=ld, b_kc=True,
                 b_s=(3 * e_s, d), c=dp, c_off=0, ldc=L, c_s=(h_s * L * L, L * L), m=L, n=L, k=d, batch=Z, zdiv=h_s,
                 out_f32=True)
            # dV = P^T dO
            _bmm(dt, a=p, a_off=0, lda=L, a_kc=False, a_s=(h_s * L * L, L * L), b=do, b_off=0, ldb=N * e_s,
                 b_kc=False, b_s=(e_s, d), c=dqkv, c_off=2 * e_s, ldc=ld, c_s=(3 * e_s, d), m=L, n=d, k=L, batch=Z,
                 zdiv=h_s)
            ds = torch.empty(Z, L, L, dtype=dt, device=x2.device)
            ops.softmax_bwd(p, dp, ds, scale)
            del dp
            # dQ = dS K
            _bmm(dt, a=ds, a_off=0, lda=L, a_kc=True, a_s=(h_s * L * L, L * L), b=qkv, b_off=e_s, ldb=ld, b_kc=False,
                 b_s=(3 * e_s, d), c=dqkv, c_off=0, ldc=ld, c_s=(3 * e_s, d), m=L, n=d, k=L, batch=Z, zdiv=h_s)
            # dK = dS^T Q
            _bmm(dt, a=ds, a_off=0, lda=L, a_kc=False, a_s=(h_s * L * L, L * L), b=qkv, b_off=0, ldb=ld, b_kc=False,
                 b_s=(3 * e_s, d), c=dqkv, c_off=e_s, ldc=ld, c_s=(3 * e_s, d), m=L, n=d, k=L, batch=Z, zdiv=h_s)
            # in-projection
            if need_dx:
                c_out, c_in = acc.target(i)
                ops.linear_dgrad(dqkv, w_in, c_out, c_in=c_in)
            rot.release(i)
            ops.linear_wgrad(dqkv, x2, g_w_in, c_in=g_w_in if accumulate else None)
            if g_b_in is not None:
                ops.colsum(dqkv, g_b_in, accumulate=accumulate)
        return (dx.view(L, N, E) if need_dx else None), None, None, None, None, None


class ParallelMultiheadAttention(RotatedLayer):
    """Signature follows rtp/module/attention.py:192-193; `MultiheadAttention_layer` imports the weights
    of an unsharded nn.MultiheadAttention.  Self-attention only (query, key and value must be the same
    tensor); key_padding_mask, 3-D masks and attention dropout are not implemented and raise."""

    def __init__(self, embed_dim, num_heads, world_size, rank, dropout=0., bias=True, add_bias_kv=False,
                 add_zero_attn=False, kdim=None, vdim=None, batch_first=False, device=None, dtype=None,
                 MultiheadAttention_layer: Optional[nn.MultiheadAttention] = None) -> None:
        super().__init__()
        self.world_size, self.rank = world_size, rank
        self.embed_dim, self.num_heads = embed_dim, num_heads
        self.dropout, self.batch_first, self.has_bias = dropout, batch_first, bias
        if MultiheadAttention_layer is not None and device is None:
            device = MultiheadAttention_layer.in_proj_weight.device
        if MultiheadAttention_layer is not None and dtype is None:
            dtype = MultiheadAttention_layer.in_proj_weight.dtype
        layers = []
        for s in range(world_size):
            sub = SubParallelMultiheadAttention(embed_dim, num_heads, world_size, s, dropout, bias, add_bias_kv,
                                                add_zero_attn, kdim, vdim, batch_first, device, dtype)
            sub.affine_weight(MultiheadAttention_layer)
            layers.append(sub)
        self.head_dim = layers[0].head_dim
        self.num_heads_per_partition = layers[0].num_heads_per_partition
        self.embed_dim_per_partition = layers[0].embed_dim_per_partition
        self._init_store(layers)
        self.layers = list(self.shards)
        self.MultiheadAttention = self.layers[self.rank]

    def forward(self, query: Tensor, key: Tensor, value: Tensor, key_padding_mask: Optional[Tensor] = None,
                need_weights: bool = True, attn_mask: Optional[Tensor] = None, average_attn_weights: bool = True,
                is_causal: bool = False, test_tensor=None) -> Tuple[Tensor, Optional[Tensor]]:
        if not (key is query and value is query):
            if not (key.data_ptr() == query.data_ptr() == value.data_ptr() and key.shape == query.shape == value.shape
                    and key.stride() == query.stride() == value.stride()):
                raise NotImplementedError("rotated attention implements self-attention only (query is key is value)")
        if key_padding_mask is not None:
            raise NotImplementedError("rotated attention: key_padding_mask is not implemented")
        if self.dropout > 0.0 and self.training:
            raise NotImplementedError("rotated attention: attention dropout is not implemented (use dropout=0)")
        if query.dim() != 3:
            raise NotImplementedError("rotated attention expects a batched [L, N, E] (or batch_first) input")
        x = query.transpose(0, 1) if self.batch_first else query
        L = x.shape[0]
        mask = None
        causal = False
        if attn_mask is not None:
            if attn_mask.dim() != 2 or tuple(attn_mask.shape) != (L, L):
                raise NotImplementedError("rotated attention: only a 2-D [L, L] attn_mask is implemented")
            mask = F._canonical_mask(mask=attn_mask, mask_name="attn_mask", other_type=None, other_name="",
                                     target_type=torch.float32)
            mask = mask.to(device=x.device, dtype=torch.float32).contiguous()
        elif is_causal:
            causal = True
        out, weights = _AttentionFn.apply(x, self._anchor, self, mask, causal, bool(need_weights))
        if need_weights and weights is not None and average_attn_weights:
            weights = weights.float().mean(dim=1).to(out.dtype)
        if self.batch_first:
            out = out.transpose(0, 1)
        return out, (weights if need_weights else None)
