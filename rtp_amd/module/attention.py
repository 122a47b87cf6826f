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
from ..ring import Rotation, ring_order, run_wgrad
from . import shard_ops as S
from .collectives import RotatedLayer
from .utils import (affine_weight, affine_weight_attention, as_rows, attention_block_index,
                    divide_and_check_no_remainder)


class SubParallelMultiheadAttention(nn.Module):
    """Parameters of one head group (rtp/module/attention.py:17-104).  Declaration order fixes the
    flat-shard layout: in_proj_weight (or q_proj_weight, k_proj_weight, v_proj_weight when keys or values have
    their own width), in_proj_bias, bias_k, bias_v (add_bias_kv), out_proj.weight, out_proj.bias -- torch's own
    order: a module's parameters before its children's.

    add_bias_kv: the reference declares bias_k / bias_v at full width [1, 1, embed_dim] in every shard and
    concatenates them to keys of width embed_dim / ws (attention.py:70-72, functional.py:711-716), which only runs
    with one shard.  Here a shard holds its head group's slice [1, 1, embed_dim / ws] of them, so that the rotated
    layer equals nn.MultiheadAttention(add_bias_kv=True) for any shard count (and the reference for one)."""

    def __init__(self, embed_dim, num_heads, world_size, rank, dropout=0., bias=True, add_bias_kv=False,
                 add_zero_attn=False, kdim=None, vdim=None, batch_first=False, device=None, dtype=None) -> None:
        if embed_dim <= 0 or num_heads <= 0:
            raise ValueError(f"embed_dim and num_heads must be greater than 0, got embed_dim={embed_dim} and "
                             f"num_heads={num_heads} instead")
        super().__init__()
        kdim = embed_dim if kdim is None else kdim
        vdim = embed_dim if vdim is None else vdim
        self.embed_dim, self.kdim, self.vdim = embed_dim, kdim, vdim
        self._qkv_same_embed_dim = kdim == embed_dim and vdim == embed_dim
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
        if self._qkv_same_embed_dim:
            self.in_proj_weight = Parameter(torch.empty((3 * e_s, embed_dim), **kw))
        else:
            # attention.py:51-55: three separate row blocks when keys or values have their own width
            self.q_proj_weight = Parameter(torch.empty((e_s, embed_dim), **kw))
            self.k_proj_weight = Parameter(torch.empty((e_s, kdim), **kw))
            self.v_proj_weight = Parameter(torch.empty((e_s, vdim), **kw))
            self.register_parameter("in_proj_weight", None)
        self.bias = bias
        if bias:
            self.in_proj_bias = Parameter(torch.empty(3 * e_s, **kw))
        else:
            self.register_parameter("in_proj_bias", None)
        self.out_proj = NonDynamicallyQuantizableLinear(e_s, embed_dim, bias=bias, **kw)
        if add_bias_kv:
            self.bias_k = Parameter(torch.empty((1, 1, e_s), **kw))
            self.bias_v = Parameter(torch.empty((1, 1, e_s), **kw))
        else:
            self.bias_k = self.bias_v = None
        self.add_zero_attn = add_zero_attn
        self._reset_parameters()

    def _reset_parameters(self) -> None:
        # The reference leaves in_proj_* as torch.empty (attention.py:57,64); give them the
        # nn.MultiheadAttention defaults instead of uninitialised memory.
        if self._qkv_same_embed_dim:
            nn.init.xavier_uniform_(self.in_proj_weight)
        else:
            for w in (self.q_proj_weight, self.k_proj_weight, self.v_proj_weight):
                nn.init.xavier_uniform_(w)
        if self.in_proj_bias is not None:
            nn.init.constant_(self.in_proj_bias, 0.)
            nn.init.constant_(self.out_proj.bias, 0.)
        if self.bias_k is not None:
            nn.init.xavier_normal_(self.bias_k)
            nn.init.xavier_normal_(self.bias_v)

    def affine_weight(self, mha) -> None:
        if mha is None:
            return
        idx = attention_block_index(self.rank, self.world_size)
        e_s = self.embed_dim_per_partition
        if self._qkv_same_embed_dim:
            affine_weight_attention(self.in_proj_weight, mha.in_proj_weight, idx, e_s, 0, self.world_size, self.rank)
        else:
            for mine, theirs in ((self.q_proj_weight, mha.q_proj_weight), (self.k_proj_weight, mha.k_proj_weight),
                                 (self.v_proj_weight, mha.v_proj_weight)):
                affine_weight(mine, theirs, e_s, 0, self.world_size, self.rank)
        if self.bias:
            affine_weight_attention(self.in_proj_bias, mha.in_proj_bias, idx, e_s, 0, self.world_size, self.rank)
        affine_weight(self.out_proj.weight, mha.out_proj.weight, e_s, 1, self.world_size, self.rank)
        if self.bias_k is not None:
            if mha.bias_k is None:
                raise ValueError("add_bias_kv: the layer to import has no bias_k / bias_v")
            with torch.no_grad():  # the head group's columns of the appended key / value
                self.bias_k.copy_(mha.bias_k[..., self.rank * e_s:(self.rank + 1) * e_s])
                self.bias_v.copy_(mha.bias_v[..., self.rank * e_s:(self.rank + 1) * e_s])
        if self.bias:
            with torch.no_grad():
                self.out_proj.bias.data.copy_(mha.out_proj.bias.data)
                self.out_proj.bias.data.div_(self.world_size)


def _bmm(dtype, *, a, a_off, lda, a_kc, a_s, a_sg, b, b_off, ldb, b_kc, b_s, b_sg, c, c_off, ldc, c_s, c_sg, m, n, k,
         batch, zdiv, groups, out_f32=False):
    esz = a.element_size()
    csz = 4 if out_f32 else esz
    ops.gemm_raw(dtype, a=a.data_ptr() + a_off * esz, b=b.data_ptr() + b_off * esz, c_out=c.data_ptr() + c_off * csz,
                 m=m, n=n, k=k, lda=lda, ldb=ldb, ldc=ldc, a_kcontig=a_kc, b_kcontig=b_kc, batch=batch, zdiv=zdiv,
                 a_s=a_s, b_s=b_s, c_s=c_s, out_f32=out_f32, groups=groups, a_sg=a_sg, b_sg=b_sg, c_sg=c_sg)


class _AttentionFn(torch.autograd.Function):
    """Buffers hold all head groups side by side: qkv [L*N, ws*3E_s] (group g at column block g, inside it
    Q | K | V of that group), p [ws*N*h_s, L, L], o [L*N, E] (= the unsharded head order).  A (group,
    batch, head) triple is addressed by strides inside the batched GEMM, so nothing is re-laid out.

    The core runs in one of three forms: bf16 with L <= 32 in one launch that keeps the scores in registers and
    stores p; bf16 with longer sequences in a running-softmax launch that stores only the log-sum-exp per
    query (not when the caller wants the attention weights back); otherwise as batched products and a softmax
    kernel with p in memory."""

    @staticmethod
    def forward(ctx, x, anchor, layer, mask, causal, want_weights, residual_grad=False, key_bias=None, drop_p=0.0):
        store = layer._store
        L, N, E = x.shape
        ws, h_s, d, e_s = layer.world_size, layer.num_heads_per_partition, layer.head_dim, layer.embed_dim_per_partition
        dt, dev = x.dtype, x.device
        x2 = as_rows(x, E)
        rows, Z = L * N, N * h_s
        scale = 1.0 / math.sqrt(d)
        off = store.offsets
        b_in_off, w_o_off, b_o_off = (off[1], off[2], off[3]) if layer.has_bias else (None, off[1], None)
        qkv = torch.empty(rows, ws * 3 * e_s, dtype=dt, device=dev)
        o = torch.empty(rows, E, dtype=dt, device=dev)
        out = torch.empty(rows, E, dtype=dt, device=dev)
        ldq = N * ws * 3 * e_s
        # attention dropout and per-head masks work on the probabilities in memory: the product + softmax form
        plain = drop_p == 0.0 and (mask is None or mask.dim() == 2)
        fused = plain and ops.attn_supported(dt, L, d)
        flash = plain and not fused and not want_weights and ops.attn_flash_supported(dt, L, d)
        if flash:
            p = torch.empty(ws * Z, L, dtype=torch.float32, device=dev)  # log-sum-exp in place of probabilities
        else:
            p = torch.empty(ws * Z, L, L, dtype=dt, device=dev)
        # drop: per-probability multiplier 0 or 1 / (1 - drop_p); pv: the probabilities that meet V
        drop = torch.empty(ws * Z, L, L, dtype=torch.float32, device=dev) if drop_p > 0.0 else None
        pv = torch.empty_like(p) if drop_p > 0.0 else p
        order = ring_order(layer.rank, ws)
        rot = Rotation(store.home, order, group=store.stage_group)
        acc = ops.ShardSum(out, sum(len(w) for w in rot.windows))
        i = 0
        for j in range(rot.steps):
            for flat, first, cnt in rot.acquire(j):
                S.col_fwd(x2, flat, 0, 3 * e_s, E, b_in_off, qkv, first * 3 * e_s)
                q0 = first * 3 * e_s
                if fused:
                    # scores, softmax and p v in one launch, one wavefront per (group, batch, head)
                    ops.attn_fwd(qkv, q0, q0 + e_s, q0 + 2 * e_s, (ldq, ws * 3 * e_s, d, 3 * e_s), o, first * e_s,
                                 (N * E, E, d, e_s), p[first * Z:(first + cnt) * Z], mask, causal, scale, L, N, h_s,
                                 d, cnt, key_bias=key_bias)
                    c_out, c_in = acc.target(i)
                    S.row_fwd(o, flat, w_o_off, E, e_s, b_o_off, c_out, first * e_s, c_in=c_in)
                    i += 1
                    continue
                if flash:
                    ops.attn_flash_fwd(qkv, q0, q0 + e_s, q0 + 2 * e_s, (ldq, ws * 3 * e_s, d, 3 * e_s), o,
                                       first * e_s, (N * E, E, d, e_s), p[first * Z:(first + cnt) * Z], mask, causal,
                                       scale, L, N, h_s, d, cnt, key_bias=key_bias)
                    c_out, c_in = acc.target(i)
                    S.row_fwd(o, flat, w_o_off, E, e_s, b_o_off, c_out, first * e_s, c_in=c_in)
                    i += 1
                    continue
                scores = torch.empty(cnt * Z, L, L, dtype=torch.float32, device=dev)
                _bmm(dt, a=qkv, a_off=q0, lda=ldq, a_kc=True, a_s=(ws * 3 * e_s, d), a_sg=3 * e_s, b=qkv,
                     b_off=q0 + e_s, ldb=ldq, b_kc=True, b_s=(ws * 3 * e_s, d), b_sg=3 * e_s, c=scores, c_off=0, ldc=L,
                     c_s=(h_s * L * L, L * L), c_sg=Z * L * L, m=L, n=L, k=d, batch=Z, zdiv=h_s, groups=cnt,
                     out_f32=True)
                p_run = p[first * Z:(first + cnt) * Z]
                if drop is not None:
                    ops.softmax_fwd(scores, p_run, mask=mask, causal=causal, scale=scale, key_bias=key_bias, heads=h_s,
                                    keep=_draw_keep(layer, drop_p, drop[first * Z:(first + cnt) * Z]),
                                    p_dropped=pv[first * Z:(first + cnt) * Z])
                else:
                    ops.softmax_fwd(scores, p_run, mask=mask, causal=causal, scale=scale, key_bias=key_bias, heads=h_s)
                del scores
                _bmm(dt, a=pv, a_off=first * Z * L * L, lda=L, a_kc=True, a_s=(h_s * L * L, L * L), a_sg=Z * L * L,
                     b=qkv, b_off=q0 + 2 * e_s, ldb=ldq, b_kc=False, b_s=(ws * 3 * e_s, d), b_sg=3 * e_s, c=o,
                     c_off=first * e_s, ldc=N * E, c_s=(E, d), c_sg=e_s, m=L, n=d, k=L, batch=Z, zdiv=h_s, groups=cnt)
                c_out, c_in = acc.target(i)
                S.row_fwd(o, flat, w_o_off, E, e_s, b_o_off, c_out, first * e_s, c_in=c_in)
                i += 1
            rot.release(j)
        weights = None
        if want_weights:
            last = order[-1]
            weights = pv[last * Z:(last + 1) * Z].view(N, h_s, L, L)  # functional.py:789-792: after dropout
        ctx.layer = layer
        ctx.dims = (L, N, E)
        ctx.residual_grad = residual_grad
        ctx.flash = (mask, causal, key_bias) if flash else None
        ctx.fused = fused
        ctx.dropped = drop is not None
        ctx.save_for_backward(x2, qkv, p, o, *((drop, pv) if drop is not None else ()))
        ctx.mark_non_differentiable(*([weights] if weights is not None else []))
        return out.view(L, N, E), weights

    @staticmethod
    def backward(ctx, dout, _dweights=None):
        layer = ctx.layer
        x2, qkv, p, o = ctx.saved_tensors[:4]
        drop, pv = ctx.saved_tensors[4:] if ctx.dropped else (None, p)
        store = layer._store
        L, N, E = ctx.dims
        ws, h_s, d, e_s = layer.world_size, layer.num_heads_per_partition, layer.head_dim, layer.embed_dim_per_partition
        dt, dev = x2.dtype, x2.device
        rows, Z = L * N, N * h_s
        scale = 1.0 / math.sqrt(d)
        off = store.offsets
        b_in_off, w_o_off, b_o_off = (off[1], off[2], off[3]) if layer.has_bias else (None, off[1], None)
        dout2 = as_rows(dout, E)
        need_dx = ctx.needs_input_grad[0]
        dx = torch.empty_like(x2) if need_dx else None
        do = torch.empty(rows, E, dtype=dt, device=dev)
        dqkv = torch.empty(rows, ws * 3 * e_s, dtype=dt, device=dev)
        ldq = N * ws * 3 * e_s
        fused = ctx.fused
        delta = torch.empty_like(p) if ctx.flash is not None else None
        order = ring_order(layer.rank, ws, reverse=True)
        rot = Rotation(store.home, order, group=store.stage_group)
        # residual_grad: the caller's y = norm(x + attention(x)) sends x's whole gradient through this function,
        # which adds the output gradient to its own input gradient in the epilogue of the last product
        init = dout2 if ctx.residual_grad else None
        acc = ops.ShardSum(dx, sum(len(w) for w in rot.windows), init=init) if need_dx else None
        i = 0
        for j in range(rot.steps):
            for flat, first, cnt in rot.acquire(j):
                q0 = first * 3 * e_s
                # out-projection: dO_g = dOut W_o,g
                S.row_dgrad(dout2, flat, w_o_off, E, e_s, do, first * e_s)
                if fused:
                    ops.attn_bwd(qkv, q0, q0 + e_s, q0 + 2 * e_s, (ldq, ws * 3 * e_s, d, 3 * e_s), do, first * e_s,
                                 (N * E, E, d, e_s), p[first * Z:(first + cnt) * Z], dqkv, scale, L, N, h_s, d, cnt)
                    if need_dx:
                        c_out, c_in = acc.target(i)
                        S.col_dgrad(dqkv, flat, 0, 3 * e_s, E, c_out, q0, c_in=c_in)
                    i += 1
                    continue
                if ctx.flash is not None:
                    mask, causal, key_bias = ctx.flash
                    ops.attn_flash_bwd(qkv, q0, q0 + e_s, q0 + 2 * e_s, (ldq, ws * 3 * e_s, d, 3 * e_s), o, do,
                                       first * e_s, (N * E, E, d, e_s), p[first * Z:(first + cnt) * Z],
                                       delta[first * Z:(first + cnt) * Z], dqkv, mask, causal, scale, L, N, h_s, d,
                                       cnt, key_bias=key_bias)
                    if need_dx:
                        c_out, c_in = acc.target(i)
                        S.col_dgrad(dqkv, flat, 0, 3 * e_s, E, c_out, q0, c_in=c_in)
                    i += 1
                    continue
                # attention core, all (group, batch, head) triples of the run in one launch each
                dp = torch.empty(cnt * Z, L, L, dtype=torch.float32, device=dev)
                _bmm(dt, a=do, a_off=first * e_s, lda=N * E, a_kc=True, a_s=(E, d), a_sg=e_s, b=qkv, b_off=q0 + 2 * e_s,
                     ldb=ldq, b_kc=True, b_s=(ws * 3 * e_s, d), b_sg=3 * e_s, c=dp, c_off=0, ldc=L,
                     c_s=(h_s * L * L, L * L), c_sg=Z * L * L, m=L, n=L, k=d, batch=Z, zdiv=h_s, groups=cnt, out_f32=True)
                p_off = first * Z * L * L
                # dV = P^T dO
                _bmm(dt, a=pv, a_off=p_off, lda=L, a_kc=False, a_s=(h_s * L * L, L * L), a_sg=Z * L * L, b=do,
                     b_off=first * e_s, ldb=N * E, b_kc=False, b_s=(E, d), b_sg=e_s, c=dqkv, c_off=q0 + 2 * e_s, ldc=ldq,
                     c_s=(ws * 3 * e_s, d), c_sg=3 * e_s, m=L, n=d, k=L, batch=Z, zdiv=h_s, groups=cnt)
                ds = torch.empty(cnt * Z, L, L, dtype=dt, device=dev)
                ops.softmax_bwd(p[first * Z:(first + cnt) * Z], dp, ds, scale,
                                keep=None if drop is None else drop[first * Z:(first + cnt) * Z])
                del dp
                # dQ = dS K
                _bmm(dt, a=ds, a_off=0, lda=L, a_kc=True, a_s=(h_s * L * L, L * L), a_sg=Z * L * L, b=qkv,
                     b_off=q0 + e_s, ldb=ldq, b_kc=False, b_s=(ws * 3 * e_s, d), b_sg=3 * e_s, c=dqkv, c_off=q0, ldc=ldq,
                     c_s=(ws * 3 * e_s, d), c_sg=3 * e_s, m=L, n=d, k=L, batch=Z, zdiv=h_s, groups=cnt)
                # dK = dS^T Q
                _bmm(dt, a=ds, a_off=0, lda=L, a_kc=False, a_s=(h_s * L * L, L * L), a_sg=Z * L * L, b=qkv, b_off=q0,
                     ldb=ldq, b_kc=False, b_s=(ws * 3 * e_s, d), b_sg=3 * e_s, c=dqkv, c_off=q0 + e_s, ldc=ldq,
                     c_s=(ws * 3 * e_s, d), c_sg=3 * e_s, m=L, n=d, k=L, batch=Z, zdiv=h_s, groups=cnt)
                # in-projection input gradient: dX += sum_g dQKV_g W_in,g
                if need_dx:
                    c_out, c_in = acc.target(i)
                    S.col_dgrad(dqkv, flat, 0, 3 * e_s, E, c_out, q0, c_in=c_in)
                i += 1
            rot.release(j)
        runs = store.grad_runs(order)

        def param_grads():
            for first, cnt, accumulate in runs:
                S.row_wgrad(dout2, o, store.grads, first, w_o_off, E, e_s, first * e_s, cnt, accumulate,
                            b_off=b_o_off if layer.has_bias else None, store=store)
                S.col_wgrad(dqkv, x2, store.grads, first, 0, 3 * e_s, E, first * 3 * e_s, cnt, accumulate,
                            b_off=b_in_off if layer.has_bias else None, store=store)
            store.grads_ready()

        run_wgrad(dev, param_grads, (dout2, o, dqkv, x2))
        return (dx.view(L, N, E) if need_dx else None), None, None, None, None, None, None, None, None


def _draw_keep(layer, drop_p: float, drop: Tensor) -> Tensor:
    """Attention dropout (functional.py:789-792 / the dropout_p of :825): every probability is kept with chance
    1 - drop_p and scaled by 1 / (1 - drop_p).  Fills `drop` with the fp32 multipliers (0 or 1 / (1 - drop_p)) that the
    softmax kernels apply, forward and backward.  The draw itself is torch's device generator (like the model's
    other dropouts); `layer.dropout_keep_fn`, if set, supplies the 0 / 1 keep mask instead."""
    keep = 1.0 - drop_p
    fn = getattr(layer, "dropout_keep_fn", None)
    if fn is not None:
        drop.copy_(fn(tuple(drop.shape)))
    else:
        drop.bernoulli_(keep)
    return drop.div_(keep)


def _shard_layout(layer):
    """Element offsets inside a flat shard of (W_q, W_k, W_v, b_in, W_o, b_o); b_in / b_o are None without biases."""
    off = layer._store.offsets
    e_s, E = layer.embed_dim_per_partition, layer.embed_dim
    if layer.separate_proj:
        wq, wk, wv, nxt = off[0], off[1], off[2], 3
    else:
        wq, wk, wv, nxt = off[0], off[0] + e_s * E, off[0] + 2 * e_s * E, 1
    kv = 2 if layer.add_bias_kv else 0  # bias_k, bias_v sit between the input projection and the output projection
    if layer.has_bias:
        return wq, wk, wv, off[nxt], off[nxt + 1 + kv], off[nxt + 2 + kv]
    return wq, wk, wv, None, off[nxt + kv], None


def _bias_kv_layout(layer):
    """Element offsets of (bias_k, bias_v) inside a flat shard."""
    off = layer._store.offsets
    nxt = (3 if layer.separate_proj else 1) + (1 if layer.has_bias else 0)
    return off[nxt], off[nxt + 1]


class _GeneralAttentionFn(torch.autograd.Function):
    """Attention whose keys and values come from their own tensors (query [L, N, E], key [S, N, kdim], value
    [S, N, vdim]; functional.py:575-609 projects them with three row blocks of the shard), optionally with the
    learned key / value bias_k / bias_v (add_bias_kv, functional.py:711-716) and then one all-zero key / value
    (add_zero_attn, functional.py:746-753) appended per batch entry.  Three projections per shard run into
    q [L*N, E], k and v [(S+z)*N, E] (group g at column block g; z appended positions); the core is batched products
    and the softmax kernel with p [ws*N*h_s, L, S+z] in memory."""

    @staticmethod
    def forward(ctx, query, key, value, anchor, layer, mask, key_bias, want_weights, drop_p=0.0):
        store = layer._store
        L, N, E = query.shape
        s_in = key.shape[0]
        zero = 1 if layer.add_zero_attn else 0
        bkv = 1 if layer.add_bias_kv else 0
        sk = s_in + bkv + zero
        ws, h_s, d, e_s = layer.world_size, layer.num_heads_per_partition, layer.head_dim, layer.embed_dim_per_partition
        dt, dev = query.dtype, query.device
        q2, k2, v2 = as_rows(query, E), as_rows(key, layer.kdim), as_rows(value, layer.vdim)
        wq, wk, wv, b_in, w_o, b_o = _shard_layout(layer)
        bq, bk, bv = (b_in, b_in + e_s, b_in + 2 * e_s) if b_in is not None else (None, None, None)
        Z = N * h_s
        scale = 1.0 / math.sqrt(d)
        qb = torch.empty(L * N, E, dtype=dt, device=dev)
        kb = torch.empty(sk * N, E, dtype=dt, device=dev)
        vb = torch.empty(sk * N, E, dtype=dt, device=dev)
        if zero:
            kb[(s_in + bkv) * N:].zero_()
            vb[(s_in + bkv) * N:].zero_()
        bk_off, bv_off = _bias_kv_layout(layer) if bkv else (None, None)
        o = torch.empty(L * N, E, dtype=dt, device=dev)
        out = torch.empty(L * N, E, dtype=dt, device=dev)
        p = torch.empty(ws * Z, L, sk, dtype=dt, device=dev)
        drop = torch.empty(ws * Z, L, sk, dtype=torch.float32, device=dev) if drop_p > 0.0 else None
        pv = torch.empty_like(p) if drop_p > 0.0 else p
        ld = N * E  # one step along the sequence in q, k, v and o
        order = ring_order(layer.rank, ws)
        rot = Rotation(store.home, order, group=store.stage_group)
        acc = ops.ShardSum(out, sum(len(w) for w in rot.windows))
        i = 0
        for j in range(rot.steps):
            for flat, first, cnt in rot.acquire(j):
                c0 = first * e_s
                S.col_fwd(q2, flat, wq, e_s, E, bq, qb, c0)
                S.col_fwd(k2, flat, wk, e_s, layer.kdim, bk, kb[:s_in * N], c0)
                S.col_fwd(v2, flat, wv, e_s, layer.vdim, bv, vb[:s_in * N], c0)
                if bkv:  # position s_in of every batch entry: the head groups' slices of bias_k / bias_v
                    kb[s_in * N:(s_in + 1) * N, c0:c0 + cnt * e_s] = flat[:, bk_off:bk_off + e_s].reshape(1, cnt * e_s)
                    vb[s_in * N:(s_in + 1) * N, c0:c0 + cnt * e_s] = flat[:, bv_off:bv_off + e_s].reshape(1, cnt * e_s)
                scores = torch.empty(cnt * Z, L, sk, dtype=torch.float32, device=dev)
                _bmm(dt, a=qb, a_off=c0, lda=ld, a_kc=True, a_s=(E, d), a_sg=e_s, b=kb, b_off=c0, ldb=ld, b_kc=True,
                     b_s=(E, d), b_sg=e_s, c=scores, c_off=0, ldc=sk, c_s=(h_s * L * sk, L * sk), c_sg=Z * L * sk,
                     m=L, n=sk, k=d, batch=Z, zdiv=h_s, groups=cnt, out_f32=True)
                if drop is not None:
                    ops.softmax_fwd(scores, p[first * Z:(first + cnt) * Z], mask=mask, causal=False, scale=scale,
                                    key_bias=key_bias, heads=h_s,
                                    keep=_draw_keep(layer, drop_p, drop[first * Z:(first + cnt) * Z]),
                                    p_dropped=pv[first * Z:(first + cnt) * Z])
                else:
                    ops.softmax_fwd(scores, p[first * Z:(first + cnt) * Z], mask=mask, causal=False, scale=scale,
                                    key_bias=key_bias, heads=h_s)
                del scores
                _bmm(dt, a=pv, a_off=first * Z * L * sk, lda=sk, a_kc=True, a_s=(h_s * L * sk, L * sk),
                     a_sg=Z * L * sk, b=vb, b_off=c0, ldb=ld, b_kc=False, b_s=(E, d), b_sg=e_s, c=o, c_off=c0, ldc=ld,
                     c_s=(E, d), c_sg=e_s, m=L, n=d, k=sk, batch=Z, zdiv=h_s, groups=cnt)
                c_out, c_in = acc.target(i)
                S.row_fwd(o, flat, w_o, E, e_s, b_o, c_out, c0, c_in=c_in)
                i += 1
            rot.release(j)
        weights = None
        if want_weights:
            last = order[-1]
            weights = pv[last * Z:(last + 1) * Z].view(N, h_s, L, sk)
        ctx.layer = layer
        ctx.dims = (L, N, E, s_in, sk)
        ctx.dropped = drop is not None
        ctx.save_for_backward(q2, k2, v2, qb, kb, vb, p, o, *((drop, pv) if drop is not None else ()))
        ctx.mark_non_differentiable(*([weights] if weights is not None else []))
        return out.view(L, N, E), weights

    @staticmethod
    def backward(ctx, dout, _dweights=None):
        layer = ctx.layer
        q2, k2, v2, qb, kb, vb, p, o = ctx.saved_tensors[:8]
        drop, pv = ctx.saved_tensors[8:] if ctx.dropped else (None, p)
        store = layer._store
        L, N, E, s_in, sk = ctx.dims
        ws, h_s, d, e_s = layer.world_size, layer.num_heads_per_partition, layer.head_dim, layer.embed_dim_per_partition
        dt, dev = q2.dtype, q2.device
        wq, wk, wv, b_in, w_o, b_o = _shard_layout(layer)
        bq, bk, bv = (b_in, b_in + e_s, b_in + 2 * e_s) if b_in is not None else (None, None, None)
        Z = N * h_s
        scale = 1.0 / math.sqrt(d)
        ld = N * E
        dout2 = as_rows(dout, E)
        do = torch.empty(L * N, E, dtype=dt, device=dev)
        dqb = torch.empty(L * N, E, dtype=dt, device=dev)
        dkb = torch.empty(sk * N, E, dtype=dt, device=dev)
        dvb = torch.empty(sk * N, E, dtype=dt, device=dev)
        order = ring_order(layer.rank, ws, reverse=True)
        rot = Rotation(store.home, order, group=store.stage_group)
        parts = sum(len(w) for w in rot.windows)
        # input gradients of the three projections, each summed over the shards; the rows of an appended zero key
        # belong to no input
        sums = []
        for need, src, rows, width, w_off in ((ctx.needs_input_grad[0], dqb, L * N, E, wq),
                                              (ctx.needs_input_grad[1], dkb, s_in * N, layer.kdim, wk),
                                              (ctx.needs_input_grad[2], dvb, s_in * N, layer.vdim, wv)):
            if need:
                dx = torch.empty(rows, width, dtype=dt, device=dev)
                sums.append((dx, ops.ShardSum(dx, parts), src[:rows], width, w_off))
            else:
                sums.append(None)
        i = 0
        for j in range(rot.steps):
            for flat, first, cnt in rot.acquire(j):
                c0 = first * e_s
                p_off = first * Z * L * sk
                p_s, p_sg = (h_s * L * sk, L * sk), Z * L * sk
                S.row_dgrad(dout2, flat, w_o, E, e_s, do, c0)
                # dP = dO V^T
                dp = torch.empty(cnt * Z, L, sk, dtype=torch.float32, device=dev)
                _bmm(dt, a=do, a_off=c0, lda=ld, a_kc=True, a_s=(E, d), a_sg=e_s, b=vb, b_off=c0, ldb=ld, b_kc=True,
                     b_s=(E, d), b_sg=e_s, c=dp, c_off=0, ldc=sk, c_s=p_s, c_sg=p_sg, m=L, n=sk, k=d, batch=Z,
                     zdiv=h_s, groups=cnt, out_f32=True)
                # dV = P^T dO
                _bmm(dt, a=pv, a_off=p_off, lda=sk, a_kc=False, a_s=p_s, a_sg=p_sg, b=do, b_off=c0, ldb=ld, b_kc=False,
                     b_s=(E, d), b_sg=e_s, c=dvb, c_off=c0, ldc=ld, c_s=(E, d), c_sg=e_s, m=sk, n=d, k=L, batch=Z,
                     zdiv=h_s, groups=cnt)
                ds = torch.empty(cnt * Z, L, sk, dtype=dt, device=dev)
                ops.softmax_bwd(p[first * Z:(first + cnt) * Z], dp, ds, scale,
                                keep=None if drop is None else drop[first * Z:(first + cnt) * Z])
                del dp
                # dQ = dS K
                _bmm(dt, a=ds, a_off=0, lda=sk, a_kc=True, a_s=p_s, a_sg=p_sg, b=kb, b_off=c0, ldb=ld, b_kc=False,
                     b_s=(E, d), b_sg=e_s, c=dqb, c_off=c0, ldc=ld, c_s=(E, d), c_sg=e_s, m=L, n=d, k=sk, batch=Z,
                     zdiv=h_s, groups=cnt)
                # dK = dS^T Q
                _bmm(dt, a=ds, a_off=0, lda=sk, a_kc=False, a_s=p_s, a_sg=p_sg, b=qb, b_off=c0, ldb=ld, b_kc=False,
                     b_s=(E, d), b_sg=e_s, c=dkb, c_off=c0, ldc=ld, c_s=(E, d), c_sg=e_s, m=sk, n=d, k=L, batch=Z,
                     zdiv=h_s, groups=cnt)
                for item in sums:
                    if item is not None:
                        _, acc, src, width, w_off = item
                        c_out, c_in = acc.target(i)
                        S.col_dgrad(src, flat, w_off, e_s, width, c_out, c0, c_in=c_in)
                i += 1
            rot.release(j)
        runs = store.grad_runs(order)
        dk_in, dv_in = dkb[:s_in * N], dvb[:s_in * N]

        def param_grads():
            for first, cnt, accumulate in runs:
                c0 = first * e_s
                S.row_wgrad(dout2, o, store.grads, first, w_o, E, e_s, c0, cnt, accumulate, b_off=b_o, store=store)
                S.col_wgrad(dqb, q2, store.grads, first, wq, e_s, E, c0, cnt, accumulate, b_off=bq, store=store)
                S.col_wgrad(dk_in, k2, store.grads, first, wk, e_s, layer.kdim, c0, cnt, accumulate, b_off=bk, store=store)
                S.col_wgrad(dv_in, v2, store.grads, first, wv, e_s, layer.vdim, c0, cnt, accumulate, b_off=bv, store=store)
                if layer.add_bias_kv:
                    # the appended position's key / value gradient, summed over the batch entries it was copied to
                    bk_off, bv_off = _bias_kv_layout(layer)
                    S.col_bgrad(dkb[s_in * N:(s_in + 1) * N], store.grads, first, bk_off, e_s, c0, cnt, accumulate)
                    S.col_bgrad(dvb[s_in * N:(s_in + 1) * N], store.grads, first, bv_off, e_s, c0, cnt, accumulate)
            store.grads_ready()

        run_wgrad(dev, param_grads, (dout2, o, dqb, dkb, dvb, q2, k2, v2))
        grads = [None if item is None else item[0] for item in sums]
        dq = None if grads[0] is None else grads[0].view(L, N, E)
        dk = None if grads[1] is None else grads[1].view(s_in, N, layer.kdim)
        dv = None if grads[2] is None else grads[2].view(s_in, N, layer.vdim)
        return dq, dk, dv, None, None, None, None, None, None


class ParallelMultiheadAttention(RotatedLayer):
    """Signature follows rtp/module/attention.py:192-193; `MultiheadAttention_layer` imports the weights
    of an unsharded nn.MultiheadAttention.  Self-attention (query, key and value the same tensor) takes the packed
    projection and the fused cores; keys / values from other tensors, kdim / vdim != embed_dim and add_zero_attn take
    three projections and the product + softmax core, and so do attention dropout while training (the probabilities
    are dropped in memory), 3-D masks [batch * heads / ws, L, S] and add_bias_kv (a shard holds its head group's slice of
    bias_k / bias_v, see SubParallelMultiheadAttention).  key_padding_mask [batch, keys] (bool or float, functional.py:615-623 and :760-768) reaches
    the kernels as a per-(batch, key) additive bias."""

    def __init__(self, embed_dim, num_heads, world_size, rank, dropout=0., bias=True, add_bias_kv=False,
                 add_zero_attn=False, kdim=None, vdim=None, batch_first=False, device=None, dtype=None,
                 MultiheadAttention_layer: Optional[nn.MultiheadAttention] = None) -> None:
        super().__init__()
        self.world_size, self.rank = world_size, rank
        self.embed_dim, self.num_heads = embed_dim, num_heads
        self.dropout, self.batch_first, self.has_bias = dropout, batch_first, bias
        if MultiheadAttention_layer is not None and device is None:
            device = MultiheadAttention_layer.out_proj.weight.device
        if MultiheadAttention_layer is not None and dtype is None:
            dtype = MultiheadAttention_layer.out_proj.weight.dtype
        layers = []
        for s in range(world_size):
            sub = SubParallelMultiheadAttention(embed_dim, num_heads, world_size, s, dropout, bias, add_bias_kv,
                                                add_zero_attn, kdim, vdim, batch_first, device, dtype)
            sub.affine_weight(MultiheadAttention_layer)
            layers.append(sub)
        self.head_dim = layers[0].head_dim
        self.kdim, self.vdim = layers[0].kdim, layers[0].vdim
        self.separate_proj = not layers[0]._qkv_same_embed_dim
        self.add_zero_attn = bool(add_zero_attn)
        self.add_bias_kv = bool(add_bias_kv)
        self.num_heads_per_partition = layers[0].num_heads_per_partition
        self.embed_dim_per_partition = layers[0].embed_dim_per_partition
        self._init_store(layers)
        self.layers = list(self.shards)
        self.MultiheadAttention = self.layers[self.rank]

    def forward(self, query: Tensor, key: Tensor, value: Tensor, key_padding_mask: Optional[Tensor] = None,
                need_weights: bool = True, attn_mask: Optional[Tensor] = None, average_attn_weights: bool = True,
                is_causal: bool = False, test_tensor=None, residual_grad: bool = False) -> Tuple[Tensor, Optional[Tensor]]:
        same = key is query and value is query
        if not same:
            same = (key.data_ptr() == query.data_ptr() == value.data_ptr() and key.shape == query.shape == value.shape
                    and key.stride() == query.stride() == value.stride())
        general = not same or self.separate_proj or self.add_zero_attn or self.add_bias_kv
        drop_p = float(self.dropout) if self.training else 0.0
        if not 0.0 <= drop_p < 1.0:
            raise ValueError(f"attention dropout probability has to be in [0, 1), got {drop_p}")
        if query.dim() != 3 or key.dim() != 3 or value.dim() != 3:
            raise NotImplementedError("rotated attention expects batched [L, N, E] (or batch_first) inputs")
        x = query.transpose(0, 1) if self.batch_first else query
        L, keys = x.shape[0], (key.shape[1] if self.batch_first else key.shape[0])
        mask = None
        causal = False
        if attn_mask is not None:
            # functional.py:690-704: [L, S], or one mask per (batch, head of a shard) [N * heads / ws, L, S], which
            # every head group of the rotation then shares
            per_head = (x.shape[1] * self.num_heads_per_partition, L, keys)
            if tuple(attn_mask.shape) not in ((L, keys), per_head):
                raise RuntimeError(f"The shape of the attn_mask is {tuple(attn_mask.shape)}, but should be "
                                   f"{(L, keys)} or {per_head}.")
            mask = F._canonical_mask(mask=attn_mask, mask_name="attn_mask", other_type=None, other_name="",
                                     target_type=torch.float32)
            mask = mask.to(device=x.device, dtype=torch.float32).contiguous()
        elif is_causal:
            if general:
                # functional.py:623-628
                raise RuntimeError("Need attn_mask if specifying the is_causal hint.")
            causal = True
        key_bias = None
        if key_padding_mask is not None:
            # functional.py:615-623, :760-768: a bool mask hides the keys where it is True, a float mask is added to the
            # scores; merged into the attention mask per batch there, handed to the kernels as a [batch, key] bias here
            if key_padding_mask.dim() != 2 or tuple(key_padding_mask.shape) != (x.shape[1], keys):
                raise ValueError(f"key_padding_mask must be [batch, keys] = {(x.shape[1], keys)}, got "
                                 f"{tuple(key_padding_mask.shape)}")
            key_bias = F._canonical_mask(mask=key_padding_mask, mask_name="key_padding_mask",
                                         other_type=F._none_or_dtype(attn_mask), other_name="attn_mask",
                                         target_type=torch.float32)
            key_bias = key_bias.to(device=x.device, dtype=torch.float32).contiguous()
        if general:
            if residual_grad:
                raise ValueError("residual_grad is for self-attention (the residual is the attention's own input)")
            k_in, v_in = (key.transpose(0, 1), value.transpose(0, 1)) if self.batch_first else (key, value)
            if k_in.shape[0] != v_in.shape[0] or k_in.shape[1] != x.shape[1] or v_in.shape[1] != x.shape[1] or \
                    x.shape[2] != self.embed_dim or k_in.shape[2] != self.kdim or v_in.shape[2] != self.vdim:
                raise ValueError(f"rotated attention: query {tuple(query.shape)}, key {tuple(key.shape)} and value "
                                 f"{tuple(value.shape)} do not fit embed_dim / kdim / vdim = "
                                 f"{(self.embed_dim, self.kdim, self.vdim)} and a common batch and key count")
            # functional.py:711-716 and :746-753: the appended bias key and the appended all-zero key are visible to
            # every query (one zero column each in both masks)
            extra = int(self.add_bias_kv) + int(self.add_zero_attn)
            if extra:
                if mask is not None:
                    mask = F.pad(mask, (0, extra))
                if key_bias is not None:
                    key_bias = F.pad(key_bias, (0, extra))
            out, weights = _GeneralAttentionFn.apply(x, k_in, v_in, self._anchor, self, mask, key_bias,
                                                     bool(need_weights), drop_p)
        else:
            out, weights = _AttentionFn.apply(x, self._anchor, self, mask, causal, bool(need_weights),
                                              bool(residual_grad), key_bias, drop_p)
        if need_weights and weights is not None and average_attn_weights:
            weights = weights.float().mean(dim=1).to(out.dtype)
        if self.batch_first:
            out = out.transpose(0, 1)
        return out, (weights if need_weights else None)
