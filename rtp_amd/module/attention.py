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
    def forward(ctx, x, anchor, layer, mask, causal, want_weights, residual_grad=False, key_bias=None):
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
        fused = ops.attn_supported(dt, L, d)
        flash = not fused and not want_weights and ops.attn_flash_supported(dt, L, d)
        if flash:
            p = torch.empty(ws * Z, L, dtype=torch.float32, device=dev)  # log-sum-exp in place of probabilities
        else:
            p = torch.empty(ws * Z, L, L, dtype=dt, device=dev)
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
                ops.softmax_fwd(scores, p_run, mask=mask, causal=causal, scale=scale, key_bias=key_bias, heads=h_s)
                del scores
                _bmm(dt, a=p, a_off=first * Z * L * L, lda=L, a_kc=True, a_s=(h_s * L * L, L * L), a_sg=Z * L * L,
                     b=qkv, b_off=q0 + 2 * e_s, ldb=ldq, b_kc=False, b_s=(ws * 3 * e_s, d), b_sg=3 * e_s, c=o,
                     c_off=first * e_s, ldc=N * E, c_s=(E, d), c_sg=e_s, m=L, n=d, k=L, batch=Z, zdiv=h_s, groups=cnt)
                c_out, c_in = acc.target(i)
                S.row_fwd(o, flat, w_o_off, E, e_s, b_o_off, c_out, first * e_s, c_in=c_in)
                i += 1
            rot.release(j)
        weights = None
        if want_weights:
            last = order[-1]
            weights = p[last * Z:(last + 1) * Z].view(N, h_s, L, L)
        ctx.layer = layer
        ctx.dims = (L, N, E)
        ctx.residual_grad = residual_grad
        ctx.flash = (mask, causal, key_bias) if flash else None
        ctx.save_for_backward(x2, qkv, p, o)
        ctx.mark_non_differentiable(*([weights] if weights is not None else []))
        return out.view(L, N, E), weights

    @staticmethod
    def backward(ctx, dout, _dweights=None):
        layer = ctx.layer
        x2, qkv, p, o = ctx.saved_tensors
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
        fused = ops.attn_supported(dt, L, d)
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
                _bmm(dt, a=p, a_off=p_off, lda=L, a_kc=False, a_s=(h_s * L * L, L * L), a_sg=Z * L * L, b=do,
                     b_off=first * e_s, ldb=N * E, b_kc=False, b_s=(E, d), b_sg=e_s, c=dqkv, c_off=q0 + 2 * e_s, ldc=ldq,
                     c_s=(ws * 3 * e_s, d), c_sg=3 * e_s, m=L, n=d, k=L, batch=Z, zdiv=h_s, groups=cnt)
                ds = torch.empty(cnt * Z, L, L, dtype=dt, device=dev)
                ops.softmax_bwd(p[first * Z:(first + cnt) * Z], dp, ds, scale)
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
                            b_off=b_o_off if layer.has_bias else None)
                S.col_wgrad(dqkv, x2, store.grads, first, 0, 3 * e_s, E, first * 3 * e_s, cnt, accumulate,
                            b_off=b_in_off if layer.has_bias else None)
            store.grads_ready()

        run_wgrad(dev, param_grads, (dout2, o, dqkv, x2))
        return (dx.view(L, N, E) if need_dx else None), None, None, None, None, None, None, None


class ParallelMultiheadAttention(RotatedLayer):
    """Signature follows rtp/module/attention.py:192-193; `MultiheadAttention_layer` imports the weights
    of an unsharded nn.MultiheadAttention.  Self-attention only (query, key and value must be the same
    tensor); 3-D masks and attention dropout are not implemented and raise.  key_padding_mask [batch, keys] (bool or
    float, functional.py:615-623 and :760-768) reaches the kernels as a per-(batch, key) additive bias."""

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
                is_causal: bool = False, test_tensor=None, residual_grad: bool = False) -> Tuple[Tensor, Optional[Tensor]]:
        if not (key is query and value is query):
            if not (key.data_ptr() == query.data_ptr() == value.data_ptr() and key.shape == query.shape == value.shape
                    and key.stride() == query.stride() == value.stride()):
                raise NotImplementedError("rotated attention implements self-attention only (query is key is value)")
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
        key_bias = None
        if key_padding_mask is not None:
            # functional.py:615-623, :760-768: a bool mask hides the keys where it is True, a float mask is added to the
            # scores; merged into the attention mask per batch there, handed to the kernels as a [batch, key] bias here
            if key_padding_mask.dim() != 2 or tuple(key_padding_mask.shape) != (x.shape[1], L):
                raise ValueError(f"key_padding_mask must be [batch, keys] = {(x.shape[1], L)}, got "
                                 f"{tuple(key_padding_mask.shape)}")
            key_bias = F._canonical_mask(mask=key_padding_mask, mask_name="key_padding_mask",
                                         other_type=F._none_or_dtype(attn_mask), other_name="attn_mask",
                                         target_type=torch.float32)
            key_bias = key_bias.to(device=x.device, dtype=torch.float32).contiguous()
        out, weights = _AttentionFn.apply(x, self._anchor, self, mask, causal, bool(need_weights), bool(residual_grad),
                                          key_bias)
        if need_weights and weights is not None and average_attn_weights:
            weights = weights.float().mean(dim=1).to(out.dtype)
        if self.batch_first:
            out = out.transpose(0, 1)
        return out, (weights if need_weights else None)
