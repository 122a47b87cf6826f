"""Rotated sharded Embedding (counterpart of rtp/module/embedding.py:33-164).

The table is split along the embedding dimension: shard s is the [V, D/ws] column block s of the
master table (embedding.py:65-71) and fills column block s of the output.  Forward gathers rows from
the staged shard; backward builds each shard's dense [V, D/ws] gradient with a sorted, segmented
scatter-add whose per-row summation order is ascending token position, which reproduces torch's CPU
nn.Embedding backward bit for bit.  The backward needs no weights, so it runs no rotation.
"""
from __future__ import annotations

from typing import Callable, Optional

import torch
import torch.nn as nn
import torch.nn.init as init

from .. import ops
from ..ring import Rotation, ring_order
from .collectives import RotatedLayer
from .shard_ops import _fused, _fused_done
from .utils import affine_weight, divide_and_check_no_remainder


class ModelParallelEmbedding(nn.Embedding):
    """One column block of the table (rtp/module/embedding.py:33-71)."""

    def __init__(self, num_embeddings: int, embedding_dim: int, world_size: int, rank: int,
                 padding_idx: Optional[int] = None, max_norm: Optional[float] = None, norm_type: float = 2.0,
                 scale_grad_by_freq: bool = False, sparse: bool = False,
                 init_method: Callable[[torch.Tensor], torch.Tensor] = init.xavier_normal_,
                 keep_master_weight_for_test: bool = False, device=None, dtype=None) -> None:
        self.world_size = world_size
        self.rank = rank
        self.embedding_dim_per_partition = divide_and_check_no_remainder(embedding_dim, world_size)
        super().__init__(num_embeddings, self.embedding_dim_per_partition, padding_idx, max_norm, norm_type,
                         scale_grad_by_freq, sparse, device=device, dtype=dtype)

    def affine_weight(self, Embedding_layer) -> None:
        if Embedding_layer is not None:
            affine_weight(self.weight, Embedding_layer.weight, self.embedding_dim_per_partition, 1, self.world_size,
                          self.rank)


class _EmbeddingFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, ids, anchor, layer, scale=1.0, pos=None):
        store = layer._store
        d_s, ws = layer.embedding_dim_per_partition, layer.world_size
        flat_ids = ids.reshape(-1).contiguous()
        out = torch.empty(flat_ids.numel(), layer.embedding_dim, dtype=store.home.dtype, device=store.home.device)
        rot = Rotation(store.home, ring_order(layer.rank, ws), group=store.stage_group)
        # tokens are [sequence, batch, ...]: every id of one position shares a positional row
        batch = flat_ids.numel() // ids.shape[0] if pos is not None else 1
        for j in range(rot.steps):
            for flat, first, cnt in rot.acquire(j):
                table = flat[0].view(layer.num_embeddings, d_s)
                cols = slice(first * d_s, (first + 1) * d_s)
                ops.embedding_gather(table, flat_ids, out[:, cols], groups=cnt, table_sg=store.numel, out_sg=d_s,
                                     scale=scale, pos=None if pos is None else pos[:, cols], pos_sg=d_s, batch=batch)
            rot.release(j)
        ctx.layer = layer
        ctx.grad_scale = scale
        ctx.save_for_backward(flat_ids)
        return out.view(*ids.shape, layer.embedding_dim)

    @staticmethod
    def backward(ctx, dout):
        layer = ctx.layer
        (flat_ids,) = ctx.saved_tensors
        store = layer._store
        d_s, ws = layer.embedding_dim_per_partition, layer.world_size
        g2 = dout.reshape(-1, layer.embedding_dim)
        if g2.stride(1) != 1:
            g2 = g2.contiguous()
        # up to a few thousand tokens: one launch per run of shards, from the raw ids; longer steps sort the ids once
        # and scatter-add per run
        onepass = ops.embedding_backward_supported(flat_ids.numel())
        workspace = None if onepass else ops.embedding_sort_ids(flat_ids)
        pad = -1 if layer.padding_idx is None else layer.padding_idx
        if store.on_backward is not None:
            store.on_backward(store)
        # runs of consecutive shards with the same overwrite / accumulate state go out as one grouped launch
        for first, cnt, accumulate in store._grad_runs(ring_order(layer.rank, ws, reverse=True)):
            table = store.grads[first, :store.numels[0]].view(store.shapes[0])
            # an optimiser that applies its update where gradients are produced: the rows the step's tokens name are
            # updated by the scatter-add itself, the dense [V, D/ws] gradient is neither zero-filled nor written
            kw = _fused(store, accumulate, first, cnt, store.offsets[0], store.numels[0])
            common = dict(padding_idx=pad, scale_by_freq=layer.scale_grad_by_freq, zero_fill=not accumulate, groups=cnt,
                          grad_out_sg=d_s, grad_table_sg=store.grads.shape[1], grad_scale=ctx.grad_scale, **kw)
            if onepass:
                ops.embedding_backward(g2[:, first * d_s:(first + 1) * d_s], flat_ids, table, **common)
            else:
                ops.embedding_scatter_add(g2[:, first * d_s:(first + 1) * d_s], flat_ids.numel(), workspace, table,
                                          **common)
            _fused_done(store, kw)
        store.grads_ready()
        return None, None, None, None, None


class ParallelEmbedding(RotatedLayer):
    """Embedding sharded along the embedding dimension and rotated.  Signature follows
    rtp/module/embedding.py:85-101; `Embedding_layer` imports the table of an unsharded nn.Embedding.
    `max_norm` and `sparse` gradients are not implemented by the kernels and raise."""

    def __init__(self, num_embeddings: int, embedding_dim: int, world_size: int, rank: int,
                 padding_idx: Optional[int] = None, max_norm: Optional[float] = None, norm_type: float = 2.0,
                 scale_grad_by_freq: bool = False, sparse: bool = False,
                 init_method: Callable[[torch.Tensor], torch.Tensor] = init.xavier_normal_,
                 keep_master_weight_for_test: bool = False, Embedding_layer: Optional[nn.Embedding] = None,
                 device=None, dtype=None) -> None:
        super().__init__()
        if max_norm is not None:
            raise NotImplementedError("ParallelEmbedding: max_norm renormalisation is not implemented")
        if sparse:
            raise NotImplementedError("ParallelEmbedding: sparse gradients are not implemented")
        self.num_embeddings = num_embeddings
        self.embedding_dim = embedding_dim
        if padding_idx is not None and padding_idx < 0:
            padding_idx = num_embeddings + padding_idx
        self.padding_idx = padding_idx
        self.max_norm = max_norm
        self.norm_type = norm_type
        self.scale_grad_by_freq = scale_grad_by_freq
        self.sparse = sparse
        self.world_size = world_size
        self.rank = rank
        self.embedding_dim_per_partition = divide_and_check_no_remainder(embedding_dim, world_size)
        if Embedding_layer is not None and device is None:
            device = Embedding_layer.weight.device
        if Embedding_layer is not None and dtype is None:
            dtype = Embedding_layer.weight.dtype
        embeddings = []
        for s in range(world_size):
            shard = ModelParallelEmbedding(num_embeddings, embedding_dim, world_size, s, padding_idx, max_norm,
                                           norm_type, scale_grad_by_freq, sparse, init_method,
                                           keep_master_weight_for_test, device=device, dtype=dtype)
            shard.affine_weight(Embedding_layer)
            embeddings.append(shard)
        self._init_store(embeddings)
        self.embeddings = list(self.shards)
        self.embedding = self.embeddings[self.rank]

    def forward(self, input_: torch.Tensor) -> torch.Tensor:
        if input_.dtype != torch.int64:
            input_ = input_.long()
        return _EmbeddingFn.apply(input_, self._anchor, self)

    def forward_scaled_positional(self, input_: torch.Tensor, scale: float, pos: torch.Tensor) -> torch.Tensor:
        """(self(input_) * scale) + pos[:input_.size(0), None, :] in one gather per shard group, with the rounding
        of the separate operations; `input_` is [sequence, batch], `pos` a [positions, embedding_dim] table of the
        layer's dtype that needs no gradient (rtp/models/transformer_lm_rtp.py:27-28 and :49)."""
        if input_.dim() != 2 or pos.dim() != 2 or pos.shape[1] != self.embedding_dim or pos.requires_grad:
            raise ValueError("forward_scaled_positional: ids must be [sequence, batch] and pos [positions, dim]")
        if input_.shape[0] > pos.shape[0]:
            raise ValueError("forward_scaled_positional: sequence longer than the positional table")
        if input_.dtype != torch.int64:
            input_ = input_.long()
        return _EmbeddingFn.apply(input_, self._anchor, self, float(scale), pos)
