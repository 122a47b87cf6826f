"""RotatedTensorParallel: shard the nn.Linear / nn.Conv2d / nn.Embedding / nn.MultiheadAttention leaves of an
existing model in place and run them as rotated layers (counterpart of
rtp/rotated_tensor_parallel.py:296-571).

Sharding rules (rotated_tensor_parallel.py:454-529):
  nn.Linear              out_features % ws == 0 -> column shards (weight rows, bias slice), outputs side by side;
                         elif in_features % ws == 0 -> row shards (weight columns, bias/ws), outputs summed;
                         else ValueError.
  nn.Conv2d              out_channels % ws == 0 -> output-channel shards, outputs concatenated on dim 1, else
                         ValueError (rotated_tensor_parallel.py:472-483).
  nn.Embedding           embedding_dim % ws == 0 -> column blocks of the table, else ValueError.
  nn.MultiheadAttention  head groups: in-projection blocks [r, r+ws, r+2ws] of a 3*ws row split,
                         out-projection column block r, out bias / ws; outputs summed.
Each replaced leaf becomes a FlyweightWarpper holding the rotated layer.
"""
from __future__ import annotations

import copy
from typing import Any, List, Optional, Sequence

import torch
import torch.nn as nn

from .module.attention import ParallelMultiheadAttention, SubParallelMultiheadAttention
from .module.collectives import RotatedLayer, emulate_shards, resolve_world
from .module.conv import ColumnParallelConv2d
from .module.embedding import ParallelEmbedding
from .module.linear import ColumnParallelLinear, RowParallelLinear

RotatedMultiheadAttention = ParallelMultiheadAttention  # rtp/module/attention.py's layer (rtp/attention.py has a twin)


def split_tensor(tensor: torch.Tensor, num_partitions: int, contiguous_split_chunks: bool = False, dim: int = -1):
    """`num_partitions` equal blocks of `tensor` along `dim` (rtp/rotated_tensor_parallel.py:40-62): how a caller cuts
    a leaf to one rank's share before wrapping it by hand."""
    if tensor.size(dim) % num_partitions != 0:
        raise AssertionError("{} is not divisible by {}".format(tensor.size(dim), num_partitions))
    chunks = torch.split(tensor, tensor.size(dim) // num_partitions, dim=dim)
    return tuple(c.contiguous() for c in chunks) if contiguous_split_chunks else chunks


def _rotated_from_shards(shards: Sequence[nn.Module], ws: int, rank: int, row_partition: bool, cat_output: bool,
                         output_partition_dim: int, input_partition_dim: int) -> nn.Module:
    """The rotated layer whose shard s holds exactly the parameters of shards[s] (leaf modules already cut to one
    rank's share, as rotated_tensor_parallel.py:454-529 cuts them before wrapping)."""
    proto = shards[0]
    p0 = next(proto.parameters())
    dev, dt = p0.device, p0.dtype

    def want(cond: bool, what: str) -> None:
        if not cond:
            raise NotImplementedError(f"FlyweightWarpper: {type(proto).__name__} shards {what}")

    with emulate_shards(ws):
        if isinstance(proto, SubParallelMultiheadAttention):
            want(not cat_output and not row_partition, "are summed: pass cat_output=False (and no row_partition)")
            rotated = RotatedMultiheadAttention(
                proto.embed_dim, proto.num_heads, ws, rank, dropout=proto.dropout, bias=proto.bias,
                add_bias_kv=proto.bias_k is not None, add_zero_attn=proto.add_zero_attn, kdim=proto.kdim,
                vdim=proto.vdim, batch_first=proto.batch_first, device=dev, dtype=dt)
        elif isinstance(proto, nn.Linear):
            if row_partition:
                want(input_partition_dim == -1, "split their input on the last dimension (input_partition_dim=-1)")
                rotated = RowParallelLinear(proto.in_features * ws, proto.out_features, bias=proto.bias is not None,
                                            device=dev, dtype=dt)
            else:
                want(cat_output and output_partition_dim == -1,
                     "lay their outputs side by side on the last dimension (cat_output, output_partition_dim=-1)")
                rotated = ColumnParallelLinear(proto.in_features, proto.out_features * ws, bias=proto.bias is not None,
                                               device=dev, dtype=dt)
        elif isinstance(proto, nn.Conv2d):
            want(cat_output and not row_partition and output_partition_dim == 1,
                 "concatenate their outputs on the channel dimension (output_partition_dim=1)")
            rotated = ColumnParallelConv2d(proto.in_channels, proto.out_channels * ws, proto.kernel_size, proto.stride,
                                           proto.padding, proto.dilation, proto.groups, proto.bias is not None,
                                           proto.padding_mode, device=dev, dtype=dt)
        elif isinstance(proto, nn.Embedding):
            want(cat_output and not row_partition and output_partition_dim == -1,
                 "lay their outputs side by side on the last dimension (cat_output, output_partition_dim=-1)")
            rotated = ParallelEmbedding(proto.num_embeddings, proto.embedding_dim * ws, ws, rank,
                                        padding_idx=proto.padding_idx, max_norm=proto.max_norm,
                                        norm_type=proto.norm_type, scale_grad_by_freq=proto.scale_grad_by_freq,
                                        sparse=proto.sparse, device=dev, dtype=dt)
        else:
            raise NotImplementedError(
                f"FlyweightWarpper: no rotated kernel path for a {type(proto).__name__} leaf (nn.Linear, nn.Conv2d, "
                "nn.Embedding and the attention shard of rtp.attention are the leaves the wrapper shards)")
    with torch.no_grad():
        for mine, given in zip(rotated.shards, shards):
            theirs = dict(given.named_parameters())
            for name, p in mine.named_parameters():
                if name not in theirs or theirs[name].shape != p.shape:
                    raise ValueError(f"FlyweightWarpper: shard parameter {name} {tuple(p.shape)} has no counterpart "
                                     "of that shape in the module handed in")
                p.copy_(theirs[name])
    return rotated


class FlyweightWarpper(nn.Module):
    """Holds the rotated replacement of one leaf module; constructor arguments as
    rtp/rotated_tensor_parallel.py:296-310.  `module` is

    * a rotated layer of this package (what RotatedTensorParallel hands in), or
    * a leaf already cut to ONE rank's share -- nn.Linear (column shard, or row shard with row_partition=True),
      nn.Conv2d (output_partition_dim=1), nn.Embedding, the attention shard of rtp.attention (cat_output=False) --
      as code that wraps a leaf by hand passes it, or a sequence of world_size such leaves, entry r being the leaf
      rank r would pass.  All ranks run in this one process, so the wrapper needs every rank's share; given a
      single leaf with world_size > 1 every rank starts from a copy of it (what each rank's deep copies hold in the
      reference before the first rotation, :341-355).

    `module` is then the home shard, `module_list` all shards, `flat_param` the home shard's flat parameter buffer.
    group: only its size is used (see resolve_world).  param_list / flat_param_names: the reference flattens
    `list(module.parameters())` when they are None, which is the one layout built here; anything else raises.
    partition_dim is carried as an attribute (the reference never reads it either); inplace selected the
    reference's blocking rotation and is accepted and ignored."""

    def __init__(self, module, group: Optional[Any] = None, param_list=None,
                 flat_param_names: Optional[List[str]] = None, partition_dim: Optional[int] = None,
                 output_partition_dim: Optional[int] = None, row_partition: bool = False,
                 input_partition_dim: Optional[int] = None, cat_output: bool = True, inplace: bool = False):
        super().__init__()
        self.partition_dim = -1 if partition_dim is None else partition_dim
        self.output_partition_dim = -1 if output_partition_dim is None else output_partition_dim
        self.input_partition_dim = -1 if input_partition_dim is None else input_partition_dim
        self.row_partition = row_partition
        self.cat_output = cat_output
        self.inplace = inplace
        self.group = group
        if isinstance(module, RotatedLayer):
            rotated = module
        else:
            ws, rank = resolve_world(group)
            shards = list(module) if isinstance(module, (list, tuple, nn.ModuleList)) else None
            if shards is None:
                shards = [module] + [copy.deepcopy(module) for _ in range(ws - 1)]
            if len(shards) != ws:
                raise ValueError(f"FlyweightWarpper: {len(shards)} shard modules for a world size of {ws}")
            if param_list is not None and [id(p) for p in param_list] != [id(p) for p in shards[rank].parameters()]:
                raise NotImplementedError("FlyweightWarpper: param_list other than list(module.parameters())")
            if flat_param_names is not None:
                raise NotImplementedError("FlyweightWarpper: flat_param_names (the reference ignores it too)")
            rotated = _rotated_from_shards(shards, ws, rank, row_partition, cat_output, self.output_partition_dim,
                                           self.input_partition_dim)
        self.rotated = rotated
        self.world_size = rotated.world_size
        self.rank = rotated.rank

    @property
    def module_list(self) -> List[nn.Module]:
        return list(self.rotated.shards)

    @property
    def module(self) -> nn.Module:
        return self.rotated.shards[self.rank]

    @property
    def flat_param(self) -> torch.Tensor:
        return self.rotated._store.home[self.rank]

    def forward(self, *args: Any, **kwargs: Any):
        return self.rotated(*args, **kwargs)


class RotatedTensorParallel(nn.Module):
    """RotatedTensorParallel(module, group=None, inplace=False): walks `module`, replaces every
    shardable leaf and forwards calls to it.  `inplace` selected the reference's blocking rotation
    variant; there is one rotation schedule here, so it is accepted and ignored."""

    def __init__(self, module: nn.Module, group: Optional[Any] = None, inplace: bool = False):
        super().__init__()
        self.group = group
        self.world_size, self.rank = resolve_world(group)
        self.module = module
        self.inplace = inplace
        self.FlyweightModule_list: List[FlyweightWarpper] = []
        self.RecursiveVisit("module", self.module, self)

    def RecursiveVisit(self, name: str, module: nn.Module, upper_module: nn.Module) -> None:
        has_parameters = any(True for _ in module.parameters())
        has_child = any(True for _ in module.children())
        is_mha = isinstance(module, nn.MultiheadAttention)
        if has_child and not is_mha:
            for child_name, child in list(module.named_children()):
                self.RecursiveVisit(child_name, child, module)
            return
        if not has_parameters:
            return
        ws = self.world_size
        wrapped = None
        with emulate_shards(ws):
            if isinstance(module, nn.Linear):
                if module.out_features % ws == 0:
                    wrapped = FlyweightWarpper(ColumnParallelLinear(
                        module.in_features, module.out_features, bias=module.bias is not None, linear_layer=module))
                elif module.in_features % ws == 0:
                    wrapped = FlyweightWarpper(RowParallelLinear(
                        module.in_features, module.out_features, bias=module.bias is not None, linear_layer=module),
                        row_partition=True)
                else:
                    raise ValueError("The input or output features of the linear layer must be divisible by the "
                                     "world size.")
            elif isinstance(module, nn.Conv2d):
                if module.out_channels % ws != 0:
                    raise ValueError("The input or output channels of the conv layer must be divisible by the world "
                                     "size.")
                wrapped = FlyweightWarpper(ColumnParallelConv2d(
                    module.in_channels, module.out_channels, module.kernel_size, module.stride, module.padding,
                    module.dilation, module.groups, module.bias is not None, module.padding_mode, Conv2d_layer=module))
            elif isinstance(module, nn.Embedding):
                if module.embedding_dim % ws != 0:
                    raise ValueError("The embedding_dim of the embedding layer must be divisible by the world size.")
                wrapped = FlyweightWarpper(ParallelEmbedding(
                    module.num_embeddings, module.embedding_dim, ws, self.rank, padding_idx=module.padding_idx,
                    max_norm=module.max_norm, norm_type=module.norm_type,
                    scale_grad_by_freq=module.scale_grad_by_freq, sparse=module.sparse, Embedding_layer=module))
            elif is_mha:
                wrapped = FlyweightWarpper(ParallelMultiheadAttention(
                    module.embed_dim, module.num_heads, ws, self.rank, dropout=module.dropout,
                    bias=module.in_proj_bias is not None, add_bias_kv=module.bias_k is not None,
                    add_zero_attn=module.add_zero_attn, kdim=module.kdim, vdim=module.vdim,
                    batch_first=module.batch_first, MultiheadAttention_layer=module), cat_output=False)
        if wrapped is not None:
            setattr(upper_module, name, wrapped)
            self.FlyweightModule_list.append(wrapped)

    def forward(self, *args: Any, **kwargs: Any):
        return self.module(*args, **kwargs)
