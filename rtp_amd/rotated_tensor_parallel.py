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

from typing import Any, List, Optional

import torch
import torch.nn as nn

from .module.attention import ParallelMultiheadAttention
from .module.collectives import emulate_shards, resolve_world
from .module.conv import ColumnParallelConv2d
from .module.embedding import ParallelEmbedding
from .module.linear import ColumnParallelLinear, RowParallelLinear


class FlyweightWarpper(nn.Module):
    """Holds the rotated replacement of one leaf module.  `module` is the home shard, `module_list` all
    shards, `flat_param` the home shard's flat parameter buffer."""

    def __init__(self, rotated: nn.Module, row_partition: bool = False, cat_output: bool = True):
        super().__init__()
        self.rotated = rotated
        self.row_partition = row_partition
        self.cat_output = cat_output
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
