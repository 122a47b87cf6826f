"""The attention leaf the auto-wrapper shards by hand (counterpart of rtp/attention.py:12-147): ONE rank's head
group -- a packed in-projection [3E/ws, E] (or three blocks when keys / values have their own width) and the
out-projection's column block [E, E/ws] -- with the world size taken from the process group instead of passed in.

It is a parameter holder: on one GPU every rank's head group runs inside one rotated layer, so wrap it,
`FlyweightWarpper(shard_or_list_of_shards, group, cat_output=False)`, as rtp/rotated_tensor_parallel.py:525 does, or
build `rtp.module.attention.ParallelMultiheadAttention` directly.  Calling the bare shard raises.
"""
from __future__ import annotations

from typing import Optional

import torch.nn as nn

from .module.attention import SubParallelMultiheadAttention
from .module.collectives import resolve_world


class ParallelMultiheadAttention(SubParallelMultiheadAttention):
    """Constructor arguments follow rtp/attention.py:18-20.  `MultiheadAttention` (an unsharded nn.MultiheadAttention,
    unused by the reference's constructor) imports this rank's blocks of its weights: in-projection blocks
    [r, r+ws, r+2ws] of a 3*ws row split, out-projection column block r, out bias / ws.  `empty_init` leaves the
    parameters as allocated."""

    def __init__(self, embed_dim, num_heads, dropout=0., bias=True, add_bias_kv=False, add_zero_attn=False, kdim=None,
                 vdim=None, batch_first=False, device=None, dtype=None,
                 MultiheadAttention: Optional[nn.MultiheadAttention] = None, empty_init=False, group=None) -> None:
        world_size, rank = resolve_world(group)
        super().__init__(embed_dim, num_heads, world_size, rank, dropout, bias, add_bias_kv, add_zero_attn, kdim, vdim,
                         batch_first, device, dtype)
        self.affine_weight(MultiheadAttention)

    def forward(self, *args, **kwargs):
        raise NotImplementedError(
            "rtp.attention.ParallelMultiheadAttention holds one rank's head group; wrap it in FlyweightWarpper(..., "
            "cat_output=False) or use rtp.module.attention.ParallelMultiheadAttention, which run all head groups of "
            "the rotation on this GPU")
