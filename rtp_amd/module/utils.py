"""Shard-layout helpers (the rules of rtp/module/utils.py:19-103)."""
from __future__ import annotations

from typing import List, Sequence

import torch


def ensure_divisibility(numerator: int, denominator: int) -> None:
    assert numerator % denominator == 0, "{} is not divisible by {}".format(numerator, denominator)


def divide_and_check_no_remainder(numerator: int, denominator: int) -> int:
    ensure_divisibility(numerator, denominator)
    return numerator // denominator


divide = divide_and_check_no_remainder


def shard_slice(master: torch.Tensor, per_partition_size: int, partition_dim: int, index: int) -> torch.Tensor:
    """Block `index` of `master` cut into blocks of `per_partition_size` along `partition_dim`
    (what affine_weight copies for rank == index, rtp/module/utils.py:33-36)."""
    return master.narrow(partition_dim, index * per_partition_size, per_partition_size)


def affine_weight(weight: torch.Tensor, master_weight: torch.Tensor, per_partition_size: int, partition_dim: int,
                  world_size: int, rank: int, stride: int = 1) -> None:
    """Copy shard `rank` of the master weight into `weight`."""
    assert stride == 1, "strided partitions are not used by the rotated layers"
    with torch.no_grad():
        weight.data.copy_(shard_slice(master_weight.data, per_partition_size, partition_dim, rank))


def attention_block_index(rank: int, world_size: int) -> List[int]:
    """Blocks of a 3*ws-way row split of a packed in-projection that belong to head-group `rank`:
    its Q rows, K rows and V rows (rtp/module/attention.py:86-100)."""
    return [rank, rank + world_size, rank + 2 * world_size]


def affine_weight_attention(weight: torch.Tensor, master_weight: torch.Tensor, index: Sequence[int],
                            per_partition_size: int, partition_dim: int, world_size: int, rank: int,
                            stride: int = 1) -> None:
    """Copy the concatenation of blocks `index` (of size per_partition_size) of the master into
    `weight` (rtp/module/utils.py:38-59)."""
    assert stride == 1
    parts = [shard_slice(master_weight.data, per_partition_size, partition_dim, i) for i in index]
    with torch.no_grad():
        weight.data.copy_(torch.cat(parts, dim=partition_dim))


def split_tensor_along_last_dim(tensor: torch.Tensor, num_partitions: int, contiguous_split_chunks: bool = False):
    last = tensor.dim() - 1
    size = divide(tensor.size(last), num_partitions)
    chunks = torch.split(tensor, size, dim=last)
    if contiguous_split_chunks:
        return tuple(c.contiguous() for c in chunks)
    return chunks


def as_rows(x: torch.Tensor, width: int) -> torch.Tensor:
    """[..., width] -> [rows, width] with unit column stride (copies only if the layout forces it)."""
    x2 = x.reshape(-1, width)
    if x2.shape[1] > 1 and x2.stride(1) != 1:
        x2 = x2.contiguous()
    if x2.shape[0] > 1 and x2.stride(0) < x2.shape[1]:
        x2 = x2.contiguous()
    return x2
