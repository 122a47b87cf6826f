"""State dicts in the reference's per-rank layout.

In the reference only a rank's own shard is a registered submodule of a rotated layer (the other flyweights sit in
a plain list, rtp/module/linear.py:187), so `model.state_dict()` on rank r holds that rank's slice under the home
attribute's name: `<layer>.linear.weight`, `<layer>.embedding.weight`, `<layer>.MultiheadAttention.in_proj_weight`,
`<layer>.experts.0...`, `<layer>.wg.weight`.  Here one process holds every shard (`<layer>.shards.<s>...`), and
the home attribute is an alias of shard `layer.rank`.  These helpers convert between the two, so that weights
trained here load into `world_size` reference ranks and back:

    rank_state_dict(model, r)          what the reference's rank r would save
    load_rank_state_dicts(model, sds)  load one such dict per rank into every shard held here

Tensors are returned as they are held (views of the flat shard buffers), like `nn.Module.state_dict()`.
"""
from __future__ import annotations

from collections import OrderedDict
from typing import Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn as nn

from .module.collectives import ShardStore


def _rotated_layers(model: nn.Module) -> List[Tuple[str, nn.Module]]:
    """(prefix, layer) of every rotated layer, longest prefixes first (a gate sits inside its MoE layer)."""
    out = []
    # every name of a module registered twice (a gate is a child of its decoder layer and of the MoE layer): the
    # state dict lists it under both
    for name, m in model.named_modules(remove_duplicate=False):
        if isinstance(getattr(m, "_store", None), ShardStore) and hasattr(m, "shards"):
            out.append((name + "." if name else "", m))
    return sorted(out, key=lambda t: -len(t[0]))


def _home_attr(layer: nn.Module) -> str:
    """Name under which the layer registers its own rank's shard (the attribute the reference registers)."""
    home = layer.shards[layer.rank]
    for name, child in layer.named_children():
        if name != "shards" and child is home:
            return name
    raise RuntimeError(f"{type(layer).__name__} does not expose its home shard as an attribute")


def _owner(layers, key: str) -> Optional[Tuple[str, nn.Module]]:
    for prefix, layer in layers:
        if key.startswith(prefix):
            return prefix, layer
    return None


def world_size_of(model: nn.Module) -> int:
    sizes = {len(layer.shards) for _, layer in _rotated_layers(model)}
    if len(sizes) > 1:
        raise ValueError(f"rotated layers of different world sizes in one model: {sorted(sizes)}")
    return sizes.pop() if sizes else 1


def rank_state_dict(model: nn.Module, rank: int) -> "OrderedDict[str, torch.Tensor]":
    """The state dict the reference's process `rank` holds for this model: its shard of every rotated layer under the
    home attribute's name, and every other parameter / buffer (replicated on all ranks) under its own name."""
    layers = _rotated_layers(model)
    for prefix, layer in layers:
        if not 0 <= rank < len(layer.shards):
            raise ValueError(f"rank {rank} outside 0..{len(layer.shards) - 1} of layer '{prefix[:-1]}'")
    out: "OrderedDict[str, torch.Tensor]" = OrderedDict()
    for key, tensor in model.state_dict().items():
        own = _owner(layers, key)
        if own is None:
            out[key] = tensor
            continue
        prefix, layer = own
        rest, home = key[len(prefix):], _home_attr(layer)
        if rest.startswith("shards."):
            s, tail = rest[len("shards."):].split(".", 1)
            if int(s) == rank:
                out[f"{prefix}{home}.{tail}"] = tensor
        elif not rest.startswith(home + "."):
            out[key] = tensor
    return out


def load_rank_state_dicts(model: nn.Module, dicts: Sequence[Dict[str, torch.Tensor]], strict: bool = True) -> None:
    """Load `world_size` per-rank state dicts (index = rank) into all shards held by `model`.  Replicated entries are
    taken from rank 0 (strict: they must agree on every rank).  Parameters are overwritten in place, so they stay
    views of the flat shard buffers; an optimiser with fp32 master copies must re-read them afterwards
    (`RotatedSGD.reload_masters()`)."""
    layers = _rotated_layers(model)
    ws = world_size_of(model)
    if len(dicts) != ws:
        raise ValueError(f"need one state dict per rank: got {len(dicts)}, world size {ws}")
    full: Dict[str, torch.Tensor] = {}
    for rank, sd in enumerate(dicts):
        for key, tensor in sd.items():
            own = _owner(layers, key)
            target = key
            if own is not None:
                prefix, layer = own
                rest, home = key[len(prefix):], _home_attr(layer)
                if rest.startswith(home + "."):
                    target = f"{prefix}shards.{rank}.{rest[len(home) + 1:]}"
            if target in full:
                if strict and not torch.equal(full[target].to(tensor.device), tensor):
                    raise ValueError(f"replicated entry '{key}' differs between rank 0 and rank {rank}")
                continue
            full[target] = tensor
    have = model.state_dict()
    aliases = set()
    for prefix, layer in layers:
        home = _home_attr(layer)
        aliases.update(k for k in have if k.startswith(f"{prefix}{home}."))
    missing, unexpected = model.load_state_dict(full, strict=False)
    missing = [k for k in missing if k not in aliases]
    if strict and (missing or unexpected):
        raise KeyError(f"load_rank_state_dicts: missing {missing}, unexpected {list(unexpected)}")
    if any(layer._store.home.is_cuda for _, layer in layers):
        from . import ring
        ring.fence(next(layer._store.home.device for _, layer in layers if layer._store.home.is_cuda))
