"""Flat-parameter flyweight storage and shard bookkeeping for the rotated layers.

Mirrors the role of rtp/module/collectives.py:19-79 (set_full_param / allign_storage / allign_grad) and
:628-640 (zero_full_grads).  In the reference every rank owns ONE flat shard that `ws` flyweight modules
alias; here one process emulates all `ws` ranks' shards, so a layer owns a home tensor [ws, numel] in
which row s is the reference's `_full_param` of shard s, packed in named_parameters() order
(collectives.py:23-35), and a gradient tensor of the same shape whose row s is `_full_grad`.
"""
from __future__ import annotations

import contextlib
import os
from typing import Iterator, List, Optional, Sequence, Tuple

import torch
import torch.distributed as dist
import torch.nn as nn

_EMULATED: List[int] = []


@contextlib.contextmanager
def emulate_shards(world_size: int) -> Iterator[None]:
    """Layers constructed inside this context are built with `world_size` rotation shards on the one
    local device (rank 0), without a process group."""
    if world_size < 1:
        raise ValueError("emulate_shards: world_size must be >= 1")
    _EMULATED.append(int(world_size))
    try:
        yield
    finally:
        _EMULATED.pop()


def resolve_world(group=None) -> Tuple[int, int]:
    """(world_size, rank) for a layer under construction: the emulation context, else the environment
    variable RTP_EMULATED_SHARDS, else an initialised process group, else (1, 0).  The reference reads
    dist.get_world_size(group) / dist.get_rank(group) (rtp/module/linear.py:180-182)."""
    if _EMULATED:
        return _EMULATED[-1], 0
    env = os.environ.get("RTP_EMULATED_SHARDS")
    if env:
        return int(env), 0
    if dist.is_available() and dist.is_initialized():
        ws = dist.get_world_size(group)
        if ws > 1:
            raise NotImplementedError(
                "this build runs all shards of a layer on one GPU; a process group with world_size > 1 is "
                "the multi-GPU ring, which is not built")
        return 1, dist.get_rank(group)
    return 1, 0


class ShardStore:
    """Home storage of the `ws` flat shards of one layer plus their gradients.

    `shard_modules[s]` is an ordinary nn.Module holding shard s's parameters; after packing, every
    parameter's `.data` is a view into home[s] and (once a backward has run) its `.grad` is a view into
    grads[s].  `module._full_param` / `module._full_grad` name those rows, as in the reference.
    """

    def __init__(self, shard_modules: Sequence[nn.Module]):
        self.modules = list(shard_modules)
        names0 = [n for n, _ in self.modules[0].named_parameters()]
        self.names = names0
        self.shapes = [tuple(p.shape) for _, p in self.modules[0].named_parameters()]
        self.numels = [p.numel() for _, p in self.modules[0].named_parameters()]
        self.offsets = [0]
        for n in self.numels:
            self.offsets.append(self.offsets[-1] + n)
        self.numel = self.offsets[-1]
        for m in self.modules[1:]:
            shapes = [tuple(p.shape) for _, p in m.named_parameters()]
            if shapes != self.shapes:
                raise ValueError("all shards of a layer must have identical parameter shapes")
        self.home: Optional[torch.Tensor] = None
        self.grads: Optional[torch.Tensor] = None
        self._overwrite = set()
        self.stage_group = None  # set by ring.group_stores
        self.fused_sgd = None  # set by an optimiser that applies its update inside the weight-gradient products
        self.on_grads_ready = None  # optional callable(store): the layer's backward has written every gradient row
        self.on_backward = None     # optional callable(store): the layer's backward has started (called at once)
        self.pack()

    # -- storage ---------------------------------------------------------------------------------
    @property
    def world_size(self) -> int:
        return len(self.modules)

    def params(self, s: int) -> List[nn.Parameter]:
        return [p for _, p in self.modules[s].named_parameters()]

    def pack(self) -> None:
        """(Re)build home storage from the parameters' current values, device and dtype, and re-point
        every parameter at its slice (set_full_param + allign_storage)."""
        p0 = self.params(0)[0]
        home = torch.empty(self.world_size, max(self.numel, 1), dtype=p0.dtype, device=p0.device)
        with torch.no_grad():
            for s in range(self.world_size):
                for p, off, n in zip(self.params(s), self.offsets, self.numels):
                    home[s, off:off + n].copy_(p.data.reshape(-1))
        self.home = home
        self.grads = None
        self._overwrite.clear()
        if home.is_cuda:
            from .. import ring
            ring.fence(home.device)
        for s in range(self.world_size):
            self.modules[s]._full_param = home[s]
            self.modules[s]._full_grad = None
            for p, off, n, shape in zip(self.params(s), self.offsets, self.numels, self.shapes):
                p.data = home[s, off:off + n].view(shape)
                p.grad = None

    def views(self, flat: torch.Tensor) -> List[torch.Tensor]:
        """Parameter-shaped views of one flat shard (home row or staged copy)."""
        return [flat[off:off + n].view(shape) for off, n, shape in zip(self.offsets, self.numels, self.shapes)]

    # -- gradients -------------------------------------------------------------------------------
    def grad_views(self, s: int) -> Tuple[List[torch.Tensor], bool]:
        """Gradient slices of shard s and whether the caller must ACCUMULATE into them.

        If the shard's parameters carry no .grad (first backward, or after zero_grad(set_to_none=True))
        the slices are handed out for overwriting and attached as the parameters' .grad (allign_grad,
        collectives.py:75-79); otherwise they hold earlier gradients that must be added to."""
        if self.grads is None or self.grads.device != self.home.device or self.grads.dtype != self.home.dtype:
            self.grads = torch.empty_like(self.home)
            for m in self.modules:
                for p in m.parameters():
                    p.grad = None
        if s in self._overwrite:
            # zeroed by mark_overwrite(): the views are still attached, their contents are to be replaced
            self._overwrite.discard(s)
            if all(p.grad is not None for p in self.params(s)):
                return self.views(self.grads[s]), False
        params = self.params(s)
        views = self.views(self.grads[s])
        fresh = any(p.grad is None for p in params)
        if fresh:
            self.modules[s]._full_grad = self.grads[s]
            for p, v in zip(params, views):
                p.grad = v
            return views, False
        for p, v in zip(params, views):
            if p.grad.data_ptr() != v.data_ptr():
                # someone replaced .grad with their own tensor: fold it in and re-attach
                v.copy_(p.grad)
                p.grad = v
        return views, True

    def mark_overwrite(self) -> None:
        """Cheap zero_grad for a training loop: keep the .grad views attached and let the next backward
        overwrite every shard's gradient instead of accumulating into it."""
        if self.grads is not None:
            self._overwrite = set(range(self.world_size))

    def settle_overwrite(self) -> None:
        """Before an optimiser reads `grads`: a shard still marked for overwriting took no part in any backward since
        zero_grad (a layer that was not used), so its row holds the previous step's gradient; torch would apply a
        zero (or no) gradient, so the row is cleared."""
        if self.grads is not None:
            for s in sorted(self._overwrite):
                self.grads[s].zero_()
        self._overwrite.clear()

    def grad_runs(self, order: Sequence[int]):
        if self.on_backward is not None:
            self.on_backward(self)
        return self._grad_runs(order)

    def _grad_runs(self, order: Sequence[int]):
        """Attach gradient storage to every shard in `order` and return maximal runs (first, count,
        accumulate) of consecutive shards that share the same accumulate flag, so that a grouped kernel can
        write a whole run of gradient rows in one launch."""
        flags = {s: self.grad_views(s)[1] for s in order}
        ids = sorted(flags)
        runs, start = [], ids[0]
        for a, b in zip(ids, ids[1:] + [None]):
            if b is None or b != a + 1 or flags[b] != flags[a]:
                runs.append((start, a - start + 1, flags[a]))
                start = b
        return runs

    def grads_ready(self) -> None:
        """Called by a layer at the end of its backward, after the last kernel that writes `grads` has been
        launched on the current stream."""
        if self.on_grads_ready is not None:
            self.on_grads_ready(self)

    def weight_bytes(self) -> int:
        return self.world_size * self.numel * self.home.element_size()


def zero_full_grads(module: nn.Module) -> None:
    """Drop the gradients of every rotated layer under `module` (the intent of the reference's
    zero_full_grads, rtp/module/collectives.py:628-640)."""
    for m in module.modules():
        store = getattr(m, "_store", None)
        if isinstance(store, ShardStore):
            for sm in store.modules:
                sm._full_grad = None
                for p in sm.parameters():
                    p.grad = None


class RotatedLayer(nn.Module):
    """Base of the rotated layers: owns a ShardStore, keeps the flat storage intact across
    .to()/.cuda()/.float()/.bfloat16(), and provides the graph anchor that makes autograd call the
    layer's backward even when its input needs no gradient."""

    def _init_store(self, shard_modules: Sequence[nn.Module]) -> None:
        self.shards = nn.ModuleList(shard_modules)
        self._store = ShardStore(shard_modules)
        self.register_load_state_dict_post_hook(RotatedLayer._after_load_state_dict)
        self._anchor = torch.zeros((), dtype=torch.float32, device=self._store.home.device, requires_grad=True)

    @staticmethod
    def _after_load_state_dict(module, incompatible_keys) -> None:
        """load_state_dict copied new values into the home rows on the current stream: staged copies made from now
        on must wait for that."""
        home = module._store.home
        if home is not None and home.is_cuda:
            from .. import ring
            ring.fence(home.device)

    def _apply(self, fn, recurse=True):
        super()._apply(fn, recurse)
        # nn.Module._apply moved every parameter separately; restore the flat aliasing on the new
        # device / dtype (the reference's cuda()/to() overrides, rtp/module/linear.py:239-305).
        self._store.pack()
        self._anchor = torch.zeros((), dtype=torch.float32, device=self._store.home.device, requires_grad=True)
        return self

    def set_full_param(self, device=None, dtype=None):
        self.to(device=device, dtype=dtype)

    def weight_bytes(self) -> int:
        return self._store.weight_bytes()


def rotated_weight_bytes(module: nn.Module) -> int:
    """Resident bytes of all rotated layers' home storage under `module` (each shard counted once)."""
    return sum(m._store.weight_bytes() for m in module.modules() if isinstance(getattr(m, "_store", None), ShardStore))
