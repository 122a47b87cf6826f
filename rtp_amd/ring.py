"""Single-GPU shard rotation: the ring of rtp/module/collectives.py:202-317 collapsed onto one device.

Every shard of a layer lives exactly once in the layer's home storage.  A rotation visits the shards
in ring order; while step i computes on the shard sitting in one slot of a two-slot staging buffer, the
copy kernel streams the shard of step i+1 into the other slot on a side stream (what a neighbour's
isend/irecv does in the multi-GPU reference).  The staging buffer is shared by all layers of a device,
so the resident weight bytes are 1x the model plus two slots of the largest shard.
"""
from __future__ import annotations

import ctypes as C
from typing import Dict, List, Optional, Sequence

import torch

from . import _lib
from ._lib import check

_SLOT_ALIGN = 256
_ELEMENT_SIZE = {torch.float32: 4, torch.bfloat16: 2}


class DeviceRing:
    """Side stream + fencing events (native) and the two staging slots (a torch allocation)."""

    def __init__(self, device: torch.device):
        _lib.require_device()
        self.device = device
        handle = C.c_void_p()
        with torch.cuda.device(device):
            check(_lib.load().rtp_ring_create(C.byref(handle)))
        self._handle = handle
        self.slot_bytes = 0
        self.staging: Optional[torch.Tensor] = None
        self.peak_slot_bytes = 0

    def reserve(self, nbytes: int) -> None:
        if nbytes <= self.slot_bytes:
            return
        # Work queued on the side stream may still read the old slots.
        torch.cuda.synchronize(self.device)
        self.slot_bytes = (nbytes + _SLOT_ALIGN - 1) // _SLOT_ALIGN * _SLOT_ALIGN
        self.staging = torch.empty(2 * self.slot_bytes, dtype=torch.uint8, device=self.device)
        self.peak_slot_bytes = max(self.peak_slot_bytes, self.slot_bytes)

    def slot_ptr(self, slot: int) -> int:
        return self.staging.data_ptr() + slot * self.slot_bytes

    def slot_view(self, slot: int, numel: int, dtype: torch.dtype) -> torch.Tensor:
        nbytes = numel * _ELEMENT_SIZE[dtype]
        return self.staging[slot * self.slot_bytes: slot * self.slot_bytes + nbytes].view(dtype)

    def __del__(self):
        try:
            if self._handle:
                _lib.load().rtp_ring_destroy(self._handle)
        except Exception:
            pass


_rings: Dict[int, DeviceRing] = {}


def device_ring(device: torch.device) -> DeviceRing:
    idx = device.index if device.index is not None else torch.cuda.current_device()
    ring = _rings.get(idx)
    if ring is None:
        ring = _rings[idx] = DeviceRing(torch.device("cuda", idx))
    return ring


def staging_bytes(device: Optional[torch.device] = None) -> int:
    """Bytes held by the two staging slots on `device` (0 before the first rotation)."""
    if device is None:
        device = torch.device("cuda", torch.cuda.current_device())
    idx = device.index if device.index is not None else torch.cuda.current_device()
    ring = _rings.get(idx)
    return 0 if ring is None else 2 * ring.slot_bytes


class Rotation:
    """One pass over the shards of a layer, in the given order.

        rot = Rotation(home, order)          # home: [ws, numel] tensor, order: shard indices
        for i in range(len(order)):
            flat = rot.acquire(i)            # staged copy of shard order[i]; prefetches order[i+1]
            ... launch kernels that read `flat` on the current stream ...
            rot.release(i)
    """

    def __init__(self, home: torch.Tensor, order: Sequence[int]):
        if home.dim() != 2 or not home.is_contiguous():
            raise ValueError("Rotation: home must be a contiguous [shards, numel] tensor")
        self.home = home
        self.order = list(order)
        self.numel = home.shape[1]
        self.nbytes = self.numel * home.element_size()
        self.ring = device_ring(home.device)
        self.ring.reserve(self.nbytes)
        self.lib = _lib.load()
        self.stream = torch.cuda.current_stream(home.device).cuda_stream
        check(self.lib.rtp_ring_begin(self.ring._handle, self.stream))
        self._prefetch(0)

    def _prefetch(self, i: int) -> None:
        src = self.home.data_ptr() + self.order[i] * self.nbytes
        check(self.lib.rtp_ring_prefetch(self.ring._handle, i & 1, self.ring.slot_ptr(i & 1), src, self.nbytes))

    def acquire(self, i: int) -> torch.Tensor:
        if i + 1 < len(self.order):
            self._prefetch(i + 1)
        check(self.lib.rtp_ring_acquire(self.ring._handle, self.stream, i & 1))
        return self.ring.slot_view(i & 1, self.numel, self.home.dtype)

    def release(self, i: int) -> None:
        check(self.lib.rtp_ring_release(self.ring._handle, self.stream, i & 1))


def ring_order(rank: int, world_size: int, reverse: bool = False) -> List[int]:
    """Shard visited at step i: (rank + i) % ws going forward (rtp/module/linear.py:212); the backward
    pass walks the same sequence from its end (autograd reverses the step order)."""
    order = [(rank + i) % world_size for i in range(world_size)]
    return order[::-1] if reverse else order
