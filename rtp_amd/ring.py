"""Single-GPU shard rotation: the ring of rtp/module/collectives.py:202-317 collapsed onto one device.

Every shard of a layer lives exactly once in the layer's home storage.  A rotation visits the shards in
ring order, `window` shards at a time: while the kernels of one window read its shards from one slot of a
two-slot staging buffer, the copy kernel streams the next window -- of this layer, or the first window
of the next layer -- into the other slot on a side stream (what a neighbour's isend/irecv does in the
multi-GPU reference).  window = 1 is the reference's step-by-step schedule; a larger window lets one
grouped kernel launch cover several ring steps.  The staging buffer is shared by all layers of a device,
so the resident weight bytes are 1x the model plus two slots of the largest window.
"""
from __future__ import annotations

import ctypes as C
import os
import weakref
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import check

_SLOT_ALIGN = 256
_ELEMENT_SIZE = {torch.float32: 4, torch.bfloat16: 2}
_window: Optional[int] = None


def set_rotation_window(window: Optional[int]) -> None:
    """Ring steps staged and computed together (None = all shards of a layer, 1 = one shard per step)."""
    global _window
    if window is not None and window < 1:
        raise ValueError("rotation window must be >= 1")
    _window = window


def rotation_window() -> Optional[int]:
    return _window


# ---- where a shard waits for its turn ----------------------------------------------------------------
# "direct" (default): the products read every shard straight from its home row.  The double buffer of the rotation is
# then the LDS stage ring inside the product kernel: its loader waves stream the tiles of the next (shard, tile) work
# item from home into LDS while the MFMA waves work on the current one, so no second copy of a shard ever exists in
# HBM (resident weights = 1.0x the model) and the weights cross the memory bus once per pass.
# "staged": every window of shards is first copied home -> staging slot by the copy kernel on the side stream while
# the previous window computes (two slots in HBM; the transport a multi-GPU ring would fill from its neighbour).
_mode = os.environ.get("RTP_ROTATION", "direct")


def set_rotation_mode(mode: str) -> None:
    global _mode
    if mode not in ("direct", "staged"):
        raise ValueError("rotation mode must be 'direct' or 'staged'")
    _mode = mode


def rotation_mode() -> str:
    return _mode


# ---- the next layer's shards arrive while the current layer computes (direct mode) ------------------------
# Read from their home rows, a layer's weights are touched once per pass, so at their turn they come from HBM, and the
# products' load pipeline (a few K slabs in flight) does not cover that latency: measured on the LM's shapes, a
# product takes 15 - 30 % longer on weights from HBM than on weights that sit in the 256 MiB memory-side cache.  With
# the switch on, a rotation that starts hands the home rows of the layer that followed this one the last time round
# to its own first product (rtp_gemm_warm_next), whose workgroups request them at their start: the one-GPU form of
# the reference's irecv of the next shard during the current step (rtp/module/linear.py:211-220).  Which layer
# follows is learned from the order of the rotations (keyed by the last two layers, so the forward and the backward
# order are told apart); nothing depends on the guess being right.  No second stream is involved: a read pass on a
# side stream (rtp_cache_warm) warms as well, but every fork of the compute stream costs ~5 us, more than it gains.
_warm_ahead = os.environ.get("RTP_WARM_AHEAD", "1") == "1"
_warm_hist: Dict[int, Tuple[int, int]] = {}
_warm_next: Dict[Tuple[int, int, int], "weakref.ref"] = {}  # (device, layer before, layer) -> the layer that followed
_warm_pending: Dict[int, Optional[torch.Tensor]] = {}       # the tensor a hint not yet launched may point into


def set_warm_ahead(on: bool) -> None:
    global _warm_ahead
    _warm_ahead = bool(on)
    _warm_hist.clear()
    _warm_next.clear()
    if _warm_pending:
        _lib.load().rtp_gemm_warm_next(None, 0)
        _warm_pending.clear()


def warm_ahead() -> bool:
    return _warm_ahead


def _warm_step(home: torch.Tensor) -> None:
    """A rotation over `home` starts (direct mode).  The table holds weak references, so it keeps no model alive; the
    one tensor a pending hint points into is held until the next rotation replaces or withdraws the hint (the
    library drops a hint with the first product launched after it, carried or not)."""
    idx = home.device.index if home.device.index is not None else torch.cuda.current_device()
    prev, cur = _warm_hist.get(idx, (0, 0))
    here = home.data_ptr()
    if here == cur:
        return  # the same layer again (its backward pass right after its forward pass)
    if len(_warm_next) > 4096:
        _warm_next.clear()  # far more layers than any model rotates: stale entries of models long gone
    _warm_next[(idx, prev, cur)] = weakref.ref(home)
    _warm_hist[idx] = (cur, here)
    ref = _warm_next.get((idx, cur, here))
    nxt = ref() if ref is not None else None
    lib = _lib.load()
    if nxt is not None and nxt.is_cuda and nxt.data_ptr() != here:
        _warm_pending[idx] = nxt
        check(lib.rtp_gemm_warm_next(nxt.data_ptr(), nxt.numel() * nxt.element_size()))
    elif _warm_pending.get(idx) is not None:
        _warm_pending[idx] = None
        check(lib.rtp_gemm_warm_next(None, 0))


# ---- weight gradients on a second stream -----------------------------------------------------------
# A layer's weight / bias gradients are needed only by the optimiser, while its input gradient is needed by
# the next layer of the backward pass.  With the switch on, the gradient products of the parameters are
# launched on a second stream (after everything already launched on the compute stream), so they fill the
# launch gaps and tails of the input-gradient chain.  The compute stream rejoins at the end of the backward
# pass (an autograd engine callback) and in join_wgrad().  Tensors produced inside `fn` on the second stream
# (workspaces) are allocated and freed there.
_wgrad_overlap = os.environ.get("RTP_WGRAD_OVERLAP", "0") == "1"
_wgrad_streams: Dict[int, "torch.cuda.Stream"] = {}
_wgrad_dirty: Dict[int, bool] = {}
_wgrad_keepalive: Dict[int, list] = {}
_wgrad_pending: Dict[int, list] = {}
_WGRAD_BATCH = int(os.environ.get("RTP_WGRAD_BATCH", "9"))  # layers per fork (three decoder blocks; measured optimum)


def set_wgrad_overlap(on: bool) -> None:
    global _wgrad_overlap
    _wgrad_overlap = bool(on)


def wgrad_overlap() -> bool:
    return _wgrad_overlap


# Work of the compute stream that is due at the end of a backward pass and does not depend on the second stream (the
# one-launch reduction of the LayerNorm parameter gradients): launched before the compute stream starts waiting for
# the second stream, it runs beside the last weight-gradient products instead of after them.
_before_join: List = []


def run_before_join(fn) -> None:
    """Register fn(device index), called at the start of every join_wgrad."""
    if fn not in _before_join:
        _before_join.append(fn)


def join_wgrad(device: Optional[torch.device] = None) -> None:
    """Launch what is still deferred and make the current stream wait for the parameter-gradient work on the
    second stream."""
    idx = torch.cuda.current_device() if device is None or device.index is None else device.index
    for fn in _before_join:
        fn(idx)
    _flush_wgrad(idx)
    _wgrad_task.pop(idx, None)
    if _wgrad_dirty.get(idx):
        torch.cuda.current_stream(idx).wait_stream(_wgrad_streams[idx])
        _wgrad_dirty[idx] = False
        _wgrad_keepalive.get(idx, []).clear()


def _flush_wgrad(idx: int) -> None:
    pending = _wgrad_pending.get(idx)
    if not pending:
        return
    aux = _wgrad_streams.get(idx)
    if aux is None:
        aux = _wgrad_streams[idx] = torch.cuda.Stream(device=idx)  # default priority
        _install_optimizer_hooks()
    aux.wait_stream(torch.cuda.current_stream(idx))
    _wgrad_dirty[idx] = True
    with torch.cuda.stream(aux):
        for fn in pending:
            fn()
    pending.clear()


_wgrad_task: Dict[int, int] = {}  # device -> id of the backward pass whose end-of-pass join is armed


def _abandon_wgrad(idx: int) -> None:
    """A backward pass ended without its join (it raised part-way): what it deferred is dropped unlaunched -- its
    gradients are incomplete anyway -- and what it already launched on the second stream is waited for."""
    _wgrad_pending.get(idx, []).clear()
    if _wgrad_dirty.get(idx):
        torch.cuda.current_stream(idx).wait_stream(_wgrad_streams[idx])
        _wgrad_dirty[idx] = False
    _wgrad_keepalive.get(idx, []).clear()
    _wgrad_task.pop(idx, None)


def run_wgrad(device: torch.device, fn, tensors: Sequence[torch.Tensor] = ()) -> None:
    """Run `fn`, which launches a layer's parameter-gradient kernels.  Without the overlap switch: now, on the
    current stream.  With it: deferred until `_WGRAD_BATCH` layers have queued up (or the backward pass ends) and
    then on the second stream -- one fork of the compute stream per batch, since every fork and join between
    two hardware queues idles the compute stream for several microseconds.  `tensors` are the operands `fn`
    reads that autograd may free or reuse when the layer's backward returns.  The join at the end of the pass is
    armed once per backward pass (by the id of the autograd engine's running task); outside a backward pass the
    launches happen at once, on the current stream."""
    task = torch._C._current_graph_task_id() if _wgrad_overlap else -1
    if task < 0:
        fn()
        return
    idx = device.index if device.index is not None else torch.cuda.current_device()
    if _wgrad_task.get(idx) != task:
        if idx in _wgrad_task or _wgrad_pending.get(idx) or _wgrad_dirty.get(idx):
            _abandon_wgrad(idx)  # leftovers of a pass that never reached its join
        torch.autograd.Variable._execution_engine.queue_callback(lambda: join_wgrad(torch.device("cuda", idx)))
        _wgrad_task[idx] = task
    # Hold the operands until the compute stream has rejoined: while a second reference exists autograd
    # neither frees a gradient buffer nor accumulates into it in place under the second stream's reads.
    _wgrad_keepalive.setdefault(idx, []).extend(t for t in tensors if t is not None)
    _wgrad_pending.setdefault(idx, []).append(fn)
    if len(_wgrad_pending[idx]) >= _WGRAD_BATCH:
        _flush_wgrad(idx)


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
        self.next_slot = 0
        self.epoch = 0
        self.holder: List[Optional["StageGroup"]] = [None, None]
        self.retired: List[torch.Tensor] = []

    def reserve(self, nbytes: int) -> None:
        if nbytes <= self.slot_bytes:
            return
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("rotation staging slots have to grow while a graph is being captured: run one eager "
                               "step of every model first, so that the slots have their final size")
        # Work queued on the side stream may still read the old slots.
        torch.cuda.synchronize(self.device)
        if self.staging is not None:
            # a graph captured earlier holds addresses inside the old slots and may be replayed again: the memory
            # stays allocated (and nobody else's) for the life of the process
            self.retired.append(self.staging)
        self.slot_bytes = (nbytes + _SLOT_ALIGN - 1) // _SLOT_ALIGN * _SLOT_ALIGN
        self.staging = torch.empty(2 * self.slot_bytes, dtype=torch.uint8, device=self.device)
        self.fence()

    def take_slot(self, stream: int = 0) -> int:
        """Next staging slot, alternating, but never one that a stage group still reads (its remaining members
        have not rotated yet); if both are held, the older group is dropped and will stage again."""
        for cand in (self.next_slot, self.next_slot ^ 1):
            g = self.holder[cand]
            if g is None or g.slot != cand or not g.remaining:
                self.holder[cand] = None
                self.next_slot = cand ^ 1
                return cand
        cand = self.next_slot
        g = self.holder[cand]
        check(_lib.load().rtp_ring_release(self._handle, stream, cand))
        g.slot = None
        self.holder[cand] = None
        self.next_slot = cand ^ 1
        return cand

    def fence(self) -> None:
        """Home storage was written by work queued on the current stream: the next staging copy waits."""
        self.epoch += 1  # staged copies made before this point are stale
        check(_lib.load().rtp_ring_fence(self._handle, torch.cuda.current_stream(self.device).cuda_stream))

    def __del__(self):
        try:
            if self._handle:
                _lib.load().rtp_ring_destroy(self._handle)
        except Exception:
            pass


_rings: Dict[int, DeviceRing] = {}
_hooks_installed = False


def _install_optimizer_hooks() -> None:
    """Any torch.optim optimiser rewrites home shards in place: before its step the deferred weight gradients are
    joined, after it every ring is fenced, so that the next staging copy is ordered after the update without the
    caller having to know about the side stream (RotatedSGD / RotatedAdam do the same themselves)."""
    global _hooks_installed
    if _hooks_installed:
        return
    _hooks_installed = True
    from torch.optim.optimizer import register_optimizer_step_post_hook, register_optimizer_step_pre_hook

    def pre(optimizer, args, kwargs):
        for idx in list(_wgrad_pending) + list(_wgrad_dirty):
            join_wgrad(torch.device("cuda", idx))

    def post(optimizer, args, kwargs):
        for r in _rings.values():
            with torch.cuda.device(r.device):
                r.fence()

    register_optimizer_step_pre_hook(pre)
    register_optimizer_step_post_hook(post)


def device_ring(device: torch.device) -> DeviceRing:
    idx = device.index if device.index is not None else torch.cuda.current_device()
    ring = _rings.get(idx)
    if ring is None:
        ring = _rings[idx] = DeviceRing(torch.device("cuda", idx))
        _install_optimizer_hooks()
    return ring


def fence(device: Optional[torch.device] = None) -> None:
    """Call after modifying rotated weights in place with your own kernels (optimizer step, weight load)
    and after ending a HIP-graph capture: orders the next staging copy after that work."""
    if device is None:
        device = torch.device("cuda", torch.cuda.current_device())
    idx = device.index if device.index is not None else torch.cuda.current_device()
    if idx in _rings:
        _rings[idx].fence()


def staging_bytes(device: Optional[torch.device] = None) -> int:
    """Bytes held by the two staging slots on `device` (0 before the first rotation)."""
    if device is None:
        device = torch.device("cuda", torch.cuda.current_device())
    idx = device.index if device.index is not None else torch.cuda.current_device()
    ring = _rings.get(idx)
    return 0 if ring is None else 2 * ring.slot_bytes


Run = Tuple[torch.Tensor, int, int]  # (staged [count, numel] view, first shard index, count)


class StageGroup:
    """Layers whose rotations always run back to back (the rotated layers of one decoder block).  When a whole
    layer is staged per rotation (window = all), the first member to rotate stages every member into one slot
    and the others find their shards there: one wait on the copy stream and one slot hand-back per block and
    pass instead of one per layer -- each is a dependency between two hardware queues, which costs several
    microseconds of idle compute stream even when the copy finished long ago."""

    def __init__(self, stores: Sequence[object]):
        self.stores = list(stores)  # objects with a `.home` [shards, numel] tensor
        for st in self.stores:
            st.stage_group = self
        self.slot: Optional[int] = None
        self.epoch = -1
        self.offsets: List[int] = []
        self.remaining: set = set()
        self.acquired = False

    def total_bytes(self) -> int:
        return sum((st.home.numel() * st.home.element_size() + _SLOT_ALIGN - 1) // _SLOT_ALIGN * _SLOT_ALIGN
                   for st in self.stores)

    def usable(self, home: torch.Tensor) -> bool:
        return all(st.home is not None and st.home.device == home.device for st in self.stores)

    def member(self, home: torch.Tensor) -> int:
        for i, st in enumerate(self.stores):
            if st.home is home:
                return i
        return -1

    def stage(self, ring: "DeviceRing", lib, stream: int) -> None:
        """Copy every member's shards into one slot (on the ring's copy stream)."""
        ring.reserve(self.total_bytes())
        if self.slot is not None and self.epoch == ring.epoch and self.remaining:
            lib.rtp_ring_release(ring._handle, stream, self.slot)  # an unfinished pass: hand its slot back first
            self.slot = None
        self.remaining = set()
        self.slot = ring.take_slot(stream)
        ring.holder[self.slot] = self
        self.epoch = ring.epoch
        self.offsets, off = [], 0
        base = ring.staging.data_ptr() + self.slot * ring.slot_bytes
        for st in self.stores:
            nb = st.home.numel() * st.home.element_size()
            check(lib.rtp_ring_prefetch(ring._handle, stream, self.slot, base + off, st.home.data_ptr(), nb))
            self.offsets.append(off)
            off += (nb + _SLOT_ALIGN - 1) // _SLOT_ALIGN * _SLOT_ALIGN
        self.remaining = set(range(len(self.stores)))
        self.acquired = False


def group_stores(stores: Sequence[object]) -> StageGroup:
    """Declare that the layers owning `stores` (ShardStore objects) always rotate one after another.
    RTP_STAGE_GROUPS=0 in the environment turns the grouping off (every layer stages for itself)."""
    if os.environ.get("RTP_STAGE_GROUPS", "1") == "0":
        return None
    return StageGroup(stores)


class Rotation:
    """One pass over the shards of a layer in ring order, `window` ring steps at a time.

        rot = Rotation(home, order)            # home: [ws, numel], order: shard index per ring step
        for j in range(rot.steps):
            for staged, first, count in rot.acquire(j):   # staged[i] is a copy of home[first + i]
                ... launch kernels that read `staged` on the current stream ...
            rot.release(j)

    A window's shards are staged in ascending index order as runs of consecutive shards, so a grouped
    kernel can address them with one stride.
    """

    def __init__(self, home: torch.Tensor, order: Sequence[int], window: Optional[int] = None,
                 group: Optional[StageGroup] = None):
        if home.dim() != 2 or not home.is_contiguous():
            raise ValueError("Rotation: home must be a contiguous [shards, numel] tensor")
        self.home = home
        self.group = None
        self.numel = home.shape[1]
        self.nbytes = self.numel * home.element_size()
        order = list(order)
        w = window if window is not None else _window
        w = len(order) if w is None else max(1, min(int(w), len(order)))
        self.windows: List[List[Tuple[int, int]]] = []
        for i in range(0, len(order), w):
            ids = sorted(order[i:i + w])
            runs, start = [], ids[0]
            for a, b in zip(ids, ids[1:] + [None]):
                if b is None or b != a + 1:
                    runs.append((start, a - start + 1))
                    start = b
            self.windows.append(runs)
        self.steps = len(self.windows)
        self.direct = _mode == "direct"
        if self.direct:
            if _warm_ahead:
                _warm_step(home)
            return
        self.ring = device_ring(home.device)
        self.lib = _lib.load()
        self.stream = torch.cuda.current_stream(home.device).cuda_stream
        self.slots = [None] * self.steps
        if group is not None and self.steps == 1 and w == home.shape[0] and group.usable(home):
            self.member = group.member(home)
            if self.member >= 0:
                self.group = group
                if group.slot is None or group.epoch != self.ring.epoch or self.member not in group.remaining:
                    group.stage(self.ring, self.lib, self.stream)
                return
        self.ring.reserve(w * self.nbytes)
        self._prefetch(0)

    def _prefetch(self, j: int) -> None:
        slot = self.slots[j] = self.ring.take_slot(self.stream)
        dst = self.ring.staging.data_ptr() + slot * self.ring.slot_bytes
        for first, count in self.windows[j]:
            check(self.lib.rtp_ring_prefetch(self.ring._handle, self.stream, slot, dst,
                                             self.home.data_ptr() + first * self.nbytes, count * self.nbytes))
            dst += count * self.nbytes

    def acquire(self, j: int) -> List[Run]:
        if self.direct:
            return [(self.home[first:first + count], first, count) for first, count in self.windows[j]]
        if self.group is not None:
            g = self.group
            if not g.acquired:
                check(self.lib.rtp_ring_acquire(self.ring._handle, self.stream, g.slot))
                g.acquired = True
            off = g.slot * self.ring.slot_bytes + g.offsets[self.member]
            nb = self.home.shape[0] * self.nbytes
            staged = self.ring.staging[off:off + nb].view(self.home.dtype).view(self.home.shape[0], self.numel)
            return [(staged, 0, self.home.shape[0])]
        if j + 1 < self.steps:
            self._prefetch(j + 1)
        slot = self.slots[j]
        check(self.lib.rtp_ring_acquire(self.ring._handle, self.stream, slot))
        out, off = [], slot * self.ring.slot_bytes
        for first, count in self.windows[j]:
            nb = count * self.nbytes
            out.append((self.ring.staging[off:off + nb].view(self.home.dtype).view(count, self.numel), first, count))
            off += nb
        return out

    def release(self, j: int) -> None:
        if self.direct:
            return
        if self.group is not None:
            g = self.group
            g.remaining.discard(self.member)
            if not g.remaining and g.slot is not None:  # the last member of the block: hand the slot back
                check(self.lib.rtp_ring_release(self.ring._handle, self.stream, g.slot))
                self.ring.holder[g.slot] = None
                g.slot = None
            return
        check(self.lib.rtp_ring_release(self.ring._handle, self.stream, self.slots[j]))


def ring_order(rank: int, world_size: int, reverse: bool = False) -> List[int]:
    """Shard visited at step i: (rank + i) % ws going forward (rtp/module/linear.py:212); the backward
    pass walks the same sequence from its end (autograd reverses the step order)."""
    order = [(rank + i) % world_size for i in range(world_size)]
    return order[::-1] if reverse else order
