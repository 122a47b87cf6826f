"""Optimiser step over the flat shard buffers (the harness step of benchmarks/rtp_benchmark.py:185-186:
clip_grad_value_ then optimizer.step), as one fused kernel launch per rotated layer.

For bf16 layers the optimiser owns an fp32 master copy of every flat shard buffer; the step updates
the master and rounds it into the bf16 weights the kernels read.  For fp32 layers the weights are
their own master.  Parameters outside rotated layers (LayerNorm) are flattened into one buffer (weights,
gradients, master) and updated by one launch.

`overlap_backward=True` applies a rotated layer's update as soon as that layer's backward has written its
gradients, on a second stream, so the memory-bound update runs under the matrix products of the layers
still to be differentiated.  The arithmetic is the same; what changes is WHEN the weights change: they are
already updated when backward() returns, and step() only waits for the updates and handles the remaining
parameters.  It therefore needs exactly one backward per step and every rotated layer applied once per
forward (gradient accumulation over several backwards raises).
"""
from __future__ import annotations

from typing import List, Optional

import torch
import torch.nn as nn

from . import ops, ring
from .module.collectives import ShardStore


class GradSink:
    """Persistent gradient slice of a parameter that is not part of a rotated layer."""

    __slots__ = ("view", "overwrite")

    def __init__(self, view: torch.Tensor):
        self.view = view
        self.overwrite = False  # True after zero_grad(): the next gradient replaces the slice's contents


class _FusedBinding:
    """Per rotated layer: where the fp32 parameters and their compute-dtype copy live, and which parameter ranges
    of which shards the weight-gradient products of the running backward pass have already updated."""

    def __init__(self, ctx: ops.FusedSgd, master: Optional[torch.Tensor]):
        self.ctx = ctx
        self.master = master       # [ws, numel] fp32, or None when the weights are fp32 themselves
        self.applied = {}          # (offset, length) -> set of shard indices
        self._last = None

    def bind(self, store: ShardStore, first: int, cnt: int, w_off: int, length: int):
        numel = store.numel
        if self.master is None:
            mptr, wptr = store.home.data_ptr() + (first * numel + w_off) * 4, 0
        else:
            mptr = self.master.data_ptr() + (first * numel + w_off) * 4
            wptr = store.home.data_ptr() + (first * numel + w_off) * store.home.element_size()
        self._last = ((w_off, length), range(first, first + cnt))
        self.ctx.missed = False
        return dict(sgd=self.ctx, sgd_master=mptr, sgd_weights=wptr)

    def confirm(self) -> None:
        key, shards = self._last
        self._last = None
        if self.ctx.missed:
            self.ctx.missed = False
            return
        self.applied.setdefault(key, set()).update(shards)


class RotatedSGD:
    """`fused_backward=True`: clip + SGD of every weight matrix of the rotated layers is applied in the epilogue of
    the weight-gradient product that computes its gradient (the gradient is consumed where it is produced: it is not
    written to memory unless keep_grads=True, and never read back); step() then only updates what no product
    covers -- biases, embedding tables, gate weights, LayerNorm.  Same arithmetic, bit-identical weights.  As with
    overlap_backward the weights change during backward(), and exactly one backward per step is allowed."""

    def __init__(self, model: nn.Module, lr: float, clip_value: float = 0.0, overlap_backward: bool = False,
                 fused_backward: bool = False, keep_grads: bool = False):
        self.lr = float(lr)
        self.clip_value = float(clip_value)
        self.overlap_backward = bool(overlap_backward)
        self.fused_backward = bool(fused_backward)
        if self.fused_backward and self.overlap_backward:
            raise ValueError("RotatedSGD: fused_backward and overlap_backward exclude each other")
        self.stores: List[ShardStore] = []
        rotated_params = set()
        for m in model.modules():
            st = getattr(m, "_store", None)
            if isinstance(st, ShardStore) and st not in self.stores:
                self.stores.append(st)
                for sm in st.modules:
                    rotated_params.update(id(p) for p in sm.parameters())
        self.other = [p for p in model.parameters() if id(p) not in rotated_params and p.requires_grad]
        self.masters = [None if st.home.dtype == torch.float32 else st.home.float() for st in self.stores]
        self._flatten_other()
        self._early = set()  # stores already updated during the current backward
        self._table = self._table_key = None
        self._table_params, self._table_dtype = 0, None
        self._aux = None
        self._rest_table = self._rest_key = None
        self._rest_params = 0
        if self.fused_backward:
            ctx = ops.FusedSgd(self.lr, self.clip_value, keep_grads, source=self)
            for st, master in zip(self.stores, self.masters):
                st.fused_sgd = _FusedBinding(ctx, master)
        if self.overlap_backward and self.stores:
            self._aux = torch.cuda.Stream(device=self.stores[0].home.device)  # default priority
            for st in self.stores:
                st.on_backward = self._announce
                st.on_grads_ready = self._update_early

    def _flatten_other(self) -> None:
        """Parameters outside rotated layers (LayerNorm) of one device and dtype are re-pointed into ONE flat
        buffer, their gradients into another (views attached as .grad for good) and their fp32 master into a
        third, so that the whole set is updated by one launch.  A parameter carries `_rtp_grad_sink`: a layer
        that computes its gradient with its own kernel (module/norm.py) may write it straight into the view."""
        self.flat = self.flat_grad = self.flat_master = None
        self.sinks: List[GradSink] = []
        if not self.other:
            return
        p0 = self.other[0]
        if any(p.device != p0.device or p.dtype != p0.dtype or not p.is_cuda for p in self.other):
            raise NotImplementedError("RotatedSGD: parameters outside rotated layers must share one CUDA device and dtype")
        sizes = [(p.numel() + 7) // 8 * 8 for p in self.other]  # 16-byte aligned slices
        total = sum(sizes)
        self.flat = torch.zeros(total, dtype=p0.dtype, device=p0.device)
        self.flat_grad = torch.zeros(total, dtype=p0.dtype, device=p0.device)
        off = 0
        with torch.no_grad():
            for p, n in zip(self.other, sizes):
                view = self.flat[off:off + p.numel()].view(p.shape)
                view.copy_(p.data)
                p.data = view
                gview = self.flat_grad[off:off + p.numel()].view(p.shape)
                sink = GradSink(gview)
                p._rtp_grad_sink = sink
                p.grad = gview
                self.sinks.append(sink)
                off += n
        self.flat_master = None if p0.dtype == torch.float32 else self.flat.float()

    @torch.no_grad()
    def reload_masters(self) -> None:
        """Re-read the fp32 master copies from the weights (after a checkpoint was loaded into the model)."""
        for st, master in zip(self.stores, self.masters):
            if master is not None:
                master.copy_(st.home)
        if self.flat_master is not None:
            self.flat_master.copy_(self.flat)

    def master_bytes(self) -> int:
        n = sum(m.numel() * 4 for m in self.masters if m is not None)
        return n + (self.flat_master.numel() * 4 if self.flat_master is not None else 0)

    def zero_grad(self) -> None:
        """Rotated layers keep their gradient views attached and overwrite them in the next backward (no
        per-parameter work); other parameters get .grad = None as torch does."""
        for st in self.stores:
            st.mark_overwrite()
        if self.flat_grad is not None:
            # one fill for all of them; the views stay attached, and a layer that writes its own gradient
            # overwrites instead of accumulating
            self.flat_grad.zero_()
            for p, sink in zip(self.other, self.sinks):
                sink.overwrite = True
                p.grad = sink.view

    def _update_store(self, st: ShardStore, master: Optional[torch.Tensor]) -> None:
        home, grads = st.home.view(-1), st.grads.view(-1)
        if master is None:
            ops.sgd_step(home, grads, None, self.lr, self.clip_value)
        else:
            ops.sgd_step(master.view(-1), grads, home, self.lr, self.clip_value)

    def _announce(self, st: ShardStore) -> None:
        """Backward-started callback of a store (runs at once, in the layer's backward)."""
        if id(st) in self._early:
            raise RuntimeError("RotatedSGD(overlap_backward=True): a rotated layer produced gradients twice before "
                               "step(); use overlap_backward=False for gradient accumulation or shared layers")
        self._early.add(id(st))

    def _fold_other_grads(self) -> None:
        for p, sink in zip(self.other, self.sinks):
            if p.grad is None:
                sink.view.zero_()  # someone dropped the gradient: nothing to apply
                p.grad = sink.view
            elif p.grad.data_ptr() != sink.view.data_ptr():
                sink.view.copy_(p.grad)  # someone attached a tensor of their own: fold it in
                p.grad = sink.view

    @torch.no_grad()
    def _update_early(self, st: ShardStore) -> None:
        """Gradient-ready callback of a store: update it on the second stream, after everything launched so far
        on the current stream (the layer's own products read the staged copy of the weights and are among it)."""
        self._aux.wait_stream(torch.cuda.current_stream(st.home.device))
        with torch.cuda.stream(self._aux):
            self._update_store(st, self.masters[self.stores.index(st)])

    def _multi_table(self):
        """Chunk table covering every buffer (rotated stores + the flat non-rotated parameters), rebuilt only when
        a buffer moved; None when a buffer cannot be updated this way."""
        items, dtype = [], None
        for st, master in zip(self.stores, self.masters):
            if st.grads is None:
                return None
            home, grads = st.home.view(-1), st.grads.view(-1)
            items.append((home, grads, None) if master is None else (master.view(-1), grads, home))
            dtype = home.dtype if dtype is None else dtype
            if home.dtype != dtype:
                return None
        if self.flat is not None:
            if dtype is not None and self.flat.dtype != dtype:
                return None
            dtype = self.flat.dtype
            items.append((self.flat, self.flat_grad, None) if self.flat_master is None
                         else (self.flat_master, self.flat_grad, self.flat))
        key = tuple(t.data_ptr() for it in items for t in it if t is not None)
        if key != self._table_key:
            self._table_key = key
            self._table = ops.sgd_chunk_table(items, items[0][0].device) if items else None
            self._table_params = sum(it[0].numel() for it in items)
            self._table_dtype = dtype
        return self._table

    def _step_rest(self) -> None:
        """fused_backward: update every parameter range the weight-gradient products of this pass did not."""
        items = []
        for st, master in zip(self.stores, self.masters):
            if st.grads is None:
                continue
            done = st.fused_sgd.applied
            for off, n in zip(st.offsets, st.numels):
                for s in range(st.world_size):
                    if s in done.get((off, n), ()):
                        continue
                    g, h = st.grads[s, off:off + n], st.home[s, off:off + n]
                    items.append((h, g, None) if master is None else (master[s, off:off + n], g, h))
            done.clear()
        if self.flat is not None:
            self._fold_other_grads()
            items.append((self.flat, self.flat_grad, None) if self.flat_master is None
                         else (self.flat_master, self.flat_grad, self.flat))
        if not items:
            return
        key = tuple(t.data_ptr() for it in items for t in it if t is not None)
        if key != self._rest_key:
            same = len({it[1].dtype for it in items}) == 1
            self._rest_key = key
            self._rest_table = ops.sgd_chunk_table(items, items[0][0].device) if same else None
            self._rest_params = sum(it[0].numel() for it in items)
        if self._rest_table is not None:
            ops.sgd_step_multi(self._rest_table, items[0][1].dtype, self.lr, self.clip_value, self._rest_params)
        else:
            for m, g, sh in items:
                ops.sgd_step(m, g, sh, self.lr, self.clip_value)

    @torch.no_grad()
    def step(self) -> None:
        if self.stores:
            ring.join_wgrad(self.stores[0].home.device)
        for st in self.stores:
            st.settle_overwrite()
        if self.fused_backward:
            self._step_rest()
            if self.stores:
                ring.fence(self.stores[0].home.device)
            return
        table = None if (self._early or self.overlap_backward) else self._multi_table()
        if table is not None:
            self._fold_other_grads()
            ops.sgd_step_multi(table, self._table_dtype, self.lr, self.clip_value, self._table_params)
            if self.stores:
                ring.fence(self.stores[0].home.device)
            return
        for st, master in zip(self.stores, self.masters):
            if st.grads is None or id(st) in self._early:
                continue
            self._update_store(st, master)
        if self._early:
            torch.cuda.current_stream(self.stores[0].home.device).wait_stream(self._aux)
            self._early.clear()
        if self.flat is not None:
            self._fold_other_grads()
            if self.flat_master is None:
                ops.sgd_step(self.flat, self.flat_grad, None, self.lr, self.clip_value)
            else:
                ops.sgd_step(self.flat_master, self.flat_grad, self.flat, self.lr, self.clip_value)
        if self.stores:
            ring.fence(self.stores[0].home.device)  # staging copies of the next step must see the new weights


class RotatedAdam(RotatedSGD):
    """The reference harness's optimiser (benchmarks/rtp_benchmark.py:41-42: torch.optim.Adam(lr 1e-3) after
    clip_grad_value_(0.05)) over the same flat buffers as RotatedSGD, fp32 moments beside the fp32 master: one launch
    over a device chunk table for all of them (or one per buffer where a buffer is not 16-byte aligned or the buffers
    differ in dtype).  The step count lives in device
    memory and the kernels form the bias corrections 1 - beta^step themselves, so step() may be recorded into a HIP
    graph and replayed (`steps` then only counts the eager calls)."""

    def __init__(self, model: nn.Module, lr: float = 1e-3, betas=(0.9, 0.999), eps: float = 1e-8,
                 weight_decay: float = 0.0, clip_value: float = 0.0):
        super().__init__(model, lr, clip_value, overlap_backward=False)
        self.betas, self.eps, self.weight_decay = (float(betas[0]), float(betas[1])), float(eps), float(weight_decay)
        self.steps = 0
        self._step_dev = None
        self._moments = {}
        self._adam_table = self._adam_key = None
        self._adam_params, self._adam_dtype = 0, None

    def state_bytes(self) -> int:
        return sum(m.numel() * 4 + v.numel() * 4 for m, v in self._moments.values())

    def _state(self, key, target: torch.Tensor):
        if key not in self._moments:
            self._moments[key] = (torch.zeros_like(target), torch.zeros_like(target))
        return self._moments[key]

    def _buffers(self):
        """(key, update target, gradients, weights to refresh or None) of every buffer that has gradients."""
        out = []
        for i, (st, master) in enumerate(zip(self.stores, self.masters)):
            if st.grads is None:
                continue
            home, grads = st.home.view(-1), st.grads.view(-1)
            out.append((i, home, grads, None) if master is None else (i, master.view(-1), grads, home))
        if self.flat is not None:
            out.append(("flat", self.flat, self.flat_grad, None) if self.flat_master is None
                       else ("flat", self.flat_master, self.flat_grad, self.flat))
        return out

    def _multi_adam_table(self, buffers):
        """Chunk table over every buffer, rebuilt only when a buffer moved; None when one launch cannot cover them."""
        if len({g.dtype for _, _, g, _ in buffers}) != 1:
            return None
        items = []
        for key, target, grads, shadow in buffers:
            m, v = self._state(key, target)
            items.append((target, grads, shadow, m, v))
        ptr_key = tuple(t.data_ptr() for it in items for t in it if t is not None)
        if ptr_key != self._adam_key:
            self._adam_key = ptr_key
            self._adam_table = ops.adam_chunk_table(items, items[0][0].device)
            self._adam_params = sum(it[0].numel() for it in items)
            self._adam_dtype = items[0][1].dtype
        return self._adam_table

    @torch.no_grad()
    def step(self) -> None:
        if self.stores:
            ring.join_wgrad(self.stores[0].home.device)
        for st in self.stores:
            st.settle_overwrite()
        if self._step_dev is None:
            buffers = [st.home for st in self.stores] + ([self.flat] if self.flat is not None else [])
            if not buffers:
                return
            self._step_dev = torch.zeros(1, dtype=torch.int64, device=buffers[0].device)
        self.steps += 1
        self._step_dev += 1
        if self.flat is not None:
            self._fold_other_grads()
        buffers = self._buffers()
        table = self._multi_adam_table(buffers) if buffers else None
        if table is not None:
            ops.adam_step_multi(table, self._adam_dtype, self._step_dev, self.lr, self.betas, self.eps,
                                self.weight_decay, self.clip_value, self._adam_params)
        else:
            for key, target, grads, shadow in buffers:
                m, v = self._state(key, target)
                ops.adam_step(target, grads, shadow, m, v, self._step_dev, self.lr, self.betas, self.eps,
                              self.weight_decay, self.clip_value)
        if self.stores:
            ring.fence(self.stores[0].home.device)  # staging copies of the next step must see the new weights
