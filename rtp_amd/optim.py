"""Optimiser step over the flat shard buffers (the harness step of benchmarks/rtp_benchmark.py:185-186:
clip_grad_value_ then optimizer.step), as one fused kernel launch per rotated layer.

For bf16 layers the optimiser owns an fp32 master copy of every flat shard buffer; the step updates
the master and rounds it into the bf16 weights the kernels read.  For fp32 layers the weights are
their own master.  Parameters outside rotated layers (LayerNorm) are flattened the same way.

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


class RotatedSGD:
    def __init__(self, model: nn.Module, lr: float, clip_value: float = 0.0, overlap_backward: bool = False):
        self.lr = float(lr)
        self.clip_value = float(clip_value)
        self.overlap_backward = bool(overlap_backward)
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
        self.other_masters = [None if p.dtype == torch.float32 else p.detach().float().clone() for p in self.other]
        self._early = set()  # stores already updated during the current backward
        self._aux = None
        if self.overlap_backward and self.stores:
            self._aux = torch.cuda.Stream(device=self.stores[0].home.device)  # default priority
            for st in self.stores:
                st.on_grads_ready = self._update_early

    def master_bytes(self) -> int:
        n = sum(m.numel() * 4 for m in self.masters if m is not None)
        return n + sum(m.numel() * 4 for m in self.other_masters if m is not None)

    def zero_grad(self) -> None:
        """Rotated layers keep their gradient views attached and overwrite them in the next backward (no
        per-parameter work); other parameters get .grad = None as torch does."""
        for st in self.stores:
            st.mark_overwrite()
        for p in self.other:
            p.grad = None

    def _update_store(self, st: ShardStore, master: Optional[torch.Tensor]) -> None:
        home, grads = st.home.view(-1), st.grads.view(-1)
        if master is None:
            ops.sgd_step(home, grads, None, self.lr, self.clip_value)
        else:
            ops.sgd_step(master.view(-1), grads, home, self.lr, self.clip_value)

    @torch.no_grad()
    def _update_early(self, st: ShardStore) -> None:
        """Gradient-ready callback of a store: update it on the second stream, after everything launched so far
        on the current stream (the layer's own products read the staged copy of the weights and are among it)."""
        if id(st) in self._early:
            raise RuntimeError("RotatedSGD(overlap_backward=True): a rotated layer produced gradients twice before "
                               "step(); use overlap_backward=False for gradient accumulation or shared layers")
        self._early.add(id(st))
        self._aux.wait_stream(torch.cuda.current_stream(st.home.device))
        with torch.cuda.stream(self._aux):
            self._update_store(st, self.masters[self.stores.index(st)])

    @torch.no_grad()
    def step(self) -> None:
        if self.stores:
            ring.join_wgrad(self.stores[0].home.device)
        for st, master in zip(self.stores, self.masters):
            if st.grads is None or id(st) in self._early:
                continue
            self._update_store(st, master)
        if self._early:
            torch.cuda.current_stream(self.stores[0].home.device).wait_stream(self._aux)
            self._early.clear()
        for p, master in zip(self.other, self.other_masters):
            if p.grad is None:
                continue
            g = p.grad.contiguous().view(-1)
            if master is None:
                ops.sgd_step(p.data.view(-1), g, None, self.lr, self.clip_value)
            else:
                ops.sgd_step(master.view(-1), g, p.data.view(-1), self.lr, self.clip_value)
        if self.stores:
            ring.fence(self.stores[0].home.device)  # staging copies of the next step must see the new weights
