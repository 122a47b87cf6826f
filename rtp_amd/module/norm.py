"""Residual add fused with LayerNorm for the post-LN decoder layers (the reference computes
norm1(x + sa_block(x)) / norm2(x + ff_block(x)) with two ATen calls each way,
rtp/models/transformer_lm_rtp.py:176-177).  The LayerNorm parameters stay ordinary nn.LayerNorm parameters."""
from __future__ import annotations

import os

import torch
import torch.nn as nn

from .. import ops
from .. import ring as _ring


class _DeferredParamGrads:
    """LayerNorm parameter gradients whose reduction waits for the end of the backward pass: each layer's backward
    leaves per-block partial sums in a buffer of its own, and ONE launch reduces all of them when autograd is done
    (nobody reads a parameter gradient earlier).  Only for gradients that go straight into an optimiser's persistent
    slices.  The device table of one set of buffers is built once and kept for good: a captured graph holds its
    address, and another model's backward pass must neither replace it nor force a host-to-device copy into a
    capture (the first, eager, step of a model builds its table)."""

    def __init__(self):
        self.pending = {}   # device index -> [(part, rows, cols, dgamma, dbeta, weight)]
        self.armed = {}     # device index -> id of the backward pass that has a callback queued
        self.tables = {}    # (device index, dtype, buffer addresses and shapes) -> (table, max_cols)

    def add(self, device: torch.device, item) -> bool:
        idx = device.index if device.index is not None else torch.cuda.current_device()
        task = torch._C._current_graph_task_id()
        if task < 0:
            return False  # not inside a backward pass: the caller reduces at once
        if self.armed.get(idx) != task:
            # leftovers of a pass that raised before its callback ran: its partial sums are dropped with it
            for it in self.pending.pop(idx, []):
                it[5]._rtp_ln_pending = False
            torch.autograd.Variable._execution_engine.queue_callback(lambda: self.flush(idx))
            self.armed[idx] = task
        self.pending.setdefault(idx, []).append(item)
        item[5]._rtp_ln_pending = True
        return True

    def flush(self, idx: int) -> None:
        self.armed.pop(idx, None)
        items = self.pending.pop(idx, [])
        if not items:
            return
        for it in items:
            it[5]._rtp_ln_pending = False
        by_dtype = {}
        for it in items:
            by_dtype.setdefault(it[3].dtype, []).append(it)
        for dtype, group in by_dtype.items():
            key = tuple((it[0].data_ptr(), it[1], it[2], it[3].data_ptr(), it[4].data_ptr() if it[4] is not None else 0)
                        for it in group)
            cached = self.tables.get((idx, dtype, key))
            if cached is None:
                cached = (ops.layernorm_final_table([it[:5] for it in group], group[0][0].device),
                          max(it[2] for it in group))
                self.tables[(idx, dtype, key)] = cached
            ops.layernorm_finalize(cached[0], dtype, cached[1])


_deferred = _DeferredParamGrads()
# reduce before the compute stream waits for the weight-gradient stream at the end of the pass, not after
_ring.run_before_join(_deferred.flush)
_DEFER = os.environ.get("RTP_LN_DEFER", "1") != "0"  # 0: reduce each LayerNorm's parameter gradients in its own backward


class _AddLayerNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, r, weight, bias, eps, x_grad_via_branch=False):
        x2, r2 = x.contiguous(), r.contiguous()
        cols = x2.shape[-1]
        rows = x2.numel() // cols
        z = torch.empty_like(x2)
        y = torch.empty_like(x2)
        mean = torch.empty(rows, dtype=torch.float32, device=x2.device)
        rstd = torch.empty(rows, dtype=torch.float32, device=x2.device)
        ops.add_layernorm_fwd(x2, r2, weight, bias, eps, z, y, mean, rstd)
        ctx.save_for_backward(z, weight, mean, rstd)
        ctx.bias = bias
        ctx.x_grad_via_branch = x_grad_via_branch
        return y

    @staticmethod
    def backward(ctx, dy):
        z, weight, mean, rstd = ctx.saved_tensors
        dz = torch.empty_like(z)
        bias = ctx.bias
        # An optimiser may have given the parameters persistent gradient slices (RotatedSGD): right after its
        # zero_grad() the kernel writes the gradients there and autograd gets nothing to accumulate.
        ws, bs = getattr(weight, "_rtp_grad_sink", None), getattr(bias, "_rtp_grad_sink", None) if bias is not None else None
        direct = ws is not None and ws.overwrite and (bias is None or (bs is not None and bs.overwrite))
        if direct:
            dgamma, dbeta = ws.view, (bs.view if bias is not None else None)
        else:
            dgamma = torch.empty_like(weight)
            dbeta = torch.empty_like(weight) if bias is not None else None
        if direct and not _DEFER:
            ops.layernorm_bwd(dy.contiguous(), z, weight, mean, rstd, dz, dgamma, dbeta)
        elif direct:
            # reduced together with every other LayerNorm's when the backward pass ends
            part = ops.layernorm_bwd_deferred(dy.contiguous(), z, weight, mean, rstd, dz,
                                              getattr(weight, "_rtp_ln_part", None))
            weight._rtp_ln_part = part
            done = _deferred.add(z.device, (part, z.numel() // z.shape[-1], z.shape[-1], dgamma, dbeta, weight))
            if not done:
                ops.layernorm_finalize(ops.layernorm_final_table(
                    [(part, z.numel() // z.shape[-1], z.shape[-1], dgamma, dbeta)], z.device), z.dtype, z.shape[-1])
        else:
            if getattr(weight, "_rtp_ln_pending", False):
                # the same LayerNorm applied twice: its first gradient must be in place before autograd adds this one
                _deferred.flush(z.device.index if z.device.index is not None else torch.cuda.current_device())
            ops.layernorm_bwd(dy.contiguous(), z, weight, mean, rstd, dz, dgamma, dbeta)
        if direct:
            ws.overwrite = False
            weight.grad = ws.view
            if bias is not None:
                bs.overwrite = False
                bias.grad = bs.view
            return (None if ctx.x_grad_via_branch else dz), dz, None, None, None, None
        return (None if ctx.x_grad_via_branch else dz), dz, dgamma, dbeta, None, None


def layer_norm_fusable(x: torch.Tensor, norm: nn.LayerNorm) -> bool:
    """Whether add_layer_norm(x, r, norm) takes the fused kernels for a branch output r shaped like x."""
    return bool(x.is_cuda and norm.elementwise_affine and len(norm.normalized_shape) == 1
                and norm.normalized_shape[0] == x.shape[-1] and norm.weight.dtype == x.dtype
                and ops.layernorm_supported(x.dtype, x.shape[-1]))


def add_layer_norm(x: torch.Tensor, r: torch.Tensor, norm: nn.LayerNorm, x_grad_via_branch: bool = False) -> torch.Tensor:
    """norm(x + r) in one kernel each way.  Rows must be whole 16-byte vectors, at most 1024 of them (8192 bf16 /
    4096 fp32 features), over the last dimension with an elementwise affine: anything else raises (there is no
    second implementation behind this one).
    x_grad_via_branch: r = f(x) was computed by a rotated layer called with residual_grad=True, whose backward
    already returns the residual part of x's gradient (added in the epilogue of its last product), so this
    function gives x no gradient of its own."""
    if not (layer_norm_fusable(x, norm) and x.shape == r.shape and x.dtype == r.dtype):
        from .._lib import RtpError
        raise RtpError(f"add_layer_norm: x {tuple(x.shape)} {x.dtype} on {x.device}, branch {tuple(r.shape)} {r.dtype}, "
                       f"LayerNorm{tuple(norm.normalized_shape)}: needs device tensors of one dtype, a LayerNorm over "
                       "the last dimension with elementwise affine, rows of whole 16-byte vectors (at most 1024)")
    return _AddLayerNormFn.apply(x, r, norm.weight, norm.bias, norm.eps, bool(x_grad_via_branch))
