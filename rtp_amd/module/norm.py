"""Residual add fused with LayerNorm for the post-LN decoder layers (the reference computes
norm1(x + sa_block(x)) / norm2(x + ff_block(x)) with two ATen calls each way,
rtp/models/transformer_lm_rtp.py:176-177).  The LayerNorm parameters stay ordinary nn.LayerNorm parameters."""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import ops


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
    """norm(x + r).  Fused on the device when the row length qualifies, else the two torch calls.
    x_grad_via_branch: r = f(x) was computed by a rotated layer called with residual_grad=True, whose backward
    already returns the residual part of x's gradient (added in the epilogue of its last product), so this
    function gives x no gradient of its own.  Only valid when layer_norm_fusable(x, norm)."""
    fused = layer_norm_fusable(x, norm) and x.shape == r.shape and x.dtype == r.dtype
    if not fused:
        if x_grad_via_branch:
            raise RuntimeError("add_layer_norm: x_grad_via_branch needs the fused path (check layer_norm_fusable)")
        return norm(x + r)
    return _AddLayerNormFn.apply(x, r, norm.weight, norm.bias, norm.eps, bool(x_grad_via_branch))
