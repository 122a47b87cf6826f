"""Fused residual add + LayerNorm against torch's fp32 layer_norm(x + r) on the same inputs."""
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from gpu_util import DEV, assert_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,cols", [(37, 2048), (5, 64), (1024, 512), (3, 8), (9, 1288)])
def test_add_layer_norm_matches_torch(dtype, rows, cols):
    from rtp_amd import ops
    from rtp_amd.module.norm import add_layer_norm
    assert ops.layernorm_supported(dtype, cols)
    gen = torch.Generator().manual_seed(rows * 7 + cols)
    x = torch.randn(rows, cols, generator=gen).to(dtype)
    r = torch.randn(rows, cols, generator=gen).to(dtype)
    g = torch.randn(rows, cols, generator=gen).to(dtype)
    norm = nn.LayerNorm(cols)
    with torch.no_grad():
        norm.weight.copy_(torch.rand(cols, generator=gen) + 0.5)
        norm.bias.copy_(torch.randn(cols, generator=gen) * 0.1)
    norm = norm.to(dtype)
    # reference in fp32 from the same (rounded) inputs; z is rounded to dtype like a separate add
    xr, rr = x.float().clone().requires_grad_(), r.float().clone().requires_grad_()
    w, b = norm.weight.detach().float().requires_grad_(), norm.bias.detach().float().requires_grad_()
    z = (xr + rr).to(dtype).float()
    ref = F.layer_norm(z, (cols,), w, b, norm.eps)
    ref.backward(g.float())
    dev_norm = nn.LayerNorm(cols).to(dtype)
    dev_norm.load_state_dict(norm.state_dict())
    dev_norm = dev_norm.to(DEV)
    xd, rd = x.detach().to(DEV).requires_grad_(), r.detach().to(DEV).requires_grad_()
    y = add_layer_norm(xd.view(rows, 1, cols), rd.view(rows, 1, cols), dev_norm).view(rows, cols)
    y.backward(g.detach().to(DEV))
    assert_close(y, ref, dtype, "y")
    assert_close(xd.grad, xr.grad, dtype, "dx")
    assert_close(rd.grad, rr.grad, dtype, "dr")
    assert_close(dev_norm.weight.grad, w.grad, dtype, "dgamma")
    assert_close(dev_norm.bias.grad, b.grad, dtype, "dbeta")


def test_add_layer_norm_falls_back_for_unsupported_rows():
    from rtp_amd import ops
    from rtp_amd.module.norm import add_layer_norm
    assert not ops.layernorm_supported(torch.float32, 4100)
    assert not ops.layernorm_supported(torch.bfloat16, 36)
    assert not ops.layernorm_supported(torch.float32, 38)
    norm = nn.LayerNorm(38).to(DEV)
    x = torch.randn(4, 38, device=DEV)
    r = torch.randn(4, 38, device=DEV)
    assert torch.equal(add_layer_norm(x, r, norm), norm(x + r))
