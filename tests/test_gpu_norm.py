"""Fused residual add + LayerNorm against torch's fp32 layer_norm(x + r) on the same inputs."""
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from gpu_util import DEV, assert_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,cols", [(37, 2048), (5, 64), (1024, 512), (3, 8), (9, 1288), (6, 4096), (5, 3080)])
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


def test_add_layer_norm_refuses_rows_the_kernels_cannot_take():
    """There is one implementation: rows that are not whole 16-byte vectors, or wider than the kernels hold in
    registers, raise instead of going through torch."""
    from rtp_amd import ops
    from rtp_amd._lib import RtpError
    from rtp_amd.module.norm import add_layer_norm
    assert ops.layernorm_supported(torch.bfloat16, 8192) and ops.layernorm_supported(torch.float32, 4096)
    assert not ops.layernorm_supported(torch.float32, 4100)
    assert not ops.layernorm_supported(torch.bfloat16, 36)
    assert not ops.layernorm_supported(torch.float32, 38)
    norm = nn.LayerNorm(38).to(DEV)
    x = torch.randn(4, 38, device=DEV)
    r = torch.randn(4, 38, device=DEV)
    with pytest.raises(RtpError, match="16-byte"):
        add_layer_norm(x, r, norm)
    with pytest.raises(RtpError):
        add_layer_norm(torch.randn(4, 64), torch.randn(4, 64), nn.LayerNorm(64))     # CPU tensors


def test_layer_norm_parameter_gradients_reduced_at_the_end_of_backward():
    """With an optimiser's persistent gradient slices, every LayerNorm's backward leaves partial sums and one launch
    at the end of the backward pass reduces all of them: same gradients as torch, also for a LayerNorm applied twice
    in one forward pass (its second gradient is accumulated by autograd after the first is in place) and over
    repeated steps (the device table is reused)."""
    import torch.nn as nn
    from rtp_amd.module.norm import add_layer_norm
    from rtp_amd.optim import RotatedSGD

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.n1, self.n2 = nn.LayerNorm(64), nn.LayerNorm(64)

        def forward(self, x, fused):
            f = (lambda a, b, n: add_layer_norm(a, b, n)) if fused else (lambda a, b, n: n(a + b))
            h = f(x, x * 0.5, self.n1)
            h = f(h, x, self.n2)
            return f(h, h * 2.0, self.n1)            # n1 a second time

    torch.manual_seed(0)
    ref = Net()
    with torch.no_grad():
        for p in ref.parameters():
            p.add_(torch.randn_like(p) * 0.1)
    net = Net().to(DEV)
    net.load_state_dict(ref.state_dict())
    opt = RotatedSGD(net, lr=0.0)
    for step in range(3):
        x = torch.randn(40, 64)
        g = torch.randn(40, 64)
        opt.zero_grad()
        ref.zero_grad()
        net(x.to(DEV), True).backward(g.to(DEV))
        ref(x, False).backward(g)
        for (k, p), q in zip(net.named_parameters(), ref.parameters()):
            assert_close(p.grad, q.grad, torch.float32, f"step {step} {k}")


def test_backward_that_raises_leaves_no_partial_layer_norm_sums_behind():
    """A backward pass that raises after a LayerNorm has left its partial sums never runs the end-of-pass reduction.
    The next pass must queue its own reduction and must not reduce the dead pass's partial sums."""
    import torch.nn as nn
    from rtp_amd.module import norm as norm_mod
    from rtp_amd.module.norm import add_layer_norm
    from rtp_amd.optim import RotatedSGD

    class Boom(torch.autograd.Function):
        @staticmethod
        def forward(ctx, x):
            return x.clone()

        @staticmethod
        def backward(ctx, g):
            raise ValueError("boom")

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.n1, self.n2 = nn.LayerNorm(64), nn.LayerNorm(64)

        def forward(self, x, fused, boom=False):
            f = (lambda a, b, n: add_layer_norm(a, b, n)) if fused else (lambda a, b, n: n(a + b))
            h = f(x, x * 0.5, self.n1)
            if boom:
                h = Boom.apply(h)
            return f(h, x, self.n2)

    torch.manual_seed(1)
    ref = Net()
    net = Net().to(DEV)
    net.load_state_dict(ref.state_dict())
    opt = RotatedSGD(net, lr=0.0)
    x = torch.randn(24, 64)
    opt.zero_grad()
    with pytest.raises(ValueError, match="boom"):
        net(x.to(DEV), True, boom=True).sum().backward()     # n2 has left partial sums; the pass dies before n1
    x, g = torch.randn(24, 64), torch.randn(24, 64)
    opt.zero_grad()
    net(x.to(DEV), True).backward(g.to(DEV))
    ref(x, False).backward(g)
    torch.cuda.synchronize()
    assert not norm_mod._deferred.pending.get(0) and 0 not in norm_mod._deferred.armed
    for (k, p), q in zip(net.named_parameters(), ref.parameters()):
        assert_close(p.grad, q.grad, torch.float32, k)
