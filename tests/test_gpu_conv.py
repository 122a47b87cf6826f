"""Rotated ColumnParallelConv2d and the wrapper's Conv2d rule against stock torch.nn.Conv2d on the CPU (the
reference's own oracle for this layer: test_net.py:135-177 compares the wrapped MNIST Net with an untouched copy),
and the implicit-GEMM entry points against products over the explicit patch matrix (F.unfold / F.fold)."""
import copy

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from gpu_util import DEV, assert_close
from oracle import rtp_oracle as O

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("rotation_window")]

GEOMS = [
    # (N, Ci, H, W, Co, kernel, stride, padding, dilation)
    (3, 1, 28, 28, 32, 3, 1, 0, 1),                   # MNIST conv1: 9-element patches, one input channel
    (2, 32, 26, 26, 64, 3, 1, 0, 1),                  # MNIST conv2: 288-element patches
    (2, 8, 13, 11, 16, (3, 2), (2, 1), (1, 2), (1, 2)),
    (1, 4, 9, 9, 8, 5, 3, 2, 1),
]


def _pair(v):
    return (v, v) if isinstance(v, int) else v


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("geom", GEOMS)
def test_implicit_products_match_the_patch_matrix_oracle(geom, dtype):
    """The three entry points on a run of two shards against products over the oracle's explicit patch matrix
    (F.unfold) and its fold back (F.fold)."""
    from rtp_amd import ops
    n, ci, h, w, co, k, s, p, d = geom
    k, s, p, d = _pair(k), _pair(s), _pair(p), _pair(d)
    gen = torch.Generator().manual_seed(h * w + co)
    x = torch.randn(n, ci, h, w, generator=gen).to(dtype)
    g = ops.conv_geom(x.shape, k, s, p, d)
    kp, shards, extra = ci * k[0] * k[1], 2, 3                         # `extra` unused elements in front of a row
    n_s = co // shards
    numel = extra + n_s * kp + n_s
    flat = (torch.randn(shards, numel, generator=gen) * 0.2).to(dtype)
    w2d = torch.cat([flat[i, extra:extra + n_s * kp].view(n_s, kp) for i in range(shards)], 0).float()
    bias = torch.cat([flat[i, extra + n_s * kp:] for i in range(shards)], 0).float()
    patches = O.conv_patches(x.float(), k, s, p, d)                    # [n*ho*wo, kp]
    to_nchw = lambda m2d, c: m2d.view(n, g.ho, g.wo, c).permute(0, 3, 1, 2)
    xd, fd = x.to(DEV), flat.to(DEV)
    # forward into the middle channels of a wider output
    y = torch.full((n, co + 2, g.ho, g.wo), 7.0, dtype=dtype, device=DEV)
    ops.conv2d_fwd(xd, g, fd, extra, extra + n_s * kp, n_s, y, 1)
    assert_close(y[:, 1:1 + co], to_nchw(patches @ w2d.t() + bias, co), dtype, "forward")
    assert bool((y[:, 0] == 7).all()) and bool((y[:, -1] == 7).all())
    y2 = torch.empty_like(y)
    ops.conv2d_fwd(xd.contiguous(memory_format=torch.channels_last), g, fd, extra, None, n_s, y2, 1)
    assert_close(y2[:, 1:1 + co], to_nchw(patches @ w2d.t(), co), dtype, "forward, channels-last input, no bias")
    # weight and bias gradients, written and then accumulated
    dy = torch.randn(n, co + 2, g.ho, g.wo, generator=gen).to(dtype)
    dy2d = dy[:, 1:1 + co].permute(0, 2, 3, 1).reshape(-1, co).float()
    grads = torch.full((shards, numel), 5.0, dtype=dtype, device=DEV)
    ops.conv2d_wgrad(dy.to(DEV), xd, g, grads, extra, extra + n_s * kp, n_s, 1, False)
    dw = torch.cat([grads[i, extra:extra + n_s * kp].view(n_s, kp) for i in range(shards)], 0)
    db = torch.cat([grads[i, extra + n_s * kp:] for i in range(shards)], 0)
    assert_close(dw, dy2d.t() @ patches, dtype, "weight gradient")
    assert_close(db, dy2d.sum(0), dtype, "bias gradient")
    assert bool((grads[:, :extra] == 5).all())
    if dtype == torch.float32:
        ops.conv2d_wgrad(dy.to(DEV), xd, g, grads, extra, extra + n_s * kp, n_s, 1, True)
        dw2 = torch.cat([grads[i, extra:extra + n_s * kp].view(n_s, kp) for i in range(shards)], 0)
        assert_close(dw2, 2 * (dy2d.t() @ patches), dtype, "accumulated weight gradient")
    # input gradient: plain, and as the last window of a sum kept in fp32
    want_dx = O.conv_fold(dy2d @ w2d, x.shape, k, s, p, d)
    dx = torch.empty(n, ci, h, w, dtype=dtype, device=DEV)
    ops.conv2d_dgrad(dy.to(DEV), g, fd, extra, n_s, 1, dx)
    assert_close(dx, want_dx, dtype, "input gradient")
    part = torch.randn(n, ci, h, w, generator=gen)
    scratch = torch.empty(n, ci, h, w, device=DEV)
    ops.conv2d_dgrad(dy.to(DEV), g, fd, extra, n_s, 1, scratch, addend=part.to(dtype).to(DEV))
    assert_close(scratch, want_dx + part.to(dtype).float(), torch.float32 if dtype == torch.float32 else dtype,
                 "input gradient into fp32 with an addend")
    ops.conv2d_dgrad(dy.to(DEV), g, fd, extra, n_s, 1, dx, addend=scratch)
    assert_close(dx, 2 * want_dx + part.to(dtype).float(), dtype, "input gradient from an fp32 addend")


def test_conv_entry_points_reject_bad_geometry():
    from rtp_amd import _lib, ops
    x = torch.zeros(1, 1, 4, 4, device=DEV)
    with pytest.raises(ValueError):
        ops.conv_geom(x.shape, (5, 5), (1, 1), (0, 0), (1, 1))
    g = ops.conv_geom(x.shape, (3, 3), (1, 1), (0, 0), (1, 1))
    flat = torch.zeros(1, 2 * 9 + 2, device=DEV)
    y = torch.zeros(1, 2, 2, 2, device=DEV)
    ops.conv2d_fwd(x, g, flat, 0, 18, 2, y, 0)
    with pytest.raises(ValueError):
        ops.conv2d_fwd(x, g, flat, 4, 18, 2, y, 0)                    # the weight does not fit the shard row
    with pytest.raises(ValueError):
        ops.conv2d_fwd(x, g, flat, 0, 18, 2, y, 1)                    # channels beyond the output
    g.ho = 3                                                          # inconsistent with the geometry
    with pytest.raises(_lib.RtpError):
        ops.conv2d_fwd(x, g, flat, 0, 18, 2, torch.zeros(1, 2, 3, 2, device=DEV), 0)


@pytest.mark.parametrize("dtype,ws", [(torch.float32, 4), (torch.float32, 1), (torch.bfloat16, 4)])
@pytest.mark.parametrize("geom", GEOMS)
def test_column_conv2d_matches_nn_conv2d(geom, dtype, ws):
    from rtp_amd import emulate_shards
    from rtp_amd.module.conv import ColumnParallelConv2d
    n, ci, h, w, co, k, s, p, d = geom
    torch.manual_seed(co + ws)
    ref = nn.Conv2d(ci, co, k, s, p, d)
    with torch.no_grad():
        for q in ref.parameters():
            q.copy_(q.to(dtype).float())
    x = torch.randn(n, ci, h, w).to(dtype)
    with emulate_shards(ws):
        layer = ColumnParallelConv2d(ci, co, k, s, p, d, Conv2d_layer=ref, device=DEV, dtype=dtype)
    assert layer.conv is layer.layers[0] and layer.conv.weight.shape[0] == co // ws
    xd = x.to(DEV).requires_grad_()
    out = layer(xd)
    xr = x.float().requires_grad_()
    want = ref(xr)
    assert out.shape == want.shape and out.is_contiguous()
    gy = torch.randn(want.shape).to(dtype)
    out.backward(gy.to(DEV))
    want.backward(gy.float())
    assert_close(out, want, dtype, "output")
    assert_close(xd.grad, xr.grad, dtype, "input grad")
    assert_close(torch.cat([l.weight.grad for l in layer.layers], 0), ref.weight.grad, dtype, "weight grad")
    assert_close(torch.cat([l.bias.grad for l in layer.layers], 0), ref.bias.grad, dtype, "bias grad")
    assert_close(out, O.column_parallel_conv2d(x.float(), ref.weight.detach(), ref.bias.detach(), ws, s, p, d), dtype,
                 "oracle")


def test_column_conv2d_options():
    from rtp_amd import emulate_shards
    from rtp_amd.module.conv import ColumnParallelConv2d
    with emulate_shards(2):
        same = ColumnParallelConv2d(2, 4, 3, padding="same", bias=False, device=DEV)
        assert same.padding == (1, 1) and same.conv.bias is None
        x = torch.randn(1, 2, 6, 5, device=DEV)
        assert same(x).shape == (1, 4, 6, 5)
        with pytest.raises(NotImplementedError):
            ColumnParallelConv2d(4, 4, 3, groups=2, device=DEV)
        with pytest.raises(NotImplementedError):
            ColumnParallelConv2d(4, 4, 3, padding_mode="reflect", device=DEV)
        with pytest.raises(AssertionError):
            ColumnParallelConv2d(4, 5, 3, device=DEV)                 # out_channels not divisible
        with pytest.raises(ValueError):
            same(torch.randn(1, 3, 6, 5, device=DEV))


class MnistNet(nn.Module):
    """The network of the reference's rtp_mnist.py / test_net.py: two convolutions and two linear layers."""

    def __init__(self):
        super().__init__()
        self.conv1 = nn.Conv2d(1, 32, 3, 1)
        self.conv2 = nn.Conv2d(32, 64, 3, 1)
        self.fc1 = nn.Linear(9216, 128)
        self.fc2 = nn.Linear(128, 10)

    def forward(self, x):
        x = F.relu(self.conv1(x))
        x = F.max_pool2d(F.relu(self.conv2(x)), 2)
        x = F.relu(self.fc1(torch.flatten(x, 1)))
        return F.log_softmax(self.fc2(x), dim=1)


def test_wrapper_shards_the_mnist_net():
    from rtp_amd import emulate_shards
    from rtp_amd.rotated_tensor_parallel import RotatedTensorParallel
    ws = 2
    torch.manual_seed(0)
    ref = MnistNet()
    with emulate_shards(ws):
        model = RotatedTensorParallel(copy.deepcopy(ref)).to(DEV)
    kinds = [type(w.rotated).__name__ for w in model.FlyweightModule_list]
    assert kinds == ["ColumnParallelConv2d", "ColumnParallelConv2d", "ColumnParallelLinear", "ColumnParallelLinear"]
    x = torch.randn(4, 1, 28, 28)
    target = torch.tensor([3, 1, 4, 1])
    loss = F.nll_loss(model(x.to(DEV)), target.to(DEV))
    loss.backward()
    ref_loss = F.nll_loss(ref(x), target)
    ref_loss.backward()
    assert abs(float(loss) - float(ref_loss)) <= 1e-5 * abs(float(ref_loss))
    m = model.module
    for name in ("conv1", "conv2", "fc1", "fc2"):
        mine = torch.cat([s.weight.grad for s in getattr(m, name).module_list], 0)
        assert_close(mine, getattr(ref, name).weight.grad, torch.float32, name)
    with emulate_shards(4), pytest.raises(ValueError):
        RotatedTensorParallel(nn.Sequential(nn.Conv2d(3, 6, 3)))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rotated_sgd_updates_conv_layers_with_and_without_fused_backward(dtype):
    """A convolution's weight gradient does not carry the optimiser's update in its own launch: under
    RotatedSGD(fused_backward=True) its parameters take the separate update, and two steps leave the same weights
    as the plain optimiser, bit for bit."""
    from rtp_amd import emulate_shards
    from rtp_amd.module.conv import ColumnParallelConv2d
    from rtp_amd.module.linear import ColumnParallelLinear
    from rtp_amd.optim import RotatedSGD
    torch.manual_seed(5)
    ref_conv, ref_fc = nn.Conv2d(3, 8, 3, padding=1), nn.Linear(8 * 6 * 6, 16)
    x = torch.randn(4, 3, 6, 6).to(dtype).to(DEV)
    models = []
    for fused in (False, True):
        with emulate_shards(2):
            conv = ColumnParallelConv2d(3, 8, 3, padding=1, Conv2d_layer=ref_conv, device=DEV, dtype=dtype)
            fc = ColumnParallelLinear(8 * 6 * 6, 16, linear_layer=ref_fc, device=DEV, dtype=dtype)
        model = nn.Sequential(conv, nn.Flatten(), fc)
        opt = RotatedSGD(model, lr=0.05, clip_value=0.05, fused_backward=fused)
        for _ in range(2):
            opt.zero_grad()
            model(x).float().square().mean().backward()
            opt.step()
        models.append(model)
    torch.cuda.synchronize()
    for a, b in zip(models[0].parameters(), models[1].parameters()):
        assert torch.equal(a, b)
    moved = (models[0][0].layers[0].weight.float().cpu() - ref_conv.weight[:4].to(dtype).float()).abs().max()
    assert float(moved) > 0


def test_conv_layer_replayed_from_a_graph_matches_eager():
    """Forward + backward of the rotated convolution recorded into a HIP graph (every entry point allocation-free and
    never synchronising; the weight gradient's partial-sum workspace comes from torch's capture-aware allocator) and
    replayed on new inputs, with eager work in between, against the same layer run eagerly: bit-identical."""
    from rtp_amd import emulate_shards, ring
    from rtp_amd.module.conv import ColumnParallelConv2d
    torch.manual_seed(11)
    with emulate_shards(2):
        layer = ColumnParallelConv2d(4, 8, 3, padding=1, device=DEV, dtype=torch.bfloat16)
    x_static = torch.randn(16, 4, 12, 12, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    gy = torch.randn(16, 8, 12, 12, device=DEV, dtype=torch.bfloat16)

    def run(x):
        layer.zero_grad(set_to_none=False)
        x.grad = None
        y = layer(x)
        y.backward(gy)
        return y.detach().clone(), x.grad.detach().clone(), layer._store.grads.detach().clone()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(x_static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    x_static.grad = None          # the captured backward then owns a gradient buffer that every replay overwrites
    with torch.cuda.graph(g):
        layer.zero_grad(set_to_none=False)
        y_g = layer(x_static)
        y_g.backward(gy)
    ring.fence(torch.device(DEV))
    for seed in (1, 2, 3):
        new = torch.randn(16, 4, 12, 12, generator=torch.Generator().manual_seed(seed)).to(torch.bfloat16).to(DEV)
        with torch.no_grad():
            x_static.copy_(new)
        g.replay()
        torch.cuda.synchronize()
        got = (y_g.detach().clone(), x_static.grad.detach().clone(), layer._store.grads.detach().clone())
        torch.zeros(1 << 20, device=DEV).add_(1.0)                    # eager work between the replays
        probe = new.clone().requires_grad_()
        want = run(probe)
        for a, b in zip(got, want):
            assert torch.equal(a, b)
