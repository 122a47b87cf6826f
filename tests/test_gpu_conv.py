"""Rotated ColumnParallelConv2d and the wrapper's Conv2d rule against stock torch.nn.Conv2d on the CPU (the
reference's own oracle for this layer: test_net.py:135-177 compares the wrapped MNIST Net with an untouched copy),
and the patch-matrix kernels against F.unfold / F.fold."""
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
    (3, 1, 28, 28, 32, 3, 1, 0, 1),                   # MNIST conv1: 9-element patches (element-wise GEMM path)
    (2, 32, 26, 26, 64, 3, 1, 0, 1),                  # MNIST conv2: 288-element patches (vector path)
    (2, 8, 13, 11, 16, (3, 2), (2, 1), (1, 2), (1, 2)),
    (1, 4, 9, 9, 8, 5, 3, 2, 1),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("geom", GEOMS)
def test_patch_kernels_match_unfold_and_fold(geom, dtype):
    from rtp_amd import ops
    n, ci, h, w, _, k, s, p, d = geom
    pair = lambda v: (v, v) if isinstance(v, int) else v
    k, s, p, d = pair(k), pair(s), pair(p), pair(d)
    gen = torch.Generator().manual_seed(h * w)
    x = torch.randn(n, ci, h, w, generator=gen).to(dtype)
    g = ops.conv_geom(x.shape, k, s, p, d)
    ref = O.conv_patches(x.float(), k, s, p, d)
    cols = torch.empty(ref.shape, dtype=dtype, device=DEV)
    ops.im2col(x.to(DEV), g, cols)
    assert torch.equal(cols.float().cpu(), ref)                       # pure data movement: bit-exact
    # a channels-last input is read through its strides
    cols2 = torch.empty_like(cols)
    ops.im2col(x.to(DEV).contiguous(memory_format=torch.channels_last), g, cols2)
    assert torch.equal(cols2, cols)
    # padded row pitch: the extra columns are zeroed
    ld = ref.shape[1] + 5
    wide = torch.full((ref.shape[0], ld), 7.0, dtype=dtype, device=DEV)
    ops.im2col(x.to(DEV), g, wide)
    assert torch.equal(wide[:, :ref.shape[1]], cols) and not wide[:, ref.shape[1]:].any()
    dcols = torch.randn(ref.shape, generator=gen).to(dtype)
    dx = torch.empty(n, ci, h, w, dtype=dtype, device=DEV)
    ops.col2im(dcols.to(DEV), g, dx)
    assert_close(dx, O.conv_fold(dcols.float(), x.shape, k, s, p, d), dtype, "col2im")


def test_patch_kernels_reject_bad_geometry():
    from rtp_amd import _lib, ops
    x = torch.zeros(1, 1, 4, 4, device=DEV)
    with pytest.raises(ValueError):
        ops.conv_geom(x.shape, (5, 5), (1, 1), (0, 0), (1, 1))
    g = ops.conv_geom(x.shape, (3, 3), (1, 1), (0, 0), (1, 1))
    g.ho = 3                                                          # inconsistent with the geometry
    with pytest.raises(_lib.RtpError):
        ops.im2col(x, g, torch.zeros(3 * 2, 9, device=DEV))


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
