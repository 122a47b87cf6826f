"""Two-kernel softmax cross-entropy against torch's F.cross_entropy on the fp32 image of the same logits."""
import pytest
import torch
import torch.nn.functional as F

from gpu_util import DEV, assert_close

pytestmark = pytest.mark.gpu


def _case(rows, cols, dtype, seed, pad=0):
    gen = torch.Generator().manual_seed(seed)
    store = (torch.randn(rows, cols + pad, generator=gen) * 3.0).to(dtype)
    target = torch.randint(0, cols, (rows,), generator=gen)
    return store, target


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,cols,pad", [(1024, 10240, 0), (7, 8, 0), (33, 1000, 24), (1, 4096, 0), (64, 50264, 8)])
def test_cross_entropy_matches_torch(dtype, rows, cols, pad):
    from rtp_amd.module.loss import cross_entropy
    store, target = _case(rows, cols, dtype, rows + cols, pad)
    ref_in = store[:, :cols].float().clone().requires_grad_()
    ref = F.cross_entropy(ref_in, target)
    ref.backward()
    dev_store = store.to(DEV)
    x = dev_store[:, :cols].detach().requires_grad_()
    assert x.stride(0) == cols + pad
    loss = cross_entropy(x, target.to(DEV))
    loss.backward()
    assert loss.dtype == torch.float32
    assert abs(loss.item() - ref.item()) <= 1e-5 * abs(ref.item())
    assert x.grad.dtype == dtype
    assert_close(x.grad, ref_in.grad, dtype, "dlogits")


@pytest.mark.parametrize("reduction", ["none", "sum", "mean"])
def test_cross_entropy_reductions_ignore_index_and_upstream_gradient(reduction):
    from rtp_amd.module.loss import CrossEntropyLoss
    rows, cols = 96, 512
    store, target = _case(rows, cols, torch.bfloat16, 5)
    target[::5] = -100
    ref_in = store.float().clone().requires_grad_()
    ref = F.cross_entropy(ref_in, target, reduction=reduction, ignore_index=-100)
    w = torch.linspace(0.5, 2.0, rows) if reduction == "none" else torch.tensor(1.7)
    (ref * w).sum().backward()
    x = store.to(DEV).requires_grad_()
    out = CrossEntropyLoss(ignore_index=-100, reduction=reduction)(x, target.to(DEV))
    (out * w.to(DEV)).sum().backward()
    assert_close(out, ref, torch.float32, "loss")
    assert_close(x.grad, ref_in.grad, torch.bfloat16, "dlogits")
    assert torch.count_nonzero(x.grad[::5]).item() == 0   # ignored rows get no gradient


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("reduction", ["none", "sum", "mean"])
@pytest.mark.parametrize("cols", [512, 37])
def test_cross_entropy_ignore_index_inside_the_class_range(dtype, reduction, cols):
    """A padding id such as 0 is a valid class index AND the ignore index: its rows give zero loss and zero gradient
    in the vector kernels (512 classes) and the element-wise ones (37), and the mean runs over the other rows."""
    from rtp_amd.module.loss import cross_entropy
    rows = 50
    store, target = _case(rows, cols, dtype, 11 + cols)
    target[::3] = 0
    ref_in = store.float().clone().requires_grad_()
    ref = F.cross_entropy(ref_in, target, reduction=reduction, ignore_index=0)
    w = torch.linspace(0.5, 2.0, rows) if reduction == "none" else torch.tensor(0.6)
    (ref * w).sum().backward()
    x = store.to(DEV).requires_grad_()
    out = cross_entropy(x, target.to(DEV), ignore_index=0, reduction=reduction)
    (out * w.to(DEV)).sum().backward()
    assert_close(out, ref, torch.float32, "loss")
    assert_close(x.grad, ref_in.grad, dtype, "dlogits")
    assert torch.count_nonzero(x.grad[::3]).item() == 0
    assert torch.count_nonzero(x.grad[1]).item() > 0


def test_linear_cross_entropy_ignore_index_inside_the_class_range():
    from rtp_amd import emulate_shards
    from rtp_amd.module.linear import ColumnParallelLinear
    from rtp_amd.module.loss import linear_cross_entropy
    gen = torch.Generator().manual_seed(21)
    rows, k, vocab = 96, 64, 512
    master = torch.nn.Linear(k, vocab)
    with emulate_shards(4):
        layer = ColumnParallelLinear(k, vocab, linear_layer=master, device=DEV, dtype=torch.float32)
    x = torch.randn(rows, k, generator=gen)
    target = torch.randint(0, vocab, (rows,), generator=gen)
    target[::4] = 0
    xd = x.to(DEV).requires_grad_()
    loss = linear_cross_entropy(xd, layer, target.to(DEV), ignore_index=0)
    loss.backward()
    xr = x.clone().requires_grad_()
    ref = F.cross_entropy(master(xr), target, ignore_index=0)
    ref.backward()
    assert abs(float(loss) - float(ref)) <= 1e-5 * abs(float(ref))
    assert_close(xd.grad, xr.grad, torch.float32, "dx")
    assert torch.count_nonzero(xd.grad[::4]).item() == 0


def test_cross_entropy_extreme_logits_stay_finite():
    from rtp_amd.module.loss import cross_entropy
    x = torch.zeros(4, 64, dtype=torch.float32)
    x[0, 3] = 3.0e4
    x[1, :] = -3.0e4
    x[2, 5] = -3.0e4
    target = torch.tensor([3, 0, 5, 1])
    ref_in = x.clone().requires_grad_()
    ref = F.cross_entropy(ref_in, target, reduction="none")
    ref.sum().backward()
    xd = x.to(DEV).requires_grad_()
    out = cross_entropy(xd, target.to(DEV), reduction="none")
    out.sum().backward()
    assert torch.isfinite(out).all() and torch.isfinite(xd.grad).all()
    assert_close(out, ref, torch.float32, "loss")
    assert_close(xd.grad, ref_in.grad, torch.float32, "dlogits")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,cols", [(6, 37), (3, 1), (17, 1001)])
def test_cross_entropy_ragged_class_counts(dtype, rows, cols):
    """Class counts that are not whole 16-byte vectors take the element-wise kernels: same results, no torch path."""
    from rtp_amd.module.loss import cross_entropy
    store, target = _case(rows, cols, dtype, 3 * rows + cols)
    ref_in = store.float().clone().requires_grad_()
    ref = F.cross_entropy(ref_in, target)
    ref.backward()
    x = store.to(DEV).requires_grad_()
    loss = cross_entropy(x, target.to(DEV).int())     # int32 class indices are accepted
    loss.backward()
    assert abs(loss.item() - ref.item()) <= 1e-5 * max(abs(ref.item()), 1e-3)
    assert_close(x.grad, ref_in.grad, dtype, "dlogits")


def test_cross_entropy_default_ignore_index_and_invalid_targets():
    """-100 is ignored by default and the mean runs over the other rows (nn.CrossEntropyLoss's defaults); a target
    outside the classes that is not the ignore index poisons the loss with NaN instead of being skipped silently."""
    from rtp_amd._lib import RtpError
    from rtp_amd.module.loss import CrossEntropyLoss, cross_entropy
    rows, cols = 40, 64
    store, target = _case(rows, cols, torch.float32, 9)
    target[::4] = -100
    ref_in = store.clone().requires_grad_()
    ref = torch.nn.CrossEntropyLoss()(ref_in, target)
    ref.backward()
    x = store.to(DEV).requires_grad_()
    out = CrossEntropyLoss()(x, target.to(DEV))
    out.backward()
    assert_close(out, ref, torch.float32, "loss")
    assert_close(x.grad, ref_in.grad, torch.float32, "dlogits")
    bad = target.clone()
    bad[1] = cols + 3
    assert torch.isnan(cross_entropy(store.to(DEV), bad.to(DEV)))
    rows_loss = cross_entropy(store.to(DEV), bad.to(DEV), reduction="none")
    assert torch.isnan(rows_loss[1]) and torch.isfinite(rows_loss[2])
    all_ignored = torch.full((rows,), -100)
    assert torch.isnan(cross_entropy(store.to(DEV), all_ignored.to(DEV)))          # 0 / 0, as torch
    assert float(cross_entropy(store.to(DEV), all_ignored.to(DEV), reduction="sum")) == 0.0
    with pytest.raises(RtpError):
        cross_entropy(store, target)                                             # CPU tensors: no fallback


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,k,vocab,ws", [(1024, 256, 10240, 8), (96, 64, 512, 4), (70, 64, 128, 2), (130, 128, 1344, 3)])
def test_linear_cross_entropy_matches_separate_layer_and_loss(dtype, rows, k, vocab, ws):
    """The logits layer fused with its loss (logits never stored) against the same layer followed by the
    cross-entropy kernels, and against torch on the CPU: loss, input gradient, weight and bias gradients, with
    ignored rows."""
    from rtp_amd import emulate_shards
    from rtp_amd.module.linear import ColumnParallelLinear
    from rtp_amd.module.loss import cross_entropy, linear_cross_entropy
    gen = torch.Generator().manual_seed(rows + vocab)
    master = torch.nn.Linear(k, vocab)
    with torch.no_grad():
        master.weight.copy_((torch.rand(vocab, k, generator=gen) * 0.2 - 0.1).to(dtype).float())
        master.bias.copy_((torch.rand(vocab, generator=gen) * 0.2 - 0.1).to(dtype).float())
    with emulate_shards(ws):
        fused = ColumnParallelLinear(k, vocab, linear_layer=master, device=DEV, dtype=dtype)
        plain = ColumnParallelLinear(k, vocab, linear_layer=master, device=DEV, dtype=dtype)
    x = (torch.randn(rows, k, generator=gen) * 2.0).to(dtype)
    target = torch.randint(0, vocab, (rows,), generator=gen)
    target[::7] = -100
    xf, xp = x.to(DEV).requires_grad_(), x.to(DEV).requires_grad_()
    lf = linear_cross_entropy(xf, fused, target.to(DEV))
    (lf * 1.5).backward()
    lp = cross_entropy(plain(xp), target.to(DEV))
    (lp * 1.5).backward()
    xr = x.float().clone().requires_grad_()
    lr = F.cross_entropy(master(xr), target)
    (lr * 1.5).backward()
    assert abs(float(lf) - float(lr)) <= (1e-5 if dtype == torch.float32 else 2e-2) * abs(float(lr))
    assert abs(float(lf) - float(lp)) <= 1e-6 * abs(float(lp))     # same rounded logits on both device paths
    assert_close(xf.grad, xr.grad, dtype, "dx vs torch")
    assert_close(xf.grad, xp.grad.float().cpu(), dtype, "dx vs separate kernels")
    gw = torch.cat([s.weight.grad for s in fused.linears], 0)
    gb = torch.cat([s.bias.grad for s in fused.linears], 0)
    assert_close(gw, master.weight.grad, dtype, "dW")
    assert_close(gb, master.bias.grad, dtype, "db")
    assert torch.count_nonzero(xf.grad[::7]).item() == 0


def test_linear_cross_entropy_refuses_shard_widths_it_cannot_block():
    from rtp_amd import emulate_shards
    from rtp_amd._lib import RtpError
    from rtp_amd.module.linear import ColumnParallelLinear
    from rtp_amd.module.loss import linear_cross_entropy
    with emulate_shards(2):
        layer = ColumnParallelLinear(64, 96, device=DEV)          # 48 columns per shard
    with pytest.raises(RtpError, match="multiple of 64"):
        linear_cross_entropy(torch.randn(8, 64, device=DEV), layer, torch.zeros(8, dtype=torch.long, device=DEV))
