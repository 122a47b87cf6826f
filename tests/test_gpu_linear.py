"""Rotated Column/RowParallelLinear through the drop-in API vs the CPU oracle (and nn.Linear), with the
reference tests' gather rules for the gradients (tests/test_linear.py:117-186)."""
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from gpu_util import DEV, assert_close, rel_err
from oracle import rtp_oracle as O

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("rotation_window")]


def _build(cls_name, master, ws, dtype):
    from rtp_amd import emulate_shards
    from rtp_amd.module import linear as L
    with emulate_shards(ws):
        layer = getattr(L, cls_name)(master.in_features, master.out_features, linear_layer=master, device=DEV,
                                     dtype=dtype)
    return layer


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ws", [1, 2, 4])
def test_column_linear_reference_shape(dtype, ws):
    """nn.Linear(8,8), data [8,8] as in tests/test_linear.py."""
    master = nn.Linear(8, 8)
    x = torch.randn(8, 8)
    g = torch.randn(8, 8)
    layer = _build("ColumnParallelLinear", master.to(dtype), ws, dtype)
    xd = x.to(DEV, dtype).requires_grad_()
    out = layer(xd)
    out.backward(g.to(DEV, dtype))
    w, b = master.weight.detach().float().requires_grad_(), master.bias.detach().float().requires_grad_()
    xo = x.to(dtype).float().requires_grad_()
    ref = O.column_parallel_linear(xo, w, b, ws)
    ref.backward(g.to(dtype).float())
    assert_close(out, ref, dtype, "output")
    assert_close(torch.cat([l.weight.grad for l in layer.linears], dim=0), w.grad, dtype, "weight grad (cat dim 0)")
    assert_close(torch.cat([l.bias.grad for l in layer.linears], dim=0), b.grad, dtype, "bias grad (cat dim 0)")
    assert_close(xd.grad, xo.grad, dtype, "input grad")
    assert layer.linear is layer.linears[0] and layer.linear.weight.shape == (8 // ws, 8)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ws", [1, 2, 4])
def test_row_linear_reference_shape(dtype, ws):
    master = nn.Linear(8, 8)
    x = torch.randn(3, 8, 8)
    g = torch.randn(3, 8, 8)
    layer = _build("RowParallelLinear", master.to(dtype), ws, dtype)
    xd = x.to(DEV, dtype).requires_grad_()
    out = layer(xd)
    out.backward(g.to(DEV, dtype))
    w, b = master.weight.detach().float().requires_grad_(), master.bias.detach().float().requires_grad_()
    xo = x.to(dtype).float().requires_grad_()
    ref = O.row_parallel_linear(xo, w, b, ws)
    ref.backward(g.to(dtype).float())
    assert_close(out, ref, dtype, "output")
    assert_close(torch.cat([l.weight.grad for l in layer.linears], dim=1), w.grad, dtype, "weight grad (cat dim 1)")
    for l in layer.linears:  # each shard stores b/ws and receives the full bias gradient
        assert_close(l.bias.grad, b.grad, dtype, "bias grad (un-gathered)")
        assert_close(l.bias * ws, b, dtype, "bias/ws")
    assert_close(xd.grad, xo.grad, dtype, "input grad")


def test_column_linear_headline_config_fp32():
    """X [1024,2048] ~N(0,1), W [2048,2048] ~U(-0.1,0.1), bias zeros, 2 column shards."""
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(1024, 2048, generator=gen)
    master = nn.Linear(2048, 2048)
    with torch.no_grad():
        master.weight.copy_(torch.rand(2048, 2048, generator=gen) * 0.2 - 0.1)
        master.bias.zero_()
    dy = torch.randn(1024, 2048, generator=gen)
    layer = _build("ColumnParallelLinear", master, 2, torch.float32)
    xd = x.to(DEV).requires_grad_()
    out = layer(xd)
    out.backward(dy.to(DEV))
    xo = x.clone().requires_grad_()
    ref = master(xo)
    ref.backward(dy)
    assert_close(out, ref, torch.float32, "output")
    assert_close(torch.cat([l.weight.grad for l in layer.linears], 0), master.weight.grad, torch.float32, "dW")
    assert_close(torch.cat([l.bias.grad for l in layer.linears], 0), master.bias.grad, torch.float32, "db")
    assert_close(xd.grad, xo.grad, torch.float32, "dX")
    # linearity: the layer is affine in x with zero bias
    out2 = layer(2 * xd.detach())
    assert_close(out2, 2 * ref, torch.float32, "linearity")


def test_grad_accumulation_and_zero_grad():
    from rtp_amd import zero_full_grads
    master = nn.Linear(16, 12)
    layer = _build("ColumnParallelLinear", master, 4, torch.float32)
    x = torch.randn(5, 16, device=DEV)
    layer(x).sum().backward()
    g1 = torch.cat([l.weight.grad for l in layer.linears], 0).clone()
    layer(x).sum().backward()  # second backward accumulates, as torch does
    g2 = torch.cat([l.weight.grad for l in layer.linears], 0)
    assert_close(g2, 2 * g1, torch.float32, "accumulated grad")
    zero_full_grads(layer)
    assert all(l.weight.grad is None for l in layer.linears)
    layer(x).sum().backward()
    assert_close(torch.cat([l.weight.grad for l in layer.linears], 0), g1, torch.float32, "grad after zeroing")
    # parameters alias the flat home storage, shard by shard
    for s, l in enumerate(layer.linears):
        assert l.weight.data_ptr() == layer._store.home[s].data_ptr()
        assert l.weight.grad.data_ptr() == layer._store.grads[s].data_ptr()
    assert len(list(layer.parameters())) == 8


def test_to_dtype_keeps_flat_storage():
    master = nn.Linear(16, 8)
    layer = _build("ColumnParallelLinear", master, 2, torch.float32)
    layer.to(torch.bfloat16)
    assert layer._store.home.dtype == torch.bfloat16 and layer.linear.weight.dtype == torch.bfloat16
    x = torch.randn(4, 16, device=DEV, dtype=torch.bfloat16)
    assert_close(layer(x), master(x.float().cpu()), torch.bfloat16, "after .to(bf16)")


def test_indivisible_raises():
    from rtp_amd import emulate_shards
    from rtp_amd.module.linear import ColumnParallelLinear
    with emulate_shards(3), pytest.raises(AssertionError):
        ColumnParallelLinear(8, 8, device=DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ws", [1, 4])
def test_column_relu_mlp_matches_separate_modules(dtype, ws):
    """column_relu_mlp(x, lin1, lin2) == lin2(relu(lin1(x))) with nn.Linear masters, outputs and every gradient
    (the ReLU lives in the epilogues of the rotated products)."""
    from rtp_amd.module.linear import column_relu_mlp
    gen = torch.Generator().manual_seed(11 + ws)
    m1, m2 = nn.Linear(64, 96), nn.Linear(96, 32)
    with torch.no_grad():
        for p in list(m1.parameters()) + list(m2.parameters()):
            p.copy_(torch.rand(p.shape, generator=gen) * 0.4 - 0.2)
    x = torch.randn(5, 7, 64, generator=gen)
    g = torch.randn(5, 7, 32, generator=gen)
    l1 = _build("ColumnParallelLinear", m1.to(dtype), ws, dtype)
    l2 = _build("ColumnParallelLinear", m2.to(dtype), ws, dtype)
    xd = x.to(DEV, dtype).requires_grad_()
    out = column_relu_mlp(xd, l1, l2)
    out.backward(g.to(DEV, dtype))
    r1, r2 = nn.Linear(64, 96), nn.Linear(96, 32)
    r1.load_state_dict({k: v.float() for k, v in m1.state_dict().items()})
    r2.load_state_dict({k: v.float() for k, v in m2.state_dict().items()})
    xo = x.to(dtype).float().requires_grad_()
    ref = r2(torch.relu(r1(xo)))
    ref.backward(g.to(dtype).float())
    assert_close(out, ref, dtype, "output")
    assert_close(xd.grad, xo.grad, dtype, "input grad")
    for layer, r in ((l1, r1), (l2, r2)):
        assert_close(torch.cat([l.weight.grad for l in layer.linears], dim=0), r.weight.grad, dtype, "weight grad")
        assert_close(torch.cat([l.bias.grad for l in layer.linears], dim=0), r.bias.grad, dtype, "bias grad")


def test_unused_layer_gets_no_stale_gradient_after_zero_grad():
    """RotatedSGD.zero_grad keeps the gradient rows attached and lets the next backward overwrite them; a rotated
    layer that takes no part in that backward must then be stepped with a zero gradient, not with last step's."""
    from rtp_amd import emulate_shards
    from rtp_amd.module.linear import ColumnParallelLinear
    from rtp_amd.optim import RotatedSGD
    with emulate_shards(2):
        used = ColumnParallelLinear(8, 8, device=DEV)
        idle = ColumnParallelLinear(8, 8, device=DEV)
    model = nn.ModuleList([used, idle])
    opt = RotatedSGD(model, lr=0.5)
    x = torch.randn(4, 8, device=DEV)
    (used(x).sum() + idle(x).sum()).backward()
    opt.step()
    w_idle = torch.cat([l.weight.detach().clone() for l in idle.linears], 0)
    w_used = torch.cat([l.weight.detach().clone() for l in used.linears], 0)
    opt.zero_grad()
    used(x).sum().backward()       # `idle` is not part of this step
    opt.step()
    torch.cuda.synchronize()
    assert torch.equal(torch.cat([l.weight.detach() for l in idle.linears], 0), w_idle)
    assert not torch.equal(torch.cat([l.weight.detach() for l in used.linears], 0), w_used)


def test_backward_that_raises_leaves_no_deferred_weight_gradients_behind():
    """With weight gradients deferred to the second stream, a backward pass that raises part-way never reaches its
    end-of-pass join; the next pass must not launch the dead pass's closures nor skip its own join."""
    from rtp_amd import emulate_shards, ring
    from rtp_amd.module.linear import ColumnParallelLinear

    class Boom(torch.autograd.Function):
        @staticmethod
        def forward(ctx, x):
            return x.clone()

        @staticmethod
        def backward(ctx, g):
            raise ValueError("boom")

    with emulate_shards(2):
        a = ColumnParallelLinear(8, 8, device=DEV)
        b = ColumnParallelLinear(8, 8, device=DEV)
    x = torch.randn(4, 8, device=DEV)
    ring.set_wgrad_overlap(True)
    try:
        with pytest.raises(ValueError, match="boom"):
            b(Boom.apply(a(x))).sum().backward()     # b's backward defers its gradients, then the pass dies
        for l in a.linears + b.linears:
            l.weight.grad = l.bias.grad = None
        x2 = torch.randn(4, 8, device=DEV)
        b(a(x2)).sum().backward()
        torch.cuda.synchronize()
        assert not ring._wgrad_pending.get(0) and not ring._wgrad_dirty.get(0) and 0 not in ring._wgrad_task
        wa = torch.cat([l.weight.detach() for l in a.linears], 0)
        ba = torch.cat([l.bias.detach() for l in a.linears], 0)
        wb = torch.cat([l.weight.detach() for l in b.linears], 0)
        h = x2 @ wa.T + ba
        want_b = torch.ones(4, 8, device=DEV).T @ h
        got_b = torch.cat([l.weight.grad for l in b.linears], 0)
        assert rel_err(got_b, want_b) <= 1e-5
        want_a = (torch.ones(4, 8, device=DEV) @ wb).T @ x2
        assert rel_err(torch.cat([l.weight.grad for l in a.linears], 0), want_a) <= 1e-5
    finally:
        ring.set_wgrad_overlap(False)


def test_column_relu_mlp_with_dropout_on_the_hidden_activations():
    """lin2(dropout(relu(lin1(x)))) (rtp/models/transformer_lm_rtp.py:88-89 with dropout > 0): the keep mask is drawn
    by torch's device generator inside the function; redrawing it from the same generator state gives the
    reference computation on the CPU."""
    from rtp_amd import emulate_shards
    from rtp_amd.module.linear import ColumnParallelLinear, column_relu_mlp
    torch.manual_seed(4)
    m1, m2 = nn.Linear(32, 48), nn.Linear(48, 32)
    with emulate_shards(4):
        l1 = ColumnParallelLinear(32, 48, linear_layer=m1, device=DEV)
        l2 = ColumnParallelLinear(48, 32, linear_layer=m2, device=DEV)
    x, g = torch.randn(10, 32), torch.randn(10, 32)
    p = 0.25
    torch.cuda.manual_seed(77)
    xd = x.to(DEV).requires_grad_()
    y = column_relu_mlp(xd, l1, l2, dropout_p=p)
    y.backward(g.to(DEV))
    torch.cuda.manual_seed(77)
    keep = torch.empty(10, 48, device=DEV).bernoulli_(1.0 - p).mul_(1.0 / (1.0 - p)).cpu()
    assert 0 < int((keep == 0).sum()) < keep.numel()
    xr = x.clone().requires_grad_()
    ref = m2(torch.relu(m1(xr)) * keep)
    ref.backward(g)
    assert_close(y, ref, torch.float32, "output")
    assert_close(xd.grad, xr.grad, torch.float32, "dx")
    assert_close(torch.cat([s.weight.grad for s in l1.linears], 0), m1.weight.grad, torch.float32, "dW1")
    assert_close(torch.cat([s.weight.grad for s in l2.linears], 0), m2.weight.grad, torch.float32, "dW2")
    assert_close(torch.cat([s.bias.grad for s in l1.linears], 0), m1.bias.grad, torch.float32, "db1")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,n_s,k,ws,bias", [(1024, 256, 2048, 8, True), (320, 32, 64, 4, True), (64, 24, 8, 1, False),
                                                (77, 40, 72, 3, True)])
def test_rotated_linear_entry_points_against_torch(dtype, rows, n_s, k, ws, bias):
    """rtp_rotated_linear_fwd / _bwd through the C ABI on a flat [shards, numel] layer (the reference's per-layer ring
    loop, rtp/module/linear.py:211-222, and its backward) against F.linear on the unsharded weight: outputs, input
    gradient with an initial value and a ReLU mask, weight and bias gradients, and the fused clip + SGD update."""
    from rtp_amd import _lib, ops
    gen = torch.Generator().manual_seed(rows + n_s)
    numel = n_s * k + (n_s if bias else 0) + 8            # some unrelated tail in every flat shard
    home = (torch.randn(ws, numel, generator=gen) * 0.1).to(dtype)
    w = home[:, :n_s * k].reshape(ws * n_s, k).float()
    b = home[:, n_s * k:n_s * k + n_s].reshape(-1).float() if bias else None
    x = torch.randn(rows, k, generator=gen).to(dtype)
    dy = torch.randn(rows, ws * n_s, generator=gen).to(dtype)
    init = torch.randn(rows, k, generator=gen).to(dtype)
    gate = torch.randn(rows, k, generator=gen).to(dtype)
    hd, xd, dyd = home.to(DEV), x.to(DEV), dy.to(DEV)
    b_off = n_s * k if bias else None
    y = torch.empty(rows, ws * n_s, dtype=dtype, device=DEV)
    ops.rotated_linear_fwd(xd, hd, 0, b_off, n_s, k, y, relu=True)
    assert_close(y, torch.relu(F.linear(x.float(), w, b)), dtype, "relu(x W^T + b)")
    dx = torch.empty(rows, k, dtype=dtype, device=DEV)
    ops.rotated_linear_bwd(dyd, None, hd, 0, b_off, n_s, k, dx=dx, dx_init=init.to(DEV), relu_gate=gate.to(DEV))
    want = (init.float() + dy.float() @ w) * (gate.float() > 0)
    assert_close(dx, want, dtype, "dx")
    grads = torch.full((ws, numel), 7.0, dtype=dtype, device=DEV)
    done = ops.rotated_linear_bwd(dyd, xd, hd, 0, b_off, n_s, k, grads=grads)
    dw = (dy.float().T @ x.float()).view(ws, n_s * k)
    assert_close(grads[:, :n_s * k], dw, dtype, "dW")
    if bias:
        if done & _lib.ROTATED_BIAS_DONE:
            assert_close(grads[:, n_s * k:n_s * k + n_s], dy.float().sum(0).view(ws, n_s), dtype, "db")
    assert bool((grads[:, -8:] == 7.0).all())            # nothing beyond the layer's own slices is touched
    # the same launch with the optimiser's update in its epilogue: fp32 parameters and their copy
    master = hd.float().clone()
    weights = hd.clone()
    sgd = ops.FusedSgd(lr=0.05, clip=0.5, keep_grads=False)
    grads2 = torch.full((ws, numel), 7.0, dtype=dtype, device=DEV)
    done = ops.rotated_linear_bwd(dyd, xd, hd, 0, b_off, n_s, k, grads=grads2, sgd=sgd, sgd_master=master.data_ptr(),
                                  sgd_weights=weights.data_ptr() if dtype != torch.float32 else 0)
    if done & _lib.ROTATED_SGD_DONE:
        g = grads[:, :n_s * k].float().clamp(-0.5, 0.5)          # the gradient as the dtype holds it
        want_m = hd.float()[:, :n_s * k] - 0.05 * g
        assert torch.equal(master[:, :n_s * k], want_m)
        assert torch.equal(master[:, n_s * k:], hd.float()[:, n_s * k:])
        if dtype != torch.float32:
            assert torch.equal(weights[:, :n_s * k], want_m.to(dtype))
        assert bool((grads2[:, :n_s * k] == 7.0).all())          # consumed, not stored
    else:
        assert rows == 64 or k % 8                               # only shapes the vector kernel does not take
