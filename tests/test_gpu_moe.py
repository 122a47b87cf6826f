"""Top-2 routing (bit-exact integers) and the rotated MoE layer vs the oracle and the reference goldens."""
import glob
import os

import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from gpu_util import DEV, assert_close, rel_err
from oracle import rtp_oracle as O

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("rotation_window")]
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _route(logits, noise):
    from rtp_amd import ops
    r = ops.top2_route(logits.to(DEV).contiguous(), noise.to(DEV).contiguous())
    torch.cuda.synchronize()
    return r


def _check_routing(logits, noise):
    g = O.top2gating(logits, noise)
    top = torch.sort(g["gates"], dim=1, descending=True).values
    assert (top[:, 0] - top[:, 1]).min() > 0, "fixture must have a non-zero top-1 margin"
    r = _route(logits, noise)
    S, E = logits.shape
    assert torch.equal(r.expert.cpu(), g["expert"]), "expert choice"
    assert torch.equal(r.keep.cpu(), g["keep"]), "capacity drop"
    assert torch.equal(r.slot.cpu(), g["slot"]), "slot"
    assert torch.equal(r.counts.cpu(), g["counts"]), "per-expert counts"
    assert rel_err(r.weight, g["weight"]) <= 1e-5
    assert rel_err(r.gates, g["gates"]) <= 1e-5
    assert abs(float(r.l_aux) - float(g["l_aux"])) <= 1e-6
    C = 2 * S // E
    st = r.slot_token.cpu().view(E, C)
    expect = torch.full((E, C), -1, dtype=torch.int32)
    for s in range(S):
        for j in range(2):
            if g["keep"][s, j]:
                expect[g["expert"][s, j], g["slot"][s, j]] = s
    assert torch.equal(st, expect), "slot -> token map"
    return r, g


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "top2gating_*.npz"))))
def test_routing_matches_reference_golden(path):
    z = np.load(path)
    r, g = _check_routing(torch.from_numpy(z["logits"]), torch.from_numpy(z["noise"]))
    from rtp_amd.module.top2gate import dense_from_routing
    combine, dispatch = dense_from_routing(r, r.weight, torch.float32)
    assert np.array_equal(dispatch.cpu().numpy(), z["dispatch_mask"])
    np.testing.assert_allclose(combine.cpu().numpy(), z["combine_weights"], rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("S,E,seed,skew", [(8, 2, 0, 0.0), (512, 8, 1, 0.0), (4096, 8, 2, 0.0), (4096, 8, 3, 2.0),
                                           (1000, 4, 4, 1.0), (768, 64, 5, 0.0)])
def test_routing_bit_exact(S, E, seed, skew):
    gen = torch.Generator().manual_seed(seed)
    logits = torch.randn(S, E, generator=gen)
    logits[:, 0] += skew
    _check_routing(logits, O.gumbel_noise((S, E), gen))


def test_routing_backward_matches_autograd_of_oracle():
    from rtp_amd.module.top2gate import top2_route
    gen = torch.Generator().manual_seed(7)
    S, E = 64, 4
    logits = torch.randn(S, E, generator=gen)
    logits[:, 2] += 1.5
    noise = O.gumbel_noise((S, E), gen)
    cw = torch.randn(S, 2, generator=gen)
    ld = logits.to(DEV).requires_grad_()
    r, weight, l_aux = top2_route(ld, noise.to(DEV))
    ((weight * cw.to(DEV)).sum() + 3.0 * l_aux).backward()
    lo = logits.clone().requires_grad_()
    g = O.top2gating(lo, noise)
    ((g["weight"] * cw).sum() + 3.0 * g["l_aux"]).backward()
    assert rel_err(ld.grad, lo.grad) <= 1e-5


def _moe_from_tensors(wg, experts, ws, dtype):
    from rtp_amd import emulate_shards
    from rtp_amd.models.transformer_lm_rtp import FeedForwardLayer_expert
    from rtp_amd.module.moe import WeightMOELayer
    from rtp_amd.module.top2gate import Top2Gate, WeightTop2Gate
    E, M = wg.shape
    Fd = experts[0][0].shape[0]
    master_gate = Top2Gate(M, E)
    with torch.no_grad():
        master_gate.wg.weight.copy_(wg)
    masters = []
    for w1, b1, w2, b2 in experts:
        m = FeedForwardLayer_expert(M, Fd, nn.ReLU(), 0.0)
        with torch.no_grad():
            m.linear1.weight.copy_(w1), m.linear1.bias.copy_(b1), m.linear2.weight.copy_(w2), m.linear2.bias.copy_(b2)
        masters.append(m)
    n_local = E // ws
    with emulate_shards(ws):
        gate = WeightTop2Gate(M, E, gate=master_gate.to(dtype), device=DEV, dtype=dtype)
        local = nn.ModuleList([FeedForwardLayer_expert(M, Fd, nn.ReLU(), 0.0) for _ in range(n_local)])
        originals = [nn.ModuleList(masters[s * n_local:(s + 1) * n_local]) for s in range(ws)]
        layer = WeightMOELayer(gate, local, device=DEV, dtype=dtype, original_experts=originals)
    return layer


def test_moe_layer_matches_reference_golden():
    """The reference's WeightMOELayer on a 2-rank gloo ring (tests/golden/moe_ws2.npz)."""
    z = np.load(os.path.join(GOLDEN, "moe_ws2.npz"))
    t = {k: torch.from_numpy(z[k]) for k in z.files}
    names = ("linear1.weight", "linear1.bias", "linear2.weight", "linear2.bias")
    experts = [tuple(t[f"expert{e}.{n}"] for n in names) for e in range(2)]
    layer = _moe_from_tensors(t["wg"], experts, 2, torch.float32)
    x = t["x"].to(DEV).requires_grad_()
    out = layer(x)
    assert rel_err(out, t["out"]) <= 1e-5
    assert abs(float(layer.l_aux) - float(t["l_aux"])) <= 1e-6
    ((out * t["coef"].to(DEV)).sum() + layer.l_aux).backward()
    for n, p in zip(names, layer.experts.parameters()):
        assert rel_err(2 * p.grad, t[f"grad_expert0.0.{n}"]) <= 1e-5, n
    assert rel_err(2 * layer.gate.wg.weight.grad, t["grad_wg0"]) <= 1e-5


@pytest.mark.parametrize("dtype,ws,E", [(torch.float32, 4, 4), (torch.float32, 2, 4), (torch.bfloat16, 4, 4)])
def test_moe_layer_vs_oracle(dtype, ws, E):
    gen = torch.Generator().manual_seed(21)
    M, Fd, S = 32, 48, 64
    wg = (torch.rand(E, M, generator=gen) * 0.2 - 0.1).to(dtype).float()
    experts = [tuple((torch.rand(s, generator=gen) * 0.2 - 0.1).to(dtype).float()
                     for s in ((Fd, M), (Fd,), (M, Fd), (M,))) for _ in range(E)]
    x = torch.randn(4, S // 4, M, generator=gen).to(dtype)
    coef = torch.randn(4, S // 4, M, generator=gen).to(dtype)
    noise = O.gumbel_noise((S, E), gen)
    layer = _moe_from_tensors(wg, experts, ws, dtype)
    xd = x.to(DEV).requires_grad_()
    out = layer(xd, noise=noise.to(DEV))
    ((out.float() * coef.to(DEV).float()).sum() + layer.l_aux.float()).backward()
    wgo = wg.clone().requires_grad_()
    eo = [tuple(p.clone().requires_grad_() for p in e) for e in experts]
    xo = x.float().requires_grad_()
    if dtype == torch.bfloat16:
        # routing is discrete: give the oracle the logits the device actually produced
        pass
    ref, l_aux = O.moe_layer(xo, wgo, eo, noise, ws)
    ((ref * coef.float()).sum() + l_aux).backward()
    assert_close(out, ref, dtype, "output")
    assert abs(float(layer.l_aux) - float(l_aux)) <= (1e-6 if dtype == torch.float32 else 2e-3)
    assert_close(xd.grad, xo.grad, dtype, "input grad")
    n_local = E // ws
    for s in range(ws):
        params = list(layer.experts_list[s].parameters())
        for j in range(n_local):
            for q, p in zip(eo[s * n_local + j], params[4 * j:4 * j + 4]):
                assert_close(p.grad, q.grad, dtype, f"expert {s * n_local + j} grad")
    assert_close(torch.cat([w.weight.grad for w in layer.gate.wgs], 0), wgo.grad, dtype, "gate grad (cat dim 0)")


def test_gate_module_dense_api():
    from rtp_amd import emulate_shards
    from rtp_amd.module.top2gate import WeightTop2Gate
    gen = torch.Generator().manual_seed(4)
    with emulate_shards(4):
        gate = WeightTop2Gate(16, 4, device=DEV)
    x = torch.randn(32, 16, generator=gen)
    noise = O.gumbel_noise((32, 4), gen)
    l_aux, combine, dispatch = gate(x.to(DEV), noise=noise.to(DEV))
    wg = torch.cat([w.weight.detach().cpu() for w in gate.wgs], 0)
    g = O.top2gating(x @ wg.t(), noise)
    assert combine.shape == (32, 4, 16) and dispatch.dtype == torch.bool
    assert torch.equal(dispatch.cpu(), g["dispatch_mask"])
    assert rel_err(combine, g["combine_weights"]) <= 1e-5


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "top2gating_*.npz"))))
def test_unsharded_top2gate_forward_matches_reference_golden(path):
    """Top2Gate.forward = top2gating(wg(input)) (rtp/module/top2gate.py:131-137).  With the gate weight an identity
    block, wg(input) reproduces the fixture's logits bit for bit (every product is x*1 or x*0), so the reference's
    own combine / dispatch tensors are the expected output; a second case with a random projection is checked
    against the oracle on the CPU-computed logits, with gradients."""
    from rtp_amd.module.top2gate import Top2Gate
    z = np.load(path)
    logits, noise = torch.from_numpy(z["logits"]), torch.from_numpy(z["noise"])
    S, E = logits.shape
    M = 16
    gate = Top2Gate(M, E)
    with torch.no_grad():
        gate.wg.weight.zero_()
        gate.wg.weight[:, :E].copy_(torch.eye(E))
    gate = gate.to(DEV)
    x = torch.zeros(S, M)
    x[:, :E] = logits
    l_aux, combine, dispatch = gate(x.to(DEV), noise=noise.to(DEV))
    assert np.array_equal(dispatch.cpu().numpy(), z["dispatch_mask"])
    np.testing.assert_allclose(combine.detach().cpu().numpy(), z["combine_weights"], rtol=1e-5, atol=1e-7)
    assert abs(float(l_aux) - float(z["l_aux"])) <= 1e-6


def test_unsharded_top2gate_gradients():
    from rtp_amd.module.top2gate import Top2Gate
    gen = torch.Generator().manual_seed(9)
    S, M, E = 48, 24, 4
    gate = Top2Gate(M, E)
    w = gate.wg.weight.detach().clone()
    gate = gate.to(DEV)
    x = torch.randn(S, M, generator=gen)
    noise = O.gumbel_noise((S, E), gen)
    coef = torch.randn(S, E, 2 * S // E, generator=gen)
    xd = x.to(DEV).requires_grad_()
    l_aux, combine, dispatch = gate(xd, noise=noise.to(DEV))
    ((combine * coef.to(DEV)).sum() + 2.0 * l_aux).backward()
    xo, wo = x.clone().requires_grad_(), w.clone().requires_grad_()
    g = O.top2gating(F.linear(xo, wo), noise)
    ((g["combine_weights"] * coef).sum() + 2.0 * g["l_aux"]).backward()
    assert torch.equal(dispatch.cpu(), g["dispatch_mask"])
    assert rel_err(combine, g["combine_weights"]) <= 1e-5
    assert rel_err(xd.grad, xo.grad) <= 1e-5 and rel_err(gate.wg.weight.grad, wo.grad) <= 1e-5


@pytest.mark.parametrize("dtype,S,M,E", [(torch.float32, 100, 64, 3), (torch.bfloat16, 4096, 2048, 8),
                                         (torch.bfloat16, 33, 136, 16), (torch.float32, 5, 4, 1)])
def test_gate_streaming_kernels_against_torch(dtype, S, M, E):
    """rtp_gate_fwd / dgrad / wgrad through the C ABI against fp32 torch products on the same inputs: the gate
    projection of the reference (an nn.Linear without bias, rtp/module/top2gate.py:202) and its backward."""
    from rtp_amd import ops
    from gpu_util import assert_close
    gen = torch.Generator().manual_seed(S + M + E)
    x = torch.randn(S, M, generator=gen).to(dtype)
    w = (torch.randn(E, M, generator=gen) * 0.1).to(dtype)
    dl = torch.randn(S, E + 2, generator=gen)                     # the run's columns sit at offset 1 of a wider matrix
    xd, wd, dld = x.to(DEV), w.to(DEV), dl.to(DEV)
    assert ops.gate_supported(xd, wd)
    logits = torch.full((S, E + 2), 7.0, device=DEV)
    ops.gate_fwd(xd, wd, logits, 1)
    assert_close(logits[:, 1:E + 1], x.float() @ w.float().T, torch.float32 if dtype == torch.float32 else dtype, "logits")
    assert bool((logits[:, 0] == 7).all()) and bool((logits[:, E + 1] == 7).all())
    dx = torch.empty(S, M, dtype=dtype, device=DEV)
    ops.gate_dgrad(dld, 1, wd, dx)
    assert_close(dx, dl[:, 1:E + 1] @ w.float(), dtype, "dx")
    # with an addend: the sum autograd would form of the two rounded tensors, bit for bit (also in place)
    other = torch.randn(S, M, generator=gen).to(dtype).to(DEV)
    dx2 = torch.empty_like(dx)
    ops.gate_dgrad(dld, 1, wd, dx2, init=other)
    assert torch.equal(dx2, other + dx)
    ops.gate_dgrad(dld, 1, wd, other, init=other)
    assert torch.equal(other, dx2)
    dw = torch.zeros(E, M, dtype=dtype, device=DEV)
    ops.gate_wgrad(dld, 1, xd, dw, False)
    want = dl[:, 1:E + 1].T @ x.float()
    assert_close(dw, want, dtype, "dw")
    first = dw.clone()
    ops.gate_wgrad(dld, 1, xd, dw, True)
    assert_close(dw, first.float().cpu() + want, dtype, "dw accumulated")
    ops.gate_wgrad(dld, 1, xd, dw, False)
    assert torch.equal(dw, first)                                  # fixed summation order: bit-identical repeat


def test_gate_streaming_kernels_limits():
    from rtp_amd import ops
    from rtp_amd._lib import RtpError
    x = torch.zeros(8, 64, dtype=torch.bfloat16, device=DEV)
    assert not ops.gate_supported(x, torch.zeros(17, 64, dtype=torch.bfloat16, device=DEV))   # too many experts
    assert not ops.gate_supported(x[:, :60], torch.zeros(4, 60, dtype=torch.bfloat16, device=DEV))  # 60 % 8 != 0
    assert not ops.gate_supported(x[:, 1:9], torch.zeros(4, 8, dtype=torch.bfloat16, device=DEV))   # misaligned rows
    with pytest.raises(RtpError):
        ops.gate_fwd(x, torch.zeros(17, 64, dtype=torch.bfloat16, device=DEV), torch.zeros(8, 17, device=DEV), 0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_moe_input_gradient_paths_meet_in_the_gate_kernel(dtype):
    """The tokens feed the gate and the dispatch; the gate's input-gradient kernel adds the dispatch path's gradient in
    its epilogue.  Same bits as autograd's own sum of the two (taken from two layers that share weights, one fed
    through a leaf per path), l_aux arrives in the layer's dtype, and a loss that uses only l_aux still works."""
    from rtp_amd import emulate_shards
    from rtp_amd.models.transformer_lm_rtp import FeedForwardLayer_expert
    from rtp_amd.module import moe as moe_mod
    from rtp_amd.module.moe import WeightMOELayer
    from rtp_amd.module.top2gate import Top2Gate, WeightTop2Gate
    gen = torch.Generator().manual_seed(4)
    M, Fd, E, ws = 64, 128, 4, 4
    mg = Top2Gate(M, E)
    masters = [FeedForwardLayer_expert(M, Fd, torch.nn.ReLU(), 0.0) for _ in range(E)]
    with emulate_shards(ws):
        gate = WeightTop2Gate(M, E, gate=mg, device=DEV, dtype=dtype)
        layer = WeightMOELayer(gate, torch.nn.ModuleList([FeedForwardLayer_expert(M, Fd, torch.nn.ReLU(), 0.0)]),
                               device=DEV, dtype=dtype, original_experts=[torch.nn.ModuleList([m]) for m in masters])
    x = torch.randn(4, 16, M, generator=gen).to(dtype).to(DEV)
    g = torch.randn(4, 16, M, generator=gen).to(dtype).to(DEV)
    u = torch.rand(64, E, generator=gen).clamp(min=1e-6, max=1 - 1e-6)
    noise = (-torch.log(-torch.log(u))).to(DEV)
    xa = x.clone().requires_grad_()
    out = layer(xa, noise=noise)
    assert layer.l_aux.dtype == dtype
    out.backward(g)
    fused = xa.grad.clone()
    # the same pass with the meeting point switched off: autograd adds the two paths itself
    try:
        moe_mod._JOIN_INPUT_GRADIENTS = False
        xb = x.clone().requires_grad_()
        layer(xb, noise=noise).backward(g)
    finally:
        moe_mod._JOIN_INPUT_GRADIENTS = True
    assert torch.equal(fused, xb.grad)
    xc = x.clone().requires_grad_()
    layer(xc, noise=noise)
    layer.l_aux.backward()                                        # only the auxiliary loss: the outputs' grads are None
    assert xc.grad is not None and torch.isfinite(xc.grad).all() and float(xc.grad.abs().sum()) > 0
