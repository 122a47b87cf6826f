"""Pins the CPU oracle (oracle/rtp_oracle.py) against independent references: stock torch layers (the
reference's own test oracle), golden vectors written from the reference's routing / MoE code, brute-force
integer loops, and closed forms.  CPU only."""
import glob
import math
import os

import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from oracle import rtp_oracle as O

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


# ---- Linear: reference oracle is nn.Linear on the unsharded problem (tests/test_linear.py:134-186) ----
@pytest.mark.parametrize("ws", [1, 2, 4])
@pytest.mark.parametrize("rank", [0, 1])
def test_column_linear_matches_nn_linear(ws, rank):
    if rank >= ws:
        pytest.skip("rank outside ring")
    lin = nn.Linear(12, 8)
    x = torch.randn(5, 3, 12, requires_grad=True)
    ref = lin(x)
    w, b = lin.weight.detach().clone().requires_grad_(), lin.bias.detach().clone().requires_grad_()
    x2 = x.detach().clone().requires_grad_()
    out = O.column_parallel_linear(x2, w, b, ws, rank)
    torch.testing.assert_close(out, ref)
    g = torch.randn_like(ref)
    ref.backward(g)
    out.backward(g)
    torch.testing.assert_close(w.grad, lin.weight.grad)
    torch.testing.assert_close(b.grad, lin.bias.grad)
    torch.testing.assert_close(x2.grad, x.grad)


@pytest.mark.parametrize("ws", [1, 2, 4])
def test_row_linear_matches_nn_linear(ws):
    lin = nn.Linear(12, 8)
    x = torch.randn(7, 12)
    ref = lin(x)
    out = O.row_parallel_linear(x, lin.weight.detach(), lin.bias.detach(), ws)
    torch.testing.assert_close(out, ref)
    # every row shard carries bias/ws (linear.py:133-135)
    shards = O.row_shards(lin.weight.detach(), lin.bias.detach(), ws)
    torch.testing.assert_close(sum(b for _, b in shards), lin.bias.detach())
    torch.testing.assert_close(torch.cat([w for w, _ in shards], dim=1), lin.weight.detach())


# ---- Embedding: nn.Embedding, bit for bit (tests/test_embedding.py:127-157) ----
@pytest.mark.parametrize("ws", [1, 2, 4])
def test_embedding_forward_is_exact_gather(ws):
    emb = nn.Embedding(37, 16)
    ids = torch.randint(0, 37, (6, 5))
    out = O.parallel_embedding(ids, emb.weight.detach(), ws)
    assert torch.equal(out, emb(ids))


def test_embedding_backward_sequential_is_torch_cpu_backward_bitwise():
    torch.manual_seed(3)
    emb = nn.Embedding(20, 24)
    ids = torch.randint(0, 20, (32, 8))  # 256 tokens over 20 rows: every row is hit many times
    g = torch.randn(32, 8, 24)
    emb(ids).backward(g)
    mine = O.embedding_backward_sequential(ids.numpy(), g.numpy(), 20)
    assert np.array_equal(mine, emb.weight.grad.numpy())
    idx_add = torch.zeros(20, 24).index_add_(0, ids.reshape(-1), g.reshape(-1, 24))
    assert np.array_equal(mine, idx_add.numpy())
    # a wrong accumulation order (descending position) differs in the last bits
    rev = O.embedding_backward_sequential(ids.numpy().reshape(-1)[::-1].copy(), g.numpy().reshape(-1, 24)[::-1].copy(), 20)
    assert not np.array_equal(rev, mine)
    np.testing.assert_allclose(rev, mine, rtol=1e-5, atol=1e-5)


def test_embedding_backward_padding_idx():
    emb = nn.Embedding(10, 4, padding_idx=3)
    ids = torch.tensor([[1, 3, 3, 2], [3, 1, 0, 9]])
    g = torch.randn(2, 4, 4)
    emb(ids).backward(g)
    mine = O.embedding_backward_sequential(ids.numpy(), g.numpy(), 10, padding_idx=3)
    assert np.array_equal(mine, emb.weight.grad.numpy())


# ---- Attention: nn.MultiheadAttention (tests/test_attention.py:133-187) ----
def _causal(L):
    return torch.triu(torch.full((L, L), float("-inf")), diagonal=1)


@pytest.mark.parametrize("ws", [1, 2, 4])
@pytest.mark.parametrize("masked", [False, True])
def test_attention_matches_nn_mha(ws, masked):
    E, H, L, N = 16, 4, 6, 3
    mha = nn.MultiheadAttention(E, H, bias=True)
    with torch.no_grad():
        mha.in_proj_bias.uniform_(-0.1, 0.1)
        mha.out_proj.bias.uniform_(-0.1, 0.1)
    x = torch.randn(L, N, E)
    mask = _causal(L) if masked else None
    ref, ref_w = mha(x, x, x, attn_mask=mask, need_weights=True, average_attn_weights=False)
    ref2, _ = mha(x, x, x, attn_mask=mask, need_weights=False)
    out, w = O.parallel_multihead_attention(x, mha.in_proj_weight.detach(), mha.in_proj_bias.detach(),
                                            mha.out_proj.weight.detach(), mha.out_proj.bias.detach(), H, ws,
                                            mask=mask, need_weights=True)
    torch.testing.assert_close(out, ref.detach())
    torch.testing.assert_close(out, ref2.detach())
    # returned weights = head average of the last shard's heads only (attention.py:267)
    h_s = H // ws
    last = O.ring_order(0, ws)[-1]
    torch.testing.assert_close(w, ref_w[:, last * h_s:(last + 1) * h_s].mean(dim=1).detach())


def test_attention_shard_grads_reinterleave_to_unsharded():
    E, H, L, N, ws = 16, 4, 5, 2, 2
    mha = nn.MultiheadAttention(E, H, bias=True)
    x = torch.randn(L, N, E)
    g = torch.randn(L, N, E)
    mha(x, x, x, need_weights=False)[0].backward(g)
    shards = []
    for s in range(ws):
        p = [t.detach().clone().requires_grad_() for t in O.attention_shard_params(
            mha.in_proj_weight.detach(), mha.in_proj_bias.detach(), mha.out_proj.weight.detach(),
            mha.out_proj.bias.detach(), ws, s)]
        shards.append(p)
    out = None
    for p in shards:
        part, _ = O._shard_attention(x, *p, H // ws, None, False)
        out = part if out is None else out + part
    out.backward(g)
    torch.testing.assert_close(O.attention_grad_reinterleave([p[0].grad for p in shards], ws), mha.in_proj_weight.grad)
    torch.testing.assert_close(O.attention_grad_reinterleave([p[1].grad for p in shards], ws), mha.in_proj_bias.grad)
    torch.testing.assert_close(torch.cat([p[2].grad for p in shards], dim=1), mha.out_proj.weight.grad)
    for p in shards:  # each shard stores b/ws but its gradient is the full db
        torch.testing.assert_close(p[3].grad, mha.out_proj.bias.grad)


# ---- Top-2 gating: golden vectors from the reference, brute force, special cases ----
@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "top2gating_*.npz"))))
def test_top2gating_matches_reference_golden(path):
    z = np.load(path)
    g = O.top2gating(torch.from_numpy(z["logits"]), torch.from_numpy(z["noise"]))
    assert np.array_equal(g["dispatch_mask"].numpy(), z["dispatch_mask"])
    np.testing.assert_array_equal(g["combine_weights"].numpy(), z["combine_weights"])
    np.testing.assert_array_equal(g["l_aux"].numpy(), z["l_aux"])
    # the compact record encodes exactly the dense tensors
    S, E, C = z["combine_weights"].shape
    dense = np.zeros((S, E, C), np.float32)
    for s in range(S):
        for j in range(2):
            if g["keep"][s, j]:
                dense[s, g["expert"][s, j], g["slot"][s, j]] += g["weight"][s, j].item()
    np.testing.assert_array_equal(dense, z["combine_weights"])


def test_golden_set_exercises_capacity_drop():
    dropped = [2 * np.load(p)["logits"].shape[0] - np.load(p)["dispatch_mask"].sum()
               for p in glob.glob(os.path.join(GOLDEN, "top2gating_*.npz"))]
    assert len(dropped) >= 4 and max(dropped) > 0


@pytest.mark.parametrize("S,E,seed", [(8, 2, 0), (16, 4, 1), (48, 8, 2), (64, 4, 3)])
def test_top2gating_matches_bruteforce(S, E, seed):
    gen = torch.Generator().manual_seed(seed)
    logits = torch.randn(S, E, generator=gen)
    if seed == 3:
        logits[:, 1] += 3.0
    noise = O.gumbel_noise((S, E), gen)
    g = O.top2gating(logits, noise)
    expert, slot, keep = O.top2_route_bruteforce(logits.numpy(), noise.numpy())
    assert np.array_equal(g["expert"].numpy(), expert)
    assert np.array_equal(g["keep"].numpy(), keep)
    assert np.array_equal(g["slot"].numpy(), slot)


def test_top2gating_two_experts_is_noise_independent():
    gen = torch.Generator().manual_seed(5)
    logits = torch.randn(32, 2, generator=gen)
    a = O.top2gating(logits, O.gumbel_noise((32, 2), gen))
    b = O.top2gating(logits, torch.zeros(32, 2))
    assert torch.equal(a["expert"], b["expert"]) and torch.equal(a["combine_weights"], b["combine_weights"])
    assert torch.equal(a["expert"][:, 0], torch.argmax(logits, dim=1).int())
    assert torch.equal(a["expert"][:, 1], 1 - a["expert"][:, 0])


def test_top2gating_l_aux_closed_form_and_weights_normalised():
    gen = torch.Generator().manual_seed(9)
    logits = torch.randn(40, 4, generator=gen)
    g = O.top2gating(logits, O.gumbel_noise((40, 4), gen))
    gates = torch.softmax(logits, dim=1)
    first = torch.bincount(gates.argmax(1), minlength=4).float() / 40
    torch.testing.assert_close(g["l_aux"], (gates.mean(0) * first).mean())
    both = (g["keep"].sum(1) == 2)
    torch.testing.assert_close(g["weight"][both].sum(1), torch.ones(int(both.sum())))
    # a uniform gate gives l_aux = 1/E^2 * E * (1/E) ... = mean_e(1/E * ce_e) = 1/E^2
    u = O.top2gating(torch.zeros(8, 4), torch.zeros(8, 4))
    assert abs(float(u["l_aux"]) - (1.0 / 4) * (1.0 / 4)) < 1e-7


# ---- MoE layer: golden from the reference's WeightMOELayer on a 2-rank gloo ring ----
def _moe_golden():
    z = np.load(os.path.join(GOLDEN, "moe_ws2.npz"))
    t = {k: torch.from_numpy(z[k]) for k in z.files}
    experts = [tuple(t[f"expert{e}.{n}"] for n in ("linear1.weight", "linear1.bias", "linear2.weight", "linear2.bias"))
               for e in range(2)]
    return t, experts


def test_moe_layer_matches_reference_golden():
    t, experts = _moe_golden()
    wg = t["wg"].clone().requires_grad_()
    experts = [tuple(p.clone().requires_grad_() for p in e) for e in experts]
    out, l_aux = O.moe_layer(t["x"], wg, experts, torch.zeros(t["x"].shape[0] * t["x"].shape[1], 2), ws=2)
    torch.testing.assert_close(out, t["out"], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(l_aux, t["l_aux"])
    ((out * t["coef"]).sum() + l_aux).backward()
    # both reference ranks fed the same batch, so its summed expert gradients are 2x one copy's
    for n, p in zip(("linear1.weight", "linear1.bias", "linear2.weight", "linear2.bias"), experts[0]):
        torch.testing.assert_close(2 * p.grad, t[f"grad_expert0.0.{n}"], rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(2 * wg.grad[0:1], t["grad_wg0"], rtol=1e-4, atol=1e-5)


def test_moe_layer_closed_form_and_empty_slots():
    gen = torch.Generator().manual_seed(11)
    S, E, M, Fd = 16, 4, 8, 12
    x3 = torch.randn(2, 8, M, generator=gen)
    wg = torch.randn(E, M, generator=gen)
    experts = [(torch.randn(Fd, M, generator=gen) * 0.3, torch.randn(Fd, generator=gen) * 0.1,
                torch.randn(M, Fd, generator=gen) * 0.3, torch.randn(M, generator=gen) * 0.1) for _ in range(E)]
    noise = O.gumbel_noise((S, E), gen)
    out, _ = O.moe_layer(x3, wg, experts, noise, ws=4)
    out1, _ = O.moe_layer(x3, wg, experts, noise, ws=1)
    out2, _ = O.moe_layer(x3, wg, experts, noise, ws=2, rank=1)
    torch.testing.assert_close(out, out1)
    torch.testing.assert_close(out, out2)
    x = x3.reshape(-1, M)
    g = O.top2gating(F.linear(x, wg), noise)
    expect = torch.zeros(S, M)
    for s in range(S):
        for j in range(2):
            if g["keep"][s, j]:
                e = int(g["expert"][s, j])
                expect[s] += g["weight"][s, j] * O.expert_ffn(x[s:s + 1], *experts[e])[0]
    torch.testing.assert_close(out.reshape(S, M), expect, rtol=1e-5, atol=1e-6)


# ---- LM: assembled from stock layers; parameter count of the headline configuration ----
def test_transformer_lm_structure_and_param_count():
    with torch.device("meta"):
        lm = O.TransformerLM(10240, 2048, 32, 2048, 10)
    n = sum(p.numel() for p in lm.parameters())
    per_layer = (3 * 2048 * 2048 + 3 * 2048 + 2048 * 2048 + 2048) + 2 * 2 * 2048 + 2 * (2048 * 2048 + 2048)
    assert n == 10240 * 2048 + 10 * per_layer + (2048 * 10240 + 10240) == 293_816_320, n
    small = O.TransformerLM(50, 16, 4, 16, 2)
    ids = torch.randint(0, 50, (7, 3))
    out = small(ids)
    assert out.shape == (7, 3, 50)
    # causal: changing a later token never changes earlier positions
    ids2 = ids.clone()
    ids2[5:] = (ids2[5:] + 1) % 50
    torch.testing.assert_close(small(ids2)[:5], out[:5])


@pytest.mark.parametrize("ws", [2, 4])
def test_transformer_lm_shard_loop_equals_the_unsharded_model(ws):
    """The model evaluated the reference's way (every rotated layer a loop over its shards) is the same function of
    the same parameters: logits, loss and every gradient agree with the stock layers at fp32 defaults."""
    torch.manual_seed(ws)
    a = O.TransformerLM(48, 16, 4, 24, 2)
    b = O.TransformerLM(48, 16, 4, 24, 2, ws=ws, shard_loop=True)
    b.load_state_dict(a.state_dict())
    ids, tgt = torch.randint(0, 48, (7, 3)), torch.randint(0, 48, (7, 3))
    la, lb = a(ids), b(ids)
    torch.testing.assert_close(lb, la)
    torch.nn.functional.cross_entropy(la.view(-1, 48), tgt.view(-1)).backward()
    torch.nn.functional.cross_entropy(lb.view(-1, 48), tgt.view(-1)).backward()
    for (n, pa), (_, pb) in zip(a.named_parameters(), b.named_parameters()):
        torch.testing.assert_close(pb.grad, pa.grad, msg=lambda m, n=n: f"{n}: {m}")


@pytest.mark.parametrize("ws", [1, 2, 4])
@pytest.mark.parametrize("stride,padding,dilation", [(1, 0, 1), (2, 1, 1), ((1, 2), (2, 0), (2, 1))])
def test_column_conv2d_matches_unsharded_conv_and_patch_product(ws, stride, padding, dilation):
    """Shards along the output channels concatenate to stock conv2d (the reference's oracle for its Conv2d rule,
    test_net.py); the patch matrix times the flattened weight is the same convolution; its transpose is F.fold."""
    torch.manual_seed(ws)
    x = torch.randn(2, 3, 9, 8, dtype=torch.float64)
    conv = torch.nn.Conv2d(3, 8, (3, 2), stride, padding, dilation).double()
    ref = conv(x)
    out = O.column_parallel_conv2d(x, conv.weight.detach(), conv.bias.detach(), ws, stride, padding, dilation)
    assert torch.allclose(out, ref, rtol=1e-12, atol=1e-12)
    p = O.conv_patches(x, (3, 2), conv.stride, conv.padding, conv.dilation)
    y = (p @ conv.weight.detach().view(8, -1).T + conv.bias.detach()).view(2, ref.shape[2], ref.shape[3], 8)
    assert torch.allclose(y.permute(0, 3, 1, 2), ref, rtol=1e-12, atol=1e-12)
    # fold is the transpose of the patch map: <patches(x), g> == <x, fold(g)>
    g = torch.randn_like(p)
    lhs = (p * g).sum()
    rhs = (x * O.conv_fold(g, x.shape, (3, 2), conv.stride, conv.padding, conv.dilation)).sum()
    assert abs(float(lhs - rhs)) < 1e-9 * max(1.0, abs(float(lhs)))


def test_conv_patches_layout_by_loops():
    """Row (n, ho, wo), column (ci, i, j), zeros outside the image: python loops on a tiny input."""
    x = torch.arange(2 * 2 * 4 * 5, dtype=torch.float32).view(2, 2, 4, 5) + 1
    kh, kw, sh, sw, ph, pw, dh, dw = 2, 3, 2, 1, 1, 2, 1, 2
    ho = (4 + 2 * ph - dh * (kh - 1) - 1) // sh + 1
    wo = (5 + 2 * pw - dw * (kw - 1) - 1) // sw + 1
    p = O.conv_patches(x, (kh, kw), (sh, sw), (ph, pw), (dh, dw))
    assert p.shape == (2 * ho * wo, 2 * kh * kw)
    for n in range(2):
        for a in range(ho):
            for b in range(wo):
                for ci in range(2):
                    for i in range(kh):
                        for j in range(kw):
                            h, w = a * sh - ph + i * dh, b * sw - pw + j * dw
                            want = float(x[n, ci, h, w]) if 0 <= h < 4 and 0 <= w < 5 else 0.0
                            assert float(p[(n * ho + a) * wo + b, (ci * kh + i) * kw + j]) == want


@pytest.mark.parametrize("ws", [2, 4])
def test_gloo_ring_column_linear_equals_unsharded_linear(ws):
    """The reference's actual execution (ws gloo ranks, shards travelling the ring with their gradients) restated in
    oracle/gloo_ring.py gives torch.nn.functional.linear on the unsharded problem: outputs, input gradients and the
    gathered weight / bias gradients (the comparison of the reference's tests/test_linear.py:134-165)."""
    from oracle import gloo_ring
    gen = torch.Generator().manual_seed(ws)
    x, w, b = torch.randn(8 * ws, 12, generator=gen), torch.randn(4 * ws, 12, generator=gen), torch.randn(4 * ws, generator=gen)
    dy = torch.randn(8 * ws, 4 * ws, generator=gen)
    res = gloo_ring.column_linear_ring(x, w, b, dy, ws=ws, steps=2)
    xr, wr, br = x.clone().requires_grad_(), w.clone().requires_grad_(), b.clone().requires_grad_()
    y = torch.nn.functional.linear(xr, wr, br)
    y.backward(dy)
    torch.testing.assert_close(res["y"], y.detach())
    torch.testing.assert_close(res["dx"], xr.grad)
    torch.testing.assert_close(res["dw"], wr.grad)
    torch.testing.assert_close(res["db"], br.grad)
    assert len(res["times"]) == 2 and all(t > 0 for t in res["times"])
    # and the one-process shard loop used by the device parity tests agrees with it
    torch.testing.assert_close(O.column_parallel_linear(x, w, b, ws), res["y"])


# ---- LM against the reference's own TransformerLM on a 2-rank gloo ring (tests/golden/make_lm_golden.py) ----
@pytest.mark.parametrize("name", ["lm_ws2.npz", "lm_moe_ws2.npz"])
def test_transformer_lm_matches_reference_golden(name):
    """Logits, loss (and l_aux) of each rank's batch; every home-shard gradient == the matching slice of the
    gradient of the SUM of the ranks' losses; LayerNorm gradients == the gradient of that rank's loss alone."""
    import lm_golden as G
    fix = G.load(name)
    c = fix["cfg"]
    ref = G.oracle_lm(fix)
    per_rank_ln = []
    total = {}
    for r in range(c["WS"]):
        for p in ref.parameters():
            p.grad = None
        logits = ref(fix["ids"][r])
        torch.testing.assert_close(logits, fix[f"rank{r}.logits"])
        loss = F.cross_entropy(logits.view(-1, c["V"]), fix["tgt"][r].view(-1))
        if c["moe"]:
            l_aux = torch.stack([ref[2 + i].l_aux for i in range(c["NDEC"])])
            torch.testing.assert_close(l_aux, fix[f"rank{r}.l_aux"])
            loss = loss + l_aux.sum()
        torch.testing.assert_close(loss, fix[f"rank{r}.loss"])
        loss.backward()
        g = {k: v.clone() for k, v in G.oracle_full_grads(ref, c).items()}
        per_rank_ln.append({k: v for k, v in g.items() if ".ln" in k})
        for k, v in g.items():
            total[k] = total[k] + v if k in total else v
    for r in range(c["WS"]):
        for k, v in G.shard_slices(total, c, r).items():
            torch.testing.assert_close(fix[f"rank{r}.grad.{k}"], v, msg=lambda m, k=k, r=r: f"rank {r} {k}: {m}")
        for k, v in per_rank_ln[r].items():
            torch.testing.assert_close(fix[f"rank{r}.grad.{k}"], v, msg=lambda m, k=k, r=r: f"rank {r} {k}: {m}")


def test_transformer_lm_golden_catches_structural_mistakes():
    """The fixture separates the reference's structure from near misses: no sqrt(ninp) scale, sin/cos swapped in the
    positions, pre-LN blocks -- each moves the logits far outside the comparison's tolerance."""
    import lm_golden as G
    fix = G.load("lm_ws2.npz")
    ref = G.oracle_lm(fix)
    want = fix["rank0.logits"]
    ids = fix["ids"][0]

    def run(scale=True, swap_pe=False, pre_ln=False):
        x = ref[0](ids) * (math.sqrt(ref.ninp) if scale else 1.0)
        pe = ref[1].pe[: x.size(0), :]
        if swap_pe:
            pe = torch.stack([pe[..., 1::2], pe[..., 0::2]], dim=-1).flatten(-2)
        x = x + pe
        for d in list(ref)[2:-1]:
            L = x.shape[0]
            mask = torch.triu(torch.full((L, L), float("-inf")), diagonal=1)
            if pre_ln:
                h = d.norm1(x)
                x = x + d.self_attn(h, h, h, attn_mask=mask, need_weights=False)[0]
                x = x + d._ff(d.norm2(x))
            else:
                x = d.norm1(x + d.self_attn(x, x, x, attn_mask=mask, need_weights=False)[0])
                x = d.norm2(x + d._ff(x))
        return ref[-1](x)

    torch.testing.assert_close(run(), want)
    for kw in (dict(scale=False), dict(swap_pe=True), dict(pre_ln=True)):
        assert (run(**kw) - want).abs().max() > 1e-2, kw
