"""The rotated TransformerLM (rtp_amd.models.transformer_lm_rtp) vs the oracle LM assembled from stock
torch layers: loss, logits and every gradient, fp32 and bf16; the SGD step; peak weight accounting."""
import math

import pytest
import torch
import torch.nn.functional as F

from gpu_util import DEV, assert_close, rel_err
from oracle import rtp_oracle as O

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("rotation_window")]


def load_unsharded(lm, ref):
    """Copy the oracle LM's weights into the rotated LM shard by shard (the *_layer= import rules)."""
    with torch.no_grad():
        for sh in lm[0].embedding.embeddings:
            sh.affine_weight(ref[0])
        n_dec = len(lm) - 3
        for i in range(n_dec):
            dec, rdec = lm[2 + i], ref[2 + i]
            for sh in dec.self_attn.layers:
                sh.affine_weight(rdec.self_attn)
            for sh in dec.ff_block.linear1.linears:
                sh.affine_weight(rdec.linear1)
            for sh in dec.ff_block.linear2.linears:
                sh.affine_weight(rdec.linear2)
            for a, b in ((dec.norm1, rdec.norm1), (dec.norm2, rdec.norm2)):
                a.weight.copy_(b.weight), a.bias.copy_(b.bias)
        for sh in lm[-1].linear.linears:
            sh.affine_weight(ref[-1])


def gathered_grads(lm, ws):
    """Unsharded gradients rebuilt with the reference tests' gather rules."""
    out = {"emb": torch.cat([s.weight.grad for s in lm[0].embedding.embeddings], 1)}
    for i in range(len(lm) - 3):
        dec = lm[2 + i]
        sa = dec.self_attn.layers
        out[f"l{i}.in_w"] = O.attention_grad_reinterleave([s.in_proj_weight.grad for s in sa], ws)
        out[f"l{i}.in_b"] = O.attention_grad_reinterleave([s.in_proj_bias.grad for s in sa], ws)
        out[f"l{i}.out_w"] = torch.cat([s.out_proj.weight.grad for s in sa], 1)
        out[f"l{i}.out_b"] = sa[0].out_proj.bias.grad
        out[f"l{i}.w1"] = torch.cat([s.weight.grad for s in dec.ff_block.linear1.linears], 0)
        out[f"l{i}.b1"] = torch.cat([s.bias.grad for s in dec.ff_block.linear1.linears], 0)
        out[f"l{i}.w2"] = torch.cat([s.weight.grad for s in dec.ff_block.linear2.linears], 0)
        out[f"l{i}.b2"] = torch.cat([s.bias.grad for s in dec.ff_block.linear2.linears], 0)
        out[f"l{i}.ln1"] = dec.norm1.weight.grad
        out[f"l{i}.ln2"] = dec.norm2.weight.grad
    out["head_w"] = torch.cat([s.weight.grad for s in lm[-1].linear.linears], 0)
    out["head_b"] = torch.cat([s.bias.grad for s in lm[-1].linear.linears], 0)
    return out


def ref_grads(ref):
    out = {"emb": ref[0].weight.grad}
    for i in range(len(ref) - 3):
        d = ref[2 + i]
        out[f"l{i}.in_w"], out[f"l{i}.in_b"] = d.self_attn.in_proj_weight.grad, d.self_attn.in_proj_bias.grad
        out[f"l{i}.out_w"], out[f"l{i}.out_b"] = d.self_attn.out_proj.weight.grad, d.self_attn.out_proj.bias.grad
        out[f"l{i}.w1"], out[f"l{i}.b1"] = d.linear1.weight.grad, d.linear1.bias.grad
        out[f"l{i}.w2"], out[f"l{i}.b2"] = d.linear2.weight.grad, d.linear2.bias.grad
        out[f"l{i}.ln1"], out[f"l{i}.ln2"] = d.norm1.weight.grad, d.norm2.weight.grad
    out["head_w"], out["head_b"] = ref[-1].weight.grad, ref[-1].bias.grad
    return out


def build_pair(V, D, H, Fd, n_dec, ws, dtype, seed=0):
    from rtp_amd.models.transformer_lm_rtp import TransformerLM
    torch.manual_seed(seed)
    ref = O.TransformerLM(V, D, H, Fd, n_dec)
    with torch.no_grad():
        for name, p in ref.named_parameters():
            if "norm" not in name:
                p.uniform_(-0.1, 0.1)
        ref[-1].bias.zero_()
        if dtype != torch.float32:
            # bf16 vs fp32 differ by ~2^-9 per activation; a ReLU input that close to zero flips its mask and
            # moves a whole weight-gradient column by O(1/sqrt(tokens)).  Keep the pre-activations away from
            # the kink (half the units well inside the active side, half well inside the inactive side) so the
            # comparison measures rounding, not the discontinuity; the fp32 cases exercise ReLU at random signs.
            for i in range(n_dec):
                b = ref[2 + i].linear1.bias
                b.copy_(torch.where(torch.arange(b.numel()) % 2 == 0, 1.5, -1.5))
            # both sides start from the same representable values
            for p in ref.parameters():
                p.copy_(p.to(dtype).float())
    lm = TransformerLM(V, D, H, Fd, 0.0, 0.1, n_dec, ws, 0, device=DEV, dtype=dtype)
    load_unsharded(lm, ref)
    return lm, ref


@pytest.mark.parametrize("dtype,ws", [(torch.float32, 4), (torch.float32, 1), (torch.bfloat16, 4)])
def test_lm_loss_and_grads(dtype, ws):
    V, D, H, Fd, n_dec, L, N = 96, 64, 4, 64, 2, 12, 5
    lm, ref = build_pair(V, D, H, Fd, n_dec, ws, dtype)
    gen = torch.Generator().manual_seed(1)
    ids = torch.randint(0, V, (L, N), generator=gen)
    tgt = torch.randint(0, V, (L, N), generator=gen)
    logits = lm(ids.to(DEV))
    loss = F.cross_entropy(logits.float().view(-1, V), tgt.to(DEV).view(-1))
    loss.backward()
    ref_logits = ref(ids)
    ref_loss = F.cross_entropy(ref_logits.view(-1, V), tgt.view(-1))
    ref_loss.backward()
    assert_close(logits, ref_logits, dtype, "logits")
    assert abs(float(loss) - float(ref_loss)) <= (1e-5 if dtype == torch.float32 else 2e-2) * abs(float(ref_loss))
    mine, theirs = gathered_grads(lm, ws), ref_grads(ref)
    errs = {k: rel_err(mine[k], theirs[k]) for k in theirs}
    print({k: f"{v:.1e}" for k, v in errs.items()})
    # the north-star bounds: 1e-5 in fp32, 2e-2 in bf16
    limit = 1e-5 if dtype == torch.float32 else 2e-2
    for k, err in errs.items():
        assert err <= limit, f"{k}: {err:.3e}"


def test_lm_sgd_step_matches_closed_form():
    from rtp_amd.optim import RotatedSGD
    V, D, H, Fd, n_dec, L, N, ws = 64, 32, 2, 32, 1, 6, 3, 2
    lm, ref = build_pair(V, D, H, Fd, n_dec, ws, torch.float32, seed=2)
    opt = RotatedSGD(lm, lr=0.1)
    ids = torch.randint(0, V, (L, N))
    before = lm[-1].linear.linears[1].weight.detach().clone()
    F.cross_entropy(lm(ids.to(DEV)).view(-1, V), ids.to(DEV).view(-1)).backward()
    g = lm[-1].linear.linears[1].weight.grad.detach().clone()
    ln_before, ln_g = lm[2].norm1.weight.detach().clone(), lm[2].norm1.weight.grad.detach().clone()
    opt.step()
    assert torch.equal(lm[-1].linear.linears[1].weight.detach(), before - 0.1 * g)
    assert torch.equal(lm[2].norm1.weight.detach(), ln_before - 0.1 * ln_g)
    # zero_grad keeps the gradient views attached and makes the next backward overwrite them
    opt.zero_grad()
    assert not lm[2].norm1.weight.grad.any()  # a zeroed slice of the optimiser's flat gradient buffer
    F.cross_entropy(lm(ids.to(DEV)).view(-1, V), ids.to(DEV).view(-1)).backward()
    g2 = lm[-1].linear.linears[1].weight.grad.detach().clone()
    opt.zero_grad()
    F.cross_entropy(lm(ids.to(DEV)).view(-1, V), ids.to(DEV).view(-1)).backward()
    assert torch.equal(lm[-1].linear.linears[1].weight.grad, g2)  # overwritten, not accumulated


def test_lm_bf16_master_weights_and_weight_bytes():
    from rtp_amd import rotated_weight_bytes, staging_bytes
    from rtp_amd.optim import RotatedSGD
    V, D, H, Fd, n_dec, L, N, ws = 64, 32, 4, 32, 1, 6, 3, 4
    lm, _ = build_pair(V, D, H, Fd, n_dec, ws, torch.bfloat16, seed=3)
    opt = RotatedSGD(lm, lr=0.5, clip_value=0.05)
    ids = torch.randint(0, V, (L, N)).to(DEV)
    w = lm[-1].linear.linears[0].weight
    master = opt.masters[-1].view(ws, -1)[0][: w.numel()].view_as(w).clone()
    F.cross_entropy(lm(ids).float().view(-1, V), ids.view(-1)).backward()
    g = w.grad.float().clamp(-0.05, 0.05)
    opt.step()
    expect = master - 0.5 * g
    assert torch.equal(w.detach(), expect.to(torch.bfloat16))
    n_rot = sum(p.numel() for n, p in lm.named_parameters() if "norm" not in n)
    assert rotated_weight_bytes(lm) == 2 * n_rot  # every shard resident exactly once, in bf16
    largest = max(m._store.numel for m in lm.modules() if hasattr(m, "_store")) * 2
    from rtp_amd import ring
    if ring.rotation_mode() == "staged":
        assert staging_bytes() >= 2 * largest


def test_lm_moe_variant_runs_and_backprops():
    from rtp_amd.models.transformer_lm_rtp import TransformerLM
    lm = TransformerLM(64, 32, 4, 48, 0.0, 0.1, 1, 4, 0, is_moe=True, device=DEV)
    ids = torch.randint(0, 64, (8, 4)).to(DEV)  # 32 tokens over 4 experts
    out = lm(ids)
    assert out.shape == (8, 4, 64) and torch.isfinite(out).all()
    (out.float().mean() + lm[2].moe_layer.l_aux).backward()
    for p in lm.parameters():
        assert p.grad is not None and torch.isfinite(p.grad).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_lm_sgd_overlapped_with_backward_is_bit_identical(dtype):
    """overlap_backward=True updates each rotated layer right after its backward on a second stream; after
    step() every weight, master and gradient equals the sequential optimiser's, step after step."""
    from rtp_amd.optim import RotatedSGD
    V, D, H, Fd, n_dec, L, N, ws = 64, 32, 4, 64, 2, 6, 3, 4
    lm_a, _ = build_pair(V, D, H, Fd, n_dec, ws, dtype, seed=5)
    lm_b, _ = build_pair(V, D, H, Fd, n_dec, ws, dtype, seed=5)
    opt_a = RotatedSGD(lm_a, lr=0.05, clip_value=0.05)
    opt_b = RotatedSGD(lm_b, lr=0.05, clip_value=0.05, overlap_backward=True)
    gen = torch.Generator().manual_seed(0)
    for step in range(3):
        ids = torch.randint(0, V, (L, N), generator=gen).to(DEV)
        for lm, opt in ((lm_a, opt_a), (lm_b, opt_b)):
            opt.zero_grad()
            F.cross_entropy(lm(ids).float().view(-1, V), ids.view(-1)).backward()
            opt.step()
        torch.cuda.synchronize()
        for (na, pa), (nb, pb) in zip(lm_a.named_parameters(), lm_b.named_parameters()):
            assert na == nb and torch.equal(pa, pb), f"step {step}: {na} differs"
            assert torch.equal(pa.grad, pb.grad), f"step {step}: grad of {na} differs"
        for ma, mb in zip(opt_a.masters, opt_b.masters):
            assert (ma is None and mb is None) or torch.equal(ma, mb)


def test_lm_sgd_overlap_rejects_gradient_accumulation():
    from rtp_amd.optim import RotatedSGD
    V, D, H, Fd, n_dec, L, N, ws = 64, 32, 2, 32, 1, 6, 3, 2
    lm, _ = build_pair(V, D, H, Fd, n_dec, ws, torch.float32, seed=6)
    opt = RotatedSGD(lm, lr=0.1, overlap_backward=True)
    ids = torch.randint(0, V, (L, N)).to(DEV)
    F.cross_entropy(lm(ids).view(-1, V), ids.view(-1)).backward()
    with pytest.raises(RuntimeError):
        F.cross_entropy(lm(ids).view(-1, V), ids.view(-1)).backward()
    opt.step()
    torch.cuda.synchronize()


def test_lm_weight_gradients_on_second_stream_are_bit_identical():
    """ring.set_wgrad_overlap(True) moves the parameter-gradient launches to a second stream that rejoins at
    the end of the backward pass: same gradients, bit for bit, readable right after backward()."""
    from rtp_amd import ring
    V, D, H, Fd, n_dec, L, N, ws = 64, 32, 4, 64, 2, 6, 3, 4
    lm_a, _ = build_pair(V, D, H, Fd, n_dec, ws, torch.bfloat16, seed=7)
    lm_b, _ = build_pair(V, D, H, Fd, n_dec, ws, torch.bfloat16, seed=7)
    ids = torch.randint(0, V, (L, N)).to(DEV)
    F.cross_entropy(lm_a(ids).float().view(-1, V), ids.view(-1)).backward()
    ring.set_wgrad_overlap(True)
    try:
        for _ in range(2):
            for p in lm_b.parameters():
                p.grad = None
            F.cross_entropy(lm_b(ids).float().view(-1, V), ids.view(-1)).backward()
    finally:
        ring.set_wgrad_overlap(False)
    for (na, pa), (nb, pb) in zip(lm_a.named_parameters(), lm_b.named_parameters()):
        assert torch.equal(pa.grad, pb.grad), f"grad of {na} differs"


def test_lm_rank_state_dicts_round_trip_on_device():
    """Per-rank state dicts in the reference's layout, saved from one LM and loaded into another: same logits bit for
    bit; the optimiser's fp32 masters re-read; the MoE variant's expert and gate keys."""
    from rtp_amd.checkpoint import load_rank_state_dicts, rank_state_dict
    from rtp_amd.models.transformer_lm_rtp import TransformerLM
    from rtp_amd.optim import RotatedSGD
    V, D, H, Fd, n_dec, L, N, ws = 64, 32, 4, 32, 1, 6, 3, 4
    a, _ = build_pair(V, D, H, Fd, n_dec, ws, torch.bfloat16, seed=7)
    b, _ = build_pair(V, D, H, Fd, n_dec, ws, torch.bfloat16, seed=8)
    opt_b = RotatedSGD(b, lr=0.1)
    ids = torch.randint(0, V, (L, N)).to(DEV)
    assert not torch.equal(a(ids), b(ids))
    dicts = [{k: v.detach().cpu().clone() for k, v in rank_state_dict(a, r).items()} for r in range(ws)]
    assert "2.self_attn.MultiheadAttention.in_proj_weight" in dicts[1] and "0.embedding.embedding.weight" in dicts[1]
    assert f"{len(a) - 1}.linear.linear.bias" in dicts[1]
    load_rank_state_dicts(b, dicts)
    assert torch.equal(a(ids), b(ids))
    opt_b.reload_masters()
    for st, master in zip(opt_b.stores, opt_b.masters):
        assert torch.equal(master.view(-1).to(torch.bfloat16), st.home.view(-1))
    moe = TransformerLM(64, 32, 4, 48, 0.0, 0.1, 1, 4, 0, is_moe=True, device=DEV)
    keys = list(rank_state_dict(moe, 3).keys())
    assert any(k.endswith("moe_layer.gate.wg.weight") for k in keys), keys
    assert any(".moe_layer.experts.0." in k for k in keys), keys
    assert not any(".shards." in k for k in keys)
    moe2 = TransformerLM(64, 32, 4, 48, 0.0, 0.1, 1, 4, 0, is_moe=True, device=DEV)
    load_rank_state_dicts(moe2, [rank_state_dict(moe, r) for r in range(4)])
    for (ka, ta), (kb, tb) in zip(moe.state_dict().items(), moe2.state_dict().items()):
        assert ka == kb and torch.equal(ta, tb)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_lm_embedding_scale_and_positions_on_the_gather_are_bit_identical(dtype):
    """The model lets the embedding gather apply * sqrt(ninp) and + pe (transformer_lm_rtp.py:27-28, :49).  A twin
    whose embedding layer has not adopted the positional layer runs the three steps as the reference does (gather,
    multiply, add: separate operations); logits and every gradient must be the same bits."""
    V, D, H, Fd, n_dec, L, N = 96, 64, 4, 64, 2, 12, 5
    gen = torch.Generator().manual_seed(1)
    ids = torch.randint(0, V, (L, N), generator=gen).to(DEV)
    tgt = torch.randint(0, V, (L, N), generator=gen).to(DEV)
    results = []
    for fused in (True, False):
        lm, _ = build_pair(V, D, H, Fd, n_dec, 4, dtype)
        assert lm[1].added_upstream and lm[0].positional is lm[1]
        if not fused:
            object.__setattr__(lm[0], "positional", None)
            lm[1].added_upstream = False
        logits = lm(ids)
        F.cross_entropy(logits.float().view(-1, V), tgt.view(-1)).backward()
        results.append((logits.detach(), gathered_grads(lm, 4)))
    assert torch.equal(results[0][0], results[1][0])
    for k, g in results[0][1].items():
        assert torch.equal(g, results[1][1][k]), k


def graph_replays_against_eager_twin(twin_lms, V, L, N, replays, lr=1e-2, fused_replayed=False):
    """Record one whole training step of twin_lms[0] into a HIP graph and replay it `replays` times with new token ids,
    eager work and synchronisation in between; twin_lms[1] (same weights) takes the same steps eagerly.  Losses and
    all weights must stay bit-identical.  `fused_replayed`: the replayed twin applies clip + SGD in the epilogues of
    its weight-gradient products while the eager twin keeps the separate update launch."""
    from rtp_amd import ring
    from rtp_amd.module.loss import cross_entropy
    from rtp_amd.optim import RotatedSGD
    twins = [(lm, RotatedSGD(lm, lr=lr, clip_value=0.05, fused_backward=fused_replayed and i == 0))
             for i, lm in enumerate(twin_lms)]
    gen = torch.Generator().manual_seed(5)
    ids = torch.randint(0, V, (L, N), generator=gen).to(DEV)
    tgt = torch.randint(0, V, (L, N), generator=gen).to(DEV)
    losses = [None, None]

    def step(i):
        lm, opt = twins[i]
        opt.zero_grad()
        loss = cross_entropy(lm(ids).view(-1, V), tgt.view(-1))
        loss.backward()
        opt.step()
        losses[i] = loss.detach()

    def same_state(what):
        assert torch.equal(losses[0], losses[1]), what
        for (na, pa), (_, pb) in zip(twins[0][0].named_parameters(), twins[1][0].named_parameters()):
            assert torch.equal(pa, pb), f"{what}: {na}"

    # both twins take their first step eagerly on a side stream (gradient accumulators are created there)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(0)
        step(1)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    ring.fence(DEV)
    same_state("first eager step")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(0)
    ring.fence(DEV)
    # the capture recorded the step without running it: twin 0 is still one step behind until the first replay
    for r in range(replays):
        if r:
            ids.copy_(torch.randint(0, V, (L, N), generator=gen))
            tgt.copy_(torch.randint(0, V, (L, N), generator=gen))
        graph.replay()
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            step(1)
        torch.cuda.synchronize()
        same_state(f"replay {r}")
        _ = (twins[0][0][2].norm1.weight.float() * 2).sum().item()  # unrelated eager work between replays
    return float(losses[0])


@pytest.mark.parametrize("overlap", [False, True])
def test_lm_step_replayed_from_a_graph_matches_eager_steps(overlap):
    """The whole training step (zero grads, forward, cross-entropy, backward on both streams, clip + SGD, the rotation
    copies on their side stream) recorded once into a HIP graph, as the benchmark times it: every replay must leave
    exactly the weights and the loss that a twin model reaches by taking the same steps eagerly."""
    from rtp_amd import ring
    V, D, H, Fd, n_dec, L, N, ws = 96, 64, 4, 64, 2, 12, 5, 4
    before = ring.wgrad_overlap()
    ring.set_wgrad_overlap(overlap)
    try:
        twins = [build_pair(V, D, H, Fd, n_dec, ws, torch.bfloat16)[0] for _ in range(2)]
        graph_replays_against_eager_twin(twins, V, L, N, replays=4)
    finally:
        ring.set_wgrad_overlap(before)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("wgrad_overlap", [False, True])
def test_lm_sgd_fused_into_weight_gradient_products_is_bit_identical(dtype, wgrad_overlap):
    """fused_backward=True applies clip + SGD in the epilogue of every weight-gradient product (the gradient is
    never stored); after step() every weight and master equals the sequential optimiser's, step after step, and
    with keep_grads=True so does every gradient."""
    from rtp_amd import ring
    from rtp_amd.optim import RotatedSGD
    # more than 256 tokens and widths of whole 16-byte vectors: the products take the kernel that carries the update
    V, D, H, Fd, n_dec, L, N, ws = 128, 64, 4, 128, 2, 16, 20, 4
    lms = [build_pair(V, D, H, Fd, n_dec, ws, dtype, seed=5)[0] for _ in range(3)]
    opts = [RotatedSGD(lms[0], lr=0.05, clip_value=0.05),
            RotatedSGD(lms[1], lr=0.05, clip_value=0.05, fused_backward=True),
            RotatedSGD(lms[2], lr=0.05, clip_value=0.05, fused_backward=True, keep_grads=True)]
    gen = torch.Generator().manual_seed(0)
    ring.set_wgrad_overlap(wgrad_overlap)
    try:
        for step in range(3):
            ids = torch.randint(0, V, (L, N), generator=gen).to(DEV)
            for lm, opt in zip(lms, opts):
                if step == 1:     # a schedule: the fused epilogues must follow the optimiser's current scalars
                    opt.lr, opt.clip_value = 0.02, 0.03
                opt.zero_grad()
                F.cross_entropy(lm(ids).float().view(-1, V), ids.view(-1)).backward()
                opt.step()
            torch.cuda.synchronize()
            for other, opt_o, grads_too in ((lms[1], opts[1], False), (lms[2], opts[2], True)):
                for (na, pa), (nb, pb) in zip(lms[0].named_parameters(), other.named_parameters()):
                    assert na == nb and torch.equal(pa, pb), f"step {step}: {na} differs"
                    if grads_too:
                        assert torch.equal(pa.grad, pb.grad), f"step {step}: grad of {na} differs"
                for ma, mb in zip(opts[0].masters, opt_o.masters):
                    assert (ma is None and mb is None) or torch.equal(ma, mb)
    finally:
        ring.set_wgrad_overlap(False)
    # the products did cover the weight matrices: what step() still updates is a small remainder
    n_all = sum(st.world_size * st.numel for st in opts[1].stores)
    assert 0 < opts[1]._rest_params < 0.35 * n_all


def test_lm_sgd_fused_rejects_gradient_accumulation():
    from rtp_amd.optim import RotatedSGD
    V, D, H, Fd, n_dec, L, N, ws = 64, 32, 2, 32, 1, 6, 3, 2
    lm, _ = build_pair(V, D, H, Fd, n_dec, ws, torch.float32, seed=2)
    RotatedSGD(lm, lr=0.1, fused_backward=True)
    ids = torch.randint(0, V, (L, N)).to(DEV)
    F.cross_entropy(lm(ids).view(-1, V), ids.view(-1)).backward()
    with pytest.raises(RuntimeError, match="fused_backward"):
        F.cross_entropy(lm(ids).view(-1, V), ids.view(-1)).backward()
