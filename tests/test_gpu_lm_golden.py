"""The rotated TransformerLM on the GPU against golden vectors written from the reference's own TransformerLM run on a
2-rank gloo ring (tests/golden/lm_ws2.npz, lm_moe_ws2.npz; script tests/golden/make_lm_golden.py).

The reference's two ranks each fed their own batch; here the one device runs the two batches one after the other and
lets the second backward accumulate, which is what the ring's travelling partial sums add up to: every home-shard
gradient == the fixture's, LayerNorm gradients == the sum of the two ranks' (the reference never reduces them)."""
import pytest
import torch
import torch.nn.functional as F

import lm_golden as G
from gpu_util import DEV, TOL, rel_err

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("rotation_window")]


def build_rotated(fix, dtype):
    from rtp_amd.models.transformer_lm_rtp import TransformerLM
    c = fix["cfg"]
    ref = G.oracle_lm(fix)  # holder of the unsharded weights with stock-layer attribute names
    lm = TransformerLM(c["V"], c["D"], c["H"], c["FF"], 0.0, 0.1, c["NDEC"], c["WS"], 0, is_moe=c["moe"],
                       device=DEV, dtype=dtype)
    with torch.no_grad():
        for sh in lm[0].embedding.embeddings:
            sh.affine_weight(ref[0])
        for sh in lm[-1].linear.linears:
            sh.affine_weight(ref[-1])
        for i in range(c["NDEC"]):
            dec, rdec = lm[2 + i], ref[2 + i]
            for sh in dec.self_attn.layers:
                sh.affine_weight(rdec.self_attn)
            for a, b in ((dec.norm1, rdec.norm1), (dec.norm2, rdec.norm2)):
                a.weight.copy_(b.weight), a.bias.copy_(b.bias)
            if c["moe"]:
                for s in range(c["WS"]):
                    dec.gate.wgs[s].weight.copy_(torch.chunk(rdec.wg.weight, c["WS"], 0)[s])
                    e = dec.moe_layer.experts_list[s][0]
                    e.linear1.weight.copy_(rdec.experts[s][0].weight), e.linear1.bias.copy_(rdec.experts[s][0].bias)
                    e.linear2.weight.copy_(rdec.experts[s][1].weight), e.linear2.bias.copy_(rdec.experts[s][1].bias)
            else:
                for sh in dec.ff_block.linear1.linears:
                    sh.affine_weight(rdec.linear1)
                for sh in dec.ff_block.linear2.linears:
                    sh.affine_weight(rdec.linear2)
    return lm


def shard_grads(lm, c, r):
    """Gradients of shard r's parameters keyed like the fixture's rank{r}.grad.* entries."""
    out = {"emb": lm[0].embedding.embeddings[r].weight.grad, "head_w": lm[-1].linear.linears[r].weight.grad,
           "head_b": lm[-1].linear.linears[r].bias.grad}
    for i in range(c["NDEC"]):
        dec = lm[2 + i]
        sa = dec.self_attn.layers[r]
        out[f"l{i}.in_w"], out[f"l{i}.in_b"] = sa.in_proj_weight.grad, sa.in_proj_bias.grad
        out[f"l{i}.out_w"], out[f"l{i}.out_b"] = sa.out_proj.weight.grad, sa.out_proj.bias.grad
        if c["moe"]:
            e = dec.moe_layer.experts_list[r][0]
            out[f"l{i}.wg"] = dec.gate.wgs[r].weight.grad
            out[f"l{i}.e_w1"], out[f"l{i}.e_b1"] = e.linear1.weight.grad, e.linear1.bias.grad
            out[f"l{i}.e_w2"], out[f"l{i}.e_b2"] = e.linear2.weight.grad, e.linear2.bias.grad
        else:
            f1, f2 = dec.ff_block.linear1.linears[r], dec.ff_block.linear2.linears[r]
            out[f"l{i}.w1"], out[f"l{i}.b1"] = f1.weight.grad, f1.bias.grad
            out[f"l{i}.w2"], out[f"l{i}.b2"] = f2.weight.grad, f2.bias.grad
    return out


# bf16 runs on the plain model only: at this fixture's width (16) a bf16 rounding of the gate logits or of a 16-wide
# LayerNorm moves the MoE model's first-layer gradients by several percent, which says nothing about the kernels; the
# MoE layer in bf16 is compared at realistic widths in test_gpu_moe.py and test_gpu_full_size.py.
@pytest.mark.parametrize("name,dtype", [("lm_ws2.npz", torch.float32), ("lm_moe_ws2.npz", torch.float32),
                                        ("lm_ws2.npz", torch.bfloat16)])
def test_rotated_lm_matches_reference_golden(name, dtype):
    fix = G.load(name)
    c = fix["cfg"]
    if dtype == torch.bfloat16:
        # start both sides from bf16-representable weights: the comparison then measures the arithmetic
        for k, v in list(fix.items()):
            if torch.is_tensor(v) and v.dtype == torch.float32 and not k.startswith("rank"):
                fix[k] = v.to(torch.bfloat16).float()
    lm = build_rotated(fix, dtype)
    tol = TOL[dtype]
    if dtype == torch.bfloat16:
        # the fixture was computed from the unrounded weights: recompute its outputs with the oracle on the rounded ones
        ref = G.oracle_lm(fix)
    for r in range(c["WS"]):
        ids, tgt = fix["ids"][r].to(DEV), fix["tgt"][r].to(DEV)
        logits = lm(ids)
        loss = F.cross_entropy(logits.float().view(-1, c["V"]), tgt.view(-1))
        if c["moe"]:
            l_aux = torch.stack([lm[2 + i].moe_layer.l_aux.float() for i in range(c["NDEC"])])
            loss = loss + l_aux.sum()
        loss.backward()
        if dtype == torch.float32:
            want_logits, want_loss = fix[f"rank{r}.logits"], fix[f"rank{r}.loss"]
            if c["moe"]:
                assert rel_err(l_aux, fix[f"rank{r}.l_aux"]) <= 1e-5
        else:
            want_logits = ref(fix["ids"][r])
            want_loss = F.cross_entropy(want_logits.view(-1, c["V"]), fix["tgt"][r].view(-1))
            if c["moe"]:
                want_loss = want_loss + sum(ref[2 + i].l_aux for i in range(c["NDEC"]))
            want_loss.backward()  # accumulates over the ranks, like the rotated model
        assert rel_err(logits, want_logits) <= tol, f"rank {r} logits"
        assert abs(float(loss) - float(want_loss)) <= tol * abs(float(want_loss)), f"rank {r} loss"
    errs = {}
    if dtype == torch.float32:
        for r in range(c["WS"]):
            for k, g in shard_grads(lm, c, r).items():
                errs[f"rank{r}.{k}"] = rel_err(g, fix[f"rank{r}.grad.{k}"])
        for i in range(c["NDEC"]):
            for nm, mod in (("ln1", lm[2 + i].norm1), ("ln2", lm[2 + i].norm2)):
                for suffix, p in (("w", mod.weight), ("b", mod.bias)):
                    want = sum(fix[f"rank{r}.grad.l{i}.{nm}_{suffix}"] for r in range(c["WS"]))
                    errs[f"l{i}.{nm}_{suffix}"] = rel_err(p.grad, want)
    else:
        full = G.oracle_full_grads(ref, c)
        for r in range(c["WS"]):
            want = G.shard_slices(full, c, r)
            for k, g in shard_grads(lm, c, r).items():
                errs[f"rank{r}.{k}"] = rel_err(g, want[k])
        for i in range(c["NDEC"]):
            for nm, mod in (("ln1", lm[2 + i].norm1), ("ln2", lm[2 + i].norm2)):
                errs[f"l{i}.{nm}_w"] = rel_err(mod.weight.grad, full[f"l{i}.{nm}_w"])
                errs[f"l{i}.{nm}_b"] = rel_err(mod.bias.grad, full[f"l{i}.{nm}_b"])
    # the north-star bounds: 1e-5 in fp32, 2e-2 in bf16
    limit = 1e-5 if dtype == torch.float32 else 2e-2
    bad = {k: f"{v:.2e}" for k, v in errs.items() if v > limit}
    assert not bad, bad
