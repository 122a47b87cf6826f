"""Writes tests/golden/lm_ws2.npz and tests/golden/lm_moe_ws2.npz: ids, targets, master weights, logits, losses and
every home-shard gradient of the reference's own TransformerLM (rtp/models/transformer_lm_rtp.py:19-242) run on a
2-rank gloo ring on CPU -- once with the column-parallel feed-forward block, once with is_moe=True (one expert per
rank, E = 2, so the Gumbel noise cannot change the routing).

Run in the build container only (needs the reference tree on disk):
    python tests/golden/make_lm_golden.py /root/reference

Every rank builds the model, then imports its home shards from seeded stock torch layers through the reference's own
`affine_weight` methods (the in-projection of its attention is torch.empty otherwise, rtp/module/attention.py:57,64).
Each rank feeds its OWN batch; its loss is the cross-entropy of its logits (+ the sum of the layers' l_aux in the MoE
model).  After backward a rank's home shard holds the gradient summed over both ranks' losses (the shards travel the
ring with their partial sums), while the unsharded LayerNorm parameters hold the gradient of that rank's loss only.
"""
import os
import sys
import tempfile

import numpy as np
import torch
import torch.distributed as dist
import torch.multiprocessing as mp
import torch.nn as nn
import torch.nn.functional as F

V, D, H, FF, NDEC, L, N, WS = 32, 16, 2, 16, 2, 6, 4, 2


def masters(is_moe: bool):
    """Seeded stock layers holding the unsharded weights (identical on every rank)."""
    g = torch.Generator().manual_seed(1234)

    def fill(t, scale=0.3):
        with torch.no_grad():
            t.copy_((torch.rand(t.shape, generator=g) * 2 - 1) * scale)

    m = {"emb": nn.Embedding(V, D), "head": nn.Linear(D, V), "dec": []}
    fill(m["emb"].weight), fill(m["head"].weight), fill(m["head"].bias, 0.1)
    for _ in range(NDEC):
        d = {"mha": nn.MultiheadAttention(D, H), "ln1": nn.LayerNorm(D), "ln2": nn.LayerNorm(D)}
        for p in d["mha"].parameters():
            fill(p)
        for ln in (d["ln1"], d["ln2"]):
            fill(ln.weight), fill(ln.bias, 0.1)
            with torch.no_grad():
                ln.weight.add_(1.0)
        if is_moe:
            d["wg"] = nn.Linear(D, WS, bias=False)
            fill(d["wg"].weight, 1.0)
            d["experts"] = []
            for _ in range(WS):
                l1, l2 = nn.Linear(D, FF), nn.Linear(FF, D)
                for p in list(l1.parameters()) + list(l2.parameters()):
                    fill(p)
                d["experts"].append((l1, l2))
        else:
            d["l1"], d["l2"] = nn.Linear(D, FF), nn.Linear(FF, D)
            for p in list(d["l1"].parameters()) + list(d["l2"].parameters()):
                fill(p)
        m["dec"].append(d)
    return m


def worker(rank: int, ws: int, ref_root: str, init_file: str, out_path: str, is_moe: bool) -> None:
    sys.path.insert(0, ref_root)
    torch.set_num_threads(1)
    dist.init_process_group("gloo", init_method=f"file://{init_file}", rank=rank, world_size=ws)
    from rtp.models.transformer_lm_rtp import TransformerLM

    class _Gate:  # what WeightTop2Gate.affine_weight reads: an object with .wg.weight
        def __init__(self, wg):
            self.wg = wg

    m = masters(is_moe)
    torch.manual_seed(100 + rank)
    lm = TransformerLM(V, D, H, FF, 0.0, 0.1, NDEC, ws, rank, is_moe=is_moe, num_local_experts=1)
    with torch.no_grad():
        lm[0].embedding.embedding.affine_weight(m["emb"])
        lm[-1].linear.linear.affine_weight(m["head"])
        for i, d in enumerate(m["dec"]):
            dec = lm[2 + i]
            dec.self_attn.MultiheadAttention.affine_weight(d["mha"])
            for mine, theirs in ((dec.norm1, d["ln1"]), (dec.norm2, d["ln2"])):
                mine.weight.copy_(theirs.weight), mine.bias.copy_(theirs.bias)
            if is_moe:
                dec.gate.affine_weight(dec.gate.wg, _Gate(d["wg"]))
                e = dec.moe_layer.experts[0]
                l1, l2 = d["experts"][rank]
                e.linear1.weight.copy_(l1.weight), e.linear1.bias.copy_(l1.bias)
                e.linear2.weight.copy_(l2.weight), e.linear2.bias.copy_(l2.bias)
            else:
                dec.ff_block.linear1.linear.affine_weight(d["l1"])
                dec.ff_block.linear2.linear.affine_weight(d["l2"])

    g = torch.Generator().manual_seed(77)
    ids_all = torch.randint(0, V, (ws, L, N), generator=g)
    tgt_all = torch.randint(0, V, (ws, L, N), generator=g)
    logits = lm(ids_all[rank])
    loss = F.cross_entropy(logits.view(-1, V), tgt_all[rank].view(-1))
    l_aux = []
    if is_moe:
        l_aux = [lm[2 + i].moe_layer.l_aux for i in range(NDEC)]
        loss = loss + sum(l_aux)
    loss.backward()

    mine = {"logits": logits.detach(), "loss": loss.detach()}
    if is_moe:
        mine["l_aux"] = torch.stack([a.detach() for a in l_aux])
    mine["grad.emb"] = lm[0].embedding.embedding.weight.grad
    mine["grad.head_w"] = lm[-1].linear.linear.weight.grad
    mine["grad.head_b"] = lm[-1].linear.linear.bias.grad
    for i in range(NDEC):
        dec = lm[2 + i]
        sa = dec.self_attn.MultiheadAttention
        mine[f"grad.l{i}.in_w"], mine[f"grad.l{i}.in_b"] = sa.in_proj_weight.grad, sa.in_proj_bias.grad
        mine[f"grad.l{i}.out_w"], mine[f"grad.l{i}.out_b"] = sa.out_proj.weight.grad, sa.out_proj.bias.grad
        mine[f"grad.l{i}.ln1_w"], mine[f"grad.l{i}.ln1_b"] = dec.norm1.weight.grad, dec.norm1.bias.grad
        mine[f"grad.l{i}.ln2_w"], mine[f"grad.l{i}.ln2_b"] = dec.norm2.weight.grad, dec.norm2.bias.grad
        if is_moe:
            e = dec.moe_layer.experts[0]
            mine[f"grad.l{i}.wg"] = dec.gate.wg.weight.grad
            mine[f"grad.l{i}.e_w1"], mine[f"grad.l{i}.e_b1"] = e.linear1.weight.grad, e.linear1.bias.grad
            mine[f"grad.l{i}.e_w2"], mine[f"grad.l{i}.e_b2"] = e.linear2.weight.grad, e.linear2.bias.grad
        else:
            f1, f2 = dec.ff_block.linear1.linear, dec.ff_block.linear2.linear
            mine[f"grad.l{i}.w1"], mine[f"grad.l{i}.b1"] = f1.weight.grad, f1.bias.grad
            mine[f"grad.l{i}.w2"], mine[f"grad.l{i}.b2"] = f2.weight.grad, f2.bias.grad
    mine = {k: v.detach().clone().numpy() for k, v in mine.items()}
    gathered = [None] * ws if rank == 0 else None
    dist.gather_object(mine, gathered, dst=0)
    if rank == 0:
        data = {"ids": ids_all.numpy(), "tgt": tgt_all.numpy(),
                "dims": np.array([V, D, H, FF, NDEC, L, N, ws], dtype=np.int64)}
        for r, part in enumerate(gathered):
            for k, v in part.items():
                data[f"rank{r}.{k}"] = v
        data["emb"] = m["emb"].weight.detach().numpy()
        data["head_w"], data["head_b"] = m["head"].weight.detach().numpy(), m["head"].bias.detach().numpy()
        for i, d in enumerate(m["dec"]):
            mha = d["mha"]
            data[f"l{i}.in_w"], data[f"l{i}.in_b"] = mha.in_proj_weight.detach().numpy(), mha.in_proj_bias.detach().numpy()
            data[f"l{i}.out_w"] = mha.out_proj.weight.detach().numpy()
            data[f"l{i}.out_b"] = mha.out_proj.bias.detach().numpy()
            for nm in ("ln1", "ln2"):
                data[f"l{i}.{nm}_w"], data[f"l{i}.{nm}_b"] = d[nm].weight.detach().numpy(), d[nm].bias.detach().numpy()
            if is_moe:
                data[f"l{i}.wg"] = d["wg"].weight.detach().numpy()
                for e, (l1, l2) in enumerate(d["experts"]):
                    data[f"l{i}.e{e}.w1"], data[f"l{i}.e{e}.b1"] = l1.weight.detach().numpy(), l1.bias.detach().numpy()
                    data[f"l{i}.e{e}.w2"], data[f"l{i}.e{e}.b2"] = l2.weight.detach().numpy(), l2.bias.detach().numpy()
            else:
                data[f"l{i}.w1"], data[f"l{i}.b1"] = d["l1"].weight.detach().numpy(), d["l1"].bias.detach().numpy()
                data[f"l{i}.w2"], data[f"l{i}.b2"] = d["l2"].weight.detach().numpy(), d["l2"].bias.detach().numpy()
        np.savez_compressed(out_path, **data)
        print("wrote", out_path, "losses", [float(p["loss"]) for p in gathered])
    dist.barrier()
    dist.destroy_process_group()


def main(ref_root: str) -> None:
    here = os.path.dirname(os.path.abspath(__file__))
    for is_moe, name in ((False, "lm_ws2.npz"), (True, "lm_moe_ws2.npz")):
        with tempfile.TemporaryDirectory() as tmp:
            mp.spawn(worker, args=(WS, ref_root, os.path.join(tmp, "rdzv"), os.path.join(here, name), is_moe),
                     nprocs=WS)


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
