"""Helpers around tests/golden/lm_ws2.npz and lm_moe_ws2.npz (written by tests/golden/make_lm_golden.py from the
reference's TransformerLM on a 2-rank gloo ring): loading the fixture into the oracle LM, and the names of the
home-shard gradients each rank saved together with the slice of the unsharded gradient they correspond to."""
import os

import numpy as np
import torch

from oracle import rtp_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))


def load(name):
    z = np.load(os.path.join(HERE, "golden", name))
    fix = {k: torch.from_numpy(z[k]) for k in z.files}
    V, D, H, FF, NDEC, L, N, WS = (int(v) for v in fix["dims"])
    fix["cfg"] = dict(V=V, D=D, H=H, FF=FF, NDEC=NDEC, L=L, N=N, WS=WS, moe="l0.wg" in fix)
    return fix


def oracle_lm(fix):
    c = fix["cfg"]
    ref = O.TransformerLM(c["V"], c["D"], c["H"], c["FF"], c["NDEC"], num_experts=c["WS"] if c["moe"] else 0, ws=c["WS"])
    with torch.no_grad():
        ref[0].weight.copy_(fix["emb"])
        ref[-1].weight.copy_(fix["head_w"]), ref[-1].bias.copy_(fix["head_b"])
        for i in range(c["NDEC"]):
            d = ref[2 + i]
            d.self_attn.in_proj_weight.copy_(fix[f"l{i}.in_w"]), d.self_attn.in_proj_bias.copy_(fix[f"l{i}.in_b"])
            d.self_attn.out_proj.weight.copy_(fix[f"l{i}.out_w"]), d.self_attn.out_proj.bias.copy_(fix[f"l{i}.out_b"])
            d.norm1.weight.copy_(fix[f"l{i}.ln1_w"]), d.norm1.bias.copy_(fix[f"l{i}.ln1_b"])
            d.norm2.weight.copy_(fix[f"l{i}.ln2_w"]), d.norm2.bias.copy_(fix[f"l{i}.ln2_b"])
            if c["moe"]:
                d.wg.weight.copy_(fix[f"l{i}.wg"])
                for e in range(c["WS"]):
                    d.experts[e][0].weight.copy_(fix[f"l{i}.e{e}.w1"]), d.experts[e][0].bias.copy_(fix[f"l{i}.e{e}.b1"])
                    d.experts[e][1].weight.copy_(fix[f"l{i}.e{e}.w2"]), d.experts[e][1].bias.copy_(fix[f"l{i}.e{e}.b2"])
            else:
                d.linear1.weight.copy_(fix[f"l{i}.w1"]), d.linear1.bias.copy_(fix[f"l{i}.b1"])
                d.linear2.weight.copy_(fix[f"l{i}.w2"]), d.linear2.bias.copy_(fix[f"l{i}.b2"])
    return ref


def _in_proj_rows(full, ws, r):
    """Rows of the packed in-projection held by shard r: blocks [r, r+ws, r+2ws] of its 3*ws row blocks
    (rtp/module/attention.py:86-100)."""
    blocks = torch.chunk(full, 3 * ws, dim=0)
    return torch.cat([blocks[r], blocks[r + ws], blocks[r + 2 * ws]], dim=0)


def shard_slices(full, cfg, r):
    """From unsharded gradients `full` (dict keyed like the fixture's master weights, experts as l{i}.e{e}.*) the
    gradients rank r's home shard holds, keyed like the fixture's `rank{r}.grad.*` entries (LayerNorm excluded)."""
    ws = cfg["WS"]
    out = {"emb": torch.chunk(full["emb"], ws, 1)[r], "head_w": torch.chunk(full["head_w"], ws, 0)[r],
           "head_b": torch.chunk(full["head_b"], ws, 0)[r]}
    for i in range(cfg["NDEC"]):
        out[f"l{i}.in_w"] = _in_proj_rows(full[f"l{i}.in_w"], ws, r)
        out[f"l{i}.in_b"] = _in_proj_rows(full[f"l{i}.in_b"], ws, r)
        out[f"l{i}.out_w"] = torch.chunk(full[f"l{i}.out_w"], ws, 1)[r]
        out[f"l{i}.out_b"] = full[f"l{i}.out_b"]  # every shard holds bias/ws and receives the whole gradient
        if cfg["moe"]:
            out[f"l{i}.wg"] = torch.chunk(full[f"l{i}.wg"], ws, 0)[r]
            for nm in ("w1", "b1", "w2", "b2"):
                out[f"l{i}.e_{nm}"] = full[f"l{i}.e{r}.{nm}"]
        else:
            for nm in ("w1", "b1", "w2", "b2"):
                out[f"l{i}.{nm}"] = torch.chunk(full[f"l{i}.{nm}"], ws, 0)[r]
    return out


def oracle_full_grads(ref, cfg):
    """Unsharded gradients of the oracle LM keyed like the fixture's master weights."""
    out = {"emb": ref[0].weight.grad, "head_w": ref[-1].weight.grad, "head_b": ref[-1].bias.grad}
    for i in range(cfg["NDEC"]):
        d = ref[2 + i]
        out[f"l{i}.in_w"], out[f"l{i}.in_b"] = d.self_attn.in_proj_weight.grad, d.self_attn.in_proj_bias.grad
        out[f"l{i}.out_w"], out[f"l{i}.out_b"] = d.self_attn.out_proj.weight.grad, d.self_attn.out_proj.bias.grad
        out[f"l{i}.ln1_w"], out[f"l{i}.ln1_b"] = d.norm1.weight.grad, d.norm1.bias.grad
        out[f"l{i}.ln2_w"], out[f"l{i}.ln2_b"] = d.norm2.weight.grad, d.norm2.bias.grad
        if cfg["moe"]:
            out[f"l{i}.wg"] = d.wg.weight.grad
            for e in range(cfg["WS"]):
                out[f"l{i}.e{e}.w1"], out[f"l{i}.e{e}.b1"] = d.experts[e][0].weight.grad, d.experts[e][0].bias.grad
                out[f"l{i}.e{e}.w2"], out[f"l{i}.e{e}.b2"] = d.experts[e][1].weight.grad, d.experts[e][1].bias.grad
        else:
            out[f"l{i}.w1"], out[f"l{i}.b1"] = d.linear1.weight.grad, d.linear1.bias.grad
            out[f"l{i}.w2"], out[f"l{i}.b2"] = d.linear2.weight.grad, d.linear2.bias.grad
    return out
