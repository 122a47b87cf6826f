"""Writes tests/golden/moe_ws2.npz: inputs, weights, output and gradients of the reference's own
WeightMOELayer + WeightTop2Gate (rtp/module/moe.py:101-187, rtp/module/top2gate.py:139-220) run on a
2-rank gloo ring on CPU, one expert per rank (E = 2, so the Gumbel noise cannot change the routing).

Run in the build container only (needs the reference tree on disk):
    python tests/golden/make_moe_golden.py /root/reference
Both ranks feed the same input, as tests/test_moe.py does, so every parameter gradient the reference
ends up with is twice the gradient of a single copy of the batch; the fixture stores them as produced.
"""
import os
import sys
import tempfile

import numpy as np
import torch
import torch.distributed as dist
import torch.multiprocessing as mp

D_MODEL, D_FF, SEQ, TOK = 8, 16, 4, 8


def worker(rank: int, ws: int, ref_root: str, init_file: str, out_path: str) -> None:
    sys.path.insert(0, ref_root)
    torch.set_num_threads(1)
    dist.init_process_group("gloo", init_method=f"file://{init_file}", rank=rank, world_size=ws)
    from rtp.module.moe import WeightMOELayer
    from rtp.module.top2gate import Top2Gate, WeightTop2Gate
    from rtp.models.transformer_lm_rtp import FeedForwardLayer_expert

    torch.manual_seed(7)
    master_gate = Top2Gate(D_MODEL, ws)
    masters = [FeedForwardLayer_expert(D_MODEL, D_FF, torch.nn.ReLU(), 0.0) for _ in range(ws)]
    x = torch.randn(SEQ, TOK, D_MODEL)
    coef = torch.randn(SEQ, TOK, D_MODEL)

    gate = WeightTop2Gate(D_MODEL, ws, gate=master_gate)
    local = FeedForwardLayer_expert(D_MODEL, D_FF, torch.nn.ReLU(), 0.0)
    layer = WeightMOELayer(gate, local, original_experts=torch.nn.ModuleList([masters[rank]]))
    out = layer(x)
    loss = (out * coef).sum() + layer.l_aux
    loss.backward()
    if rank == 0:
        data = {"x": x.numpy(), "coef": coef.numpy(), "wg": master_gate.wg.weight.detach().numpy(),
                "out": out.detach().numpy(), "l_aux": layer.l_aux.detach().numpy(),
                "grad_wg0": gate.wg.weight.grad.numpy()}
        for e, m in enumerate(masters):
            for n, p in m.named_parameters():
                data[f"expert{e}.{n}"] = p.detach().numpy()
        for n, p in layer.experts.named_parameters():
            data[f"grad_expert0.{n}"] = p.grad.numpy()
        np.savez_compressed(out_path, **data)
        print("wrote", out_path, "l_aux", float(layer.l_aux))
    dist.barrier()
    dist.destroy_process_group()


def main(ref_root: str) -> None:
    here = os.path.dirname(os.path.abspath(__file__))
    with tempfile.TemporaryDirectory() as tmp:
        mp.spawn(worker, args=(2, ref_root, os.path.join(tmp, "rdzv"), os.path.join(here, "moe_ws2.npz")), nprocs=2)


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
