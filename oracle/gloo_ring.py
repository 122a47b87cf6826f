"""TEST / BASELINE INFRASTRUCTURE ONLY -- nothing shipped imports this file.

CPU restatement of the reference's rotated column-parallel Linear as it actually runs: `ws` processes on a
torch.distributed gloo ring, each holding one home shard of the weight and its own slice of the batch rows.

  forward   (rtp/module/linear.py:204-224): at ring step i a rank computes output block (rank + i) % ws with the shard
            it currently holds while that shard moves on to rank - 1 and the next one arrives from rank + 1
            (rtp/module/collectives.py:221-238 `_left_shift_buffer`, batch_isend_irecv of the flat shard);
  backward  (rtp/module/collectives.py:264-317): the shards travel the other way (`_right_shift_buffer`, :202-219) and
            carry their partial weight / bias gradients with them, every rank adding its batch slice's share; after ws
            steps each rank holds its home shard again together with the complete gradient.

Pinned by tests/test_oracle.py: outputs, input gradients and gathered weight gradients equal torch.nn.functional.linear
on the unsharded problem (the oracle of the reference's own tests/test_linear.py:134-165).  bench.py times it as the CPU
baseline of the column-parallel Linear workload.
"""
from __future__ import annotations

import os
import socket
import time
from typing import Dict, List

import torch
import torch.distributed as dist
import torch.multiprocessing as mp
import torch.nn.functional as F


def _free_port() -> int:
    with socket.socket(socket.AF_INET, socket.SOCK_STREAM) as s:
        s.bind(("127.0.0.1", 0))
        return s.getsockname()[1]


def _shift(tensors: List[torch.Tensor], to_rank: int, from_rank: int):
    """Start sending `tensors` to one neighbour and receiving their replacements from the other."""
    recv = [torch.empty_like(t) for t in tensors]
    ops = [dist.P2POp(dist.isend, t, to_rank) for t in tensors]
    ops += [dist.P2POp(dist.irecv, r, from_rank) for r in recv]
    return recv, dist.batch_isend_irecv(ops)


def _step(rank: int, ws: int, xr, dyr, home_w, home_b):
    rows, n_s = xr.shape[0], home_w.shape[0]
    left, right = (rank - 1) % ws, (rank + 1) % ws
    y = torch.empty(rows, n_s * ws, dtype=xr.dtype)
    w, b = home_w, home_b
    for i in range(ws):
        idx = (rank + i) % ws
        if i + 1 < ws:
            nxt, reqs = _shift([w, b], left, right)
        y[:, idx * n_s:(idx + 1) * n_s] = F.linear(xr, w, b)
        if i + 1 < ws:
            for r in reqs:
                r.wait()
            w, b = nxt
    # the rank now holds shard (rank + ws - 1) % ws; the backward pass walks the ring the other way
    dx = torch.zeros_like(xr)
    gw, gb = torch.zeros_like(w), torch.zeros_like(b)
    for i in range(ws):
        idx = (rank + ws - 1 - i) % ws
        dyb = dyr[:, idx * n_s:(idx + 1) * n_s]
        dx += dyb @ w
        gw += dyb.t() @ xr
        gb += dyb.sum(0)
        if i + 1 < ws:
            nxt, reqs = _shift([w, b, gw, gb], right, left)
            for r in reqs:
                r.wait()
            w, b, gw, gb = nxt
    return y, dx, gw, gb


def _worker(rank: int, ws: int, port: int, threads: int, x, w, b, dy, steps: int, warmup: int, out_dir: str):
    torch.set_num_threads(threads)
    dist.init_process_group("gloo", init_method=f"tcp://127.0.0.1:{port}", rank=rank, world_size=ws)
    rows, n_s = x.shape[0] // ws, w.shape[0] // ws
    xr, dyr = x[rank * rows:(rank + 1) * rows].contiguous(), dy[rank * rows:(rank + 1) * rows].contiguous()
    home_w, home_b = w[rank * n_s:(rank + 1) * n_s].clone(), b[rank * n_s:(rank + 1) * n_s].clone()
    for _ in range(warmup):
        _step(rank, ws, xr, dyr, home_w, home_b)
    times = []
    for _ in range(steps):
        dist.barrier()
        t0 = time.perf_counter()
        res = _step(rank, ws, xr, dyr, home_w, home_b)
        dist.barrier()
        times.append(time.perf_counter() - t0)
    y, dx, gw, gb = res
    torch.save({"y": y, "dx": dx, "gw": gw, "gb": gb, "times": times}, os.path.join(out_dir, f"rank{rank}.pt"))
    dist.destroy_process_group()


def column_linear_ring(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, dy: torch.Tensor, ws: int = 2, steps: int = 1,
                       warmup: int = 0, threads_per_rank: int = 1) -> Dict[str, object]:
    """Run fwd+bwd of the rotated column-parallel Linear on `ws` local gloo ranks (loopback rendezvous).
    x [M, K], w [N, K], b [N], dy [M, N] are the unsharded problem; rank r takes batch rows [r*M/ws, (r+1)*M/ws) and
    home shard r.  Returns the re-assembled y [M, N], dx [M, K], dw [N, K], db [N] and the per-step wall times
    (max over ranks)."""
    import tempfile
    assert x.shape[0] % ws == 0 and w.shape[0] % ws == 0
    port = _free_port()
    with tempfile.TemporaryDirectory() as tmp:
        mp.spawn(_worker, args=(ws, port, threads_per_rank, x, w, b, dy, steps, warmup, tmp), nprocs=ws, join=True)
        parts = [torch.load(os.path.join(tmp, f"rank{r}.pt"), weights_only=True) for r in range(ws)]
    times = [max(p["times"][i] for p in parts) for i in range(steps)]
    return {"y": torch.cat([p["y"] for p in parts], 0), "dx": torch.cat([p["dx"] for p in parts], 0),
            "dw": torch.cat([p["gw"] for p in parts], 0), "db": torch.cat([p["gb"] for p in parts], 0),
            "times": times}
