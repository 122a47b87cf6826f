"""Adam over the flat shard buffers (the reference harness's optimiser, benchmarks/rtp_benchmark.py:41-42 and
:185-186: clip_grad_value_(0.05) then torch.optim.Adam(lr 1e-3).step()) against torch.optim.Adam on the CPU fed
with the same gradients.  fp32 arithmetic in the same order as torch's single-tensor form: the results agree to
rounding of single operations (rtol 1e-6, atol 1e-7 stated below), not bit for bit (sqrt / divide / lerp are not
pinned to one instruction sequence on either side)."""
import pytest
import torch
import torch.nn.functional as F

from gpu_util import DEV

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("rotation_window")]

RTOL, ATOL = 1e-6, 1e-7


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,offset", [(4096, 0), (1003, 0), (1024, 1)])  # 16-byte path, ragged, misaligned start
@pytest.mark.parametrize("clip,wd", [(0.0, 0.0), (0.05, 0.0), (0.05, 0.01)])
def test_adam_step_matches_torch(dtype, n, offset, clip, wd):
    from rtp_amd import ops
    gen = torch.Generator().manual_seed(n + offset)
    w0 = torch.randn(n, generator=gen)
    if dtype == torch.bfloat16:
        w0 = w0.to(dtype).float()
    ref = torch.nn.Parameter(w0.clone())
    opt = torch.optim.Adam([ref], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=wd)

    def dev_slice(t):
        buf = torch.zeros(n + 8, dtype=t.dtype, device=DEV)
        buf[offset:offset + n].copy_(t)
        return buf[offset:offset + n]

    master, m, v = dev_slice(w0), dev_slice(torch.zeros(n)), dev_slice(torch.zeros(n))
    shadow = dev_slice(w0.to(dtype)) if dtype != torch.float32 else None
    for step in range(1, 4):
        g = (torch.randn(n, generator=gen) * 0.1).to(dtype)
        ref.grad = g.float().clone()
        if clip > 0:
            torch.nn.utils.clip_grad_value_([ref], clip)
        opt.step()
        ops.adam_step(master, dev_slice(g), shadow, m, v, step, 1e-3, (0.9, 0.999), 1e-8, wd, clip)
        torch.testing.assert_close(master.cpu(), ref.detach(), rtol=RTOL, atol=ATOL)
    state = opt.state[ref]
    torch.testing.assert_close(m.cpu(), state["exp_avg"], rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(v.cpu(), state["exp_avg_sq"], rtol=RTOL, atol=1e-10)
    if shadow is not None:
        assert torch.equal(shadow, master.to(dtype))


def test_adam_step_rejects_bad_arguments():
    from rtp_amd import ops
    from rtp_amd._lib import RtpError
    w, g = torch.zeros(16, device=DEV), torch.zeros(16, device=DEV)
    m, v = torch.zeros(16, device=DEV), torch.zeros(16, device=DEV)
    with pytest.raises(RtpError):
        ops.adam_step(w, g, None, m, v, 0, 1e-3)          # steps count from 1
    with pytest.raises(RtpError):
        ops.adam_step(w, g, None, m, v, 1, 1e-3, betas=(1.0, 0.999))
    with pytest.raises(ValueError):
        ops.adam_step(w, g, None, m[:8], v, 1, 1e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rotated_adam_harness_step(dtype):
    """zero grads -> forward -> cross-entropy -> backward -> clip 0.05 -> Adam(1e-3), three times, on the rotated LM;
    every parameter (shards of rotated layers and LayerNorm) tracks a torch.optim.Adam on the CPU that is handed
    this model's own gradients.  bf16: the fp32 master tracks, the bf16 weights are its rounding."""
    from test_gpu_lm import build_pair
    from rtp_amd.optim import RotatedAdam
    V, D, H, Fd, n_dec, L, N, ws = 64, 32, 4, 32, 2, 6, 3, 4
    lm, _ = build_pair(V, D, H, Fd, n_dec, ws, dtype, seed=5)
    opt = RotatedAdam(lm, lr=1e-3, clip_value=0.05)
    params = list(lm.parameters())
    clones = [torch.nn.Parameter(p.detach().float().cpu().clone()) for p in params]
    ref_opt = torch.optim.Adam(clones, lr=1e-3)
    gen = torch.Generator().manual_seed(9)
    for _ in range(3):
        ids = torch.randint(0, V, (L, N), generator=gen).to(DEV)
        opt.zero_grad()
        F.cross_entropy(lm(ids).float().view(-1, V), ids.view(-1)).backward()
        for p, c in zip(params, clones):
            c.grad = p.grad.detach().float().cpu().clone()
        torch.nn.utils.clip_grad_value_(clones, 0.05)
        ref_opt.step()
        opt.step()
    assert opt.steps == 3 and opt.state_bytes() > 0
    for p, c in zip(params, clones):
        if dtype == torch.float32:
            torch.testing.assert_close(p.detach().cpu(), c.detach(), rtol=RTOL, atol=ATOL)
        else:
            # the weight is the rounding of an fp32 master that tracks the CPU's to the tolerance above: it may land
            # on the neighbouring bf16 value where the master sits on a rounding boundary
            torch.testing.assert_close(p.detach().float().cpu(), c.detach(), rtol=2 ** -7, atol=1e-6)
    if dtype != torch.float32:
        for st, master in zip(opt.stores, opt.masters):
            assert torch.equal(st.home.view(-1), master.view(-1).to(dtype))


def test_adam_device_step_counter_follows_graph_replays():
    """The step count read from device memory: one launch recorded into a HIP graph and replayed moves on with the
    caller's counter (bias corrections of steps 2, 3, 4 ...), every replay checked against torch.optim.Adam, with
    eager work and synchronisation between the replays."""
    from rtp_amd import ops
    n = 2048
    gen = torch.Generator().manual_seed(3)
    w0 = torch.randn(n, generator=gen)
    ref = torch.nn.Parameter(w0.clone())
    opt = torch.optim.Adam([ref], lr=1e-3)
    master, m, v = w0.to(DEV), torch.zeros(n, device=DEV), torch.zeros(n, device=DEV)
    g_dev = torch.zeros(n, device=DEV)
    step_dev = torch.zeros(1, dtype=torch.int64, device=DEV)

    def one():
        step_dev.add_(1)
        ops.adam_step(master, g_dev, None, m, v, step_dev, 1e-3)

    def feed():
        g = torch.randn(n, generator=gen) * 0.1
        ref.grad = g.clone()
        opt.step()
        g_dev.copy_(g)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    feed()
    with torch.cuda.stream(side):
        one()                                   # step 1, eager
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    torch.testing.assert_close(master.cpu(), ref.detach(), rtol=RTOL, atol=ATOL)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        one()
    for step in range(2, 6):
        feed()
        graph.replay()
        torch.cuda.synchronize()
        assert int(step_dev) == step
        torch.testing.assert_close(master.cpu(), ref.detach(), rtol=RTOL, atol=ATOL)
        _ = (master * 2).sum().item()           # unrelated eager work between replays
