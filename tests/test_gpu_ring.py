"""The two-slot staged rotation: staged bytes equal the home shard, every shard is visited once in ring
order, and the fencing survives many back-to-back rotations that reuse the slots."""
import pytest
import torch

from gpu_util import DEV

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _staged_mode():
    """These tests are about the two HBM slots; the last one checks the direct schedule."""
    from rtp_amd import ring
    ring.set_rotation_mode("staged")
    yield
    ring.set_rotation_mode("direct")


@pytest.mark.parametrize("window", [1, 3, None])
def test_rotation_delivers_each_shard_in_ring_order(window):
    from rtp_amd.ring import Rotation, ring_order
    ws, numel = 8, 100_003
    home = torch.randn(ws, numel, device=DEV)
    seen = []
    for rank in (0, 3):
        order = ring_order(rank, ws)
        assert sorted(order) == list(range(ws)) and order[0] == rank
        rot = Rotation(home, order, window=window)
        visited = []
        for j in range(rot.steps):
            for flat, first, cnt in rot.acquire(j):
                assert flat.shape == (cnt, numel)
                seen.append((first, cnt, flat.clone()))
                visited += list(range(first, first + cnt))
            rot.release(j)
        assert sorted(visited) == list(range(ws))
        w = window or ws
        for j, win in enumerate(rot.windows):  # window j holds ring steps j*w .. j*w+w-1
            assert sorted(s for f, c in win for s in range(f, f + c)) == sorted(order[j * w:(j + 1) * w])
    torch.cuda.synchronize()
    for first, cnt, flat in seen:
        assert torch.equal(flat, home[first:first + cnt])
    assert ring_order(2, 4, reverse=True) == [1, 0, 3, 2]


@pytest.mark.parametrize("window", [1, 2])
def test_rotation_fencing_under_slot_reuse(window):
    """A slow consumer (large matmul) reads a slot while later prefetches want it again, across several
    back-to-back rotations that share the two slots: what each step consumed must be its own shards."""
    from rtp_amd.ring import Rotation, ring_order
    ws, numel = 6, 4_000_000
    home = torch.arange(1, ws + 1, device=DEV, dtype=torch.float32).view(ws, 1).repeat(1, numel).contiguous()
    sums = []
    for _ in range(5):
        rot = Rotation(home, ring_order(0, ws), window=window)
        for j in range(rot.steps):
            for flat, first, cnt in rot.acquire(j):
                for i in range(cnt):
                    a = flat[i].view(2000, 2000)
                    sums.append((first + i, (a @ a[:, :64]).sum()))  # heavy kernel reading the slot
            rot.release(j)
    torch.cuda.synchronize()
    for idx, s in sums:
        expect = 2000 * 2000 * 64.0 * (idx + 1) ** 2
        assert abs(float(s) - expect) <= 1e-3 * expect, (idx, float(s), expect)


def test_fence_orders_staging_after_weight_update():
    """Weights rewritten by a kernel on the compute stream, then fence(): the next rotation stages the new
    values, not the old ones."""
    from rtp_amd import ring
    from rtp_amd.ring import Rotation, ring_order
    home = torch.zeros(4, 1_000_000, device=DEV)
    for step in range(1, 4):
        big = torch.randn(3000, 3000, device=DEV)
        (big @ big).sum()  # keep the compute stream busy ahead of the update
        home.fill_(float(step))
        ring.fence()
        rot = Rotation(home, ring_order(0, 4))
        (flat, first, cnt), = rot.acquire(0)
        got = flat.sum().item()
        rot.release(0)
        assert got == step * 4 * 1_000_000.0


def test_copy_and_zero_kernels_ragged():
    from rtp_amd import ops
    for n in (1, 15, 16, 17, 4099, 1 << 20):
        src = torch.randint(0, 255, (n + 3,), dtype=torch.uint8, device=DEV)
        dst = torch.zeros(n + 3, dtype=torch.uint8, device=DEV)
        ops.shard_copy(dst[:n], src[:n])
        assert torch.equal(dst[:n], src[:n]) and dst[n:].sum() == 0
        dst2 = torch.full((n + 4,), 7, dtype=torch.uint8, device=DEV)
        ops.shard_copy(dst2[1:n + 1], src[:n])  # misaligned destination
        assert torch.equal(dst2[1:n + 1], src[:n]) and dst2[0] == 7 and dst2[n + 1] == 7
        ops.zero_(dst2[1:n + 1])
        assert dst2[1:n + 1].sum() == 0 and dst2[0] == 7 and dst2[n + 1] == 7


def test_stage_group_partial_use_and_restage():
    """Layers of a stage group may also be used alone, out of order, or after a weight update: a member that
    finds no valid staged copy of itself stages the group again, and a finished pass hands the slot back."""
    import torch.nn as nn
    from rtp_amd import emulate_shards, ring
    from rtp_amd.module.linear import ColumnParallelLinear
    torch.manual_seed(0)
    with emulate_shards(4):
        a = ColumnParallelLinear(32, 64, device=DEV)
        b = ColumnParallelLinear(64, 32, device=DEV)
    ring.group_stores([a._store, b._store])
    x = torch.randn(5, 32, device=DEV)

    def ref(layer, inp):
        w = torch.cat([l.weight for l in layer.linears], 0)
        bias = torch.cat([l.bias for l in layer.linears], 0)
        return inp @ w.t() + bias

    saved = ring.rotation_window()
    ring.set_rotation_window(None)
    try:
        with torch.no_grad():
            ya = a(x)                      # stages the group, uses one member only
            ya2 = a(x)                     # the same member again: stages again
            yb = b(ya)                     # the other member of that staging
            assert torch.allclose(ya, ref(a, x), atol=1e-5) and torch.equal(ya, ya2)
            assert torch.allclose(yb, ref(b, ya), atol=1e-5)
            for l in b.linears:            # weights change under the staged copy
                l.weight.mul_(2.0)
            ring.fence(x.device)
            yb2 = b(ya)
            assert torch.allclose(yb2, ref(b, ya), atol=1e-5)
            yb3 = b(ya)                    # b, then a: reverse order of the declaration
            ya3 = a(x)
            assert torch.equal(yb3, yb2) and torch.equal(ya3, ya)
    finally:
        ring.set_rotation_window(saved)
    torch.cuda.synchronize()


def test_staging_growth_during_capture_is_refused():
    """A layer whose shards do not fit the staging slots yet cannot take its first step inside a graph capture (the
    slots would have to be reallocated under the graph): a clear error, nothing recorded, and the layer works
    eagerly afterwards."""
    from rtp_amd import emulate_shards, ring
    from rtp_amd.module.linear import ColumnParallelLinear
    dev = torch.device(DEV)
    slot = ring.device_ring(dev).slot_bytes
    n = max(512, (int((slot / 4) ** 0.5) // 256 + 2) * 256)  # an fp32 [n, n] weight larger than one slot
    with emulate_shards(2):
        layer = ColumnParallelLinear(n, n, device=DEV, dtype=torch.float32)
    x = torch.randn(8, n, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _ = x * 2  # the capture below needs a warmed-up allocator, not a warmed-up layer
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="eager step"):
        with torch.cuda.graph(graph):
            layer(x)
    torch.cuda.synchronize()
    y = layer(x)
    ref = torch.nn.functional.linear(x.cpu(), torch.cat([l.weight for l in layer.linears], 0).cpu(),
                                     torch.cat([l.bias for l in layer.linears], 0).cpu())
    torch.testing.assert_close(y.cpu(), ref, rtol=1e-4, atol=1e-4)
    assert ring.device_ring(dev).slot_bytes >= n * n * 4


@pytest.mark.parametrize("window", [None, 1, 3])
def test_direct_rotation_reads_home_rows_and_stages_nothing(window):
    """In the direct schedule a window's shards are handed out as views of their home rows, in the same window /
    run structure as the staged schedule, and no staging memory is touched or reserved."""
    from rtp_amd import ring
    from rtp_amd.ring import Rotation, ring_order
    ring.set_rotation_mode("direct")
    before = ring.staging_bytes()
    ws, numel = 8, 1000
    home = torch.randn(ws, numel, device=DEV)
    for rank in (0, 5):
        order = ring_order(rank, ws)
        rot = Rotation(home, order, window=window)
        visited = []
        for j in range(rot.steps):
            for flat, first, cnt in rot.acquire(j):
                assert flat.data_ptr() == home[first].data_ptr() and flat.shape == (cnt, numel)
                visited += list(range(first, first + cnt))
            rot.release(j)
        assert sorted(visited) == list(range(ws))
        w = window or ws
        for j, win in enumerate(rot.windows):
            assert sorted(s for f, c in win for s in range(f, f + c)) == sorted(order[j * w:(j + 1) * w])
    assert ring.staging_bytes() == before


def test_warm_ahead_learns_the_layer_order_and_changes_no_result():
    """Direct rotation with the next layer's shards handed to the current layer's first product: after one pass the
    table knows, for the forward and for the backward order, which layer follows which; outputs and gradients are
    bit-identical with the switch off; the table keeps no layer alive."""
    import gc
    import weakref
    from rtp_amd import emulate_shards, ring
    from rtp_amd.module.linear import ColumnParallelLinear
    ring.set_rotation_mode("direct")
    ws, d = 4, 256
    gen = torch.Generator().manual_seed(11)
    with emulate_shards(ws):
        layers = [ColumnParallelLinear(d, d, device=DEV, dtype=torch.bfloat16) for _ in range(3)]
    x = (torch.randn(130, d, generator=gen) * 0.3).to(torch.bfloat16).to(DEV)

    def run():
        xi = x.clone().requires_grad_(True)
        h = xi
        for lyr in layers:
            h = lyr(h)
        h.float().square().mean().backward()
        out = [h.detach().clone(), xi.grad.clone()] + [p.grad.clone() for lyr in layers for p in lyr.parameters()]
        for lyr in layers:
            lyr.zero_grad(set_to_none=True)
        return out

    try:
        ring.set_warm_ahead(False)
        want = run()
        ring.set_warm_ahead(True)
        for _ in range(3):
            got = run()
            assert all(torch.equal(a, b) for a, b in zip(want, got))
        homes = [lyr._store.home.data_ptr() for lyr in layers]
        idx = torch.device(DEV).index or 0
        follows = {(k[1], k[2]): v().data_ptr() for k, v in ring._warm_next.items() if k[0] == idx and v() is not None}
        assert follows[(homes[0], homes[1])] == homes[2]       # forward order
        assert follows[(homes[2], homes[1])] == homes[0]       # backward order
        probe = weakref.ref(layers[1]._store.home)
        del layers[:], got, want
        gc.collect()
        ring.set_warm_ahead(True)  # clears what may still be pending
        gc.collect()
        assert probe() is None
    finally:
        ring.set_warm_ahead(True)
