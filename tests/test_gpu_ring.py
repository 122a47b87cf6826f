"""The two-slot staged rotation: staged bytes equal the home shard, every shard is visited once in ring
order, and the fencing survives many back-to-back rotations that reuse the slots."""
import pytest
import torch

from gpu_util import DEV

pytestmark = pytest.mark.gpu


def test_rotation_delivers_each_shard_in_ring_order():
    from rtp_amd.ring import Rotation, ring_order
    ws, numel = 8, 100_003
    home = torch.randn(ws, numel, device=DEV)
    seen = []
    for rank in (0, 3):
        order = ring_order(rank, ws)
        assert sorted(order) == list(range(ws)) and order[0] == rank
        rot = Rotation(home, order)
        for i, idx in enumerate(order):
            flat = rot.acquire(i)
            seen.append((idx, flat.clone()))
            rot.release(i)
    torch.cuda.synchronize()
    for idx, flat in seen:
        assert torch.equal(flat, home[idx])
    assert ring_order(2, 4, reverse=True) == [1, 0, 3, 2]


def test_rotation_fencing_under_slot_reuse():
    """A slow consumer (large reduction) reads slot s while the prefetch of step i+2 wants the same slot:
    the checksum of what each step consumed must be the checksum of its own shard."""
    from rtp_amd.ring import Rotation, ring_order
    ws, numel = 6, 4_000_000
    home = torch.arange(ws, device=DEV, dtype=torch.float32).view(ws, 1).repeat(1, numel).contiguous()
    sums = []
    for _ in range(5):
        order = ring_order(0, ws)
        rot = Rotation(home, order)
        for i, idx in enumerate(order):
            flat = rot.acquire(i)
            a = flat.view(2000, 2000)
            sums.append((idx, (a @ a[:, :64]).sum() / max(idx, 1) ** 2))  # heavy kernel reading the slot
            rot.release(i)
    torch.cuda.synchronize()
    for idx, s in sums:
        expect = 0.0 if idx == 0 else 2000 * 2000 * 64.0
        assert abs(float(s) - expect) <= 1e-3 * max(expect, 1.0), (idx, float(s), expect)


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
