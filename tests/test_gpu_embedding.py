"""Rotated ParallelEmbedding: gather and deterministic scatter-add must be bit-exact against the oracle
(== torch CPU nn.Embedding), including the headline configuration and edge cases."""
import numpy as np
import pytest
import torch
import torch.nn as nn

from gpu_util import DEV
from oracle import rtp_oracle as O

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("rotation_window")]


def _layer(master, ws, dtype=torch.float32, **kw):
    from rtp_amd.module.embedding import ParallelEmbedding
    return ParallelEmbedding(master.num_embeddings, master.embedding_dim, ws, 0, Embedding_layer=master, device=DEV,
                             dtype=dtype, **kw)


def _check(master, ids, g, ws, padding_idx=None):
    layer = _layer(master, ws, padding_idx=padding_idx)
    out = layer(ids.to(DEV))
    ref = O.parallel_embedding(ids, master.weight.detach(), ws)
    assert torch.equal(out.cpu(), ref), "gather is not bit-exact"
    out.backward(g.to(DEV))
    dw = torch.cat([e.weight.grad for e in layer.embeddings], dim=1).cpu().numpy()  # gather rule: cat on dim 1
    ref_dw = O.embedding_backward_sequential(ids.numpy(), g.numpy(), master.num_embeddings, padding_idx)
    assert np.array_equal(dw, ref_dw), f"scatter-add differs in {(dw != ref_dw).sum()} elements"
    return layer


@pytest.mark.parametrize("ws", [1, 2, 4])
def test_embedding_reference_shape(ws):
    """nn.Embedding(8,8), ids [8,8] in [0,7) as in tests/test_embedding.py: every row is hit ~9 times."""
    master = nn.Embedding(8, 8)
    ids = torch.randint(0, 7, (8, 8))
    layer = _check(master, ids, torch.randn(8, 8, 8), ws)
    assert layer.embedding.weight.shape == (8, 8 // ws)


def test_embedding_headline_config():
    """table [10240,2048] ~U(-0.1,0.1), 4 shards, ids [32,32], upstream grad ~N(0,1)."""
    gen = torch.Generator().manual_seed(0)
    master = nn.Embedding(10240, 2048)
    with torch.no_grad():
        master.weight.copy_(torch.rand(10240, 2048, generator=gen) * 0.2 - 0.1)
    ids = torch.randint(0, 10240, (32, 32), generator=gen)
    g = torch.randn(32, 32, 2048, generator=gen)
    layer = _check(master, ids, g, 4)
    # and against torch's own CPU backward
    master(ids).backward(g)
    dw = torch.cat([e.weight.grad for e in layer.embeddings], dim=1).cpu()
    assert torch.equal(dw, master.weight.grad)


def test_embedding_heavy_duplicates_ragged_and_padding():
    master = nn.Embedding(5, 12)
    ids = torch.randint(0, 5, (257,))  # long segments, odd length
    _check(master, ids, torch.randn(257, 12), 4)
    _check(master, torch.full((64,), 3), torch.randn(64, 12), 2)  # a single segment
    _check(master, ids, torch.randn(257, 12), 2, padding_idx=2)
    _check(master, torch.tensor([4]), torch.randn(1, 12), 1)  # one token


def test_embedding_bf16_and_idempotence():
    master = nn.Embedding(50, 32)
    ids = torch.randint(0, 50, (9, 7))
    layer = _layer(master.to(torch.bfloat16), 4, torch.bfloat16)
    out = layer(ids.to(DEV))
    assert torch.equal(out.cpu(), master.weight.detach()[ids]), "bf16 gather is not bit-exact"
    assert torch.equal(layer(ids.to(DEV)), out)


def test_embedding_unsupported_options_raise():
    from rtp_amd.module.embedding import ParallelEmbedding
    with pytest.raises(NotImplementedError):
        ParallelEmbedding(8, 8, 2, 0, max_norm=1.0, device=DEV)
    with pytest.raises(NotImplementedError):
        ParallelEmbedding(8, 8, 2, 0, sparse=True, device=DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ws", [1, 4])
def test_embedding_scaled_positional_is_bit_exact(dtype, ws):
    """(embedding(ids) * sqrt(d) + pe[:L]) and its backward, as the language model applies them
    (rtp/models/transformer_lm_rtp.py:27-28, :49), against the same three torch CPU operations: each step
    rounds to the element type, so equality is exact in fp32 and in bf16."""
    import math
    gen = torch.Generator().manual_seed(3)
    v, d, seq, batch = 37, 48, 11, 5
    master = nn.Embedding(v, d).to(dtype)
    pe = torch.randn(seq + 3, d, generator=gen).to(dtype)
    ids = torch.randint(0, v, (seq, batch), generator=gen)
    g = torch.randn(seq, batch, d, generator=gen).to(dtype)
    scale = math.sqrt(d)
    layer = _layer(master, ws, dtype)
    out = layer.forward_scaled_positional(ids.to(DEV), scale, pe.to(DEV))
    ref = master(ids) * scale + pe[:seq, None, :]
    assert out.dtype == dtype and torch.equal(out.cpu(), ref.detach())
    out.backward(g.to(DEV))
    ref.backward(g)
    dw = torch.cat([e.weight.grad for e in layer.embeddings], dim=1).cpu()
    if dtype == torch.float32:
        assert torch.equal(dw, master.weight.grad)
    else:
        # torch's CPU bf16 index_add_ rounds the running sum after every add; the device sums in fp32 and rounds
        # once, so compare with the fp32 ordered sum of the bf16-rounded scaled rows
        scaled = (g * scale).float().numpy()
        want = O.embedding_backward_sequential(ids.numpy(), scaled, v, None)
        want_t = torch.from_numpy(want).to(dw.dtype)  # the gradient buffer is fp32 or the layer's dtype
        assert torch.equal(dw, want_t)
    with pytest.raises(ValueError):
        layer.forward_scaled_positional(ids.to(DEV), scale, pe[:seq - 1].to(DEV))


@pytest.mark.parametrize("n,vocab", [(1, 5), (2, 3), (1000, 7), (1024, 10240), (4097, 50), (8192, 1 << 30), (8193, 100),
                                     (40000, 977)])
def test_sorted_token_ids_are_the_stable_sort_by_id(n, vocab):
    """rtp_embedding_sort_ids leaves (id, position) pairs ordered by id, equal ids by ascending position -- the order
    the scatter-add sums in.  Up to 8192 ids are sorted by one workgroup in LDS, more by the device-wide radix sort."""
    from rtp_amd import _lib
    gen = torch.Generator().manual_seed(n)
    ids = torch.randint(0, vocab, (n,), generator=gen)
    lib = _lib.load()
    _lib.require_device()
    nbytes = lib.rtp_embedding_scatter_workspace_bytes(n)
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=DEV)
    dev_ids = ids.to(DEV)
    _lib.check(lib.rtp_embedding_sort_ids(torch.cuda.current_stream().cuda_stream, dev_ids.data_ptr(), n, ws.data_ptr(),
                                          nbytes))
    arr = (n * 4 + 255) // 256 * 256
    keys = ws[2 * arr:2 * arr + 4 * n].view(torch.int32).cpu()
    vals = ws[3 * arr:3 * arr + 4 * n].view(torch.int32).cpu()
    order = torch.sort(ids, stable=True).indices
    assert torch.equal(keys.long(), ids[order]) and torch.equal(vals.long(), order)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_update_applied_by_the_scatter_add_is_bit_identical(dtype):
    """RotatedSGD(fused_backward=True): the rows the step's tokens name are updated by the scatter-add itself and the
    others left alone; weights after two steps equal those of the separate gradient + update launches bit for bit,
    with a padding row, repeated ids and gradient scaling by frequency."""
    from rtp_amd.module.embedding import ParallelEmbedding
    from rtp_amd.optim import RotatedSGD
    V, D, ws = 300, 64, 4
    gen = torch.Generator().manual_seed(23)
    master = torch.nn.Embedding(V, D, padding_idx=7, scale_grad_by_freq=True)
    with torch.no_grad():
        master.weight.copy_((torch.randn(V, D, generator=gen) * 0.5).to(dtype).float())
    twins = []
    for fused in (False, True):
        emb = ParallelEmbedding(V, D, ws, 0, padding_idx=7, scale_grad_by_freq=True, Embedding_layer=master,
                                device=DEV, dtype=dtype)
        twins.append((emb, RotatedSGD(emb, lr=0.1, clip_value=0.05, fused_backward=fused)))
    for step in range(2):
        ids = torch.randint(0, V, (9, 5), generator=gen)
        ids[0, :3] = 7          # padding rows
        ids[1:4, 0] = 11        # a repeated id
        coef = torch.randn(9, 5, D, generator=gen).to(dtype).to(DEV)
        for emb, opt in twins:
            opt.zero_grad()
            (emb(ids.to(DEV)) * coef).sum().backward()
            opt.step()
        torch.cuda.synchronize()
        for (a, _), (b, _) in zip(*[[(p, None) for p in t[0].parameters()] for t in twins]):
            assert torch.equal(a, b), f"step {step}"
    # the fused twin never filled or wrote its dense gradient table
    assert twins[1][0]._store.fused_sgd is not None


@pytest.mark.parametrize("dtype,table_f32", [(torch.float32, False), (torch.bfloat16, False), (torch.bfloat16, True)])
@pytest.mark.parametrize("n,vocab,cols,groups", [(1024, 10240, 512, 4), (257, 5, 12, 2), (64, 3, 8, 1), (4096, 50, 24, 3),
                                                 (1, 9, 7, 1), (300, 40, 33, 2)])
def test_one_launch_backward_equals_sort_and_scatter(dtype, table_f32, n, vocab, cols, groups):
    """rtp_embedding_backward (no sort, ids staged in LDS, zero fill in the same launch) against
    rtp_embedding_sort_ids + rtp_embedding_scatter_add_*: bit for bit, overwriting and accumulating, with a padding
    id, frequency scaling, a gradient scale, a shard that owns only part of the vocabulary rows, and column counts that
    are not whole 16-byte vectors (the element-wise form)."""
    from rtp_amd import ops
    gen = torch.Generator().manual_seed(n + cols)
    ids = torch.randint(0, vocab, (n,), generator=gen)
    if n > 8:
        ids[n // 2:n // 2 + 3] = ids[0]                                  # repeats far apart
    g = torch.randn(n, groups * cols, generator=gen).to(dtype).to(DEV)
    tdt = torch.float32 if table_f32 else dtype
    row_begin, rows = (vocab // 4, vocab // 2) if vocab >= 8 else (0, vocab)  # a shard of the vocabulary rows
    start = torch.randn(groups, rows, cols, generator=gen).to(tdt).to(DEV)
    dev_ids = ids.to(DEV)
    ws = ops.embedding_sort_ids(dev_ids)
    for zero_fill, by_freq, scale, pad in ((True, False, 1.0, -1), (False, False, 1.0, int(ids[0])), (True, True, 0.25, -1),
                                           (False, True, 3.0, int(ids[-1]))):
        a, b = start.clone(), start.clone()
        kw = dict(row_begin=row_begin, padding_idx=pad, scale_by_freq=by_freq, zero_fill=zero_fill, groups=groups,
                  grad_out_sg=cols, grad_table_sg=rows * cols, grad_scale=scale)
        ops.embedding_scatter_add(g[:, :cols], n, ws, a[0], **kw)
        ops.embedding_backward(g[:, :cols], dev_ids, b[0], **kw)
        torch.cuda.synchronize()
        assert torch.equal(a, b), f"zero_fill={zero_fill} by_freq={by_freq} scale={scale} pad={pad}"
    assert ops.embedding_backward_supported(4096) and not ops.embedding_backward_supported(4097)


def test_long_steps_take_the_sorted_path_and_stay_bit_exact():
    """More tokens than the one-launch backward stages in LDS: the module sorts the ids once and scatter-adds."""
    master = nn.Embedding(97, 24)
    ids = torch.randint(0, 97, (5000,))
    _check(master, ids, torch.randn(5000, 24), 4)
