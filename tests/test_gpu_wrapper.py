"""RotatedTensorParallel: wrap a stock torch model in place and compare it with an untouched copy
(the structure of the reference's test.py:126-195 and test_net.py:135-177)."""
import copy

import pytest
import torch
import torch.nn as nn

from gpu_util import DEV, assert_close
from oracle import rtp_oracle as O

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("rotation_window")]


class Net(nn.Module):
    def __init__(self):
        super().__init__()
        self.emb = nn.Embedding(40, 16)
        self.attn = nn.MultiheadAttention(16, 4)
        self.fc1 = nn.Linear(16, 24)   # out_features % ws == 0 -> column shards
        self.fc2 = nn.Linear(24, 6)    # 6 % 4 != 0 but 24 % 4 == 0 -> row shards
        self.norm = nn.LayerNorm(16)

    def forward(self, ids):
        x = self.emb(ids)
        x = self.norm(x + self.attn(x, x, x, need_weights=False)[0])
        return self.fc2(torch.relu(self.fc1(x)))


def test_wrapper_matches_unwrapped_model():
    from rtp_amd import emulate_shards
    from rtp_amd.rotated_tensor_parallel import FlyweightWarpper, RotatedTensorParallel
    ws = 4
    ref = Net()
    with emulate_shards(ws):
        model = RotatedTensorParallel(copy.deepcopy(ref)).to(DEV)
    kinds = [type(w.rotated).__name__ for w in model.FlyweightModule_list]
    assert kinds == ["ParallelEmbedding", "ParallelMultiheadAttention", "ColumnParallelLinear", "RowParallelLinear"]
    assert isinstance(model.module.fc2, FlyweightWarpper) and model.module.fc2.row_partition
    assert isinstance(model.module.norm, nn.LayerNorm)
    ids = torch.randint(0, 40, (7, 3))
    g = torch.randn(7, 3, 6)
    out = model(ids.to(DEV))
    out.backward(g.to(DEV))
    ref_out = ref(ids)
    ref_out.backward(g)
    assert_close(out, ref_out, torch.float32, "output")
    m = model.module
    # rank-r shard gradient == the matching slice of the unsharded gradient (test.py:182-193)
    assert_close(torch.cat([s.weight.grad for s in m.fc1.module_list], 0), ref.fc1.weight.grad, torch.float32, "fc1")
    assert_close(torch.cat([s.weight.grad for s in m.fc2.module_list], 1), ref.fc2.weight.grad, torch.float32, "fc2")
    assert_close(m.fc2.module.bias.grad, ref.fc2.bias.grad, torch.float32, "fc2 bias")
    assert_close(torch.cat([s.weight.grad for s in m.emb.module_list], 1), ref.emb.weight.grad, torch.float32, "emb")
    assert_close(O.attention_grad_reinterleave([s.in_proj_weight.grad for s in m.attn.module_list], ws),
                 ref.attn.in_proj_weight.grad, torch.float32, "attn in_proj")
    assert_close(m.norm.weight.grad, ref.norm.weight.grad, torch.float32, "layernorm")
    assert m.fc1.flat_param.data_ptr() == m.fc1.module.weight.data_ptr()


def test_wrapper_indivisible_linear_raises():
    from rtp_amd import emulate_shards
    from rtp_amd.rotated_tensor_parallel import RotatedTensorParallel
    with emulate_shards(4), pytest.raises(ValueError):
        RotatedTensorParallel(nn.Sequential(nn.Linear(6, 7)))


def test_wrapper_on_stock_transformer_decoder_layer():
    """torch.nn.TransformerDecoderLayer wrapped in place: its self-attention, its attention over the encoder memory
    (keys and values from another tensor, with a key padding mask) and both feed-forward projections become rotated
    layers; output and the gradients reaching both inputs must match the untouched copy."""
    from rtp_amd import emulate_shards
    from rtp_amd.rotated_tensor_parallel import RotatedTensorParallel
    torch.manual_seed(0)
    ref = nn.TransformerDecoderLayer(d_model=32, nhead=4, dim_feedforward=64, dropout=0.0)
    with emulate_shards(4):
        model = RotatedTensorParallel(copy.deepcopy(ref)).to(DEV)
    kinds = sorted(type(w.rotated).__name__ for w in model.FlyweightModule_list)
    assert kinds == ["ColumnParallelLinear", "ColumnParallelLinear", "ParallelMultiheadAttention",
                     "ParallelMultiheadAttention"]
    tgt, mem, g = torch.randn(6, 3, 32), torch.randn(9, 3, 32), torch.randn(6, 3, 32)
    causal = torch.triu(torch.full((6, 6), float("-inf")), diagonal=1)
    mem_pad = torch.zeros(3, 9, dtype=torch.bool)
    mem_pad[1, 7:] = True
    a, b = tgt.to(DEV).requires_grad_(), mem.to(DEV).requires_grad_()
    out = model(a, b, tgt_mask=causal.to(DEV), memory_key_padding_mask=mem_pad.to(DEV))
    out.backward(g.to(DEV))
    ra, rb = tgt.clone().requires_grad_(), mem.clone().requires_grad_()
    want = ref(ra, rb, tgt_mask=causal, memory_key_padding_mask=mem_pad)
    want.backward(g)
    assert_close(out, want, torch.float32, "output")
    assert_close(a.grad, ra.grad, torch.float32, "target grad")
    assert_close(b.grad, rb.grad, torch.float32, "memory grad")
    m = model.module
    assert_close(O.attention_grad_reinterleave([s.in_proj_weight.grad for s in m.multihead_attn.module_list], 4),
                 ref.multihead_attn.in_proj_weight.grad, torch.float32, "memory attention in_proj")


@pytest.mark.parametrize("overlap", [False, True])
def test_wrapped_model_trains_with_a_stock_optimizer(overlap):
    """Three steps of torch.optim.SGD + clip_grad_value_ on model.parameters() (what the reference harness does,
    benchmarks/rtp_benchmark.py:185-186) against the untouched copy on the CPU: nobody calls ring.fence() or
    join_wgrad() here, the optimiser hooks order the staging copies and the second-stream weight gradients."""
    from rtp_amd import emulate_shards, ring
    from rtp_amd.rotated_tensor_parallel import RotatedTensorParallel
    class ColumnNet(nn.Module):
        """Only layers whose shards partition the parameters: a row-parallel bias (and the attention's output bias)
        is held as bias/ws by every shard and each copy receives the whole gradient (rtp/module/linear.py:133-135),
        so after an optimiser step such a model no longer equals its unsharded twin -- in the reference as here."""

        def __init__(self):
            super().__init__()
            self.emb = nn.Embedding(40, 16)
            self.norm = nn.LayerNorm(16)
            self.fc1 = nn.Linear(16, 24)
            self.fc2 = nn.Linear(24, 8)

        def forward(self, ids):
            return self.fc2(torch.relu(self.fc1(self.norm(self.emb(ids)))))

    ws = 4
    torch.manual_seed(3)
    ref = ColumnNet()
    with emulate_shards(ws):
        model = RotatedTensorParallel(copy.deepcopy(ref)).to(DEV)
    assert [type(w.rotated).__name__ for w in model.FlyweightModule_list] == \
        ["ParallelEmbedding", "ColumnParallelLinear", "ColumnParallelLinear"]
    opt = torch.optim.SGD(model.parameters(), lr=0.1)
    ref_opt = torch.optim.SGD(ref.parameters(), lr=0.1)
    gen = torch.Generator().manual_seed(5)
    ring.set_wgrad_overlap(overlap)
    try:
        for step in range(3):
            ids = torch.randint(0, 40, (7, 3), generator=gen)
            g = torch.randn(7, 3, 8, generator=gen)
            big = torch.randn(2048, 2048, device=DEV)
            (big @ big).sum()  # the compute stream is busy when the step starts: the side stream runs ahead of it
            opt.zero_grad()
            out = model(ids.to(DEV))
            out.backward(g.to(DEV))
            torch.nn.utils.clip_grad_value_(model.parameters(), 0.05)
            opt.step()
            ref_opt.zero_grad()
            ref_out = ref(ids)
            ref_out.backward(g)
            torch.nn.utils.clip_grad_value_(ref.parameters(), 0.05)
            ref_opt.step()
            assert_close(out, ref_out, torch.float32, f"step {step} output")
    finally:
        ring.set_wgrad_overlap(False)
    m = model.module
    assert_close(torch.cat([s.weight for s in m.fc1.module_list], 0), ref.fc1.weight, torch.float32, "fc1 after 3 steps")
    assert_close(torch.cat([s.weight for s in m.emb.module_list], 1), ref.emb.weight, torch.float32, "emb after 3 steps")


def test_leaves_wrapped_by_hand_with_the_reference_constructor():
    """Code that cuts a leaf to a rank's share and wraps it itself (rtp/rotated_tensor_parallel.py:454-470 done by
    hand): column shards of one Linear and row shards of the next, through the reference's import path."""
    from rtp.rotated_tensor_parallel import FlyweightWarpper, split_tensor
    from rtp_amd import emulate_shards
    ws = 4
    torch.manual_seed(1)
    fc1, fc2 = nn.Linear(16, 24), nn.Linear(24, 6)
    cols, rows = [], []
    for r in range(ws):
        leaf = nn.Linear(16, 6)
        leaf.weight = nn.Parameter(split_tensor(fc1.weight, ws, dim=0)[r].clone())
        leaf.bias = nn.Parameter(split_tensor(fc1.bias, ws, dim=0)[r].clone())
        cols.append(leaf.to(DEV))
        leaf = nn.Linear(6, 6)
        leaf.weight = nn.Parameter(split_tensor(fc2.weight, ws, dim=-1)[r].clone())
        leaf.bias = nn.Parameter(fc2.bias.detach() / ws)
        rows.append(leaf.to(DEV))
    with emulate_shards(ws):
        w1 = FlyweightWarpper(cols, None)
        w2 = FlyweightWarpper(rows, None, row_partition=True, input_partition_dim=-1)
    x, g = torch.randn(9, 16), torch.randn(9, 6)
    xd = x.to(DEV).requires_grad_()
    out = w2(torch.relu(w1(xd)))
    out.backward(g.to(DEV))
    xr = x.clone().requires_grad_()
    want = fc2(torch.relu(fc1(xr)))
    want.backward(g)
    assert_close(out, want, torch.float32, "output")
    assert_close(xd.grad, xr.grad, torch.float32, "input grad")
    assert_close(torch.cat([s.weight.grad for s in w1.module_list], 0), fc1.weight.grad, torch.float32, "fc1")
    assert_close(torch.cat([s.weight.grad for s in w2.module_list], 1), fc2.weight.grad, torch.float32, "fc2")
    assert_close(w2.module.bias.grad, fc2.bias.grad, torch.float32, "fc2 bias")


def test_language_model_through_the_reference_import_path():
    """`from rtp.models.transformer_lm_rtp import TransformerLM` with the reference's argument list builds the
    rotated model of this library and runs a step on the device."""
    from rtp.models.transformer_lm_rtp import TransformerLM
    from rtp.module.collectives import zero_full_grads
    from rtp_amd.models import transformer_lm_rtp as mine
    assert TransformerLM is mine.TransformerLM
    V, ws = 64, 2
    lm = TransformerLM(V, 32, 2, 32, 0.0, 0.1, 1, ws, 0, device=DEV, dtype=torch.float32)
    ids = torch.randint(0, V, (6, 3)).to(DEV)
    logits = lm(ids)
    assert logits.shape == (6, 3, V)
    torch.nn.functional.cross_entropy(logits.view(-1, V), ids.view(-1)).backward()
    assert all(s.weight.grad is not None for s in lm[-1].linear.linears)
    zero_full_grads(lm)
    assert all(s.weight.grad is None for s in lm[-1].linear.linears)
