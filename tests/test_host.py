"""Host-side logic that needs no GPU: shard layouts, flat-parameter aliasing, ring order, world-size
resolution and the drop-in constructor surface."""
import inspect

import pytest
import torch
import torch.nn as nn

from oracle import rtp_oracle as O
from rtp_amd import emulate_shards
from rtp_amd.module import attention, collectives, conv, embedding, linear, moe, top2gate, utils
from rtp_amd.ring import ring_order


def test_ring_order_forward_and_backward():
    assert ring_order(0, 4) == [0, 1, 2, 3]
    assert ring_order(2, 4) == [2, 3, 0, 1] == O.ring_order(2, 4)
    assert ring_order(2, 4, reverse=True) == [1, 0, 3, 2]
    assert ring_order(0, 1) == [0]


def test_resolve_world_precedence(monkeypatch):
    monkeypatch.delenv("RTP_EMULATED_SHARDS", raising=False)
    assert collectives.resolve_world() == (1, 0)
    monkeypatch.setenv("RTP_EMULATED_SHARDS", "8")
    assert collectives.resolve_world() == (8, 0)
    with emulate_shards(2):
        assert collectives.resolve_world() == (2, 0)
        with emulate_shards(4):
            assert collectives.resolve_world() == (4, 0)
        assert collectives.resolve_world() == (2, 0)
    with pytest.raises(ValueError):
        with emulate_shards(0):
            pass


def test_attention_with_own_key_and_value_widths_keeps_three_projection_blocks():
    """kdim / vdim != embed_dim (rtp/module/attention.py:51-55, :81-84): q / k / v_proj_weight row blocks of shard s,
    the packed bias re-interleaved as for the packed weight, and the rank state dict under the reference's names."""
    from rtp_amd.checkpoint import rank_state_dict
    mha = nn.MultiheadAttention(8, 4, kdim=6, vdim=10)
    with torch.no_grad():
        mha.in_proj_bias.copy_(torch.randn(24))
    layer = attention.ParallelMultiheadAttention(8, 4, 2, 0, kdim=6, vdim=10, MultiheadAttention_layer=mha)
    assert layer._store.names == ["q_proj_weight", "k_proj_weight", "v_proj_weight", "in_proj_bias", "out_proj.weight",
                                  "out_proj.bias"]
    for s, sub in enumerate(layer.layers):
        rows = slice(4 * s, 4 * s + 4)
        assert torch.equal(sub.q_proj_weight, mha.q_proj_weight[rows]) and sub.in_proj_weight is None
        assert torch.equal(sub.k_proj_weight, mha.k_proj_weight[rows]) and sub.k_proj_weight.shape == (4, 6)
        assert torch.equal(sub.v_proj_weight, mha.v_proj_weight[rows]) and sub.v_proj_weight.shape == (4, 10)
        b = mha.in_proj_bias.detach().view(3, 2, 4)[:, s].reshape(-1)
        assert torch.equal(sub.in_proj_bias, b)
    holder = nn.Module()
    holder.attn = layer
    sd = rank_state_dict(holder, 1)
    assert torch.equal(sd["attn.MultiheadAttention.k_proj_weight"], mha.k_proj_weight[4:8])


def test_column_row_shard_layouts_match_oracle():
    master = nn.Linear(12, 8)
    with emulate_shards(4):
        col = linear.ColumnParallelLinear(12, 8, linear_layer=master)
        row = linear.RowParallelLinear(12, 8, linear_layer=master)
    for s, (w, b) in enumerate(O.column_shards(master.weight.detach(), master.bias.detach(), 4)):
        assert torch.equal(col.linears[s].weight, w) and torch.equal(col.linears[s].bias, b)
    for s, (w, b) in enumerate(O.row_shards(master.weight.detach(), master.bias.detach(), 4)):
        assert torch.equal(row.linears[s].weight, w) and torch.allclose(row.linears[s].bias, b)
    assert col.linear is col.linears[0] and col.world_size == 4 and col.rank == 0
    assert col.linear.weight.shape == (2, 12) and row.linear.weight.shape == (8, 3)


def test_flat_param_order_and_aliasing():
    """One flat buffer per shard in named_parameters() order; parameters are views of it."""
    mha = nn.MultiheadAttention(8, 4)
    layer = attention.ParallelMultiheadAttention(8, 4, 2, 0, MultiheadAttention_layer=mha)
    st = layer._store
    assert st.names == ["in_proj_weight", "in_proj_bias", "out_proj.weight", "out_proj.bias"]
    assert st.numel == 12 * 8 + 12 + 8 * 4 + 8 and st.home.shape == (2, st.numel)
    for s, sub in enumerate(layer.layers):
        assert sub._full_param.data_ptr() == st.home[s].data_ptr()
        off = 0
        for p in sub.parameters():
            assert p.data_ptr() == st.home[s].data_ptr() + off * 4
            off += p.numel()
        w_in, b_in, w_o, b_o = O.attention_shard_params(mha.in_proj_weight.detach(), mha.in_proj_bias.detach(),
                                                         mha.out_proj.weight.detach(), mha.out_proj.bias.detach(), 2, s)
        assert torch.equal(sub.in_proj_weight, w_in) and torch.equal(sub.in_proj_bias, b_in)
        assert torch.equal(sub.out_proj.weight, w_o) and torch.allclose(sub.out_proj.bias, b_o)
    # writing through a parameter view changes the flat buffer (flyweight)
    with torch.no_grad():
        layer.layers[1].in_proj_bias.fill_(3.0)
    assert float(st.home[1, 96]) == 3.0
    assert len(list(layer.parameters())) == 8  # every shard's parameters, once


def test_attention_block_index_is_q_k_v_rows_of_the_head_group():
    E, ws = 8, 2
    in_w = torch.arange(3 * E * E, dtype=torch.float32).view(3 * E, E)
    for s in range(ws):
        w_in, _, _, _ = O.attention_shard_params(in_w, None, torch.zeros(E, E), None, ws, s)
        e_s = E // ws
        expect = torch.cat([in_w[s * e_s:(s + 1) * e_s], in_w[E + s * e_s:E + (s + 1) * e_s],
                            in_w[2 * E + s * e_s:2 * E + (s + 1) * e_s]])
        assert torch.equal(w_in, expect)
        assert utils.attention_block_index(s, ws) == [s, s + ws, s + 2 * ws]


def test_embedding_shards_are_column_blocks():
    master = nn.Embedding(10, 8)
    layer = embedding.ParallelEmbedding(10, 8, 4, 0, Embedding_layer=master)
    assert layer.embedding.weight.shape == (10, 2)
    assert torch.equal(torch.cat([e.weight for e in layer.embeddings], 1), master.weight)


def test_repack_after_dtype_change_keeps_values_and_aliasing():
    master = nn.Linear(6, 4)
    with emulate_shards(2):
        col = linear.ColumnParallelLinear(6, 4, linear_layer=master)
    col.to(torch.bfloat16)
    assert col._store.home.dtype == torch.bfloat16
    assert col.linears[1].weight.data_ptr() == col._store.home[1].data_ptr()
    assert torch.equal(col.linears[1].weight, master.weight[2:4].to(torch.bfloat16))


def test_moe_and_gate_shards():
    from rtp_amd.models.transformer_lm_rtp import FeedForwardLayer_expert
    g = top2gate.Top2Gate(8, 4)
    with emulate_shards(2):
        gate = top2gate.WeightTop2Gate(8, 4, gate=g)
        local = FeedForwardLayer_expert(8, 16, nn.ReLU(), 0.0)
        layer = moe.WeightMOELayer(gate, local)
    assert torch.equal(torch.cat([w.weight for w in gate.wgs], 0), g.wg.weight)
    assert gate.wg.weight.shape == (2, 8) and layer.num_local_experts == 1 and len(layer.experts_list) == 2
    assert layer._store.names == ["0.linear1.weight", "0.linear1.bias", "0.linear2.weight", "0.linear2.bias"]
    with pytest.raises(NotImplementedError):
        with emulate_shards(2):
            moe.WeightMOELayer(gate, nn.Linear(8, 8))


def test_top2gate_state_dict_has_the_reference_key_set():
    """The unsharded gate's state dict is {'wg.weight'} (rtp/module/top2gate.py:124): a plain dict of that form
    loads strictly, the flat home row follows, and dtype moves keep the aliasing."""
    g = top2gate.Top2Gate(8, 4)
    assert list(g.state_dict().keys()) == ["wg.weight"]
    assert [n for n, _ in g.named_parameters()] == ["wg.weight"]
    w = torch.arange(32, dtype=torch.float32).view(4, 8)
    g.load_state_dict({"wg.weight": w}, strict=True)
    assert torch.equal(g.wg.weight, w) and torch.equal(g._store.home.view(4, 8), w)
    g.to(torch.bfloat16)
    assert g.wg.weight.data_ptr() == g._store.home.data_ptr() and g.shards[0] is g.wg


def test_forward_without_gpu_fails_loudly():
    from rtp_amd._lib import RtpError
    with emulate_shards(2):
        col = linear.ColumnParallelLinear(4, 4)
    with pytest.raises((RtpError, RuntimeError)):
        col(torch.zeros(2, 4))


@pytest.mark.parametrize("cls,expected", [
    (linear.ColumnParallelLinear, ["in_features", "out_features", "bias", "gather_weight", "init_method", "stride",
                                   "keep_master_weight_for_test", "device", "dtype", "group", "linear_layer"]),
    (linear.RowParallelLinear, ["in_features", "out_features", "bias", "gather_weight", "init_method", "stride",
                                "keep_master_weight_for_test", "device", "dtype", "group", "linear_layer"]),
    (embedding.ParallelEmbedding, ["num_embeddings", "embedding_dim", "world_size", "rank", "padding_idx", "max_norm",
                                   "norm_type", "scale_grad_by_freq", "sparse", "init_method",
                                   "keep_master_weight_for_test", "Embedding_layer", "device", "dtype"]),
    (attention.ParallelMultiheadAttention, ["embed_dim", "num_heads", "world_size", "rank", "dropout", "bias",
                                            "add_bias_kv", "add_zero_attn", "kdim", "vdim", "batch_first", "device",
                                            "dtype", "MultiheadAttention_layer"]),
    (top2gate.WeightTop2Gate, ["model_dim", "num_experts", "gate", "device", "dtype"]),
    (moe.WeightMOELayer, ["gate", "experts", "group", "device", "dtype", "original_experts"]),
    (conv.ColumnParallelConv2d, ["in_channels", "out_channels", "kernel_size", "stride", "padding", "dilation",
                                 "groups", "bias", "padding_mode", "device", "dtype", "group", "gather_output",
                                 "Conv2d_layer"]),
])
def test_constructor_signatures_match_reference(cls, expected):
    params = [p for p in inspect.signature(cls.__init__).parameters if p != "self"]
    assert params == expected


def test_reference_import_paths_resolve_to_the_same_objects():
    """Every import path of the reference's hot path (rtp/rotated_tensor_parallel.py, rtp/attention.py,
    rtp/module/*.py, rtp/models/transformer_lm_rtp.py) resolves here, to the very objects of rtp_amd."""
    import importlib
    pairs = {
        "rtp.rotated_tensor_parallel": ["RotatedTensorParallel", "FlyweightWarpper", "split_tensor"],
        "rtp.attention": ["ParallelMultiheadAttention"],
        "rtp.module.linear": ["ColumnParallelLinear", "RowParallelLinear", "ModelParallelLinear", "ModelParallelLinear2"],
        "rtp.module.embedding": ["ParallelEmbedding", "ModelParallelEmbedding"],
        "rtp.module.attention": ["ParallelMultiheadAttention", "SubParallelMultiheadAttention"],
        "rtp.module.moe": ["WeightMOELayer"],
        "rtp.module.top2gate": ["top2gating", "Top2Gate", "WeightTop2Gate", "gumbel_rsample"],
        "rtp.module.collectives": ["zero_full_grads"],
        "rtp.module.conv": ["ColumnParallelConv2d", "ModelParallelConv2d"],
        "rtp.module.utils": ["affine_weight", "affine_weight_attention", "divide_and_check_no_remainder",
                             "ensure_divisibility", "split_tensor_along_last_dim"],
        "rtp.models.transformer_lm_rtp": ["TransformerLM", "EmbeddingLayer", "PositionalEncodingLayer",
                                          "FeedForwardLayer", "FeedForwardLayer_expert", "TransformerDecoderLayer",
                                          "TransformerEncoderLayer", "LinearLayer"],
    }
    for path, names in pairs.items():
        theirs = importlib.import_module(path)
        mine = importlib.import_module(path.replace("rtp.", "rtp_amd.", 1))
        assert theirs is mine, path
        for n in names:
            assert getattr(theirs, n) is getattr(mine, n), f"{path}.{n}"
    from rtp.module.linear import ColumnParallelLinear as C1   # the `from ... import` form as well
    assert C1 is linear.ColumnParallelLinear
    import rtp.attention
    import rtp.module.attention
    assert rtp.attention.ParallelMultiheadAttention is not rtp.module.attention.ParallelMultiheadAttention


def test_flyweight_wrapper_takes_the_reference_constructor_arguments():
    """rtp/rotated_tensor_parallel.py:296-310, and a leaf cut to one rank's share by hand (:454-529)."""
    from rtp_amd.rotated_tensor_parallel import FlyweightWarpper, split_tensor
    params = [p for p in inspect.signature(FlyweightWarpper.__init__).parameters if p != "self"]
    assert params == ["module", "group", "param_list", "flat_param_names", "partition_dim", "output_partition_dim",
                      "row_partition", "input_partition_dim", "cat_output", "inplace"]
    ws = 2
    master = nn.Linear(6, 4)
    leaves = []
    for r in range(ws):       # what rank r of the reference does before wrapping a column shard
        leaf = nn.Linear(6, 2)
        leaf.weight = nn.Parameter(split_tensor(master.weight, ws, dim=0)[r].clone())
        leaf.bias = nn.Parameter(split_tensor(master.bias, ws, dim=0)[r].clone())
        leaves.append(leaf)
    with emulate_shards(ws):
        col = FlyweightWarpper(leaves, None)
        one = FlyweightWarpper(leaves[0])                     # a single leaf: every rank starts from a copy
        rows = []
        for r in range(ws):   # row shards: weight columns, bias / ws
            leaf = nn.Linear(3, 4)
            leaf.weight = nn.Parameter(split_tensor(master.weight, ws, dim=-1)[r].clone())
            leaf.bias = nn.Parameter(master.bias.detach() / ws)
            rows.append(leaf)
        row = FlyweightWarpper(rows, None, row_partition=True, input_partition_dim=-1)
        with pytest.raises(NotImplementedError):
            FlyweightWarpper(nn.LayerNorm(4))
        with pytest.raises(ValueError):
            FlyweightWarpper(leaves + leaves)
        with pytest.raises(NotImplementedError):
            FlyweightWarpper(nn.Conv2d(2, 4, 3))              # conv outputs concatenate on dim 1
        convw = FlyweightWarpper(nn.Conv2d(2, 4, 3), output_partition_dim=1)
        emb = FlyweightWarpper(nn.Embedding(10, 3))
    assert type(col.rotated) is linear.ColumnParallelLinear and col.world_size == ws and col.rank == 0
    assert torch.equal(torch.cat([m.weight for m in col.module_list], 0), master.weight)
    assert torch.equal(torch.cat([m.bias for m in col.module_list], 0), master.bias)
    assert col.flat_param.data_ptr() == col.module.weight.data_ptr() and col.partition_dim == -1
    assert torch.equal(one.module_list[1].weight, leaves[0].weight)
    assert type(row.rotated) is linear.RowParallelLinear and row.row_partition
    assert torch.equal(torch.cat([m.weight for m in row.module_list], 1), master.weight)
    assert type(convw.rotated) is conv.ColumnParallelConv2d and convw.rotated.out_channels == 8
    assert type(emb.rotated) is embedding.ParallelEmbedding and emb.rotated.embedding_dim == 6


def test_attention_leaf_of_the_wrapper_module():
    """rtp/attention.py's ParallelMultiheadAttention is one rank's head group; wrapped, it is the rotated layer."""
    from rtp_amd.attention import ParallelMultiheadAttention as Leaf
    from rtp_amd.rotated_tensor_parallel import FlyweightWarpper
    params = [p for p in inspect.signature(Leaf.__init__).parameters if p != "self"]
    assert params == ["embed_dim", "num_heads", "dropout", "bias", "add_bias_kv", "add_zero_attn", "kdim", "vdim",
                      "batch_first", "device", "dtype", "MultiheadAttention", "empty_init", "group"]
    mha = nn.MultiheadAttention(8, 4)
    ws = 2
    with emulate_shards(ws):
        leaf = Leaf(8, 4, MultiheadAttention=mha)
        assert leaf.in_proj_weight.shape == (12, 8) and leaf.out_proj.weight.shape == (8, 4) and leaf.rank == 0
        leaves = [leaf]
        for r in range(1, ws):
            other = Leaf(8, 4)
            other.rank = r
            other.affine_weight(mha)
            leaves.append(other)
        wrapped = FlyweightWarpper(leaves, None, cat_output=False)
        with pytest.raises(NotImplementedError):
            FlyweightWarpper(leaves, None)                    # attention outputs are summed, not concatenated
    assert type(wrapped.rotated) is attention.ParallelMultiheadAttention
    direct = attention.ParallelMultiheadAttention(8, 4, ws, 0, MultiheadAttention_layer=mha)
    for a, b in zip(wrapped.rotated._store.home, direct._store.home):
        assert torch.equal(a, b)
    with pytest.raises(NotImplementedError):
        leaf(torch.zeros(2, 1, 8), torch.zeros(2, 1, 8), torch.zeros(2, 1, 8))


def test_rank_state_dicts_follow_the_reference_layout_and_round_trip():
    """What rank r of the reference saves (its own shard under the home attribute's name, rtp/module/linear.py:187:
    only `self.linear` is a registered submodule) and loading ws such dicts back into all shards held here."""
    from rtp_amd.checkpoint import load_rank_state_dicts, rank_state_dict, world_size_of

    class Net(nn.Module):
        def __init__(self, lin, mha, emb):
            super().__init__()
            self.emb = embedding.ParallelEmbedding(10, 8, 4, 0, Embedding_layer=emb)
            self.attn = attention.ParallelMultiheadAttention(8, 4, 4, 0, MultiheadAttention_layer=mha)
            with emulate_shards(4):
                self.fc = linear.ColumnParallelLinear(8, 12, linear_layer=lin)
            self.norm = nn.LayerNorm(8)

    torch.manual_seed(0)
    lin, mha, emb = nn.Linear(8, 12), nn.MultiheadAttention(8, 4), nn.Embedding(10, 8)
    net = Net(lin, mha, emb)
    assert world_size_of(net) == 4
    dicts = [rank_state_dict(net, r) for r in range(4)]
    assert list(dicts[2].keys()) == [
        "emb.embedding.weight", "attn.MultiheadAttention.in_proj_weight", "attn.MultiheadAttention.in_proj_bias",
        "attn.MultiheadAttention.out_proj.weight", "attn.MultiheadAttention.out_proj.bias", "fc.linear.weight",
        "fc.linear.bias", "norm.weight", "norm.bias"]
    for r in range(4):
        assert torch.equal(dicts[r]["fc.linear.weight"], lin.weight[3 * r:3 * r + 3])          # output rows
        assert torch.equal(dicts[r]["fc.linear.bias"], lin.bias[3 * r:3 * r + 3])
        assert torch.equal(dicts[r]["emb.embedding.weight"], emb.weight[:, 2 * r:2 * r + 2])   # embedding columns
        assert torch.equal(dicts[r]["attn.MultiheadAttention.out_proj.weight"], mha.out_proj.weight[:, 2 * r:2 * r + 2])
        w = O.attention_shard_params(mha.in_proj_weight.detach(), mha.in_proj_bias.detach(),
                                     mha.out_proj.weight.detach(), mha.out_proj.bias.detach(), 4, r)
        assert torch.equal(dicts[r]["attn.MultiheadAttention.in_proj_weight"], w[0])
    # into a differently initialised model of the same architecture
    other = Net(nn.Linear(8, 12), nn.MultiheadAttention(8, 4), nn.Embedding(10, 8))
    saved = [{k: v.clone() for k, v in d.items()} for d in dicts]
    load_rank_state_dicts(other, saved)
    for (ka, a), (kb, b) in zip(net.state_dict().items(), other.state_dict().items()):
        assert ka == kb and torch.equal(a, b)
    st = other.fc._store
    assert other.fc.linears[1].weight.data_ptr() == st.home[1].data_ptr()   # still views of the flat buffer
    # strictness: a replicated entry that differs between ranks, a missing rank, a foreign key
    saved[3]["norm.weight"] = saved[3]["norm.weight"] + 1
    with pytest.raises(ValueError):
        load_rank_state_dicts(other, saved)
    with pytest.raises(ValueError):
        load_rank_state_dicts(other, saved[:3])
    saved[3]["norm.weight"] = saved[0]["norm.weight"]
    saved[0]["nope.weight"] = torch.zeros(1)
    with pytest.raises(KeyError):
        load_rank_state_dicts(other, saved)
    with pytest.raises(ValueError):
        rank_state_dict(net, 4)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asking for more exits with a message instead of a number."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                         timeout=120)
    assert res.returncode == 2 and "one GPU" in res.stderr and res.stdout.strip() == ""
