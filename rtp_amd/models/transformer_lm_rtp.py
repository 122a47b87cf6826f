"""GPT-2 style nn.Sequential language model built from the rotated layers (counterpart of
rtp/models/transformer_lm_rtp.py:19-242): embedding * sqrt(ninp) -> sinusoidal positions -> N post-LN
decoder layers (rotated self-attention + rotated ReLU FFN or rotated MoE) -> rotated logits projection.
Residual add + LayerNorm is one fused kernel each way (module/norm.py); the FFN's ReLU is folded into its two
products (module/linear.py); the embedding's scale and the positional rows ride on its gather; dropout masks are
drawn by torch's device generator and applied element-wise."""
from __future__ import annotations

import math

import torch
import torch.nn as nn

from .. import ring
from ..module.attention import ParallelMultiheadAttention
from ..module.collectives import emulate_shards
from ..module.embedding import ParallelEmbedding
from ..module.linear import ColumnParallelLinear, column_relu_mlp
from ..module.moe import WeightMOELayer
from ..module.norm import add_layer_norm, layer_norm_fusable
from ..module.top2gate import WeightTop2Gate


class EmbeddingLayer(nn.Module):
    def __init__(self, ntoken, ninp, initrange, world_size, rank, device=None, dtype=None):
        super().__init__()
        self.embedding = ParallelEmbedding(ntoken, ninp, world_size=world_size, rank=rank, device=device, dtype=dtype)
        with torch.no_grad():
            for shard in self.embedding.embeddings:
                shard.weight.data.uniform_(-initrange, initrange)
        self.ninp_sqrt = math.sqrt(ninp)
        self.positional = None  # set by adopt_positional

    def adopt_positional(self, layer: "PositionalEncodingLayer") -> None:
        """Take over the addition of the positional rows from the layer that follows (which then only applies its
        dropout), so that scale and addition ride on the gather instead of two passes over the activations."""
        object.__setattr__(self, "positional", layer)  # plain attribute: the layer stays registered once, in the model
        layer.added_upstream = True

    def forward(self, src):
        pos = self.positional
        if pos is None:  # on its own, as the reference's layer: the next layer adds the positions
            return self.embedding(src) * self.ninp_sqrt
        if src.dim() != 2:
            raise ValueError("EmbeddingLayer: token ids must be [sequence, batch]")
        return self.embedding.forward_scaled_positional(src, self.ninp_sqrt, pos.pe[:, 0, :])


class PositionalEncodingLayer(nn.Module):
    def __init__(self, d_model, dropout=0.1, max_len=5000, device=None, dtype=None):
        super().__init__()
        self.dropout = nn.Dropout(p=dropout)
        pe = torch.zeros(max_len, d_model)
        position = torch.arange(0, max_len, dtype=torch.float).unsqueeze(1)
        div_term = torch.exp(torch.arange(0, d_model, 2).float() * (-math.log(10000.0) / d_model))
        pe[:, 0::2] = torch.sin(position * div_term)
        pe[:, 1::2] = torch.cos(position * div_term)
        pe = pe.unsqueeze(0).transpose(0, 1)
        self.register_buffer("pe", pe.to(device=device, dtype=dtype))
        self.added_upstream = False  # True once the embedding layer before this one adds the rows itself

    def forward(self, x):
        if not self.added_upstream:
            x = x + self.pe[: x.size(0), :]
        return self.dropout(x)


class FeedForwardLayer_expert(nn.Module):
    """One MoE expert: Linear -> ReLU -> Linear (rtp/models/transformer_lm_rtp.py:63-75)."""

    def __init__(self, d_model, dim_feedforward, activation, dropout, device=None, dtype=None) -> None:
        super().__init__()
        self.linear1 = nn.Linear(d_model, dim_feedforward, device=device, dtype=dtype)
        self.activation = activation
        self.dropout1 = nn.Dropout(dropout)
        self.linear2 = nn.Linear(dim_feedforward, d_model, device=device, dtype=dtype)
        self.dropout2 = nn.Dropout(dropout)

    def forward(self, x):
        return self.dropout2(self.linear2(self.dropout1(self.activation(self.linear1(x)))))


class FeedForwardLayer(nn.Module):
    """Linear -> ReLU -> dropout -> Linear -> dropout over two rotated column-parallel layers
    (rtp/models/transformer_lm_rtp.py:77-89).  The ReLU lives in the epilogues of the two layers' products, so the
    activation must be nn.ReLU (what the reference's TransformerLM always passes)."""

    def __init__(self, d_model, dim_feedforward, activation, dropout, world_size, rank, device=None, dtype=None):
        super().__init__()
        if not isinstance(activation, nn.ReLU):
            raise NotImplementedError("FeedForwardLayer: the rotated feed-forward block computes ReLU inside its products; "
                                      f"got activation {type(activation).__name__}")
        with emulate_shards(world_size):
            self.linear1 = ColumnParallelLinear(d_model, dim_feedforward, device=device, dtype=dtype)
            self.linear2 = ColumnParallelLinear(dim_feedforward, d_model, device=device, dtype=dtype)
        self.activation = activation
        self.dropout1 = nn.Dropout(dropout)
        self.dropout2 = nn.Dropout(dropout)

    def forward(self, x, residual_grad=False):
        p1 = self.dropout1.p if self.training else 0.0
        y = column_relu_mlp(x, self.linear1, self.linear2, residual_grad=residual_grad, dropout_p=p1)
        return y if self.dropout2.p == 0.0 or not self.training else self.dropout2(y)


class TransformerEncoderLayer(nn.Module):
    def __init__(self, d_model, nhead, dim_feedforward=2048, dropout=0.1, activation=nn.ReLU(), layer_norm_eps=1e-5,
                 norm_first=False, is_moe=False, num_local_experts=1, world_size=1, rank=0, device=None, dtype=None):
        super().__init__()
        self.self_attn = ParallelMultiheadAttention(d_model, nhead, dropout=dropout, world_size=world_size,
                                                    rank=rank, device=device, dtype=dtype)
        self.norm_first = norm_first
        self.norm1 = nn.LayerNorm(d_model, eps=layer_norm_eps, device=device, dtype=dtype)
        self.norm2 = nn.LayerNorm(d_model, eps=layer_norm_eps, device=device, dtype=dtype)
        self.dropout = nn.Dropout(dropout)
        self.is_moe = is_moe
        if is_moe:
            num_global_experts = num_local_experts * world_size
            with emulate_shards(world_size):
                self.gate = WeightTop2Gate(d_model, num_global_experts, device=device, dtype=dtype)
                experts = nn.ModuleList([
                    FeedForwardLayer_expert(d_model, dim_feedforward, activation, dropout, device=device, dtype=dtype)
                    for _ in range(num_local_experts)])
                self.moe_layer = WeightMOELayer(self.gate, experts, device=device, dtype=dtype)
        else:
            self.ff_block = FeedForwardLayer(d_model, dim_feedforward, activation, dropout, world_size=world_size,
                                             rank=rank, device=device, dtype=dtype)

        # the block's rotated layers always run back to back: stage them together (one copy-stream wait per block)
        members = [self.self_attn._store]
        if is_moe:
            members += [self.gate._store, self.moe_layer._store]
        else:
            members += [self.ff_block.linear1._store, self.ff_block.linear2._store]
        ring.group_stores(members)

    def forward(self, src, src_mask=None, src_key_padding_mask=None):
        x = src
        if self.norm_first:
            x = x + self._sa_block(self.norm1(x), src_mask, src_key_padding_mask)
            x = x + self._ff_block(self.norm2(x))
        else:
            # With the fused add + LayerNorm, x's gradient is routed through the branch: its last input-gradient
            # product adds the residual part in its epilogue instead of a separate elementwise add.
            no_drop = self.dropout.p == 0.0 or not self.training  # nothing between a branch and its LayerNorm
            via = layer_norm_fusable(x, self.norm1) and x.requires_grad and torch.is_grad_enabled() and no_drop
            x = add_layer_norm(x, self._sa_block(x, src_mask, src_key_padding_mask, residual_grad=via), self.norm1,
                               x_grad_via_branch=via)
            via = via and not self.is_moe and (self.ff_block.dropout2.p == 0.0 or not self.training)
            x = add_layer_norm(x, self.ff_block(x, residual_grad=True) if via else self._ff_block(x), self.norm2,
                               x_grad_via_branch=via)
        return x

    def _sa_block(self, x, attn_mask, key_padding_mask, residual_grad=False):
        x = self.self_attn(x, x, x, attn_mask=attn_mask, key_padding_mask=key_padding_mask, need_weights=False,
                           residual_grad=residual_grad)[0]
        return x if self.dropout.p == 0.0 or not self.training else self.dropout(x)

    def _ff_block(self, x):
        return self.moe_layer(x) if self.is_moe else self.ff_block(x)


class TransformerDecoderLayer(TransformerEncoderLayer):
    """Encoder layer with a cached square subsequent (-inf above the diagonal) float mask."""

    def __init__(self, ninp, nhead, nhid, dropout, is_moe=False, num_local_experts=1, world_size=1, rank=0,
                 device=None, dtype=None):
        super().__init__(ninp, nhead, nhid, dropout, is_moe=is_moe, num_local_experts=num_local_experts,
                         world_size=world_size, rank=rank, device=device, dtype=dtype)
        self.src_mask = None

    def _generate_square_subsequent_mask(self, sz):
        mask = (torch.triu(torch.ones(sz, sz)) == 1).transpose(0, 1)
        return mask.float().masked_fill(mask == 0, float("-inf")).masked_fill(mask == 1, float(0.0))

    def forward(self, src):
        if self.src_mask is None or self.src_mask.size(0) != len(src) or self.src_mask.device != src.device:
            self.src_mask = self._generate_square_subsequent_mask(len(src)).to(src.device)
        return super().forward(src, self.src_mask)


class LinearLayer(nn.Module):
    def __init__(self, ninp, ntoken, initrange, world_size, rank, device=None, dtype=None):
        super().__init__()
        with emulate_shards(world_size):
            self.linear = ColumnParallelLinear(ninp, ntoken, device=device, dtype=dtype)
        with torch.no_grad():
            for shard in self.linear.linears:
                shard.bias.data.zero_()
                shard.weight.data.uniform_(-initrange, initrange)

    def forward(self, src):
        return self.linear(src)


class TransformerLM(nn.Sequential):
    """Constructor follows rtp/models/transformer_lm_rtp.py:233.  `world_size` is the number of rotation
    shards emulated on the one device; `rank` must be 0."""

    def __init__(self, ntokens, ninp, nhead, nhid, dropout, initrange, ndecoder, world_size, rank, is_moe=False,
                 num_local_experts=1, device=None, dtype=None):
        layers = [
            EmbeddingLayer(ntokens, ninp, initrange, world_size, rank, device=device, dtype=dtype),
            PositionalEncodingLayer(ninp, dropout, device=device, dtype=dtype),
        ]
        for _ in range(ndecoder):
            layers.append(TransformerDecoderLayer(ninp, nhead, nhid, dropout, is_moe, num_local_experts,
                                                  world_size=world_size, rank=rank, device=device, dtype=dtype))
        layers.append(LinearLayer(ninp, ntokens, initrange, world_size, rank, device=device, dtype=dtype))
        super().__init__(*layers)
        layers[0].adopt_positional(layers[1])
