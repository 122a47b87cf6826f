"""CPU restatement of RTP's rotated-shard layer algorithms -- TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package imports this module: it is the checker used by tests/, by
__graft_entry__.smoke() and by the cpu_baseline leg of bench.py, never the thing measured or shipped.

Every function follows the reference file:line it cites (paths relative to the reference tree) and is
written with plain torch CPU ops (F.linear / F.embedding / softmax / einsum) or python/numpy loops,
float32 unless the caller passes float64 tensors.  How each function is pinned (tests/test_oracle.py):

  column_parallel_linear / row_parallel_linear   == torch.nn.Linear on the unsharded problem
                                                    (the reference's own oracle, tests/test_linear.py:134-186)
  parallel_embedding / embedding_backward_sequential
                                                 == torch.nn.Embedding forward / CPU backward, bit for bit
                                                    (tests/test_embedding.py:127-157)
  attention_shard_params / parallel_multihead_attention
                                                 == torch.nn.MultiheadAttention, both need_weights paths, and
                                                    the gradient re-interleave rule of tests/test_attention.py:145-176
  top2gating                                     == golden vectors written from the reference's own top2gating
                                                    (tests/golden/top2gating_*.npz), == top2_route_bruteforce
                                                    (independent integer loops) and, for E=2, noise independence
  moe_layer                                      == golden vectors written from the reference's WeightMOELayer run on a
                                                    2-rank gloo ring (tests/golden/moe_ws2.npz), and the closed form
                                                    out[s] = w1*y[e1,slot1] + w2*y[e2,slot2]
  column_parallel_conv2d / conv_patches / conv_fold
                                                 == torch.nn.functional.conv2d on the unsharded problem, F.unfold / F.fold,
                                                    and python loops over a tiny input (patch layout and zero padding)
  TransformerLM (with and without MoE blocks)    == golden vectors written from the reference's own TransformerLM run on
                                                    a 2-rank gloo ring (tests/golden/lm_ws2.npz, lm_moe_ws2.npz: logits,
                                                    losses, l_aux and every home-shard gradient), plus parameter count
                                                    and causality; shard_loop=True (the per-shard loops of the
                                                    functions above inside the model) == shard_loop=False
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F


def ring_order(rank: int, ws: int) -> List[int]:
    """Shard index visited at step i of the forward rotation: (rank + i) % ws (rtp/module/linear.py:212)."""
    return [(rank + i) % ws for i in range(ws)]


# ------------------------------------------------------------------------------------------------
# Linear (rtp/module/linear.py)
# ------------------------------------------------------------------------------------------------
def column_shards(weight: torch.Tensor, bias: Optional[torch.Tensor], ws: int):
    """Row blocks of W[N,K] and b[N] (linear.py:78-82 via utils.py:33-36, partition dim 0)."""
    n_s = weight.shape[0] // ws
    assert n_s * ws == weight.shape[0]
    return [(weight[s * n_s:(s + 1) * n_s], None if bias is None else bias[s * n_s:(s + 1) * n_s]) for s in range(ws)]


def column_parallel_linear(x, weight, bias, ws: int, rank: int = 0):
    """linear.py:204-236: per step F.linear with the shard in hand, outputs placed by shard index, cat."""
    shards = column_shards(weight, bias, ws)
    outs = [None] * ws
    for idx in ring_order(rank, ws):
        w, b = shards[idx]
        outs[idx] = F.linear(x, w, b)
    return torch.cat(outs, dim=-1)


def row_shards(weight, bias, ws: int):
    """Column blocks of W[N,K] (partition dim 1) and bias/ws in every shard (linear.py:130-135)."""
    k_s = weight.shape[1] // ws
    assert k_s * ws == weight.shape[1]
    return [(weight[:, s * k_s:(s + 1) * k_s], None if bias is None else bias / ws) for s in range(ws)]


def row_parallel_linear(x, weight, bias, ws: int, rank: int = 0):
    """linear.py:374-407: input split on the last dim, partial outputs summed as `output + running`."""
    shards = row_shards(weight, bias, ws)
    k_s = weight.shape[1] // ws
    out = None
    for i, idx in enumerate(ring_order(rank, ws)):
        w, b = shards[idx]
        part = F.linear(x[..., idx * k_s:(idx + 1) * k_s], w, b)
        out = part if i == 0 else part + out
    return out


# ------------------------------------------------------------------------------------------------
# Embedding (rtp/module/embedding.py)
# ------------------------------------------------------------------------------------------------
def parallel_embedding(ids, table, ws: int, rank: int = 0):
    """embedding.py:134-152: shard s is table[:, s*D/ws:(s+1)*D/ws]; outputs cat on the last dim."""
    d_s = table.shape[1] // ws
    assert d_s * ws == table.shape[1]
    outs = [None] * ws
    for idx in ring_order(rank, ws):
        outs[idx] = F.embedding(ids, table[:, idx * d_s:(idx + 1) * d_s])
    return torch.cat(outs, dim=-1)


def embedding_backward_sequential(ids: np.ndarray, grad_out: np.ndarray, num_embeddings: int,
                                  padding_idx: Optional[int] = None) -> np.ndarray:
    """Dense gradient of F.embedding as a sequential loop: for flattened position t ascending,
    dW[ids[t]] += g[t] in float32.  (Autograd of embedding.py:146.)"""
    flat = ids.reshape(-1)
    g = grad_out.reshape(flat.shape[0], -1).astype(np.float32)
    dw = np.zeros((num_embeddings, g.shape[1]), dtype=np.float32)
    for t in range(flat.shape[0]):
        if padding_idx is not None and flat[t] == padding_idx:
            continue
        dw[flat[t]] = dw[flat[t]] + g[t]
    return dw


# ------------------------------------------------------------------------------------------------
# Attention (rtp/module/attention.py, rtp/module/functional.py)
# ------------------------------------------------------------------------------------------------
def attention_shard_params(in_w, in_b, out_w, out_b, ws: int, s: int):
    """Head group s: in-proj blocks [s, s+ws, s+2ws] of a 3*ws-way row split, concatenated
    (attention.py:86-100, utils.py:55-59); out-proj column block s; out bias / ws (attention.py:101-104)."""
    e = out_w.shape[0]
    e_s = e // ws
    assert e_s * ws == e
    blocks_w = torch.split(in_w, e_s, dim=0)
    w_in = torch.cat([blocks_w[s], blocks_w[s + ws], blocks_w[s + 2 * ws]], dim=0)
    b_in = None
    if in_b is not None:
        blocks_b = torch.split(in_b, e_s, dim=0)
        b_in = torch.cat([blocks_b[s], blocks_b[s + ws], blocks_b[s + 2 * ws]], dim=0)
    w_o = out_w[:, s * e_s:(s + 1) * e_s]
    b_o = None if out_b is None else out_b / ws
    return w_in, b_in, w_o, b_o


def attention_grad_reinterleave(shard_grads: Sequence[torch.Tensor], ws: int) -> torch.Tensor:
    """Rebuild the unsharded in-projection gradient from per-shard gradients: cat on dim 0 in shard
    order, split into 3*ws blocks, reorder with orders = [j*3+i] (tests/test_attention.py:145-147,170-176)."""
    cat = torch.cat(list(shard_grads), dim=0)
    blocks = torch.split(cat, cat.shape[0] // (3 * ws), dim=0)
    orders = [j * 3 + i for i in range(3) for j in range(ws)]
    return torch.cat([blocks[o] for o in orders], dim=0)


def _shard_attention(x, w_in, b_in, w_o, b_o, heads_s: int, mask, need_weights: bool):
    """functional.py:464-833 for one shard with the packed in-projection (:303-308) and E_div."""
    L, N, _ = x.shape
    e_s = w_o.shape[1]
    d = e_s // heads_s
    proj = F.linear(x, w_in, b_in)                                   # [L,N,3E_s]
    q, k, v = proj.split(e_s, dim=-1)
    q = q.reshape(L, N * heads_s, d).transpose(0, 1)                 # [N*h_s, L, d]  (functional.py:726-737)
    k = k.reshape(L, N * heads_s, d).transpose(0, 1)
    v = v.reshape(L, N * heads_s, d).transpose(0, 1)
    scores = torch.bmm(q / math.sqrt(d), k.transpose(1, 2))          # functional.py:779-787
    if mask is not None:
        scores = scores + mask
    p = torch.softmax(scores, dim=-1)
    o = torch.bmm(p, v)                                              # [N*h_s, L, d]
    o = o.transpose(0, 1).reshape(L * N, e_s)
    out = F.linear(o, w_o, b_o).view(L, N, -1)
    weights = p.view(N, heads_s, L, L) if need_weights else None
    return out, weights


def parallel_multihead_attention(x, in_w, in_b, out_w, out_b, num_heads: int, ws: int, mask=None,
                                 need_weights: bool = False, rank: int = 0):
    """attention.py:240-267: per-shard attention, outputs summed (`output + running`); the returned
    weights are the head-average of the LAST shard visited only (:267)."""
    heads_s = num_heads // ws
    out, weights = None, None
    for i, idx in enumerate(ring_order(rank, ws)):
        params = attention_shard_params(in_w, in_b, out_w, out_b, ws, idx)
        part, weights = _shard_attention(x, *params, heads_s, mask, need_weights)
        out = part if i == 0 else part + out
    if weights is not None:
        weights = weights.mean(dim=1)
    return out, weights


# ------------------------------------------------------------------------------------------------
# Top-2 gating (rtp/module/top2gate.py:43-105)
# ------------------------------------------------------------------------------------------------
def column_parallel_conv2d(x, weight, bias, ws: int, stride=1, padding=0, dilation=1, rank: int = 0):
    """Out-channel shards visited in ring order, outputs concatenated on dim 1 in shard order
    (rtp/module/conv.py:99-114; shard = rows [s*Co/ws, (s+1)*Co/ws) of weight and bias, conv.py:43-47)."""
    n_s = weight.shape[0] // ws
    assert n_s * ws == weight.shape[0]
    outs: List[Optional[torch.Tensor]] = [None] * ws
    for s in ring_order(rank, ws):
        b = None if bias is None else bias[s * n_s:(s + 1) * n_s]
        outs[s] = F.conv2d(x, weight[s * n_s:(s + 1) * n_s], b, stride, padding, dilation)
    return torch.cat(outs, dim=1).contiguous()


def conv_patches(x, kernel_size, stride, padding, dilation):
    """Patch matrix [N*Ho*Wo, Ci*kh*kw] of an NCHW input: row (n, ho, wo), column (ci, i, j), zero padding --
    the operand with which conv2d is the product patches @ weight.view(Co, -1).T (+ bias)."""
    u = F.unfold(x, kernel_size, dilation, padding, stride)        # [N, Ci*kh*kw, Ho*Wo]
    return u.transpose(1, 2).reshape(-1, u.shape[1])


def conv_fold(dpatches, x_shape, kernel_size, stride, padding, dilation):
    """Transpose of conv_patches: patch gradients [N*Ho*Wo, Ci*kh*kw] summed back onto the NCHW input."""
    n, c, h, w = x_shape
    u = dpatches.reshape(n, -1, dpatches.shape[1]).transpose(1, 2)
    return F.fold(u, (h, w), kernel_size, dilation, padding, stride)


def gumbel_noise(shape, generator: torch.Generator) -> torch.Tensor:
    """-log(-log U), U ~ Uniform(tiny, 1-eps): torch.distributions.Gumbel(0,1).rsample (top2gate.py:25-32)
    with an explicit CPU generator so the noise is an input."""
    finfo = torch.finfo(torch.float32)
    u = torch.rand(shape, generator=generator, dtype=torch.float32)
    u = u.clamp(min=finfo.tiny, max=1 - finfo.eps)
    return -torch.log(-torch.log(u))


def _one_hot(idx: torch.Tensor, n: int) -> torch.Tensor:
    out = torch.zeros(idx.shape + (n,), dtype=idx.dtype)
    out.scatter_(-1, idx.unsqueeze(-1), 1)
    return out


def top2gating(logits: torch.Tensor, noise: torch.Tensor) -> Dict[str, torch.Tensor]:
    """Step-for-step restatement of top2gating with the Gumbel sample passed in.  Returns the
    reference's outputs (l_aux, combine_weights[S,E,C], dispatch_mask) and the per-token compact
    record (expert, slot, keep, weight) that the dense tensors encode."""
    gates = F.softmax(logits, dim=1, dtype=torch.float)                      # :46
    S, E = gates.shape
    C = 2 * S // E                                                           # :52
    assert S % E == 0                                                        # :53
    idx1 = torch.argmax(gates, dim=1)                                        # :56
    mask1 = _one_hot(idx1, E)
    noisy = logits + noise                                                   # :61
    idx2 = torch.argmax(noisy.masked_fill(mask1.bool(), float("-inf")), dim=1)  # :63-64
    mask2 = _one_hot(idx2, E)
    loc1 = torch.cumsum(mask1, dim=0) - 1                                    # :68
    loc2 = torch.cumsum(mask2, dim=0) - 1 + torch.sum(mask1, dim=0, keepdim=True)  # :69-71
    me = torch.mean(gates, dim=0)                                            # :74-76
    ce = torch.mean(mask1.float(), dim=0)
    l_aux = torch.mean(me * ce)
    mask1 = mask1 * torch.lt(loc1, C)                                        # :79-80
    mask2 = mask2 * torch.lt(loc2, C)
    loc1_s = torch.sum(loc1 * mask1, dim=1)                                  # :83-84
    loc2_s = torch.sum(loc2 * mask2, dim=1)
    g1 = (gates * mask1).sum(dim=1)                                          # :87-93
    g2 = (gates * mask2).sum(dim=1)
    den = torch.clamp(g1 + g2, min=torch.finfo(gates.dtype).eps)
    g1 = g1 / den
    g2 = g2 / den
    gates1 = g1.unsqueeze(-1) * mask1                                        # :96-103
    gates2 = g2.unsqueeze(-1) * mask2
    combine = gates1.unsqueeze(2) * _one_hot(loc1_s, C).unsqueeze(1) + \
        gates2.unsqueeze(2) * _one_hot(loc2_s, C).unsqueeze(1)
    dispatch = combine.bool()
    keep1 = (mask1.sum(dim=1) > 0) & (g1 != 0)
    keep2 = (mask2.sum(dim=1) > 0) & (g2 != 0)
    return {
        "l_aux": l_aux.to(logits.dtype), "combine_weights": combine.to(logits.dtype), "dispatch_mask": dispatch,
        "gates": gates,
        "expert": torch.stack([idx1, idx2], dim=1).to(torch.int32),
        "slot": torch.stack([loc1_s * keep1, loc2_s * keep2], dim=1).to(torch.int32),
        "keep": torch.stack([keep1, keep2], dim=1).to(torch.int32),
        "weight": torch.stack([g1 * keep1, g2 * keep2], dim=1),
        "counts": torch.cat([_one_hot(idx1, E).sum(0), _one_hot(idx2, E).sum(0)]).to(torch.int32),
    }


def top2_route_bruteforce(logits: np.ndarray, noise: np.ndarray):
    """Independent integer-loop derivation of the routing decisions from the GShard description:
    first choice = most probable expert; second = argmax of logits+noise over the others; tokens take
    capacity slots in token order, all first choices of an expert before any second choice; a choice
    whose slot index reaches C = 2S/E is dropped."""
    S, E = logits.shape
    C = 2 * S // E
    l64 = logits.astype(np.float64)
    probs = np.exp(l64 - l64.max(axis=1, keepdims=True))
    probs /= probs.sum(axis=1, keepdims=True)
    e1 = [int(np.argmax(probs[s])) for s in range(S)]
    e2 = []
    for s in range(S):
        v = (logits[s] + noise[s]).astype(np.float32).copy()
        v[e1[s]] = -np.inf
        e2.append(int(np.argmax(v)))
    first_total = [sum(1 for s in range(S) if e1[s] == e) for e in range(E)]
    fill1, fill2 = [0] * E, [0] * E
    expert, slot, keep = [], [], []
    for s in range(S):
        l1 = fill1[e1[s]]
        fill1[e1[s]] += 1
        l2 = first_total[e2[s]] + fill2[e2[s]]
        fill2[e2[s]] += 1
        k1, k2 = l1 < C, l2 < C
        expert.append((e1[s], e2[s]))
        keep.append((int(k1), int(k2)))
        slot.append((l1 if k1 else 0, l2 if k2 else 0))
    return np.array(expert, np.int32), np.array(slot, np.int32), np.array(keep, np.int32)


# ------------------------------------------------------------------------------------------------
# MoE layer (rtp/module/moe.py:138-187)
# ------------------------------------------------------------------------------------------------
def expert_ffn(x, w1, b1, w2, b2):
    """FeedForwardLayer_expert with dropout 0 (rtp/models/transformer_lm_rtp.py:63-75)."""
    return F.linear(F.relu(F.linear(x, w1, b1)), w2, b2)


def moe_layer(x3: torch.Tensor, wg: torch.Tensor, experts: Sequence[Tuple[torch.Tensor, ...]], noise: torch.Tensor,
              ws: int, rank: int = 0):
    """WeightMOELayer.forward with one local expert per shard: rotated gate projection (top2gate.py:195-207),
    dense dispatch einsum (moe.py:148), per-shard expert on its capacity slab (:150-169), dense combine (:174).
    `experts[e]` = (w1, b1, w2, b2) of global expert e.  Returns (output, l_aux)."""
    E = wg.shape[0]
    n_local = E // ws
    d_model = x3.shape[2]
    x = x3.reshape(-1, d_model)
    logit_parts = [None] * ws
    for idx in ring_order(rank, ws):
        logit_parts[idx] = F.linear(x, wg[idx * n_local:(idx + 1) * n_local])
    logits = torch.cat(logit_parts, dim=-1)
    g = top2gating(logits, noise)
    dispatched = torch.einsum("sec,sm->ecm", g["dispatch_mask"].to(x.dtype), x)
    outs = [None] * E
    for idx in ring_order(rank, ws):
        for j in range(n_local):
            e = idx * n_local + j
            outs[e] = expert_ffn(dispatched[e], *experts[e])
    expert_output = torch.stack(outs, dim=0)
    combined = torch.einsum("sec,ecm->sm", g["combine_weights"], expert_output)
    return combined.reshape(x3.shape), g["l_aux"]


# ------------------------------------------------------------------------------------------------
# Transformer LM (rtp/models/transformer_lm_rtp.py) from stock torch layers
# ------------------------------------------------------------------------------------------------
class _PositionalEncoding(nn.Module):
    def __init__(self, d_model, max_len=5000):
        super().__init__()
        pe = torch.zeros(max_len, d_model)
        position = torch.arange(0, max_len, dtype=torch.float).unsqueeze(1)
        div_term = torch.exp(torch.arange(0, d_model, 2).float() * (-math.log(10000.0) / d_model))
        pe[:, 0::2] = torch.sin(position * div_term)
        pe[:, 1::2] = torch.cos(position * div_term)
        self.register_buffer("pe", pe.unsqueeze(0).transpose(0, 1))

    def forward(self, x):
        return x + self.pe[: x.size(0), :]


class _DecoderLayer(nn.Module):
    """Post-LN block x = LN1(x + SA(x)); x = LN2(x + FFN(x)) (transformer_lm_rtp.py:176-177), dropout 0.  With
    `num_experts` > 0 the feed-forward block is the MoE layer (:151-158, :191-195): gate projection `wg`, experts
    `experts[e]` = (linear1, linear2); the routing noise is the attribute `noise` ([S, E], zeros if unset -- with two
    experts the noise cannot change the routing) and the layer keeps `l_aux` as the reference's moe_layer does."""

    def __init__(self, ninp, nhead, nhid, num_experts=0, ws=1, shard_loop=False):
        super().__init__()
        self.nhead, self.shard_loop = nhead, shard_loop
        self.self_attn = nn.MultiheadAttention(ninp, nhead, dropout=0.0)
        self.norm1 = nn.LayerNorm(ninp)
        self.norm2 = nn.LayerNorm(ninp)
        self.num_experts, self.ws, self.noise, self.l_aux = num_experts, ws, None, None
        if num_experts:
            self.wg = nn.Linear(ninp, num_experts, bias=False)
            self.experts = nn.ModuleList(nn.ModuleList([nn.Linear(ninp, nhid), nn.Linear(nhid, ninp)])
                                         for _ in range(num_experts))
        else:
            self.linear1 = nn.Linear(ninp, nhid)
            self.linear2 = nn.Linear(nhid, ninp)

    def _ff(self, x):
        if not self.num_experts:
            if self.shard_loop:      # FeedForwardLayer of two ColumnParallelLinear (transformer_lm_rtp.py:82-89)
                h = F.relu(column_parallel_linear(x, self.linear1.weight, self.linear1.bias, self.ws))
                return column_parallel_linear(h, self.linear2.weight, self.linear2.bias, self.ws)
            return self.linear2(F.relu(self.linear1(x)))
        S = x.shape[0] * x.shape[1]
        noise = self.noise if self.noise is not None else torch.zeros(S, self.num_experts, dtype=x.dtype)
        experts = [(e[0].weight, e[0].bias, e[1].weight, e[1].bias) for e in self.experts]
        out, self.l_aux = moe_layer(x, self.wg.weight, experts, noise, self.ws)
        return out

    def forward(self, x):
        L = x.shape[0]
        mask = torch.triu(torch.full((L, L), float("-inf"), dtype=x.dtype), diagonal=1)      # :201-204
        if self.shard_loop:          # ParallelMultiheadAttention's loop over head groups (attention.py:240-267)
            a = self.self_attn
            sa = parallel_multihead_attention(x, a.in_proj_weight, a.in_proj_bias, a.out_proj.weight, a.out_proj.bias,
                                              self.nhead, self.ws, mask=mask)[0]
        else:
            sa = self.self_attn(x, x, x, attn_mask=mask, need_weights=False)[0]
        x = self.norm1(x + sa)
        return self.norm2(x + self._ff(x))


class TransformerLM(nn.Sequential):
    """Unsharded LM with the rotated LM's structure; weights are copied in by the tests so both sides
    start from identical values.  num_experts > 0 builds the is_moe=True model (one gate + `num_experts` experts per
    decoder layer, `ws` shards in the MoE layer's ring order).  shard_loop=True evaluates every rotated layer the way
    the reference does -- a loop over `ws` shards per layer with the per-shard F.linear / F.embedding / attention and the
    concatenation or running sum of the partial results -- on the same unsharded parameters: the same function, in the
    reference's operation count (what bench.py times as the CPU baseline)."""

    def __init__(self, ntokens, ninp, nhead, nhid, ndecoder, num_experts=0, ws=1, shard_loop=False):
        self.ninp, self.ws, self.shard_loop = ninp, ws, shard_loop
        layers = [nn.Embedding(ntokens, ninp), _PositionalEncoding(ninp)]
        layers += [_DecoderLayer(ninp, nhead, nhid, num_experts, ws, shard_loop) for _ in range(ndecoder)]
        layers.append(nn.Linear(ninp, ntokens))
        super().__init__(*layers)

    def forward(self, ids):
        if self.shard_loop:
            x = parallel_embedding(ids, self[0].weight, self.ws) * math.sqrt(self.ninp)
        else:
            x = self[0](ids) * math.sqrt(self.ninp)                           # :29
        for layer in list(self)[1:-1]:
            x = layer(x)
        if self.shard_loop:                                                   # LinearLayer = ColumnParallelLinear, :223
            return column_parallel_linear(x, self[-1].weight, self[-1].bias, self.ws)
        return self[-1](x)
