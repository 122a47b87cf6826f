"""Rotated ParallelMultiheadAttention vs the CPU oracle / nn.MultiheadAttention, with the reference
test's gradient re-interleave (tests/test_attention.py:145-183)."""
import pytest
import torch
import torch.nn as nn

from gpu_util import DEV, assert_close
from oracle import rtp_oracle as O

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("rotation_window")]


def _causal(L):
    return torch.triu(torch.full((L, L), float("-inf")), diagonal=1)


def _master(E, H, dtype, gen):
    mha = nn.MultiheadAttention(E, H, bias=True)
    with torch.no_grad():
        for p in mha.parameters():
            p.copy_(torch.rand(p.shape, generator=gen) * 0.2 - 0.1)
    return mha.to(dtype)


def _run(E, H, L, N, ws, dtype, masked, need_weights, seed=0):
    from rtp_amd.module.attention import ParallelMultiheadAttention
    gen = torch.Generator().manual_seed(seed)
    mha = _master(E, H, dtype, gen)
    x = torch.randn(L, N, E, generator=gen).to(dtype)
    g = torch.randn(L, N, E, generator=gen).to(dtype)
    mask = _causal(L) if masked else None
    layer = ParallelMultiheadAttention(E, H, ws, 0, MultiheadAttention_layer=mha, device=DEV, dtype=dtype)
    xd = x.to(DEV).requires_grad_()
    out, w = layer(xd, xd, xd, attn_mask=None if mask is None else mask.to(DEV), need_weights=need_weights)
    out.backward(g.to(DEV))
    ref_m = nn.MultiheadAttention(E, H, bias=True)
    ref_m.load_state_dict({k: v.float() for k, v in mha.state_dict().items()})
    xo = x.float().requires_grad_()
    ref, _ = ref_m(xo, xo, xo, attn_mask=mask, need_weights=False)
    ref.backward(g.float())
    assert_close(out, ref, dtype, "output")
    assert_close(xd.grad, xo.grad, dtype, "input grad")
    assert_close(O.attention_grad_reinterleave([l.in_proj_weight.grad for l in layer.layers], ws),
                 ref_m.in_proj_weight.grad, dtype, "in_proj_weight grad")
    assert_close(O.attention_grad_reinterleave([l.in_proj_bias.grad for l in layer.layers], ws),
                 ref_m.in_proj_bias.grad, dtype, "in_proj_bias grad")
    assert_close(torch.cat([l.out_proj.weight.grad for l in layer.layers], dim=1), ref_m.out_proj.weight.grad, dtype,
                 "out_proj.weight grad")
    for l in layer.layers:
        assert_close(l.out_proj.bias.grad, ref_m.out_proj.bias.grad, dtype, "out_proj.bias grad")
    if need_weights:
        _, w_ref = O.parallel_multihead_attention(
            x.float(), ref_m.in_proj_weight.detach(), ref_m.in_proj_bias.detach(), ref_m.out_proj.weight.detach(),
            ref_m.out_proj.bias.detach(), H, ws, mask=mask, need_weights=True)
        assert_close(w, w_ref, dtype, "attention weights of the last shard")
    else:
        assert w is None
    return layer


@pytest.mark.parametrize("ws", [1, 2, 4])
@pytest.mark.parametrize("masked", [False, True])
def test_attention_reference_shape_fp32(ws, masked):
    """nn.MultiheadAttention(8, 4 heads), data [8,8,8] (L,N,E), need_weights=True path."""
    _run(8, 4, 8, 8, ws, torch.float32, masked, True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_lm_shape(dtype):
    """The LM's call: float -inf mask, need_weights=False, head_dim 64, ragged L."""
    _run(256, 4, 31, 5, 2, dtype, True, False, seed=1)


def test_attention_causal_flag_equals_float_mask():
    from rtp_amd.module.attention import ParallelMultiheadAttention
    gen = torch.Generator().manual_seed(2)
    mha = _master(64, 4, torch.float32, gen)
    layer = ParallelMultiheadAttention(64, 4, 2, 0, MultiheadAttention_layer=mha, device=DEV)
    x = torch.randn(20, 3, 64, generator=gen).to(DEV)
    a, _ = layer(x, x, x, attn_mask=_causal(20).to(DEV), need_weights=False)
    b, _ = layer(x, x, x, is_causal=True, need_weights=False)
    assert torch.equal(a, b)


def test_attention_headline_config_bf16():
    """d_model 2048, 32 heads in 8 shard groups, batch 8, seq 512, causal, bf16 with fp32 accumulation;
    oracle in fp32 on the CPU (nn.MultiheadAttention)."""
    _run(2048, 32, 512, 8, 8, torch.bfloat16, True, False, seed=3)


def test_attention_unsupported_raise():
    from rtp_amd.module.attention import ParallelMultiheadAttention
    layer = ParallelMultiheadAttention(8, 2, 2, 0, device=DEV)
    x = torch.randn(4, 2, 8, device=DEV)
    with pytest.raises(NotImplementedError):
        layer(x, x.clone(), x)
    with pytest.raises(NotImplementedError):
        layer(x, x, x, key_padding_mask=torch.zeros(2, 4, dtype=torch.bool, device=DEV))
    with pytest.raises(NotImplementedError):
        ParallelMultiheadAttention(8, 2, 2, 0, kdim=4, device=DEV)
