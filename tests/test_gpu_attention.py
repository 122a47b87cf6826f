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
    with pytest.raises(RuntimeError):
        layer(x, x, x, attn_mask=torch.zeros(4, 4, 4, device=DEV))  # a 3-D mask is [batch * heads / ws, L, S] = [2, 4, 4]
    with pytest.raises(ValueError):
        layer(x, x, x, key_padding_mask=torch.zeros(3, 4, dtype=torch.bool, device=DEV))   # [batch, keys] = [2, 4]
    with pytest.raises(NotImplementedError):
        layer(x[:, 0], x[:, 0], x[:, 0])  # unbatched [L, E] inputs


@pytest.mark.parametrize("E,H,L,N,ws,masked,need_weights", [
    (128, 4, 32, 3, 2, True, False),     # head_dim 32, full 32-token tile
    (256, 4, 7, 5, 4, False, True),      # head_dim 64, ragged L, returned weights
    (512, 4, 19, 2, 2, True, True),      # head_dim 128
    (2048, 32, 32, 4, 8, True, False),   # the LM layer: 32 heads in 8 groups, seq 32
])
def test_attention_fused_short_sequence_bf16(E, H, L, N, ws, masked, need_weights):
    """bf16 with L <= 32 takes the fused core (one wavefront per head); same oracle, same tolerance."""
    from rtp_amd import ops
    assert ops.attn_supported(torch.bfloat16, L, E // H)
    _run(E, H, L, N, ws, torch.bfloat16, masked, need_weights, seed=4)


@pytest.mark.parametrize("L,d,causal,use_mask", [(32, 64, True, False), (13, 32, False, True), (32, 128, False, False),
                                                 (1, 64, True, False)])
def test_attn_core_against_torch_fp32(L, d, causal, use_mask):
    """rtp_attn_fwd / rtp_attn_bwd through the C ABI on a packed [L, N, G*3*H*d] projection, against plain
    fp32 torch attention on the same bf16 inputs (tolerance 2e-2 of the largest reference entry)."""
    from rtp_amd import ops
    gen = torch.Generator().manual_seed(L * 131 + d)
    N, H, G = 3, 2, 2
    e_s = H * d
    qkv = (torch.randn(L, N, G * 3 * e_s, generator=gen) * 0.5).to(torch.bfloat16)
    dout = torch.randn(L, N, G * e_s, generator=gen).to(torch.bfloat16)
    mask = (torch.randn(L, L, generator=gen) * 2.0) if use_mask else None
    scale = 1.0 / d ** 0.5
    # reference
    x = qkv.float().view(L, N, G, 3, H, d).requires_grad_()
    q, k, v = x[:, :, :, 0], x[:, :, :, 1], x[:, :, :, 2]                 # [L, N, G, H, d]
    s = torch.einsum("lnghd,mnghd->nghlm", q, k) * scale
    if mask is not None:
        s = s + mask
    if causal:
        s = s + _causal(L)
    p_ref = torch.softmax(s, dim=-1)
    o_ref = torch.einsum("nghlm,mnghd->lnghd", p_ref, v).reshape(L, N, G * e_s)
    o_ref.backward(dout.float())
    # device
    qd, dd = qkv.to(DEV), dout.to(DEV)
    o = torch.empty(L, N, G * e_s, dtype=torch.bfloat16, device=DEV)
    p = torch.empty(G * N * H, L, L, dtype=torch.bfloat16, device=DEV)
    dqkv = torch.zeros_like(qd)
    ld = G * 3 * e_s
    qs, os_ = (N * ld, ld, d, 3 * e_s), (N * G * e_s, G * e_s, d, e_s)
    ops.attn_fwd(qd, 0, e_s, 2 * e_s, qs, o, 0, os_, p, None if mask is None else mask.to(DEV), causal, scale,
                 L, N, H, d, G)
    ops.attn_bwd(qd, 0, e_s, 2 * e_s, qs, dd, 0, os_, p, dqkv, scale, L, N, H, d, G)
    assert_close(o, o_ref, torch.bfloat16, "o")
    assert_close(p.view(G, N, H, L, L), p_ref.permute(1, 0, 2, 3, 4), torch.bfloat16, "p")
    assert_close(dqkv, x.grad.reshape(L, N, ld), torch.bfloat16, "dqkv")


def test_attn_core_rejects_unsupported():
    from rtp_amd import ops
    from rtp_amd._lib import RtpError
    assert not ops.attn_supported(torch.float32, 16, 64)
    assert not ops.attn_supported(torch.bfloat16, 33, 64)
    assert not ops.attn_supported(torch.bfloat16, 16, 48)
    qkv = torch.zeros(33, 1, 3 * 64, dtype=torch.bfloat16, device=DEV)
    o = torch.zeros(33, 1, 64, dtype=torch.bfloat16, device=DEV)
    p = torch.zeros(1, 33, 33, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RtpError):
        ops.attn_fwd(qkv, 0, 64, 128, (192, 192, 64, 192), o, 0, (64, 64, 64, 64), p, None, False, 0.125, 33, 1, 1,
                     64, 1)


@pytest.mark.parametrize("L,d,causal,mask_kind", [
    (33, 64, False, None),        # one full key block and a block of a single key
    (64, 32, True, None),
    (100, 64, True, None),        # ragged last block, causal: block counts differ per wavefront
    (100, 128, False, "float"),
    (96, 64, False, "neg_inf"),   # the causal pattern handed over as a -inf float mask (L % 4 == 0: 16-byte loads)
    (97, 32, False, "neg_inf"),   # same, scalar mask loads
    (17, 128, True, "float"),     # shorter than one block
    (512, 64, True, None),
])
def test_attn_flash_core_against_torch_fp32(L, d, causal, mask_kind):
    """rtp_attn_flash_fwd / rtp_attn_flash_bwd through the C ABI on a packed [L, N, G*3*H*d] projection, against
    plain fp32 torch attention on the same bf16 inputs (tolerance 2e-2 of the largest reference entry); the
    log-sum-exp against torch.logsumexp to 1e-3."""
    from rtp_amd import ops
    gen = torch.Generator().manual_seed(L * 131 + d)
    N, H, G = 2, 3, 2
    e_s = H * d
    qkv = (torch.randn(L, N, G * 3 * e_s, generator=gen) * 0.5).to(torch.bfloat16)
    dout = torch.randn(L, N, G * e_s, generator=gen).to(torch.bfloat16)
    mask = {None: None, "float": torch.randn(L, L, generator=gen) * 2.0, "neg_inf": _causal(L)}[mask_kind]
    scale = 1.0 / d ** 0.5
    x = qkv.float().view(L, N, G, 3, H, d).requires_grad_()
    q, k, v = x[:, :, :, 0], x[:, :, :, 1], x[:, :, :, 2]
    s = torch.einsum("lnghd,mnghd->nghlm", q, k) * scale
    if mask is not None:
        s = s + mask
    if causal:
        s = s + _causal(L)
    p_ref = torch.softmax(s, dim=-1)
    lse_ref = torch.logsumexp(s.detach(), dim=-1).permute(1, 0, 2, 3)       # [G, N, H, L]
    o_ref = torch.einsum("nghlm,mnghd->lnghd", p_ref, v).reshape(L, N, G * e_s)
    o_ref.backward(dout.float())
    qd, dd = qkv.to(DEV), dout.to(DEV)
    o = torch.empty(L, N, G * e_s, dtype=torch.bfloat16, device=DEV)
    lse = torch.empty(G * N * H, L, dtype=torch.float32, device=DEV)
    delta = torch.empty_like(lse)
    dqkv = torch.zeros_like(qd)
    ld = G * 3 * e_s
    qs, os_ = (N * ld, ld, d, 3 * e_s), (N * G * e_s, G * e_s, d, e_s)
    md = None if mask is None else mask.to(DEV)
    assert ops.attn_flash_supported(torch.bfloat16, L, d)
    ops.attn_flash_fwd(qd, 0, e_s, 2 * e_s, qs, o, 0, os_, lse, md, causal, scale, L, N, H, d, G)
    ops.attn_flash_bwd(qd, 0, e_s, 2 * e_s, qs, o, dd, 0, os_, lse, delta, dqkv, md, causal, scale, L, N, H, d, G)
    assert_close(o, o_ref, torch.bfloat16, "o")
    assert (lse.cpu().view(G, N, H, L) - lse_ref).abs().max().item() < 1e-3
    delta_ref = (dout.float() * o.float().cpu()).view(L, N, G, H, d).sum(-1).permute(2, 1, 3, 0)
    assert (delta.cpu().view(G, N, H, L) - delta_ref).abs().max().item() < 1e-3 * max(1.0, delta_ref.abs().max().item())
    assert_close(dqkv, x.grad.reshape(L, N, ld), torch.bfloat16, "dqkv")


def test_attn_flash_matches_short_sequence_core():
    """On a sequence both cores take (L <= 32) they agree to bf16 rounding of the same fp32 results."""
    from rtp_amd import ops
    gen = torch.Generator().manual_seed(77)
    L, N, H, G, d = 29, 2, 2, 1, 64
    e_s, ld = H * d, 3 * H * d
    qd = (torch.randn(L, N, ld, generator=gen) * 0.5).to(torch.bfloat16).to(DEV)
    dd = torch.randn(L, N, e_s, generator=gen).to(torch.bfloat16).to(DEV)
    qs, os_ = (N * ld, ld, d, 3 * e_s), (N * e_s, e_s, d, e_s)
    o1, o2 = (torch.empty(L, N, e_s, dtype=torch.bfloat16, device=DEV) for _ in range(2))
    p = torch.empty(N * H, L, L, dtype=torch.bfloat16, device=DEV)
    lse = torch.empty(N * H, L, dtype=torch.float32, device=DEV)
    d1, d2 = torch.zeros_like(qd), torch.zeros_like(qd)
    ops.attn_fwd(qd, 0, e_s, 2 * e_s, qs, o1, 0, os_, p, None, True, 0.125, L, N, H, d, G)
    ops.attn_bwd(qd, 0, e_s, 2 * e_s, qs, dd, 0, os_, p, d1, 0.125, L, N, H, d, G)
    ops.attn_flash_fwd(qd, 0, e_s, 2 * e_s, qs, o2, 0, os_, lse, None, True, 0.125, L, N, H, d, G)
    ops.attn_flash_bwd(qd, 0, e_s, 2 * e_s, qs, o2, dd, 0, os_, lse, torch.empty_like(lse), d2, None, True, 0.125, L,
                       N, H, d, G)
    assert_close(o2, o1.float(), torch.bfloat16, "o")
    assert_close(d2, d1.float(), torch.bfloat16, "dqkv")


@pytest.mark.parametrize("E,H,L,N,ws,masked,need_weights", [
    (256, 4, 100, 3, 2, True, False),    # running-softmax core, ragged last block, -inf float mask
    (512, 4, 70, 2, 4, False, False),    # head_dim 128
    (128, 4, 48, 2, 2, True, True),      # returned weights: the products-and-softmax form with p in memory
])
def test_attention_long_sequence_bf16(E, H, L, N, ws, masked, need_weights):
    _run(E, H, L, N, ws, torch.bfloat16, masked, need_weights, seed=6)


def test_attn_flash_rejects_unsupported():
    from rtp_amd import ops
    from rtp_amd._lib import RtpError
    assert not ops.attn_flash_supported(torch.float32, 64, 64)
    assert not ops.attn_flash_supported(torch.bfloat16, 64, 48)
    qkv = torch.zeros(40, 1, 3 * 64, dtype=torch.bfloat16, device=DEV)
    o = torch.zeros(40, 1, 64, dtype=torch.bfloat16, device=DEV)
    lse = torch.zeros(1, 40, dtype=torch.float32, device=DEV)
    with pytest.raises(RtpError):   # stride not a multiple of 8 elements
        ops.attn_flash_fwd(qkv, 0, 64, 128, (192, 192, 60, 192), o, 0, (64, 64, 64, 64), lse, None, False, 0.125, 40, 1,
                           1, 64, 1)
    with pytest.raises(ValueError):
        ops.attn_flash_fwd(qkv, 0, 64, 128, (192, 192, 64, 192), o, 0, (64, 64, 64, 64), lse[:, :39], None, False,
                           0.125, 40, 1, 1, 64, 1)


@pytest.mark.parametrize("E,H,L,N,ws,dtype,masked,need_weights", [
    (128, 4, 20, 3, 2, torch.bfloat16, False, False),   # short-sequence core
    (128, 4, 20, 3, 2, torch.bfloat16, True, True),     # ... with the causal float mask, weights returned
    (256, 4, 100, 3, 2, torch.bfloat16, False, False),  # running-softmax core
    (256, 4, 100, 3, 4, torch.bfloat16, True, False),
    (64, 4, 40, 2, 2, torch.float32, True, False),      # products and softmax kernel
    (128, 4, 48, 2, 2, torch.bfloat16, False, True),    # weights returned beyond 32 positions
])
def test_attention_key_padding_mask(E, H, L, N, ws, dtype, masked, need_weights):
    """key_padding_mask [batch, keys] (bool: True hides the key) against nn.MultiheadAttention; each batch row pads a
    different tail, key 0 stays visible so no query loses all its keys."""
    from rtp_amd.module.attention import ParallelMultiheadAttention
    gen = torch.Generator().manual_seed(8)
    mha = _master(E, H, dtype, gen)
    x = torch.randn(L, N, E, generator=gen).to(dtype)
    g = torch.randn(L, N, E, generator=gen).to(dtype)
    kpm = torch.zeros(N, L, dtype=torch.bool)
    for b in range(N):
        kpm[b, L - 1 - 3 * b:] = True
    mask = _causal(L) if masked else None
    layer = ParallelMultiheadAttention(E, H, ws, 0, MultiheadAttention_layer=mha, device=DEV, dtype=dtype)
    xd = x.to(DEV).requires_grad_()
    out, w = layer(xd, xd, xd, attn_mask=None if mask is None else mask.to(DEV), key_padding_mask=kpm.to(DEV),
                   need_weights=need_weights)
    out.backward(g.to(DEV))
    ref_m = nn.MultiheadAttention(E, H, bias=True)
    ref_m.load_state_dict({k: v.float() for k, v in mha.state_dict().items()})
    xo = x.float().requires_grad_()
    ref, w_ref = ref_m(xo, xo, xo, attn_mask=mask, key_padding_mask=kpm, need_weights=True, average_attn_weights=False)
    ref.backward(g.float())
    assert_close(out, ref, dtype, "output")
    assert_close(xd.grad, xo.grad, dtype, "input grad")
    assert_close(O.attention_grad_reinterleave([l.in_proj_weight.grad for l in layer.layers], ws),
                 ref_m.in_proj_weight.grad, dtype, "in_proj_weight grad")
    assert_close(torch.cat([l.out_proj.weight.grad for l in layer.layers], dim=1), ref_m.out_proj.weight.grad, dtype,
                 "out_proj.weight grad")
    if need_weights:
        h_s = H // ws
        assert_close(w, w_ref[:, (ws - 1) * h_s:].mean(1), dtype, "attention weights of the last shard")
        hidden = kpm.to(DEV)[:, None, :].expand(N, L, L)
        assert not w[hidden].any()                        # padded keys get exactly zero weight
    # a float key_padding_mask is added to the scores: the same -inf pattern gives the same result
    xf = x.to(DEV)
    with torch.no_grad():
        out_f, _ = layer(xf, xf, xf, attn_mask=None if mask is None else mask.to(DEV), need_weights=need_weights,
                         key_padding_mask=torch.zeros(N, L).masked_fill(kpm, float("-inf")).to(DEV))
    assert torch.equal(out_f, out.detach())


def _attention_with_keep_masks(x, mha, H, ws, keep, drop_p, mask):
    """Per-shard attention (functional.py:779-800) with the given 0 / 1 keep mask [ws * N * H/ws, L, L] applied to the
    softmax probabilities and scaled by 1 / (1 - drop_p), on the CPU with autograd."""
    import math
    import torch.nn.functional as F
    L, N, E = x.shape
    h_s, e_s = H // ws, E // ws
    d = E // H
    Z = N * h_s
    out = 0
    for g in range(ws):
        w_in, b_in, w_o, b_o = O.attention_shard_params(mha.in_proj_weight, mha.in_proj_bias, mha.out_proj.weight,
                                                         mha.out_proj.bias, ws, g)
        q, k, v = F.linear(x, w_in, b_in).split(e_s, dim=-1)
        q, k, v = (t.reshape(L, Z, d).transpose(0, 1) for t in (q, k, v))
        s = torch.bmm(q / math.sqrt(d), k.transpose(1, 2))
        p = torch.softmax(s if mask is None else s + mask, dim=-1) * keep[g * Z:(g + 1) * Z] / (1.0 - drop_p)
        o = torch.bmm(p, v).transpose(0, 1).reshape(L * N, e_s)
        out = out + F.linear(o, w_o, b_o).view(L, N, E)
    return out


@pytest.mark.parametrize("ws", [1, 2, 4])
def test_attention_dropout_with_recorded_masks(ws):
    """Attention dropout while training: the layer draws keep masks (recorded here through dropout_keep_fn), the CPU
    restatement applies the same masks; output and every gradient must agree.  eval() switches dropout off."""
    from rtp_amd.module.attention import ParallelMultiheadAttention
    E, H, L, N, drop_p = 32, 4, 6, 3, 0.3
    gen = torch.Generator().manual_seed(11)
    mha = _master(E, H, torch.float32, gen)
    layer = ParallelMultiheadAttention(E, H, ws, 0, dropout=drop_p, MultiheadAttention_layer=mha, device=DEV)
    drawn = []
    mask_gen = torch.Generator().manual_seed(12)

    def keep_fn(shape):
        m = (torch.rand(shape, generator=mask_gen) >= drop_p).float()
        drawn.append(m)
        return m.to(DEV)
    layer.dropout_keep_fn = keep_fn
    x = torch.randn(L, N, E, generator=gen)
    g = torch.randn(L, N, E, generator=gen)
    xd = x.to(DEV).requires_grad_()
    out, w = layer(xd, xd, xd, attn_mask=_causal(L).to(DEV), need_weights=True, average_attn_weights=False)
    out.backward(g.to(DEV))
    keep = torch.cat(drawn, 0)  # ring order of home rank 0 = ascending shard index
    assert keep.shape == (N * H, L, L)
    xo = x.clone().requires_grad_()
    want = _attention_with_keep_masks(xo, mha, H, ws, keep, drop_p, _causal(L))
    want.backward(g)
    assert_close(out, want, torch.float32, "output")
    assert_close(xd.grad, xo.grad, torch.float32, "input grad")
    assert_close(O.attention_grad_reinterleave([l.in_proj_weight.grad for l in layer.layers], ws),
                 mha.in_proj_weight.grad, torch.float32, "in_proj_weight grad")
    assert_close(torch.cat([l.out_proj.weight.grad for l in layer.layers], dim=1), mha.out_proj.weight.grad,
                 torch.float32, "out_proj.weight grad")
    # the returned weights are the dropped ones of the last shard visited (functional.py:789-800)
    h_s = H // ws
    zero_where_dropped = w.cpu()[keep[(ws - 1) * N * h_s:].view(N, h_s, L, L) == 0]
    assert torch.count_nonzero(zero_where_dropped) == 0
    # without the hook the device generator draws: about drop_p of the visible probabilities become zero
    layer.dropout_keep_fn = None
    _, w2 = layer(xd, xd, xd, need_weights=True, average_attn_weights=False)
    frac = float((w2 == 0).float().mean())
    assert 0.15 < frac < 0.45, frac
    layer.eval()
    a, _ = layer(xd, xd, xd, attn_mask=_causal(L).to(DEV), need_weights=False)
    ref, _ = mha(x, x, x, attn_mask=_causal(L), need_weights=False)
    assert_close(a, ref, torch.float32, "eval output")


def test_attention_dropout_bf16_and_other_key_tensor():
    """bf16, and keys / values from another tensor: with an all-ones keep mask the probabilities are only scaled by
    1 / (1 - p), so (out - b_o) is the dropout-free result divided by (1 - p)."""
    from rtp_amd.module.attention import ParallelMultiheadAttention
    E, H, drop_p = 64, 4, 0.25
    gen = torch.Generator().manual_seed(13)
    mha = _master(E, H, torch.bfloat16, gen)
    layer = ParallelMultiheadAttention(E, H, 2, 0, dropout=drop_p, MultiheadAttention_layer=mha, device=DEV,
                                       dtype=torch.bfloat16)
    layer.dropout_keep_fn = lambda shape: torch.ones(shape, device=DEV)
    q = torch.randn(9, 2, E, generator=gen).to(torch.bfloat16)
    k = torch.randn(14, 2, E, generator=gen).to(torch.bfloat16)
    ref_m = nn.MultiheadAttention(E, H)
    ref_m.load_state_dict({n: v.float() for n, v in mha.state_dict().items()})
    for key in (q, k):
        out, _ = layer(q.to(DEV), key.to(DEV), key.to(DEV), need_weights=False)
        ref, _ = ref_m(q.float(), key.float(), key.float(), need_weights=False)
        b_o = ref_m.out_proj.bias.detach()
        assert_close(out.float().cpu() - b_o, (ref.detach() - b_o) / (1 - drop_p), torch.bfloat16, "scaled output")


def test_lm_trains_with_dropout():
    """The language model with the reference's default dropout 0.1 (transformer_lm_rtp.py:128, :139 hands it to the
    attention as well): a training step runs and the loss is finite; eval() is deterministic."""
    import torch.nn.functional as F
    from rtp_amd.models.transformer_lm_rtp import TransformerLM
    torch.manual_seed(0)
    lm = TransformerLM(64, 32, 4, 32, 0.1, 0.1, 2, 2, 0, device=DEV)
    ids = torch.randint(0, 64, (10, 3), device=DEV)
    loss = F.cross_entropy(lm(ids).view(-1, 64), ids.view(-1))
    loss.backward()
    assert torch.isfinite(loss)
    assert all(torch.isfinite(p.grad).all() for p in lm.parameters() if p.grad is not None)
    lm.eval()
    assert torch.equal(lm(ids), lm(ids))
