"""Rotated ParallelMultiheadAttention with keys / values from their own tensors, kdim / vdim != embed_dim and
add_zero_attn, against torch.nn.MultiheadAttention on the CPU (the oracle the reference's own
tests/test_attention.py:133-187 uses), with that test's gather rules for the sharded gradients."""
import pytest
import torch
import torch.nn as nn

from gpu_util import DEV, assert_close
from oracle import rtp_oracle as O

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("rotation_window")]


def _master(E, H, gen, dtype, **kw):
    mha = nn.MultiheadAttention(E, H, bias=True, **kw)
    with torch.no_grad():
        for p in mha.parameters():
            p.copy_(torch.rand(p.shape, generator=gen) * 0.2 - 0.1)
        for p in mha.parameters():  # both sides start from values the compute dtype holds exactly
            p.copy_(p.to(dtype).float())
    return mha


def _check(E, H, L, S, N, ws, dtype, *, kdim=None, vdim=None, zero=False, shared_kv=False, mask=False, pad=False,
           need_weights=False, batch_first=False, seed=0, bias_kv=False):
    from rtp_amd.module.attention import ParallelMultiheadAttention
    gen = torch.Generator().manual_seed(seed)
    ref = _master(E, H, gen, dtype, kdim=kdim, vdim=vdim, add_zero_attn=zero, batch_first=batch_first,
                  add_bias_kv=bias_kv)
    kd, vd = ref.kdim, ref.vdim
    shape = (lambda n, w: (N, n, w)) if batch_first else (lambda n, w: (n, N, w))
    q = torch.randn(shape(L, E), generator=gen).to(dtype)
    k = torch.randn(shape(S, kd), generator=gen).to(dtype)
    v = k if shared_kv else torch.randn(shape(S, vd), generator=gen).to(dtype)
    g = torch.randn(shape(L, E), generator=gen).to(dtype)
    attn_mask = None
    if mask:  # float mask with -inf entries; column 0 stays visible so no row is empty
        attn_mask = torch.where(torch.rand(L, S, generator=gen) < 0.3, float("-inf"), 0.0)
        attn_mask += torch.randn(L, S, generator=gen) * 0.5
        attn_mask[:, 0] = 0.0
    kpm = None
    if pad:  # bool key padding: the last keys of some batch entries are hidden
        kpm = torch.zeros(N, S, dtype=torch.bool)
        for n in range(N):
            kpm[n, S - (n % 3):] = n % 3 > 0
    layer = ParallelMultiheadAttention(E, H, ws, 0, kdim=kdim, vdim=vdim, add_zero_attn=zero, batch_first=batch_first,
                                       add_bias_kv=bias_kv, MultiheadAttention_layer=ref.to(dtype) if dtype != torch.float32 else ref,
                                       device=DEV, dtype=dtype)
    ref = ref.float()
    qd = q.to(DEV).requires_grad_()
    kd_ = k.to(DEV).requires_grad_()
    vd_ = kd_ if shared_kv else v.to(DEV).requires_grad_()
    out, w = layer(qd, kd_, vd_, attn_mask=None if attn_mask is None else attn_mask.to(DEV),
                   key_padding_mask=None if kpm is None else kpm.to(DEV), need_weights=need_weights,
                   average_attn_weights=False)
    out.backward(g.to(DEV))
    qo = q.float().requires_grad_()
    ko = k.float().requires_grad_()
    vo = ko if shared_kv else v.float().requires_grad_()
    want, _ = ref(qo, ko, vo, attn_mask=attn_mask, key_padding_mask=kpm, need_weights=False)
    want.backward(g.float())
    assert_close(out, want, dtype, "output")
    assert_close(qd.grad, qo.grad, dtype, "query grad")
    assert_close(kd_.grad, ko.grad, dtype, "key grad")
    if not shared_kv:
        assert_close(vd_.grad, vo.grad, dtype, "value grad")
    subs = layer.layers
    if ref._qkv_same_embed_dim:
        assert_close(O.attention_grad_reinterleave([l.in_proj_weight.grad for l in subs], ws), ref.in_proj_weight.grad,
                     dtype, "in_proj_weight grad")
    else:
        for name in ("q_proj_weight", "k_proj_weight", "v_proj_weight"):
            assert_close(torch.cat([getattr(l, name).grad for l in subs], dim=0), getattr(ref, name).grad, dtype,
                         name + " grad")
    assert_close(O.attention_grad_reinterleave([l.in_proj_bias.grad for l in subs], ws), ref.in_proj_bias.grad, dtype,
                 "in_proj_bias grad")
    assert_close(torch.cat([l.out_proj.weight.grad for l in subs], dim=1), ref.out_proj.weight.grad, dtype,
                 "out_proj.weight grad")
    for l in subs:
        assert_close(l.out_proj.bias.grad, ref.out_proj.bias.grad, dtype, "out_proj.bias grad")
    if bias_kv:  # a shard holds its head group's columns of the appended key / value
        assert_close(torch.cat([l.bias_k.grad for l in subs], dim=2), ref.bias_k.grad, dtype, "bias_k grad")
        assert_close(torch.cat([l.bias_v.grad for l in subs], dim=2), ref.bias_v.grad, dtype, "bias_v grad")
    if need_weights:
        # per-head weights of the last head group the rotation visits (shard ws-1 when the home rank is 0)
        with torch.no_grad():
            _, w_all = ref(qo, ko, vo, attn_mask=attn_mask, key_padding_mask=kpm, need_weights=True,
                           average_attn_weights=False)
        h_s = H // ws
        assert_close(w, w_all[:, (ws - 1) * h_s:], dtype, "attention weights of the last shard")
    else:
        assert w is None


@pytest.mark.parametrize("ws", [1, 2, 4])
@pytest.mark.parametrize("shared_kv", [False, True])
def test_cross_attention_fp32(ws, shared_kv):
    """Encoder-decoder attention: 7 queries over 11 keys; key is value, or three different tensors."""
    _check(32, 4, 7, 11, 3, ws, torch.float32, shared_kv=shared_kv, need_weights=True)


@pytest.mark.parametrize("ws", [1, 4])
def test_cross_attention_masks_fp32(ws):
    _check(32, 4, 9, 13, 5, ws, torch.float32, mask=True, pad=True, seed=1)
    _check(32, 4, 9, 13, 5, ws, torch.float32, pad=True, need_weights=True, seed=2)


@pytest.mark.parametrize("ws", [1, 2])
def test_attention_own_key_and_value_widths_fp32(ws):
    """kdim / vdim != embed_dim: three separate projection blocks per shard (attention.py:51-55)."""
    _check(32, 4, 6, 10, 3, ws, torch.float32, kdim=24, vdim=40, mask=True, seed=3)
    _check(32, 4, 6, 10, 3, ws, torch.float32, kdim=24, vdim=24, shared_kv=True, need_weights=True, seed=4)


@pytest.mark.parametrize("ws", [1, 2, 4])
def test_attention_add_zero_attn_fp32(ws):
    """One all-zero key / value appended per batch entry (functional.py:746-753), self- and cross-attention."""
    _check(32, 4, 8, 8, 3, ws, torch.float32, zero=True, mask=True, pad=True, seed=5)
    _check(32, 4, 5, 12, 2, ws, torch.float32, zero=True, need_weights=True, seed=6)


@pytest.mark.parametrize("ws", [1, 2, 4])
def test_attention_add_bias_kv_fp32(ws):
    """The learned key / value bias_k / bias_v appended per batch entry (functional.py:711-716), alone, together with
    the all-zero key, under masks, with own key / value widths; against nn.MultiheadAttention(add_bias_kv=True), which
    is what the reference computes with one shard (its shards keep bias_k at full width and cannot run with more)."""
    _check(32, 4, 8, 8, 3, ws, torch.float32, bias_kv=True, mask=True, pad=True, seed=11)
    _check(32, 4, 5, 12, 2, ws, torch.float32, bias_kv=True, zero=True, need_weights=True, seed=12)
    if ws <= 2:
        _check(32, 4, 6, 10, 3, ws, torch.float32, bias_kv=True, kdim=24, vdim=40, pad=True, seed=13)


def test_attention_add_bias_kv_bf16_and_self_attention_input():
    _check(128, 4, 33, 47, 3, 4, torch.bfloat16, bias_kv=True, pad=True, seed=14)
    from rtp_amd.module.attention import ParallelMultiheadAttention
    gen = torch.Generator().manual_seed(15)
    ref = _master(64, 4, gen, torch.float32, add_bias_kv=True)
    layer = ParallelMultiheadAttention(64, 4, 2, 0, add_bias_kv=True, MultiheadAttention_layer=ref, device=DEV)
    x = torch.randn(10, 3, 64, generator=gen)
    xd = x.to(DEV).requires_grad_()
    out, _ = layer(xd, xd, xd, need_weights=False)
    out.sum().backward()
    xo = x.clone().requires_grad_()
    want, _ = ref(xo, xo, xo, need_weights=False)
    want.sum().backward()
    assert_close(out, want, torch.float32, "output")
    assert_close(xd.grad, xo.grad, torch.float32, "input grad")
    assert_close(torch.cat([l.bias_k.grad for l in layer.layers], dim=2), ref.bias_k.grad, torch.float32, "bias_k grad")


def test_add_zero_attn_on_self_attention_input():
    """query is key is value with add_zero_attn: the general path, same tensor three times."""
    from rtp_amd.module.attention import ParallelMultiheadAttention
    gen = torch.Generator().manual_seed(7)
    ref = _master(64, 4, gen, torch.float32, add_zero_attn=True)
    layer = ParallelMultiheadAttention(64, 4, 2, 0, add_zero_attn=True, MultiheadAttention_layer=ref, device=DEV)
    x = torch.randn(10, 3, 64, generator=gen)
    xd = x.to(DEV).requires_grad_()
    out, _ = layer(xd, xd, xd, need_weights=False)
    out.sum().backward()
    xo = x.clone().requires_grad_()
    want, _ = ref(xo, xo, xo, need_weights=False)
    want.sum().backward()
    assert_close(out, want, torch.float32, "output")
    assert_close(xd.grad, xo.grad, torch.float32, "input grad")


def test_cross_attention_batch_first_and_bf16():
    _check(64, 4, 12, 20, 3, 2, torch.float32, batch_first=True, mask=True, seed=8)
    _check(128, 4, 33, 47, 3, 4, torch.bfloat16, pad=True, seed=9)
    _check(128, 4, 16, 40, 2, 2, torch.bfloat16, kdim=96, vdim=64, zero=True, seed=10)


def test_general_attention_argument_checks():
    from rtp_amd.module.attention import ParallelMultiheadAttention
    layer = ParallelMultiheadAttention(32, 4, 2, 0, device=DEV)
    q = torch.randn(5, 2, 32, device=DEV)
    k = torch.randn(7, 2, 32, device=DEV)
    with pytest.raises(RuntimeError):
        layer(q, k, k, is_causal=True)  # the hint needs its mask (functional.py:623-628)
    with pytest.raises(ValueError):
        layer(q, k, torch.randn(8, 2, 32, device=DEV))  # keys and values must pair up
    with pytest.raises(ValueError):
        layer(q, k, k, key_padding_mask=torch.zeros(2, 5, dtype=torch.bool, device=DEV))
    with pytest.raises(RuntimeError):
        layer(q, k, k, attn_mask=torch.zeros(8, 5, 7, device=DEV))  # 3-D masks are [batch * heads / ws, L, S]
    with pytest.raises(ValueError):  # importing a layer without bias_k / bias_v into one that has them
        ParallelMultiheadAttention(32, 4, 2, 0, add_bias_kv=True, MultiheadAttention_layer=nn.MultiheadAttention(32, 4),
                                   device=DEV)


@pytest.mark.parametrize("ws", [1, 2, 4])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_one_mask_per_batch_entry_and_head(ws, dtype):
    """3-D attn_mask (functional.py:701-704).  A shard sees heads / ws heads, so the mask is [batch * heads / ws, L, S]
    and every head group of the rotation shares it; the unsharded layer gets the same masks laid out over all heads.
    Keys from another tensor (fp32) and self-attention (also bf16, where 2-D masks would take the fused core)."""
    from rtp_amd.module.attention import ParallelMultiheadAttention
    E, H, L, N = 64, 4, 7, 3
    h_s = H // ws
    gen = torch.Generator().manual_seed(20 + ws)
    ref = _master(E, H, gen, dtype)
    layer = ParallelMultiheadAttention(E, H, ws, 0, MultiheadAttention_layer=ref.to(dtype) if dtype != torch.float32 else ref,
                                       device=DEV, dtype=dtype)
    ref = ref.float()
    for S, same in ((L, True), (10, False)):
        m = torch.where(torch.rand(N * h_s, L, S, generator=gen) < 0.3, float("-inf"), 0.0)
        m += torch.randn(N * h_s, L, S, generator=gen)
        m[:, :, 0] = 0.0
        full = m.view(N, 1, h_s, L, S).expand(N, ws, h_s, L, S).reshape(N * H, L, S)
        q = torch.randn(L, N, E, generator=gen).to(dtype)
        k = q if same else torch.randn(S, N, E, generator=gen).to(dtype)
        g = torch.randn(L, N, E, generator=gen).to(dtype)
        qd = q.to(DEV).requires_grad_()
        kd = qd if same else k.to(DEV).requires_grad_()
        out, _ = layer(qd, kd, kd, attn_mask=m.to(DEV), need_weights=False)
        out.backward(g.to(DEV))
        qo = q.float().requires_grad_()
        ko = qo if same else k.float().requires_grad_()
        want, _ = ref(qo, ko, ko, attn_mask=full, need_weights=False)
        want.backward(g.float())
        assert_close(out, want, dtype, "output")
        assert_close(qd.grad, qo.grad, dtype, "query grad")
        if not same:
            assert_close(kd.grad, ko.grad, dtype, "key grad")
