"""Grouped launches over a run of consecutive shards staged as `flat` = [count, numel].

A weight matrix of the layer is described by (offset inside a flat shard, rows, cols); shard g of the run
is found `numel` elements after shard g-1, which is the group / K-segment stride handed to rtp_gemm.
Column-style matrices (output features sharded) use one group per shard; row-style matrices (input
features sharded) contract over the shards as K segments, so their cross-shard sum stays in the MFMA
accumulators.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import _lib, ops


def _rows(t: torch.Tensor):
    m, n, ld = ops._mat(t, "operand")
    return m, n, ld


def col_fwd(x2, flat, w_off, n_s, k, bias_off, out, col0, *, relu=False):
    """out[:, col0 + g*n_s : col0 + (g+1)*n_s] = x2 @ W_g^T (+ b_g), g over the run: the run is a rotated
    column-parallel layer of its own (rtp_rotated_linear_fwd) whose outputs start at column col0."""
    ops.rotated_linear_fwd(x2, flat, w_off, bias_off, n_s, k, out[:, col0:], relu=relu)


def col_dgrad(dy2, flat, w_off, n_s, k, out, col0, c_in: Optional[torch.Tensor] = None, gate=None):
    """out[M, k] = (c_in +) sum_g dy2[:, col0 + g*n_s : ...] @ W_g   (contraction segmented over shards)."""
    ops.rotated_linear_bwd(dy2[:, col0:], None, flat, w_off, None, n_s, k, dx=out, dx_init=c_in, relu_gate=gate)


def _fused(store, accumulate, first, cnt, w_off, length):
    """Keyword arguments that make a weight-gradient product of `store` apply the optimiser's update itself (when
    an optimiser has asked for that, RotatedSGD(fused_backward=True)), and the note of what it covers."""
    f = getattr(store, "fused_sgd", None) if store is not None else None
    if f is None:
        return {}
    if accumulate:
        raise RuntimeError("RotatedSGD(fused_backward=True): a rotated layer produced gradients twice before step(); "
                           "use fused_backward=False for gradient accumulation or shared layers")
    return f.bind(store, first, cnt, w_off, length)


def _fused_done(store, kw):
    """After the launch: if the library could not fuse the update for these operands, take the note back (the
    optimiser then updates that range itself)."""
    if kw:
        store.fused_sgd.confirm()


def col_wgrad(dy2, x2, grads, first, w_off, n_s, k, col0, cnt, accumulate, b_off: Optional[int] = None, store=None):
    """grads[first+g, w_off : w_off + n_s*k] (+)= dy2[:, col0 + g*n_s : ...]^T @ x2, g < cnt; with `b_off` also the
    bias gradients grads[first+g, b_off : b_off + n_s] (+)= column sums of the same block of dy2.  `store`: the
    layer's ShardStore, for an optimiser that applies its update inside this launch."""
    numel = grads.shape[1]
    es = grads.element_size()
    m, _, lda = _rows(dy2)
    _, _, ldb = _rows(x2)
    c = grads.data_ptr() + (first * numel + w_off) * es
    if n_s == 1 and cnt > 1:
        # one output row per shard (a gate with one expert per shard): the run is a single product whose
        # output rows are the shards' gradient rows, `numel` apart -- vector loads instead of 1-row groups
        ops.gemm_raw(grads.dtype, a=dy2.data_ptr() + col0 * es, b=x2.data_ptr(), c_out=c, m=cnt, n=k, k=m, lda=lda,
                     ldb=ldb, ldc=numel, a_kcontig=False, b_kcontig=False,
                     c_in=c if accumulate else None, ld_cin=numel, stream_out=True)
        if b_off is not None:
            col_bgrad(dy2, grads, first, b_off, n_s, col0, cnt, accumulate)
        return
    # one launch for the run (rtp_rotated_linear_bwd): the weight gradients, the bias gradients as the row sums of the
    # product's first operand dy^T, and the optimiser's update where one asked for it
    kw = _fused(store, accumulate, first, cnt, w_off, n_s * k)
    if kw:  # bound to the weight's own address; the entry point takes the run's base and adds w_off itself
        kw = dict(sgd=kw["sgd"], sgd_master=kw["sgd_master"] - w_off * 4,
                  sgd_weights=kw["sgd_weights"] - w_off * es if kw["sgd_weights"] else 0)
    run = grads[first:first + cnt]  # the weight-gradient half reads no weights: the gradient rows give the layout
    done = ops.rotated_linear_bwd(dy2[:, col0:], x2, run, w_off, b_off, n_s, k, grads=run, accumulate=accumulate, **kw)
    if kw:
        if not done & _lib.ROTATED_SGD_DONE:
            kw["sgd"].missed = True
        _fused_done(store, kw)
    if b_off is not None and not done & _lib.ROTATED_BIAS_DONE:
        col_bgrad(dy2, grads, first, b_off, n_s, col0, cnt, accumulate)


def col_bgrad(dy2, grads, first, b_off, n_s, col0, cnt, accumulate):
    """grads[first+g, b_off : b_off+n_s] (+)= column sums of dy2[:, col0 + g*n_s : ...]."""
    numel = grads.shape[1]
    block = dy2[:, col0:col0 + cnt * n_s]
    ops.colsum(block, grads[first, b_off:b_off + n_s], accumulate=accumulate, seg=n_s, seg_stride=numel)


def row_fwd(x2, flat, w_off, n, k_s, bias_off, out, col0, c_in: Optional[torch.Tensor] = None):
    """out[M, n] = (c_in +) sum_g x2[:, col0 + g*k_s : ...] @ W_g^T + sum_g b_g."""
    cnt, numel = flat.shape
    es = flat.element_size()
    m, _, lda = _rows(x2)
    _, _, ldc = _rows(out)
    kw = ops._epilogue_args(flat.dtype, out, c_in, None, None)
    ops.gemm_raw(flat.dtype, a=x2.data_ptr() + col0 * es, b=flat.data_ptr() + w_off * es, c_out=out.data_ptr(), m=m,
                 n=n, k=k_s, lda=lda, ldb=k_s, ldc=ldc, a_kcontig=True, b_kcontig=True,
                 bias=None if bias_off is None else flat.data_ptr() + bias_off * es, bias_sk=numel, ksegs=cnt,
                 a_sk=k_s, b_sk=numel, **kw)


def row_dgrad(dy2, flat, w_off, n, k_s, out, col0):
    """out[:, col0 + g*k_s : ...] = dy2 @ W_g, g over the run."""
    cnt, numel = flat.shape
    es = flat.element_size()
    m, _, lda = _rows(dy2)
    _, _, ldc = _rows(out)
    ops.gemm_raw(flat.dtype, a=dy2.data_ptr(), b=flat.data_ptr() + w_off * es, c_out=out.data_ptr() + col0 * es, m=m,
                 n=k_s, k=n, lda=lda, ldb=k_s, ldc=ldc, a_kcontig=True, b_kcontig=False, groups=cnt, b_sg=numel,
                 c_sg=k_s)


def row_wgrad(dy2, x2, grads, first, w_off, n, k_s, col0, cnt, accumulate, b_off: Optional[int] = None, store=None):
    """grads[first+g, w_off : w_off + n*k_s] (+)= dy2^T @ x2[:, col0 + g*k_s : ...]; with `b_off` also the bias
    gradients grads[first+g, b_off : b_off + n] (+)= column sums of dy2 (every shard of a row-style layer stores
    bias/ws and receives the full sum, tests/test_linear.py:181-186)."""
    numel = grads.shape[1]
    es = grads.element_size()
    m, _, lda = _rows(dy2)
    _, _, ldb = _rows(x2)
    c = grads.data_ptr() + (first * numel + w_off) * es
    rs = None if b_off is None else grads.data_ptr() + (first * numel + b_off) * es
    kw = _fused(store, accumulate, first, cnt, w_off, n * k_s)
    fused = ops.gemm_raw(grads.dtype, a=dy2.data_ptr(), b=x2.data_ptr() + col0 * es, c_out=c, m=n, n=k_s, k=m, lda=lda,
                         ldb=ldb, ldc=k_s, a_kcontig=False, b_kcontig=False, groups=cnt, b_sg=k_s, c_sg=numel,
                         c_in=c if accumulate else None, ld_cin=k_s, cin_sg=numel, stream_out=True,
                         rowsum=rs, rowsum_sg=numel, rowsum_accum=accumulate, **kw)
    _fused_done(store, kw)
    if b_off is not None and not fused:
        row_bgrad(dy2, grads, first, b_off, n, cnt, accumulate)


def row_bgrad(dy2, grads, first, b_off, n, cnt, accumulate):
    """grads[first+g, b_off : b_off + n] (+)= column sums of dy2 for every shard g of the run."""
    tmp = torch.empty(n, dtype=grads.dtype, device=grads.device)
    ops.colsum(dy2, tmp)
    dst = grads[first:first + cnt, b_off:b_off + n]
    if accumulate:
        dst.add_(tmp)
    else:
        dst.copy_(tmp.expand(cnt, n))
