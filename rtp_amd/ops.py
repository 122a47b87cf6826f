"""Tensor-level wrappers over the C ABI: they validate shapes/strides on the host, pass raw device
pointers plus the current torch stream to librtp_hip.so, and never compute anything themselves."""
from __future__ import annotations

import ctypes as C
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import (GEMM_CIN_F32, GEMM_OUT_F32, GEMM_RELU, GEMM_ROWSUM_ACCUM, GEMM_STREAM_OUT, RTP_BF16, RTP_F32, GemmDesc,
                   check)

_DT = {torch.float32: RTP_F32, torch.bfloat16: RTP_BF16}


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DT[dt]
    except KeyError:
        raise TypeError(f"rtp_amd kernels support float32 and bfloat16, got {dt}") from None


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _dev(t: torch.Tensor) -> None:
    if not t.is_cuda:
        raise _lib.RtpError("rtp_amd kernels run on the GPU only; got a CPU tensor (there is no CPU path)")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _mat(t: torch.Tensor, what: str):
    """(rows, cols, ld) of a 2-D tensor whose last dim is contiguous."""
    if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        raise ValueError(f"{what}: need a 2-D tensor with unit column stride, got shape {tuple(t.shape)} "
                         f"strides {t.stride()}")
    ld = t.stride(0) if t.shape[0] > 1 else max(t.shape[1], 1)
    return t.shape[0], t.shape[1], max(ld, 1)


def gemm_raw(dtype: torch.dtype, *, a: int, b: int, c_out: int, m: int, n: int, k: int, lda: int, ldb: int,
             ldc: int, a_kcontig: bool, b_kcontig: bool, c_in: Optional[int] = None, ld_cin: int = 0,
             bias: Optional[int] = None, gate: Optional[int] = None, ld_gate: int = 0, alpha: float = 1.0,
             relu: bool = False, out_f32: bool = False, cin_f32: bool = False, batch: int = 1, zdiv: int = 1,
             a_s=(0, 0), b_s=(0, 0), c_s=(0, 0), cin_s=(0, 0), gate_s=(0, 0), bias_s=(0, 0), groups: int = 1,
             a_sg: int = 0, b_sg: int = 0, c_sg: int = 0, cin_sg: int = 0, gate_sg: int = 0, bias_sg: int = 0,
             ksegs: int = 1, a_sk: int = 0, b_sk: int = 0, bias_sk: int = 0, stream_out: bool = False,
             rowsum: Optional[int] = None, rowsum_sg: int = 0, rowsum_accum: bool = False,
             sgd: Optional["FusedSgd"] = None, sgd_master: int = 0, sgd_weights: int = 0) -> bool:
    """One rtp_gemm call on raw device addresses (see include/rtp_hip.h for the operand rules).

    `sgd` (with the addresses of the fp32 parameters and of their compute-dtype copy that match c_out) asks for the
    clip + SGD update in the product's epilogue; if the library cannot fuse it for these operands the product runs
    without it and `sgd.missed` is set.

    `rowsum` asks for the row sums of A (the bias gradient of a weight-gradient product) from the same launch.
    Returns whether they were produced: False means the library cannot fuse them for these operands, the
    product ran without them and the caller owes a separate column sum."""
    _lib.require_device()
    d = GemmDesc()
    d.a, d.b, d.c_out, d.c_in, d.bias, d.gate = a, b, c_out, c_in, bias, gate
    d.m, d.n, d.k = m, n, k
    d.lda, d.ldb, d.ldc, d.ld_cin, d.ld_gate = lda, ldb, ldc, ld_cin, ld_gate
    d.batch, d.zdiv = batch, zdiv
    d.a_so, d.a_si = a_s
    d.b_so, d.b_si = b_s
    d.c_so, d.c_si = c_s
    d.cin_so, d.cin_si = cin_s
    d.gate_so, d.gate_si = gate_s
    d.bias_so, d.bias_si = bias_s
    d.groups, d.ksegs = groups, ksegs
    d.a_sg, d.b_sg, d.c_sg, d.cin_sg, d.gate_sg, d.bias_sg = a_sg, b_sg, c_sg, cin_sg, gate_sg, bias_sg
    d.a_sk, d.b_sk, d.bias_sk = a_sk, b_sk, bias_sk
    d.alpha = alpha
    d.flags = (GEMM_OUT_F32 if out_f32 else 0) | (GEMM_CIN_F32 if cin_f32 else 0) | (GEMM_RELU if relu else 0) | \
        (GEMM_STREAM_OUT if stream_out else 0) | (GEMM_ROWSUM_ACCUM if rowsum_accum else 0)
    d.a_kcontig, d.b_kcontig = int(a_kcontig), int(b_kcontig)
    lib = _lib.load()
    if sgd is not None:
        if lib.rtp_gemm_sgd_fused(dtype_code(dtype), C.byref(d)):
            d.sgd_master, d.sgd_weights = sgd_master, (sgd_weights or None)
            d.sgd_lr, d.sgd_clip = sgd.lr, sgd.clip
            if not sgd.keep_grads:
                d.flags |= _lib.GEMM_SGD_SKIP_OUT
        else:
            sgd.missed = True
    fused = rowsum is not None and bool(lib.rtp_gemm_rowsum_fused(dtype_code(dtype), C.byref(d)))
    d.a_rowsum, d.rowsum_sg = (rowsum, rowsum_sg) if fused else (None, 0)
    check(lib.rtp_gemm(_stream(), dtype_code(dtype), C.byref(d)))
    return fused


def _rotated_layer(home: torch.Tensor, w_off: int, bias_off: Optional[int], n_s: int, k: int) -> "_lib.RotatedLinear":
    if home.dim() != 2 or not home.is_contiguous():
        raise ValueError("rotated_linear: home must be the contiguous [shards, numel] buffer of the layer")
    _dev(home)
    return _lib.RotatedLinear(home.data_ptr(), home.shape[1], home.shape[0], w_off, -1 if bias_off is None else bias_off,
                              n_s, k)


def rotated_linear_fwd(x2: torch.Tensor, home: torch.Tensor, w_off: int, bias_off: Optional[int], n_s: int, k: int,
                       y: torch.Tensor, relu: bool = False) -> None:
    """y[rows, shards * n_s] = x2 @ W_g^T + b_g for every shard g of `home` [shards, numel], one launch; y in the
    shards' dtype or fp32."""
    layer = _rotated_layer(home, w_off, bias_off, n_s, k)
    rows, kk, ldx = _mat(x2, "x")
    ry, ny, ldy = _mat(y, "y")
    if kk != k or ry != rows or ny < n_s * home.shape[0] or x2.dtype != home.dtype or \
            y.dtype not in (home.dtype, torch.float32):
        raise ValueError("rotated_linear_fwd: x [rows, k] in the shards' dtype, y [rows, >= shards * n_s] (or fp32)")
    flags = (GEMM_RELU if relu else 0) | (GEMM_OUT_F32 if y.dtype != home.dtype else 0)
    _lib.require_device()
    check(_lib.load().rtp_rotated_linear_fwd(_stream(), dtype_code(home.dtype), C.byref(layer), x2.data_ptr(), ldx, rows,
                                             y.data_ptr(), ldy, flags))


def rotated_linear_bwd(dy2: torch.Tensor, x2: Optional[torch.Tensor], home: torch.Tensor, w_off: int,
                       bias_off: Optional[int], n_s: int, k: int, *, dx: Optional[torch.Tensor] = None,
                       dx_init: Optional[torch.Tensor] = None, relu_gate: Optional[torch.Tensor] = None,
                       grads: Optional[torch.Tensor] = None, accumulate: bool = False, sgd: Optional["FusedSgd"] = None,
                       sgd_master: int = 0, sgd_weights: int = 0) -> int:
    """The backward of rotated_linear_fwd, either half or both: dx [rows, k] (= dx_init + sum over the shards, masked
    where relu_gate <= 0) and / or the gradient rows `grads` [shards, numel] (weights, and the bias where the layer
    has one), with the clip + SGD update `sgd` applied in the same launch to the fp32 parameters at address
    sgd_master and their compute-dtype copy at sgd_weights (both laid out like home).  Returns the library's
    done flags (ROTATED_BIAS_DONE, ROTATED_SGD_DONE): what is missing there is left to the caller."""
    layer = _rotated_layer(home, w_off, bias_off, n_s, k)
    rows, ny, ldy = _mat(dy2, "dy")
    if ny < n_s * home.shape[0] or dy2.dtype != home.dtype:
        raise ValueError("rotated_linear_bwd: dy must be [rows, >= shards * n_s] in the shards' dtype")
    a = _lib.RotatedLinearBwdArgs()
    done = C.c_int32(0)
    a.done = C.pointer(done)
    if dx is not None:
        r, c, ld = _mat(dx, "dx")
        if (r, c) != (rows, k):
            raise ValueError("rotated_linear_bwd: dx must be [rows, k]")
        a.dx, a.ld_dx = dx.data_ptr(), ld
        for name, t in (("dx_init", dx_init), ("relu_gate", relu_gate)):
            if t is not None:
                r, c, ld = _mat(t, name)
                if (r, c) != (rows, k):
                    raise ValueError(f"rotated_linear_bwd: {name} must match dx")
                setattr(a, name, t.data_ptr())
                setattr(a, "ld_" + name, ld)
        for t, what in ((dx, "dx"), (dx_init, "dx_init")):
            if t is not None and t.dtype not in (home.dtype, torch.float32):
                raise TypeError(f"rotated_linear_bwd: {what} must be {home.dtype} or float32")
        if relu_gate is not None and relu_gate.dtype != home.dtype:
            raise TypeError("rotated_linear_bwd: relu_gate must be in the shards' dtype")
        a.dx_flags = (GEMM_OUT_F32 if dx.dtype != home.dtype else 0) | \
            (GEMM_CIN_F32 if dx_init is not None and dx_init.dtype != home.dtype else 0)
    if grads is not None:
        if grads.shape != home.shape or grads.dtype != home.dtype or not grads.is_contiguous() or x2 is None:
            raise ValueError("rotated_linear_bwd: grads must be laid out like home, and the layer's input is needed")
        a.grads, a.accumulate = grads.data_ptr(), int(accumulate)
        if sgd is not None:
            a.sgd_master, a.sgd_weights = sgd_master, (sgd_weights or None)
            a.sgd_lr, a.sgd_clip, a.sgd_skip_grad_store = sgd.lr, sgd.clip, int(not sgd.keep_grads)
    xr = _mat(x2, "x") if x2 is not None else (rows, k, k)
    _lib.require_device()
    check(_lib.load().rtp_rotated_linear_bwd(_stream(), dtype_code(home.dtype), C.byref(layer), dy2.data_ptr(), ldy,
                                             _ptr(x2), xr[2], rows, C.byref(a)))
    return done.value


def rotated_linear_xent_fwd(x2: torch.Tensor, home: torch.Tensor, w_off: int, bias_off: Optional[int], n_s: int, k: int,
                            target: torch.Tensor, ignore_index: int = -100) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-row cross-entropy loss (fp32 [rows]) and {max, sum exp} (fp32 [rows, 2]) of the logits
    x2 @ W_g^T + b_g over all shards g of `home`, without the logits reaching memory."""
    layer = _rotated_layer(home, w_off, bias_off, n_s, k)
    rows, kk, ldx = _mat(x2, "x")
    if kk != k or x2.dtype != home.dtype:
        raise ValueError("rotated_linear_xent_fwd: x must be [rows, k] in the shards' dtype")
    if target.dtype != torch.int64 or target.numel() != rows or not target.is_contiguous() or target.device != x2.device:
        raise ValueError("rotated_linear_xent_fwd: target must be contiguous int64 [rows] on the device")
    lib = _lib.load()
    nbytes = lib.rtp_rotated_linear_xent_workspace_bytes(C.byref(layer), rows)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x2.device)
    loss = torch.empty(rows, dtype=torch.float32, device=x2.device)
    stats = torch.empty(rows, 2, dtype=torch.float32, device=x2.device)
    _lib.require_device()
    check(lib.rtp_rotated_linear_xent_fwd(_stream(), dtype_code(home.dtype), C.byref(layer), x2.data_ptr(), ldx, rows,
                                          target.data_ptr(), int(ignore_index), loss.data_ptr(), stats.data_ptr(),
                                          ws.data_ptr(), nbytes))
    return loss, stats


def rotated_linear_xent_bwd(x2: torch.Tensor, home: torch.Tensor, w_off: int, bias_off: Optional[int], n_s: int, k: int,
                            target: torch.Tensor, ignore_index: int, stats: torch.Tensor, dloss: torch.Tensor,
                            scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The logits' gradient [rows, shards * n_s] = (softmax - onehot(target)) * dloss * scale in the shards' dtype, from
    the logits product run once more with the rows' statistics."""
    layer = _rotated_layer(home, w_off, bias_off, n_s, k)
    rows, kk, ldx = _mat(x2, "x")
    if kk != k or x2.dtype != home.dtype or stats.shape != (rows, 2) or stats.dtype != torch.float32 or \
            not stats.is_contiguous() or dloss.dtype != torch.float32 or dloss.numel() != 1:
        raise ValueError("rotated_linear_xent_bwd: x [rows, k], stats fp32 [rows, 2], dloss one fp32 element")
    out = torch.empty(rows, n_s * home.shape[0], dtype=home.dtype, device=x2.device)
    _lib.require_device()
    check(_lib.load().rtp_rotated_linear_xent_bwd(_stream(), dtype_code(home.dtype), C.byref(layer), x2.data_ptr(), ldx,
                                                  rows, target.data_ptr(), int(ignore_index), stats.data_ptr(),
                                                  dloss.data_ptr(), _ptr(scale), out.data_ptr(), out.stride(0)))
    return out


def _epilogue_args(dtype, out, c_in, bias, gate):
    kw = {}
    if out.dtype == torch.float32 and dtype != torch.float32:
        kw["out_f32"] = True
    elif out.dtype != dtype:
        raise TypeError(f"gemm output must be {dtype} or float32, got {out.dtype}")
    if c_in is not None:
        _, _, ld = _mat(c_in, "c_in")
        if c_in.shape != out.shape:
            raise ValueError(f"c_in shape {tuple(c_in.shape)} != output shape {tuple(out.shape)}")
        kw["c_in"], kw["ld_cin"] = c_in.data_ptr(), ld
        if c_in.dtype == torch.float32 and dtype != torch.float32:
            kw["cin_f32"] = True
        elif c_in.dtype != dtype:
            raise TypeError(f"c_in must be {dtype} or float32, got {c_in.dtype}")
    if bias is not None:
        if bias.dtype != dtype or bias.dim() != 1 or bias.shape[0] != out.shape[1] or not bias.is_contiguous():
            raise ValueError("bias must be a contiguous vector of the output width and the compute dtype")
        kw["bias"] = bias.data_ptr()
    if gate is not None:
        _, _, ld = _mat(gate, "gate")
        if gate.shape != out.shape or gate.dtype != dtype:
            raise ValueError("gate must match the output shape and the compute dtype")
        kw["gate"], kw["ld_gate"] = gate.data_ptr(), ld
    return kw


def linear_fwd(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, *, bias=None, c_in=None, relu=False,
               alpha: float = 1.0) -> None:
    """out[M,N] = epilogue(x[M,K] @ w[N,K]^T)   (F.linear of one shard)."""
    for t in (x, w, out):
        _dev(t)
    m, k, lda = _mat(x, "x")
    n, k2, ldb = _mat(w, "w")
    mo, no, ldc = _mat(out, "out")
    if k != k2 or mo != m or no != n or x.dtype != w.dtype:
        raise ValueError(f"linear_fwd: x {tuple(x.shape)} {x.dtype}, w {tuple(w.shape)} {w.dtype}, "
                         f"out {tuple(out.shape)}")
    gemm_raw(x.dtype, a=x.data_ptr(), b=w.data_ptr(), c_out=out.data_ptr(), m=m, n=n, k=k, lda=lda, ldb=ldb,
             ldc=ldc, a_kcontig=True, b_kcontig=True, relu=relu, alpha=alpha,
             **_epilogue_args(x.dtype, out, c_in, bias, None))


def linear_dgrad(dy: torch.Tensor, w: torch.Tensor, out: torch.Tensor, *, c_in=None, gate=None) -> None:
    """out[M,K] = epilogue(dy[M,N] @ w[N,K])   (input gradient of F.linear)."""
    for t in (dy, w, out):
        _dev(t)
    m, n, lda = _mat(dy, "dy")
    n2, k, ldb = _mat(w, "w")
    mo, ko, ldc = _mat(out, "out")
    if n != n2 or mo != m or ko != k or dy.dtype != w.dtype:
        raise ValueError(f"linear_dgrad: dy {tuple(dy.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
    # contraction index is n: A = dy (n contiguous), B(kk, n) = w[n, kk] (stored n-major -> not k-contig)
    gemm_raw(dy.dtype, a=dy.data_ptr(), b=w.data_ptr(), c_out=out.data_ptr(), m=m, n=k, k=n, lda=lda, ldb=ldb,
             ldc=ldc, a_kcontig=True, b_kcontig=False, **_epilogue_args(dy.dtype, out, c_in, None, gate))


def linear_wgrad(dy: torch.Tensor, x: torch.Tensor, out: torch.Tensor, *, c_in=None) -> None:
    """out[N,K] = epilogue(dy[M,N]^T @ x[M,K])   (weight gradient of F.linear)."""
    for t in (dy, x, out):
        _dev(t)
    m, n, lda = _mat(dy, "dy")
    m2, k, ldb = _mat(x, "x")
    no, ko, ldc = _mat(out, "out")
    if m != m2 or no != n or ko != k or dy.dtype != x.dtype:
        raise ValueError(f"linear_wgrad: dy {tuple(dy.shape)}, x {tuple(x.shape)}, out {tuple(out.shape)}")
    gemm_raw(dy.dtype, a=dy.data_ptr(), b=x.data_ptr(), c_out=out.data_ptr(), m=n, n=k, k=m, lda=lda, ldb=ldb,
             ldc=ldc, a_kcontig=False, b_kcontig=False, **_epilogue_args(dy.dtype, out, c_in, None, None))


def colsum(x: torch.Tensor, out: torch.Tensor, accumulate: bool = False, seg: int = 0, seg_stride: int = 0) -> None:
    """Column sums of x[M,N] (bias gradients).  With seg == 0: out[N] (+)= sums.  With seg > 0 column c goes
    to out.view(-1)[(c // seg) * seg_stride + c % seg]: `out` is then the first segment's destination inside
    a larger buffer that holds one segment per shard, seg_stride elements apart."""
    _dev(x)
    _dev(out)
    m, n, ld = _mat(x, "x")
    if seg == 0 and (out.dim() != 1 or out.shape[0] != n or not out.is_contiguous()):
        raise ValueError("colsum: out must be a contiguous vector of x's width")
    if seg and (n % seg != 0 or seg_stride < seg):
        raise ValueError("colsum: width must be a multiple of seg and seg_stride >= seg")
    if out.dtype not in (x.dtype, torch.float32):
        raise TypeError("colsum: out must be the input dtype or float32")
    _lib.require_device()
    lib = _lib.load()
    nbytes = lib.rtp_colsum_workspace_bytes(m, n)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    check(lib.rtp_colsum(_stream(), dtype_code(x.dtype), x.data_ptr(), m, n, ld, out.data_ptr(),
                         int(out.dtype == torch.float32), int(accumulate), seg, seg_stride, ws.data_ptr(), nbytes))


def shard_copy(dst: torch.Tensor, src: torch.Tensor) -> None:
    """dst <- src with the rotation copy kernel on the current stream."""
    _dev(dst)
    _dev(src)
    if not (dst.is_contiguous() and src.is_contiguous()) or dst.numel() * dst.element_size() != \
            src.numel() * src.element_size():
        raise ValueError("shard_copy: need contiguous tensors of equal byte size")
    _lib.require_device()
    check(_lib.load().rtp_shard_copy_async(_stream(), dst.data_ptr(), src.data_ptr(),
                                           src.numel() * src.element_size()))


def zero_(t: torch.Tensor) -> None:
    _dev(t)
    if not t.is_contiguous():
        raise ValueError("zero_: need a contiguous tensor")
    _lib.require_device()
    check(_lib.load().rtp_zero_async(_stream(), t.data_ptr(), t.numel() * t.element_size()))


def embedding_gather(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, row_begin: int = 0, groups: int = 1,
                     table_sg: int = 0, out_sg: int = 0, *, scale: float = 1.0, pos: Optional[torch.Tensor] = None,
                     pos_sg: int = 0, batch: int = 1) -> None:
    """out[t, :] = table[ids[t] - row_begin, :] for ids inside the shard's row range.  With groups > 1,
    `table` / `out` are shard 0's table and output block; shard g sits table_sg / out_sg elements further.
    With `pos` ([positions, cols] block of a positional table, shard g at pos_sg elements further) the row is
    scaled and the positional row of token t (position t // batch) added, rounding after each step."""
    for t in (table, ids, out):
        _dev(t)
    rows, cols, ld_t = _mat(table, "table")
    n, cols_o, ld_o = _mat(out, "out")
    if ids.dtype != torch.int64 or not ids.is_contiguous() or ids.numel() != n or cols_o != cols or \
            out.dtype != table.dtype:
        raise ValueError("embedding_gather: ids must be contiguous int64 with one id per output row")
    _lib.require_device()
    if pos is not None:
        _dev(pos)
        p_rows, p_cols, ld_p = _mat(pos, "pos")
        if pos.dtype != table.dtype or p_cols != cols or batch < 1 or (n + batch - 1) // batch > p_rows:
            raise ValueError("embedding_gather: pos must hold one row of the table's dtype per position")
        check(_lib.load().rtp_embedding_gather_scale_pos(
            _stream(), dtype_code(table.dtype), table.data_ptr(), ld_t, row_begin, rows, cols, ids.data_ptr(), n,
            out.data_ptr(), ld_o, groups, table_sg, out_sg, float(scale), pos.data_ptr(), ld_p, pos_sg, batch))
        return
    if scale != 1.0:
        raise ValueError("embedding_gather: a scale needs the positional table")
    check(_lib.load().rtp_embedding_gather(_stream(), dtype_code(table.dtype), table.data_ptr(), ld_t, row_begin,
                                           rows, cols, ids.data_ptr(), n, out.data_ptr(), ld_o, groups, table_sg,
                                           out_sg))


def embedding_sort_ids(ids: torch.Tensor) -> torch.Tensor:
    """Sorted (id, position) workspace shared by the scatter-adds of all shards of one backward."""
    _dev(ids)
    if ids.dtype != torch.int64 or not ids.is_contiguous():
        raise ValueError("embedding_sort_ids: ids must be contiguous int64")
    _lib.require_device()
    lib = _lib.load()
    nbytes = lib.rtp_embedding_scatter_workspace_bytes(ids.numel())
    ws = torch.empty(nbytes, dtype=torch.uint8, device=ids.device)
    check(lib.rtp_embedding_sort_ids(_stream(), ids.data_ptr(), ids.numel(), ws.data_ptr(), nbytes))
    return ws


def embedding_backward_supported(n_ids: int) -> bool:
    """Whether a step of n_ids tokens fits the one-launch embedding backward (its ids are staged in LDS)."""
    return bool(_lib.load().rtp_embedding_backward_supported(int(n_ids)))


def embedding_backward(grad_out: torch.Tensor, ids: torch.Tensor, grad_table: torch.Tensor, *, row_begin: int = 0,
                       padding_idx: int = -1, scale_by_freq: bool = False, zero_fill: bool = True, groups: int = 1,
                       grad_out_sg: int = 0, grad_table_sg: int = 0, grad_scale: float = 1.0,
                       sgd: Optional["FusedSgd"] = None, sgd_master: int = 0, sgd_weights: int = 0) -> None:
    """embedding_sort_ids + embedding_scatter_add in one launch, from the raw ids (contiguous int64, one per row of
    grad_out): same arguments, same results bit for bit; rows no token names are cleared by the same launch when
    zero_fill.  Only for steps embedding_backward_supported() accepts."""
    for t in (grad_out, ids, grad_table):
        _dev(t)
    n, cols, ld_go = _mat(grad_out, "grad_out")
    rows, cols_t, ld_gt = _mat(grad_table, "grad_table")
    if ids.dtype != torch.int64 or not ids.is_contiguous() or ids.numel() != n or cols != cols_t:
        raise ValueError("embedding_backward: ids must be contiguous int64, one per row of grad_out; tables [rows, cols]")
    if grad_table.dtype not in (grad_out.dtype, torch.float32):
        raise TypeError("embedding_backward: grad_table must be the grad dtype or float32")
    if sgd is not None and (not zero_fill or grad_table.dtype != grad_out.dtype):
        raise ValueError("embedding_backward: the fused update takes the whole gradient of the step, in the table's "
                         "own dtype")
    _lib.require_device()
    check(_lib.load().rtp_embedding_backward(
        _stream(), dtype_code(grad_out.dtype), grad_out.data_ptr(), ld_go, n, ids.data_ptr(), grad_table.data_ptr(),
        ld_gt, int(grad_table.dtype == torch.float32), row_begin, rows, cols,
        -1 if padding_idx is None else padding_idx, int(scale_by_freq), int(zero_fill), groups, grad_out_sg,
        grad_table_sg, float(grad_scale), (sgd_master or None) if sgd is not None else None,
        (sgd_weights or None) if sgd is not None else None, sgd.lr if sgd is not None else 0.0,
        sgd.clip if sgd is not None else 0.0, int(sgd.keep_grads) if sgd is not None else 1))


def embedding_scatter_add(grad_out: torch.Tensor, n_ids: int, workspace: torch.Tensor, grad_table: torch.Tensor,
                          *, row_begin: int = 0, padding_idx: int = -1, scale_by_freq: bool = False,
                          zero_fill: bool = True, groups: int = 1, grad_out_sg: int = 0,
                          grad_table_sg: int = 0, grad_scale: float = 1.0, sgd: Optional["FusedSgd"] = None,
                          sgd_master: int = 0, sgd_weights: int = 0) -> None:
    """grad_table[id] (+)= sum of the grad_out rows whose token is id, in ascending position order.  With
    groups > 1, group g reads grad_out + g*grad_out_sg and writes grad_table + g*grad_table_sg (elements):
    all shards of an embedding in one launch.  grad_scale != 1 sums grad_out * grad_scale, each product rounded
    to grad_out's dtype first (the gradient a scaled embedding receives).

    `sgd` (with the addresses of the fp32 table and of its compute-dtype copy that match grad_table): the rows some
    token names are updated by clip + SGD right here, the others are left alone (their gradient is zero), and the
    dense gradient is only filled and written when sgd.keep_grads."""
    for t in (grad_out, workspace, grad_table):
        _dev(t)
    n, cols, ld_go = _mat(grad_out, "grad_out")
    rows, cols_t, ld_gt = _mat(grad_table, "grad_table")
    if n != n_ids or cols != cols_t:
        raise ValueError("embedding_scatter_add: shape mismatch")
    if grad_table.dtype not in (grad_out.dtype, torch.float32):
        raise TypeError("embedding_scatter_add: grad_table must be the grad dtype or float32")
    _lib.require_device()
    args = (_stream(), dtype_code(grad_out.dtype), grad_out.data_ptr(), ld_go, n_ids, workspace.data_ptr(),
            grad_table.data_ptr(), ld_gt, int(grad_table.dtype == torch.float32), row_begin, rows, cols,
            -1 if padding_idx is None else padding_idx, int(scale_by_freq), int(zero_fill), groups, grad_out_sg,
            grad_table_sg)
    if sgd is not None:
        if not zero_fill or grad_table.dtype != grad_out.dtype:
            raise ValueError("embedding_scatter_add: the fused update takes the whole gradient of the step, in the "
                             "table's own dtype")
        check(_lib.load().rtp_embedding_scatter_add_sgd(
            _stream(), dtype_code(grad_out.dtype), grad_out.data_ptr(), ld_go, n_ids, workspace.data_ptr(),
            grad_table.data_ptr(), ld_gt, row_begin, rows, cols, -1 if padding_idx is None else padding_idx,
            int(scale_by_freq), groups, grad_out_sg, grad_table_sg, float(grad_scale), sgd_master, sgd_weights or None,
            sgd.lr, sgd.clip, int(sgd.keep_grads)))
        return
    if grad_scale != 1.0:
        check(_lib.load().rtp_embedding_scatter_add_scaled(*args, float(grad_scale)))
    else:
        check(_lib.load().rtp_embedding_scatter_add_det(*args))


def _key_bias_ptr(who: str, key_bias: Optional[torch.Tensor], n_batch: int, keys: int):
    if key_bias is None:
        return None
    if key_bias.dtype != torch.float32 or tuple(key_bias.shape) != (n_batch, keys) or not key_bias.is_contiguous():
        raise ValueError(f"{who}: key_bias must be a contiguous fp32 [batch, keys] tensor")
    return key_bias.data_ptr()


def _keep_ptr(who: str, keep: Optional[torch.Tensor], like: torch.Tensor):
    if keep is None:
        return None
    if keep.dtype != torch.float32 or keep.shape != like.shape or not keep.is_contiguous() or keep.device != like.device:
        raise ValueError(f"{who}: keep must be a contiguous fp32 tensor of the probabilities' shape")
    return keep.data_ptr()


def softmax_fwd(scores: torch.Tensor, p: torch.Tensor, *, mask: Optional[torch.Tensor], causal: bool,
                scale: float, key_bias: Optional[torch.Tensor] = None, heads: int = 1,
                keep: Optional[torch.Tensor] = None, p_dropped: Optional[torch.Tensor] = None) -> None:
    """p[Z,L,S] = softmax(scale*scores + mask + key_bias[b]) row-wise; scores fp32, mask fp32 [L,S] (one for all
    problems) or [M,L,S] (problem z takes mask[z % M]) or None, key_bias fp32 [N,S] or None with
    Z = groups * N * heads (problem z belongs to batch (z // heads) % N).  Attention dropout: `keep` (fp32, 0 or
    1 / (1 - rate) per probability) and `p_dropped` (receives p * keep) go together."""
    _dev(scores)
    _dev(p)
    if scores.dtype != torch.float32 or scores.dim() != 3 or not scores.is_contiguous() or \
            p.shape != scores.shape or not p.is_contiguous():
        raise ValueError("softmax_fwd: scores must be contiguous fp32 [Z,L,S] and p the same shape")
    z, l, s = scores.shape
    masks = 1
    if mask is not None:
        if mask.dtype != torch.float32 or tuple(mask.shape[-2:]) != (l, s) or mask.dim() not in (2, 3) or \
                not mask.is_contiguous():
            raise ValueError("softmax_fwd: mask must be contiguous fp32 [L,S] or [M,L,S]")
        if mask.dim() == 3:
            masks = mask.shape[0]
            if masks < 1 or z % masks:
                raise ValueError(f"softmax_fwd: {masks} masks do not divide {z} problems")
    n_batch = key_bias.shape[0] if key_bias is not None else 1
    kb = _key_bias_ptr("softmax_fwd", key_bias, n_batch, s)
    _lib.require_device()
    if (keep is None) != (p_dropped is None):
        raise ValueError("softmax_fwd: keep and p_dropped go together")
    if p_dropped is not None and (p_dropped.shape != p.shape or p_dropped.dtype != p.dtype or
                                  not p_dropped.is_contiguous()):
        raise ValueError("softmax_fwd: p_dropped must match p")
    check(_lib.load().rtp_softmax_fwd_masks(_stream(), dtype_code(p.dtype), scores.data_ptr(), _ptr(mask), masks, kb,
                                            n_batch, heads, int(causal), scale, z, l, s, p.data_ptr(),
                                            _keep_ptr("softmax_fwd", keep, p), _ptr(p_dropped)))


def softmax_bwd(p: torch.Tensor, dp: torch.Tensor, ds: torch.Tensor, scale: float,
                keep: Optional[torch.Tensor] = None) -> None:
    """ds = scale * p * (g - sum_j g * p) with g = dp, or dp * keep when the probabilities were dropped."""
    _dev(p)
    if dp.dtype != torch.float32 or p.dim() != 3 or dp.shape != p.shape or ds.shape != p.shape or \
            ds.dtype != p.dtype or not (p.is_contiguous() and dp.is_contiguous() and ds.is_contiguous()):
        raise ValueError("softmax_bwd: need contiguous p/ds [Z,L,S] of one dtype and fp32 dp")
    z, l, s = p.shape
    _lib.require_device()
    check(_lib.load().rtp_softmax_bwd(_stream(), dtype_code(p.dtype), p.data_ptr(), dp.data_ptr(),
                                      _keep_ptr("softmax_bwd", keep, p), scale, z, l, s, ds.data_ptr()))


def attn_supported(dtype: torch.dtype, L: int, d: int) -> bool:
    """Whether the fused short-sequence attention core handles this shape (bf16, L <= 32, d in {32, 64, 128})."""
    if dtype != torch.bfloat16:
        return False
    return bool(_lib.load().rtp_attn_supported(dtype_code(dtype), L, d))


def attn_fwd(qkv: torch.Tensor, q_off: int, k_off: int, v_off: int, qkv_strides, o: torch.Tensor, o_off: int,
             o_strides, p: torch.Tensor, mask: Optional[torch.Tensor], causal: bool, scale: float, L: int, N: int,
             H: int, d: int, G: int, key_bias: Optional[torch.Tensor] = None) -> None:
    """Fused q k^T -> softmax -> p v for G*N*H (group, batch, head) problems addressed by element strides
    (s_l, s_b, s_h, s_g) into the packed projection `qkv` (offsets in elements) and `o`; p [G*N*H, L, L]."""
    _dev(qkv)
    esz = qkv.element_size()
    if p.dtype != qkv.dtype or o.dtype != qkv.dtype or not p.is_contiguous() or p.numel() != G * N * H * L * L:
        raise ValueError("attn_fwd: p must be contiguous [G*N*H, L, L] of the operand dtype")
    if mask is not None and (mask.dtype != torch.float32 or tuple(mask.shape) != (L, L) or not mask.is_contiguous()):
        raise ValueError("attn_fwd: mask must be a contiguous fp32 [L, L] tensor")
    _lib.require_device()
    base = qkv.data_ptr()
    check(_lib.load().rtp_attn_fwd(_stream(), dtype_code(qkv.dtype), base + q_off * esz, base + k_off * esz,
                                   base + v_off * esz, *qkv_strides, o.data_ptr() + o_off * esz, *o_strides,
                                   p.data_ptr(), mask.data_ptr() if mask is not None else None,
                                   _key_bias_ptr("attn_fwd", key_bias, N, L), int(causal), scale, L, N, H, d, G))


def attn_bwd(qkv: torch.Tensor, q_off: int, k_off: int, v_off: int, qkv_strides, dout: torch.Tensor, o_off: int,
             o_strides, p: torch.Tensor, dqkv: torch.Tensor, scale: float, L: int, N: int, H: int, d: int,
             G: int) -> None:
    """Backward of attn_fwd: writes dq, dk, dv into `dqkv` (same layout and offsets as `qkv`)."""
    _dev(qkv)
    esz = qkv.element_size()
    if dqkv.dtype != qkv.dtype or dqkv.shape != qkv.shape or dqkv.stride() != qkv.stride() or dout.dtype != qkv.dtype:
        raise ValueError("attn_bwd: dqkv must match qkv, dout must share its dtype")
    _lib.require_device()
    base, dbase = qkv.data_ptr(), dqkv.data_ptr()
    check(_lib.load().rtp_attn_bwd(_stream(), dtype_code(qkv.dtype), base + q_off * esz, base + k_off * esz,
                                   base + v_off * esz, *qkv_strides, dout.data_ptr() + o_off * esz, *o_strides,
                                   p.data_ptr(), dbase + q_off * esz, dbase + k_off * esz, dbase + v_off * esz, scale,
                                   L, N, H, d, G))


def attn_flash_supported(dtype: torch.dtype, L: int, d: int) -> bool:
    """Whether the running-softmax attention core handles this shape (bf16, any L, d in {32, 64, 128})."""
    if dtype != torch.bfloat16:
        return False
    return bool(_lib.load().rtp_attn_flash_supported(dtype_code(dtype), L, d))


def _flash_rows(name: str, t: torch.Tensor, G: int, N: int, H: int, L: int) -> None:
    if t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != G * N * H * L:
        raise ValueError(f"{name} must be a contiguous fp32 [G*N*H, L] tensor")


def _flash_mask(mask: Optional[torch.Tensor], L: int):
    if mask is None:
        return None
    if mask.dtype != torch.float32 or tuple(mask.shape) != (L, L) or not mask.is_contiguous():
        raise ValueError("attention mask must be a contiguous fp32 [L, L] tensor")
    return mask.data_ptr()


def attn_flash_fwd(qkv: torch.Tensor, q_off: int, k_off: int, v_off: int, qkv_strides, o: torch.Tensor, o_off: int,
                   o_strides, lse: torch.Tensor, mask: Optional[torch.Tensor], causal: bool, scale: float, L: int,
                   N: int, H: int, d: int, G: int, key_bias: Optional[torch.Tensor] = None) -> None:
    """attn_fwd for any L: o = softmax(scale q k^T + mask) v without storing the probabilities; lse [G*N*H, L]
    fp32 receives the log-sum-exp of each query's scores."""
    _dev(qkv)
    esz = qkv.element_size()
    if o.dtype != qkv.dtype:
        raise ValueError("attn_flash_fwd: o must share the operand dtype")
    _flash_rows("attn_flash_fwd: lse", lse, G, N, H, L)
    mask_ptr = _flash_mask(mask, L)
    _lib.require_device()
    base = qkv.data_ptr()
    check(_lib.load().rtp_attn_flash_fwd(_stream(), dtype_code(qkv.dtype), base + q_off * esz, base + k_off * esz,
                                         base + v_off * esz, *qkv_strides, o.data_ptr() + o_off * esz, *o_strides,
                                         lse.data_ptr(), mask_ptr, _key_bias_ptr("attn_flash_fwd", key_bias, N, L),
                                         int(causal), scale, L, N, H, d, G))


def attn_flash_bwd(qkv: torch.Tensor, q_off: int, k_off: int, v_off: int, qkv_strides, o: torch.Tensor,
                   dout: torch.Tensor, o_off: int, o_strides, lse: torch.Tensor, delta: torch.Tensor,
                   dqkv: torch.Tensor, mask: Optional[torch.Tensor], causal: bool, scale: float, L: int, N: int,
                   H: int, d: int, G: int, key_bias: Optional[torch.Tensor] = None) -> None:
    """Backward of attn_flash_fwd: writes dq, dk, dv into `dqkv` (layout and offsets of `qkv`); `o` and `dout`
    share layout and offset; `delta` [G*N*H, L] fp32 is scratch."""
    _dev(qkv)
    esz = qkv.element_size()
    if dqkv.dtype != qkv.dtype or dqkv.shape != qkv.shape or dqkv.stride() != qkv.stride():
        raise ValueError("attn_flash_bwd: dqkv must match qkv")
    if dout.dtype != qkv.dtype or o.dtype != qkv.dtype or dout.shape != o.shape or dout.stride() != o.stride():
        raise ValueError("attn_flash_bwd: o and dout must share dtype and layout")
    _flash_rows("attn_flash_bwd: lse", lse, G, N, H, L)
    _flash_rows("attn_flash_bwd: delta", delta, G, N, H, L)
    mask_ptr = _flash_mask(mask, L)
    _lib.require_device()
    base, dbase = qkv.data_ptr(), dqkv.data_ptr()
    check(_lib.load().rtp_attn_flash_bwd(_stream(), dtype_code(qkv.dtype), base + q_off * esz, base + k_off * esz,
                                         base + v_off * esz, *qkv_strides, o.data_ptr() + o_off * esz,
                                         dout.data_ptr() + o_off * esz, *o_strides, lse.data_ptr(), delta.data_ptr(),
                                         dbase + q_off * esz, dbase + k_off * esz, dbase + v_off * esz, mask_ptr,
                                         _key_bias_ptr("attn_flash_bwd", key_bias, N, L), int(causal), scale, L, N, H,
                                         d, G))


def layernorm_supported(dtype: torch.dtype, cols: int) -> bool:
    if dtype not in (torch.float32, torch.bfloat16):
        return False
    return bool(_lib.load().rtp_layernorm_supported(dtype_code(dtype), cols))


def add_layernorm_fwd(x: torch.Tensor, r: Optional[torch.Tensor], gamma: torch.Tensor, beta: Optional[torch.Tensor],
                      eps: float, z: Optional[torch.Tensor], y: torch.Tensor, mean: torch.Tensor,
                      rstd: torch.Tensor) -> None:
    """y = LayerNorm(x + r) over the last axis; z receives x + r; mean / rstd are fp32 [rows]."""
    _dev(x)
    cols = x.shape[-1]
    rows = x.numel() // max(cols, 1)
    tensors = [t for t in (x, r, z, y) if t is not None]
    if any(t.dtype != x.dtype or t.shape != x.shape or not t.is_contiguous() for t in tensors):
        raise ValueError("add_layernorm_fwd: x, r, z, y must be contiguous, of one shape and dtype")
    if gamma.dtype != x.dtype or gamma.numel() != cols or (beta is not None and (beta.dtype != x.dtype or
                                                                                  beta.numel() != cols)):
        raise ValueError("add_layernorm_fwd: gamma / beta must be vectors of the row length in x's dtype")
    if mean.dtype != torch.float32 or rstd.dtype != torch.float32 or mean.numel() != rows or rstd.numel() != rows:
        raise ValueError("add_layernorm_fwd: mean / rstd must be fp32 [rows]")
    _lib.require_device()
    check(_lib.load().rtp_add_layernorm_fwd(
        _stream(), dtype_code(x.dtype), x.data_ptr(), r.data_ptr() if r is not None else None, gamma.data_ptr(),
        beta.data_ptr() if beta is not None else None, eps, rows, cols, z.data_ptr() if z is not None else None,
        y.data_ptr(), mean.data_ptr(), rstd.data_ptr()))


def layernorm_bwd(dy: torch.Tensor, z: torch.Tensor, gamma: torch.Tensor, mean: torch.Tensor, rstd: torch.Tensor,
                  dz: torch.Tensor, dgamma: torch.Tensor, dbeta: Optional[torch.Tensor]) -> None:
    _dev(dy)
    cols = z.shape[-1]
    rows = z.numel() // max(cols, 1)
    if any(t.dtype != z.dtype or t.shape != z.shape or not t.is_contiguous() for t in (dy, dz)) or \
            not z.is_contiguous():
        raise ValueError("layernorm_bwd: dy, z, dz must be contiguous, of one shape and dtype")
    _lib.require_device()
    lib = _lib.load()
    nbytes = lib.rtp_layernorm_bwd_workspace_bytes(rows, cols)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=z.device)
    check(lib.rtp_layernorm_bwd(_stream(), dtype_code(z.dtype), dy.data_ptr(), z.data_ptr(), gamma.data_ptr(),
                                mean.data_ptr(), rstd.data_ptr(), rows, cols, dz.data_ptr(), dgamma.data_ptr(),
                                dbeta.data_ptr() if dbeta is not None else None, ws.data_ptr(), nbytes))


def layernorm_bwd_deferred(dy: torch.Tensor, z: torch.Tensor, gamma: torch.Tensor, mean: torch.Tensor,
                           rstd: torch.Tensor, dz: torch.Tensor, part: Optional[torch.Tensor]) -> torch.Tensor:
    """layernorm_bwd without the reduction of the parameter gradients: writes dz and leaves the per-block partial sums
    in `part` (allocated when None or too small; the caller keeps it until layernorm_finalize has run)."""
    _dev(dy)
    cols = z.shape[-1]
    rows = z.numel() // max(cols, 1)
    if any(t.dtype != z.dtype or t.shape != z.shape or not t.is_contiguous() for t in (dy, dz)) or \
            not z.is_contiguous():
        raise ValueError("layernorm_bwd_deferred: dy, z, dz must be contiguous, of one shape and dtype")
    _lib.require_device()
    lib = _lib.load()
    nbytes = lib.rtp_layernorm_bwd_workspace_bytes(rows, cols)
    if part is None or part.numel() < nbytes or part.device != z.device:
        part = torch.empty(nbytes, dtype=torch.uint8, device=z.device)
    check(lib.rtp_layernorm_bwd(_stream(), dtype_code(z.dtype), dy.data_ptr(), z.data_ptr(), gamma.data_ptr(),
                                mean.data_ptr(), rstd.data_ptr(), rows, cols, dz.data_ptr(), None, None,
                                part.data_ptr(), part.numel()))
    return part


def _device_table(rows, device) -> torch.Tensor:
    """int64 rows -> device tensor.  The upload cannot be recorded into a graph: a model's first step, which builds
    its tables, has to run eagerly."""
    if torch.cuda.is_current_stream_capturing():
        raise RuntimeError("a device table (optimiser chunks / LayerNorm reduction) has to be built while a graph is "
                           "being captured: run one eager step of the model and its optimiser first")
    return torch.tensor(rows, dtype=torch.int64).to(device)


def layernorm_final_table(items, device) -> torch.Tensor:
    """Device table for layernorm_finalize: items = [(part, rows, cols, dgamma, dbeta or None), ...]."""
    lib = _lib.load()
    rows = []
    for part, n_rows, cols, dgamma, dbeta in items:
        rows.append([part.data_ptr(), lib.rtp_layernorm_bwd_blocks(n_rows), cols, dgamma.data_ptr(),
                     dbeta.data_ptr() if dbeta is not None else 0])
    return _device_table(rows, device)


def layernorm_finalize(table: torch.Tensor, dtype: torch.dtype, max_cols: int) -> None:
    """dgamma / dbeta of every LayerNorm in `table` from its partial sums, one launch."""
    _dev(table)
    _lib.require_device()
    check(_lib.load().rtp_layernorm_bwd_finalize(_stream(), dtype_code(dtype), table.data_ptr(), table.shape[0],
                                                 max_cols))


def _xent_check(who: str, logits: torch.Tensor, target: torch.Tensor) -> None:
    _dev(logits)
    if logits.dtype not in (torch.float32, torch.bfloat16) or logits.dim() != 2 or logits.shape[1] < 1 or \
            (logits.shape[1] > 1 and logits.stride(1) != 1) or \
            (logits.shape[0] > 1 and logits.stride(0) < logits.shape[1]):
        raise ValueError(f"{who}: logits must be fp32 / bf16 [rows, classes] with unit column stride")
    if target.dtype != torch.int64 or target.numel() != logits.shape[0] or not target.is_contiguous() or \
            target.device != logits.device:
        raise ValueError(f"{who}: target must be contiguous int64 [rows] on the logits' device")


def softmax_xent_fwd(logits: torch.Tensor, target: torch.Tensor,
                     ignore_index: int = -100) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-row cross-entropy loss (fp32 [rows]; 0 where target == ignore_index, NaN for any other target outside
    the classes) and softmax statistics {max, sum exp} (fp32 [rows, 2])."""
    _xent_check("softmax_xent_fwd", logits, target)
    rows, cols = logits.shape
    loss = torch.empty(rows, dtype=torch.float32, device=logits.device)
    stats = torch.empty((rows, 2), dtype=torch.float32, device=logits.device)
    _lib.require_device()
    check(_lib.load().rtp_softmax_xent_fwd(_stream(), dtype_code(logits.dtype), logits.data_ptr(),
                                           logits.stride(0) if rows > 1 else cols, rows, cols, target.data_ptr(),
                                           int(ignore_index), loss.data_ptr(), stats.data_ptr()))
    return loss, stats


def softmax_xent_reduce(loss_rows: torch.Tensor, target: torch.Tensor, ignore_index: int,
                        mean: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    """(fp32 scalar, fp32 [1]): the sum of the per-row losses (their mean over the rows not ignored when `mean`), and
    the factor the backward pass scales with (1 / number of rows not ignored, or 1)."""
    _dev(loss_rows)
    if loss_rows.dtype != torch.float32 or not loss_rows.is_contiguous() or target.numel() != loss_rows.numel():
        raise ValueError("softmax_xent_reduce: loss_rows must be contiguous fp32 [rows] and target int64 [rows]")
    out = torch.empty((), dtype=torch.float32, device=loss_rows.device)
    scale = torch.empty(1, dtype=torch.float32, device=loss_rows.device)
    _lib.require_device()
    check(_lib.load().rtp_softmax_xent_reduce(_stream(), loss_rows.data_ptr(), target.data_ptr(), int(ignore_index),
                                              loss_rows.numel(), int(mean), out.data_ptr(), scale.data_ptr()))
    return out, scale


def softmax_xent_bwd(logits: torch.Tensor, target: torch.Tensor, stats: torch.Tensor, dloss: torch.Tensor,
                     out: Optional[torch.Tensor] = None, scale: Optional[torch.Tensor] = None,
                     ignore_index: int = -100) -> torch.Tensor:
    """dlogits = (softmax(logits) - onehot(target)) * dloss[row] (* scale[0]); dloss fp32 [rows] with stride 0 or
    1, or one element for all rows; scale: an fp32 device scalar.  Rows whose target equals `ignore_index` (also one
    inside the class range, such as a padding id) get a zero gradient."""
    _xent_check("softmax_xent_bwd", logits, target)
    rows, cols = logits.shape
    if dloss.dtype != torch.float32 or dloss.numel() not in (1, rows) or dloss.dim() > 1:
        raise ValueError("softmax_xent_bwd: dloss must be fp32 [rows] or a single fp32 element")
    if stats.dtype != torch.float32 or stats.shape != (rows, 2) or not stats.is_contiguous():
        raise ValueError("softmax_xent_bwd: stats must be the contiguous fp32 [rows, 2] of softmax_xent_fwd")
    stride = 0 if (dloss.numel() == 1 or dloss.dim() == 0) else dloss.stride(0)
    if rows > 1 and stride not in (0, 1):
        raise ValueError("softmax_xent_bwd: dloss stride must be 0 or 1")
    if scale is not None and (scale.dtype != torch.float32 or scale.numel() != 1 or scale.device != logits.device):
        raise ValueError("softmax_xent_bwd: scale must be one fp32 element on the logits' device")
    if out is None:
        out = torch.empty(rows, cols, dtype=logits.dtype, device=logits.device)
    elif out.shape != logits.shape or out.dtype != logits.dtype or (cols > 1 and out.stride(1) != 1):
        raise ValueError("softmax_xent_bwd: out must match the logits' shape and dtype")
    _lib.require_device()
    check(_lib.load().rtp_softmax_xent_bwd(_stream(), dtype_code(logits.dtype), logits.data_ptr(),
                                           logits.stride(0) if rows > 1 else cols, rows, cols, target.data_ptr(),
                                           int(ignore_index), stats.data_ptr(), dloss.data_ptr(),
                                           0 if rows <= 1 else stride,
                                           _ptr(scale), out.data_ptr(), out.stride(0) if rows > 1 else cols))
    return out


def sgd_step(master: torch.Tensor, grad: torch.Tensor, shadow: Optional[torch.Tensor], lr: float,
             clip: float = 0.0) -> None:
    _dev(master)
    if master.dtype != torch.float32 or not master.is_contiguous() or not grad.is_contiguous() or \
            grad.numel() != master.numel():
        raise ValueError("sgd_step: master must be contiguous fp32 and grad the same length")
    if shadow is not None and (shadow.dtype != grad.dtype or shadow.numel() != master.numel() or
                               not shadow.is_contiguous()):
        raise ValueError("sgd_step: shadow must match grad dtype and master length")
    _lib.require_device()
    check(_lib.load().rtp_sgd_step(_stream(), dtype_code(grad.dtype), master.data_ptr(), grad.data_ptr(),
                                   _ptr(shadow), master.numel(), lr, clip))


def gate_supported(x2: torch.Tensor, w_rows: torch.Tensor) -> bool:
    """Whether the streaming gate kernels take logits = x2 @ w_rows^T: at most 16 expert rows, model dimension a
    multiple of 16 bytes, 16-byte aligned rows on both sides."""
    if x2.dtype not in (torch.float32, torch.bfloat16) or w_rows.dtype != x2.dtype or x2.dim() != 2 or w_rows.dim() != 2:
        return False
    vec = 16 // x2.element_size()
    ok = all(t.stride(1) == 1 and t.stride(0) % vec == 0 and t.data_ptr() % 16 == 0 for t in (x2, w_rows))
    return ok and bool(_lib.load().rtp_gate_supported(dtype_code(x2.dtype), w_rows.shape[0], x2.shape[1]))


def gate_fwd(x2: torch.Tensor, w_rows: torch.Tensor, logits: torch.Tensor, col0: int) -> None:
    """logits[:, col0 : col0 + E] = x2 @ w_rows^T (fp32 logits, E = w_rows.shape[0] <= 16)."""
    _dev(x2)
    if logits.dtype != torch.float32 or logits.stride(1) != 1 or logits.shape[0] != x2.shape[0] or \
            col0 + w_rows.shape[0] > logits.shape[1]:
        raise ValueError("gate_fwd: logits must be fp32 [S, >= col0 + E]")
    _lib.require_device()
    check(_lib.load().rtp_gate_fwd(_stream(), dtype_code(x2.dtype), x2.data_ptr(), x2.stride(0), w_rows.data_ptr(),
                                   w_rows.stride(0), x2.shape[0], x2.shape[1], w_rows.shape[0],
                                   logits.data_ptr() + 4 * col0, logits.stride(0)))


def gate_dgrad(d_logits: torch.Tensor, col0: int, w_rows: torch.Tensor, dx: torch.Tensor,
               init: Optional[torch.Tensor] = None) -> None:
    """dx = (init +) d_logits[:, col0 : col0 + E] @ w_rows (d_logits fp32; dx in the weights' dtype, fully
    overwritten; `init`: an addend of dx's shape and dtype, e.g. the gradient that reached the same input along
    another path -- added to the rounded product and rounded again, as autograd's own sum of the two would be)."""
    _dev(dx)
    if init is not None and (init.shape != dx.shape or init.dtype != dx.dtype or init.stride(1) != 1):
        raise ValueError("gate_dgrad: init must match dx")
    if d_logits.dtype != torch.float32 or d_logits.stride(1) != 1 or dx.dtype != w_rows.dtype or dx.stride(1) != 1 or \
            d_logits.shape[0] != dx.shape[0] or dx.shape[1] != w_rows.shape[1]:
        raise ValueError("gate_dgrad: need fp32 d_logits [S, E] and dx [S, M] of the weights' dtype")
    _lib.require_device()
    check(_lib.load().rtp_gate_dgrad(_stream(), dtype_code(dx.dtype), d_logits.data_ptr() + 4 * col0, d_logits.stride(0),
                                     w_rows.data_ptr(), w_rows.stride(0), dx.shape[0], dx.shape[1], w_rows.shape[0],
                                     dx.data_ptr(), dx.stride(0), _ptr(init),
                                     init.stride(0) if init is not None else 0))


def gate_wgrad(d_logits: torch.Tensor, col0: int, x2: torch.Tensor, dw_rows: torch.Tensor, accumulate: bool) -> None:
    """dw_rows[E, M] (+)= d_logits[:, col0 : col0 + E]^T @ x2, summed over the tokens in a fixed order."""
    _dev(x2)
    e, m = dw_rows.shape
    if d_logits.dtype != torch.float32 or d_logits.stride(1) != 1 or dw_rows.dtype != x2.dtype or \
            dw_rows.stride(1) != 1 or x2.shape[1] != m or d_logits.shape[0] != x2.shape[0]:
        raise ValueError("gate_wgrad: need fp32 d_logits [S, E], x2 [S, M] and dw_rows [E, M] of x2's dtype")
    lib = _lib.load()
    nbytes = lib.rtp_gate_wgrad_workspace_bytes(x2.shape[0], m, e)
    ws = torch.empty(nbytes // 4, dtype=torch.float32, device=x2.device)
    _lib.require_device()
    check(lib.rtp_gate_wgrad(_stream(), dtype_code(x2.dtype), d_logits.data_ptr() + 4 * col0, d_logits.stride(0),
                             x2.data_ptr(), x2.stride(0), x2.shape[0], m, e, dw_rows.data_ptr(), dw_rows.stride(0),
                             int(accumulate), ws.data_ptr(), nbytes))


def conv_geom(x_shape, kernel_size, stride, padding, dilation) -> "_lib.ConvGeom":
    """Geometry record of a zero-padded 2-D convolution over an NCHW input (output size as torch computes it)."""
    n, c, h, w = (int(v) for v in x_shape)
    (kh, kw), (sh, sw), (ph, pw), (dh, dw) = kernel_size, stride, padding, dilation
    ho = (h + 2 * ph - dh * (kh - 1) - 1) // sh + 1
    wo = (w + 2 * pw - dw * (kw - 1) - 1) // sw + 1
    if ho < 1 or wo < 1:
        raise ValueError(f"convolution kernel {kh}x{kw} (dilation {dh},{dw}) larger than the padded input {h}x{w}")
    return _lib.ConvGeom(n, c, h, w, kh, kw, sh, sw, ph, pw, dh, dw, ho, wo)


def _conv_run(who: str, flat: torch.Tensor, n_s: int, geom, w_off: int, bias_off: Optional[int]):
    """(numel, shards, element size) of a run of shard rows [shards, numel] that holds a [n_s, C, kh, kw] weight at
    w_off and, if bias_off is given, a bias [n_s]."""
    _dev(flat)
    if flat.dim() != 2 or flat.stride(1) != 1 or (flat.shape[0] > 1 and flat.stride(0) != flat.shape[1]):
        raise ValueError(f"{who}: the shards of a run are the rows of a dense [shards, numel] tensor")
    kp = geom.c * geom.kh * geom.kw
    if w_off < 0 or w_off + n_s * kp > flat.shape[1] or (bias_off is not None and bias_off + n_s > flat.shape[1]):
        raise ValueError(f"{who}: weight / bias offsets outside a shard row of {flat.shape[1]} elements")
    return flat.shape[1], flat.shape[0], flat.element_size()


def conv2d_fwd(x: torch.Tensor, geom, flat: torch.Tensor, w_off: int, bias_off: Optional[int], n_s: int,
               y: torch.Tensor, co_first: int) -> None:
    """y[:, co_first : co_first + shards*n_s] (contiguous NCHW `y` with all the layer's channels) = conv2d(x, W_g) + b_g
    for the shards g of the run `flat` [shards, numel]; x in any memory format.  Implicit GEMM: no patch matrix."""
    numel, shards, _ = _conv_run("conv2d_fwd", flat, n_s, geom, w_off, bias_off)
    _dev(x)
    if x.dim() != 4 or tuple(x.shape) != (geom.n, geom.c, geom.h, geom.w) or x.dtype != flat.dtype or \
            y.dtype != flat.dtype or not y.is_contiguous() or y.dim() != 4 or \
            (y.shape[0], y.shape[2], y.shape[3]) != (geom.n, geom.ho, geom.wo) or co_first + shards * n_s > y.shape[1]:
        raise ValueError("conv2d_fwd: x [N,C,H,W] and a contiguous y [N,Co,Ho,Wo] of the weights' dtype")
    _lib.require_device()
    check(_lib.load().rtp_conv2d_fwd(_stream(), dtype_code(x.dtype), x.data_ptr(), *x.stride(), geom, flat.data_ptr(),
                                     numel, shards, w_off, -1 if bias_off is None else bias_off, n_s, y.data_ptr(),
                                     co_first, y.shape[1]))


def conv2d_wgrad(dy: torch.Tensor, x: torch.Tensor, geom, grads: torch.Tensor, w_off: int, bias_off: Optional[int],
                 n_s: int, co_first: int, accumulate: bool) -> None:
    """The gradient rows `grads` [shards, numel] of a run of shards: weight gradients at w_off, bias gradients at
    bias_off (if given), from dy[:, co_first : co_first + shards*n_s] and the layer input x (both in any memory
    format); added to what is there when `accumulate`."""
    numel, shards, _ = _conv_run("conv2d_wgrad", grads, n_s, geom, w_off, bias_off)
    _dev(x)
    _dev(dy)
    if x.dim() != 4 or tuple(x.shape) != (geom.n, geom.c, geom.h, geom.w) or dy.dim() != 4 or \
            (dy.shape[0], dy.shape[2], dy.shape[3]) != (geom.n, geom.ho, geom.wo) or \
            co_first + shards * n_s > dy.shape[1] or x.dtype != grads.dtype or dy.dtype != grads.dtype:
        raise ValueError("conv2d_wgrad: x [N,C,H,W] and dy [N,Co,Ho,Wo] of the gradients' dtype")
    _lib.require_device()
    lib = _lib.load()
    nbytes = lib.rtp_conv2d_wgrad_workspace_bytes(geom, shards, n_s)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
    check(lib.rtp_conv2d_wgrad(_stream(), dtype_code(x.dtype), dy.data_ptr(), *dy.stride(), x.data_ptr(),
                               *x.stride(), geom, grads.data_ptr(), numel, shards, w_off,
                               -1 if bias_off is None else bias_off, n_s, co_first, int(accumulate), ws.data_ptr(),
                               nbytes))


def conv2d_dgrad(dy: torch.Tensor, geom, flat: torch.Tensor, w_off: int, n_s: int, co_first: int, dx: torch.Tensor,
                 addend: Optional[torch.Tensor] = None) -> None:
    """dx [N,C,H,W] (contiguous; the weights' dtype or fp32) = addend + the input gradient through the shards of the
    run `flat`, which own dy's channels co_first .. co_first + shards*n_s - 1."""
    numel, shards, _ = _conv_run("conv2d_dgrad", flat, n_s, geom, w_off, None)
    _dev(dy)
    _dev(dx)
    ok = (torch.float32, flat.dtype)
    if dy.dim() != 4 or (dy.shape[0], dy.shape[2], dy.shape[3]) != (geom.n, geom.ho, geom.wo) or \
            co_first + shards * n_s > dy.shape[1] or dy.dtype != flat.dtype or not dx.is_contiguous() or \
            tuple(dx.shape) != (geom.n, geom.c, geom.h, geom.w) or dx.dtype not in ok or \
            (addend is not None and (addend.shape != dx.shape or not addend.is_contiguous() or addend.dtype not in ok)):
        raise ValueError("conv2d_dgrad: dy [N,Co,Ho,Wo] of the weights' dtype, contiguous dx / addend [N,C,H,W]")
    _lib.require_device()
    check(_lib.load().rtp_conv2d_dgrad(_stream(), dtype_code(dy.dtype), dy.data_ptr(), *dy.stride(), geom,
                                       flat.data_ptr(), numel, shards, w_off, n_s, co_first, dx.data_ptr(),
                                       int(dx.dtype == torch.float32), None if addend is None else addend.data_ptr(),
                                       int(addend is not None and addend.dtype == torch.float32)))


def adam_step(master: torch.Tensor, grad: torch.Tensor, shadow: Optional[torch.Tensor], exp_avg: torch.Tensor,
              exp_avg_sq: torch.Tensor, step, lr: float, betas=(0.9, 0.999), eps: float = 1e-8,
              weight_decay: float = 0.0, clip: float = 0.0) -> None:
    """One torch.optim.Adam update (optionally preceded by clip_grad_value_) of a flat fp32 master buffer and
    its fp32 moments; `shadow` receives the master rounded to the gradient's dtype.  `step` counts from 1: an int,
    or a one-element int64 device tensor that the kernel reads when it runs (for launches recorded into a graph)."""
    _dev(master)
    n = master.numel()
    for name, t in (("master", master), ("exp_avg", exp_avg), ("exp_avg_sq", exp_avg_sq)):
        if t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != n:
            raise ValueError(f"adam_step: {name} must be contiguous fp32 of the master's length")
    if not grad.is_contiguous() or grad.numel() != n:
        raise ValueError("adam_step: grad must be contiguous and of the master's length")
    if shadow is not None and (shadow.dtype != grad.dtype or shadow.numel() != n or not shadow.is_contiguous()):
        raise ValueError("adam_step: shadow must match grad dtype and master length")
    step_dev = None
    if isinstance(step, torch.Tensor):
        if step.dtype != torch.int64 or step.numel() != 1 or step.device != master.device:
            raise ValueError("adam_step: a device step count must be one int64 element on the master's device")
        step_dev, step = step.data_ptr(), 0
    _lib.require_device()
    check(_lib.load().rtp_adam_step(_stream(), dtype_code(grad.dtype), master.data_ptr(), grad.data_ptr(),
                                    _ptr(shadow), exp_avg.data_ptr(), exp_avg_sq.data_ptr(), n, lr, betas[0],
                                    betas[1], eps, weight_decay, int(step), step_dev, clip))


SGD_CHUNK = 16384  # parameters per workgroup of the multi-buffer update


def sgd_chunk_table(items, device) -> Optional[torch.Tensor]:
    """Device table for sgd_step_multi from (master, grad, shadow-or-None) triples of flat tensors, or None when
    some buffer does not allow 16-byte accesses (then update the buffers one by one)."""
    rows = []
    for master, grad, shadow in items:
        n = master.numel()
        ptrs = [master.data_ptr(), grad.data_ptr()] + ([shadow.data_ptr()] if shadow is not None else [])
        if n % 4 or any(p % 16 for p in ptrs) or grad.numel() != n or (shadow is not None and shadow.numel() != n):
            return None
        gs = grad.element_size()
        for off in range(0, n, SGD_CHUNK):
            cnt = min(SGD_CHUNK, n - off)
            rows.append((master.data_ptr() + off * 4, grad.data_ptr() + off * gs,
                         shadow.data_ptr() + off * gs if shadow is not None else 0, cnt))
    if not rows:
        return None
    return _device_table(rows, device)


def adam_chunk_table(items, device) -> Optional[torch.Tensor]:
    """Device table for adam_step_multi from (master, grad, shadow-or-None, exp_avg, exp_avg_sq) tuples of flat
    tensors, or None when some buffer does not allow 16-byte accesses (then update the buffers one by one)."""
    rows = []
    for master, grad, shadow, m, v in items:
        n = master.numel()
        ptrs = [master.data_ptr(), grad.data_ptr(), m.data_ptr(), v.data_ptr()] + \
               ([shadow.data_ptr()] if shadow is not None else [])
        if n % 4 or any(p % 16 for p in ptrs) or any(t.numel() != n for t in (grad, m, v)) or \
                (shadow is not None and shadow.numel() != n):
            return None
        gs = grad.element_size()
        for off in range(0, n, SGD_CHUNK):
            cnt = min(SGD_CHUNK, n - off)
            rows.append((master.data_ptr() + off * 4, grad.data_ptr() + off * gs,
                         shadow.data_ptr() + off * gs if shadow is not None else 0, m.data_ptr() + off * 4,
                         v.data_ptr() + off * 4, cnt))
    if not rows:
        return None
    return _device_table(rows, device)


def adam_step_multi(table: torch.Tensor, dtype: torch.dtype, step, lr: float, betas, eps: float, weight_decay: float,
                    clip: float, total_params: int) -> None:
    """adam_step for every chunk of `table` in one launch; `step` as for adam_step."""
    _dev(table)
    step_dev = None
    if isinstance(step, torch.Tensor):
        if step.dtype != torch.int64 or step.numel() != 1 or step.device != table.device:
            raise ValueError("adam_step_multi: a device step count must be one int64 element on the table's device")
        step_dev, step = step.data_ptr(), 0
    _lib.require_device()
    check(_lib.load().rtp_adam_step_multi(_stream(), dtype_code(dtype), table.data_ptr(), table.shape[0], lr, betas[0],
                                          betas[1], eps, weight_decay, int(step), step_dev, clip, float(total_params)))


def sgd_step_multi(table: torch.Tensor, dtype: torch.dtype, lr: float, clip: float, total_params: int) -> None:
    _dev(table)
    _lib.require_device()
    check(_lib.load().rtp_sgd_step_multi(_stream(), dtype_code(dtype), table.data_ptr(), table.shape[0], lr, clip,
                                         float(total_params)))


def cast(src: torch.Tensor, dst: torch.Tensor) -> None:
    _dev(src)
    _dev(dst)
    if not (src.is_contiguous() and dst.is_contiguous()) or src.numel() != dst.numel():
        raise ValueError("cast: need contiguous tensors of equal length")
    _lib.require_device()
    check(_lib.load().rtp_cast(_stream(), dtype_code(src.dtype), src.data_ptr(), dtype_code(dst.dtype),
                               dst.data_ptr(), src.numel()))


class FusedSgd:
    """What a weight-gradient product needs to apply clip + SGD in its own epilogue: the step's scalars, whether the
    gradient is still to be stored, and the record of what was (or could not be) updated this way."""

    def __init__(self, lr: float, clip: float, keep_grads: bool = False, source=None):
        """`source`: an object whose `lr` / `clip_value` attributes are read at every launch (the optimiser), so that a
        learning-rate schedule reaches the fused epilogues like every other update; without one the two scalars
        given here stay fixed."""
        self._lr, self._clip, self.keep_grads = float(lr), float(clip), bool(keep_grads)
        self._source = source
        self.missed = False

    @property
    def lr(self) -> float:
        return float(self._source.lr) if self._source is not None else self._lr

    @property
    def clip(self) -> float:
        return float(self._source.clip_value) if self._source is not None else self._clip


class ShardSum:
    """Accumulation plan for a result that is summed over the shard steps of a rotation
    (row-parallel outputs, attention out-projections, input gradients).  fp32 results accumulate in
    place; bf16 results accumulate in an fp32 scratch and are rounded once, by the last step."""

    def __init__(self, out: torch.Tensor, steps: int, init: Optional[torch.Tensor] = None):
        """`init`, if given, is an addend of the sum (the first step reads it as its c_in)."""
        self.out = out
        self.steps = steps
        self.init = init
        self.scratch = None
        if out.dtype != torch.float32 and steps > 1:
            self.scratch = torch.empty(out.shape, dtype=torch.float32, device=out.device)

    def target(self, i: int):
        """(c_out, c_in) for step i."""
        if self.scratch is None:
            return self.out, (self.out if i > 0 else self.init)
        if i == self.steps - 1:
            return self.out, self.scratch
        return self.scratch, (self.scratch if i > 0 else self.init)


class Routing:
    """Compact result of top-2 routing for S tokens over E experts with capacity C = 2S/E."""

    __slots__ = ("s", "e", "capacity", "expert", "slot", "keep", "weight", "gates", "slot_token", "l_aux", "counts",
                 "l_aux_typed")


def top2_route(logits: torch.Tensor, noise: torch.Tensor, l_aux_dtype: Optional[torch.dtype] = None) -> Routing:
    """Run the routing kernels on fp32 logits[S,E] and noise[S,E].  l_aux_dtype=torch.bfloat16: the routing also
    leaves `l_aux_typed`, the auxiliary loss in that dtype (what a bf16 layer hands on), from the same kernels."""
    _dev(logits)
    _dev(noise)
    if logits.dtype != torch.float32 or noise.dtype != torch.float32 or logits.dim() != 2 or \
            noise.shape != logits.shape or not (logits.is_contiguous() and noise.is_contiguous()):
        raise ValueError("top2_route: logits and noise must be contiguous fp32 [S,E]")
    s, e = logits.shape
    assert s % e == 0, "num_tokens must be a multiple of num_experts"
    dev = logits.device
    r = Routing()
    r.s, r.e, r.capacity = s, e, 2 * s // e
    r.expert = torch.empty(s, 2, dtype=torch.int32, device=dev)
    r.slot = torch.empty(s, 2, dtype=torch.int32, device=dev)
    r.keep = torch.empty(s, 2, dtype=torch.int32, device=dev)
    r.weight = torch.empty(s, 2, dtype=torch.float32, device=dev)
    r.gates = torch.empty(s, e, dtype=torch.float32, device=dev)
    r.slot_token = torch.empty(2 * s, dtype=torch.int32, device=dev)
    r.l_aux = torch.empty((), dtype=torch.float32, device=dev)
    r.counts = torch.empty(2 * e, dtype=torch.int32, device=dev)
    r.l_aux_typed = torch.empty((), dtype=torch.bfloat16, device=dev) if l_aux_dtype == torch.bfloat16 else None
    _lib.require_device()
    lib = _lib.load()
    nbytes = lib.rtp_top2_route_workspace_bytes(s, e)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    check(lib.rtp_top2_route(_stream(), logits.data_ptr(), noise.data_ptr(), s, e, r.expert.data_ptr(),
                             r.slot.data_ptr(), r.keep.data_ptr(), r.weight.data_ptr(), r.gates.data_ptr(),
                             r.slot_token.data_ptr(), r.l_aux.data_ptr(), r.counts.data_ptr(), ws.data_ptr(), nbytes,
                             _ptr(r.l_aux_typed)))
    return r


def top2_route_bwd(r: Routing, d_weight: Optional[torch.Tensor], d_l_aux: Optional[torch.Tensor]) -> torch.Tensor:
    if d_weight is None:  # only the auxiliary loss was used
        d_weight = torch.zeros(r.s, 2, dtype=torch.float32, device=r.gates.device)
    d_weight = d_weight.contiguous().float()
    d_logits = torch.empty(r.s, r.e, dtype=torch.float32, device=r.gates.device)
    if d_l_aux is not None:
        d_l_aux = d_l_aux.contiguous().float()
    check(_lib.load().rtp_top2_route_bwd(_stream(), r.gates.data_ptr(), r.expert.data_ptr(), r.keep.data_ptr(),
                                         r.counts.data_ptr(), d_weight.data_ptr(), _ptr(d_l_aux), r.s, r.e,
                                         d_logits.data_ptr()))
    return d_logits


def moe_dispatch(x: torch.Tensor, r: Routing, out: torch.Tensor, weight: Optional[torch.Tensor] = None) -> None:
    """out[E*C, M]: row e*C+c = x[token in that slot] (times its combine weight if `weight`), else 0."""
    _dev(x)
    rows, cols, ld_x = _mat(x, "x")
    n_slots, cols_o, ld_o = _mat(out, "out")
    if rows != r.s or cols != cols_o or n_slots != r.e * r.capacity or out.dtype != x.dtype:
        raise ValueError("moe_dispatch: shape mismatch")
    check(_lib.load().rtp_moe_dispatch(_stream(), dtype_code(x.dtype), x.data_ptr(), ld_x, r.slot_token.data_ptr(),
                                       r.expert.data_ptr(), r.slot.data_ptr(), _ptr(weight), n_slots, r.capacity,
                                       cols, out.data_ptr(), ld_o))


def moe_combine(y: torch.Tensor, r: Routing, out: torch.Tensor, weight: Optional[torch.Tensor]) -> None:
    """out[s,:] = sum over the kept choices of token s of weight * y[expert*C + slot, :]."""
    _dev(y)
    n_slots, cols, ld_y = _mat(y, "y")
    rows, cols_o, ld_o = _mat(out, "out")
    if rows != r.s or cols != cols_o or n_slots != r.e * r.capacity or out.dtype != y.dtype:
        raise ValueError("moe_combine: shape mismatch")
    check(_lib.load().rtp_moe_combine(_stream(), dtype_code(y.dtype), y.data_ptr(), ld_y, r.expert.data_ptr(),
                                      r.slot.data_ptr(), r.keep.data_ptr(), _ptr(weight), r.s, r.capacity, cols,
                                      out.data_ptr(), ld_o))


def moe_combine_dweight(dout: torch.Tensor, y: torch.Tensor, r: Routing) -> torch.Tensor:
    _dev(dout)
    rows, cols, ld_d = _mat(dout, "dout")
    n_slots, cols_y, ld_y = _mat(y, "y")
    if rows != r.s or cols != cols_y or dout.dtype != y.dtype:
        raise ValueError("moe_combine_dweight: shape mismatch")
    dw = torch.empty(r.s, 2, dtype=torch.float32, device=dout.device)
    check(_lib.load().rtp_moe_combine_dweight(_stream(), dtype_code(y.dtype), dout.data_ptr(), ld_d, y.data_ptr(),
                                              ld_y, r.expert.data_ptr(), r.slot.data_ptr(), r.keep.data_ptr(), r.s,
                                              r.capacity, cols, dw.data_ptr()))
    return dw
