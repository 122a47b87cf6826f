"""ctypes binding of librtp_hip.so (the C ABI declared in include/rtp_hip.h).

The library is the only compute backend of this package: there is no PyTorch or CPU fallback, and
`load()` raises if the shared object is missing or the device is not gfx950.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
# RTP_HIP_LIB in the environment names another build of the library (same ABI)
LIB_PATH = os.environ.get("RTP_HIP_LIB") or os.path.join(_HERE, "lib", "librtp_hip.so")

RTP_F32 = 0
RTP_BF16 = 1

GEMM_OUT_F32 = 1
GEMM_CIN_F32 = 2
GEMM_RELU = 4
GEMM_STREAM_OUT = 8
GEMM_ROWSUM_ACCUM = 16
GEMM_SGD_SKIP_OUT = 32
ROTATED_BIAS_DONE, ROTATED_SGD_DONE = 1, 2
GATE_WGRAD_STATIC_MAX_BYTES = 8 << 20  # RTP_GATE_WGRAD_STATIC_MAX_BYTES of include/rtp_hip.h


class RtpError(RuntimeError):
    """A call into librtp_hip.so returned a negative status."""


class ConvGeom(C.Structure):
    """rtp_conv_geom of include/rtp_hip.h."""
    _fields_ = [(n, C.c_int64) for n in ("n", "c", "h", "w", "kh", "kw", "sh", "sw", "ph", "pw", "dh", "dw", "ho", "wo")]


class GemmDesc(C.Structure):
    _fields_ = [
        ("a", C.c_void_p), ("b", C.c_void_p), ("c_out", C.c_void_p), ("c_in", C.c_void_p),
        ("bias", C.c_void_p), ("gate", C.c_void_p),
        ("m", C.c_int64), ("n", C.c_int64), ("k", C.c_int64),
        ("lda", C.c_int64), ("ldb", C.c_int64), ("ldc", C.c_int64), ("ld_cin", C.c_int64),
        ("ld_gate", C.c_int64),
        ("batch", C.c_int64), ("zdiv", C.c_int64),
        ("a_so", C.c_int64), ("a_si", C.c_int64), ("b_so", C.c_int64), ("b_si", C.c_int64),
        ("c_so", C.c_int64), ("c_si", C.c_int64), ("cin_so", C.c_int64), ("cin_si", C.c_int64),
        ("gate_so", C.c_int64), ("gate_si", C.c_int64), ("bias_so", C.c_int64), ("bias_si", C.c_int64),
        ("groups", C.c_int64), ("ksegs", C.c_int64),
        ("a_sg", C.c_int64), ("b_sg", C.c_int64), ("c_sg", C.c_int64), ("cin_sg", C.c_int64),
        ("gate_sg", C.c_int64), ("bias_sg", C.c_int64), ("a_sk", C.c_int64), ("b_sk", C.c_int64),
        ("bias_sk", C.c_int64),
        ("alpha", C.c_float), ("flags", C.c_int32), ("a_kcontig", C.c_int32), ("b_kcontig", C.c_int32),
        ("a_rowsum", C.c_void_p), ("rowsum_sg", C.c_int64),
        ("sgd_master", C.c_void_p), ("sgd_weights", C.c_void_p), ("sgd_lr", C.c_float), ("sgd_clip", C.c_float),
        ("xent_mode", C.c_int32), ("xent_reserved", C.c_int32), ("xent_target", C.c_void_p), ("xent_ignore", C.c_int64),
        ("xent_part", C.c_void_p), ("xent_tlogit", C.c_void_p), ("xent_stats", C.c_void_p), ("xent_dloss", C.c_void_p),
        ("xent_scale", C.c_void_p),
    ]


class RotatedLinear(C.Structure):
    """rtp_rotated_linear of include/rtp_hip.h: where the shards of a column-parallel layer live."""
    _fields_ = [("home", C.c_void_p), ("numel", C.c_int64), ("shards", C.c_int64), ("w_off", C.c_int64),
                ("bias_off", C.c_int64), ("n_s", C.c_int64), ("k", C.c_int64)]


class RotatedLinearBwdArgs(C.Structure):
    """rtp_rotated_linear_bwd_args of include/rtp_hip.h."""
    _fields_ = [("dx", C.c_void_p), ("ld_dx", C.c_int64), ("dx_init", C.c_void_p), ("ld_dx_init", C.c_int64),
                ("relu_gate", C.c_void_p), ("ld_relu_gate", C.c_int64), ("dx_flags", C.c_int64), ("grads", C.c_void_p),
                ("accumulate", C.c_int32), ("sgd_skip_grad_store", C.c_int32), ("sgd_master", C.c_void_p),
                ("sgd_weights", C.c_void_p), ("sgd_lr", C.c_float), ("sgd_clip", C.c_float),
                ("colsum_workspace", C.c_void_p), ("colsum_workspace_bytes", C.c_size_t),
                ("done", C.POINTER(C.c_int32))]


class KernelStat(C.Structure):
    _fields_ = [("name", C.c_char * 64), ("launches", C.c_int64), ("total_ms", C.c_double),
                ("flops", C.c_double), ("bytes", C.c_double), ("phase_ms", C.c_double * 4)]


_vp, _i, _i64, _sz, _f = C.c_void_p, C.c_int, C.c_int64, C.c_size_t, C.c_float

# name -> (restype, argtypes); every symbol include/rtp_hip.h declares.
PROTOTYPES = {
    "rtp_last_error": (C.c_char_p, []),
    "rtp_abi_version": (_i, []),
    "rtp_device_check": (_i, [C.c_char_p, _i]),
    "rtp_rotated_linear_fwd": (_i, [_vp, _i, C.POINTER(RotatedLinear), _vp, _i64, _i64, _vp, _i64, _i]),
    "rtp_rotated_linear_bwd": (_i, [_vp, _i, C.POINTER(RotatedLinear), _vp, _i64, _vp, _i64, _i64,
                                    C.POINTER(RotatedLinearBwdArgs)]),
    "rtp_rotated_linear_xent_workspace_bytes": (_sz, [C.POINTER(RotatedLinear), _i64]),
    "rtp_rotated_linear_xent_fwd": (_i, [_vp, _i, C.POINTER(RotatedLinear), _vp, _i64, _i64, _vp, _i64, _vp, _vp, _vp, _sz]),
    "rtp_rotated_linear_xent_bwd": (_i, [_vp, _i, C.POINTER(RotatedLinear), _vp, _i64, _i64, _vp, _i64, _vp, _vp, _vp, _vp,
                                         _i64]),
    "rtp_softmax_xent_combine": (_i, [_vp, _vp, _i64, _vp, _vp, _i64, _i64, _vp, _vp]),
    "rtp_gemm": (_i, [_vp, _i, C.POINTER(GemmDesc)]),
    "rtp_gemm_warm_next": (_i, [_vp, _sz]),
    "rtp_probe_mfma_rate": (_i, [_vp, _i, _i, C.POINTER(C.c_double)]),
    "rtp_gemm_rowsum_fused": (_i, [_i, C.POINTER(GemmDesc)]),
    "rtp_gemm_sgd_fused": (_i, [_i, C.POINTER(GemmDesc)]),
    "rtp_gemm_desc_size": (_sz, []),
    "rtp_colsum_workspace_bytes": (_sz, [_i64, _i64]),
    "rtp_colsum": (_i, [_vp, _i, _vp, _i64, _i64, _i64, _vp, _i, _i, _i64, _i64, _vp, _sz]),
    "rtp_ring_create": (_i, [C.POINTER(_vp)]),
    "rtp_ring_destroy": (_i, [_vp]),
    "rtp_ring_fence": (_i, [_vp, _vp]),
    "rtp_ring_prefetch": (_i, [_vp, _vp, _i, _vp, _vp, _sz]),
    "rtp_cache_warm": (_i, [_vp, _vp, _sz, _i]),
    "rtp_ring_acquire": (_i, [_vp, _vp, _i]),
    "rtp_ring_release": (_i, [_vp, _vp, _i]),
    "rtp_shard_copy_async": (_i, [_vp, _vp, _vp, _sz]),
    "rtp_zero_async": (_i, [_vp, _vp, _sz]),
    "rtp_embedding_gather": (_i, [_vp, _i, _vp, _i64, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _i64, _i64, _i64]),
    "rtp_embedding_gather_scale_pos": (_i, [_vp, _i, _vp, _i64, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _i64, _i64,
                                            _i64, _f, _vp, _i64, _i64, _i64]),
    "rtp_embedding_scatter_workspace_bytes": (_sz, [_i64]),
    "rtp_embedding_sort_ids": (_i, [_vp, _vp, _i64, _vp, _sz]),
    "rtp_embedding_scatter_add_det": (_i, [_vp, _i, _vp, _i64, _i64, _vp, _vp, _i64, _i, _i64, _i64, _i64,
                                           _i64, _i, _i, _i64, _i64, _i64]),
    "rtp_embedding_scatter_add_scaled": (_i, [_vp, _i, _vp, _i64, _i64, _vp, _vp, _i64, _i, _i64, _i64, _i64,
                                              _i64, _i, _i, _i64, _i64, _i64, _f]),
    "rtp_embedding_scatter_add_sgd": (_i, [_vp, _i, _vp, _i64, _i64, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i, _i64,
                                           _i64, _i64, _f, _vp, _vp, _f, _f, _i]),
    "rtp_embedding_backward_supported": (_i, [_i64]),
    "rtp_embedding_backward": (_i, [_vp, _i, _vp, _i64, _i64, _vp, _vp, _i64, _i, _i64, _i64, _i64, _i64, _i, _i, _i64,
                                    _i64, _i64, _f, _vp, _vp, _f, _f, _i]),
    "rtp_softmax_fwd": (_i, [_vp, _i, _vp, _vp, _vp, _i64, _i64, _i, _f, _i64, _i64, _i64, _vp]),
    "rtp_softmax_fwd_masks": (_i, [_vp, _i, _vp, _vp, _i64, _vp, _i64, _i64, _i, _f, _i64, _i64, _i64, _vp, _vp, _vp]),
    "rtp_softmax_bwd": (_i, [_vp, _i, _vp, _vp, _vp, _f, _i64, _i64, _i64, _vp]),
    "rtp_attn_supported": (_i, [_i, _i64, _i64]),
    "rtp_attn_fwd": (_i, [_vp, _i, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _i,
                          _f, _i64, _i64, _i64, _i64, _i64]),
    "rtp_attn_bwd": (_i, [_vp, _i, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _vp,
                          _f, _i64, _i64, _i64, _i64, _i64]),
    "rtp_attn_flash_supported": (_i, [_i, _i64, _i64]),
    "rtp_attn_flash_fwd": (_i, [_vp, _i, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _vp,
                                _i, _f, _i64, _i64, _i64, _i64, _i64]),
    "rtp_attn_flash_bwd": (_i, [_vp, _i, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _i64, _i64, _i64, _i64, _vp,
                                _vp, _vp, _vp, _vp, _vp, _vp, _i, _f, _i64, _i64, _i64, _i64, _i64]),
    "rtp_layernorm_supported": (_i, [_i, _i64]),
    "rtp_add_layernorm_fwd": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _f, _i64, _i64, _vp, _vp, _vp, _vp]),
    "rtp_layernorm_bwd_workspace_bytes": (_sz, [_i64, _i64]),
    "rtp_layernorm_bwd_blocks": (_i64, [_i64]),
    "rtp_layernorm_bwd_finalize": (_i, [_vp, _i, _vp, _i64, _i64]),
    "rtp_layernorm_bwd": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _vp, _vp, _vp, _vp, _sz]),
    "rtp_softmax_xent_fwd": (_i, [_vp, _i, _vp, _i64, _i64, _i64, _vp, _i64, _vp, _vp]),
    "rtp_softmax_xent_reduce": (_i, [_vp, _vp, _vp, _i64, _i64, _i, _vp, _vp]),
    "rtp_softmax_xent_bwd": (_i, [_vp, _i, _vp, _i64, _i64, _i64, _vp, _i64, _vp, _vp, _i64, _vp, _vp, _i64]),
    "rtp_top2_route_workspace_bytes": (_sz, [_i64, _i64]),
    "rtp_top2_route": (_i, [_vp, _vp, _vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "rtp_top2_route_bwd": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _vp]),
    "rtp_moe_dispatch": (_i, [_vp, _i, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _i64]),
    "rtp_moe_combine": (_i, [_vp, _i, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _i64]),
    "rtp_moe_combine_dweight": (_i, [_vp, _i, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "rtp_gate_supported": (_i, [_i, _i64, _i64]),
    "rtp_gate_fwd": (_i, [_vp, _i, _vp, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _i64]),
    "rtp_gate_dgrad": (_i, [_vp, _i, _vp, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _i64, _vp, _i64]),
    "rtp_gate_wgrad_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "rtp_gate_wgrad": (_i, [_vp, _i, _vp, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _i64, _i, _vp, _sz]),
    "rtp_gate_wgrad_static": (_i, [_vp, _i, _vp, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _i64, _i]),
    "rtp_conv2d_fwd": (_i, [_vp, _i, _vp, _i64, _i64, _i64, _i64, C.POINTER(ConvGeom), _vp, _i64, _i64, _i64, _i64, _i64,
                            _vp, _i64, _i64]),
    "rtp_conv2d_wgrad": (_i, [_vp, _i, _vp, _i64, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64, C.POINTER(ConvGeom), _vp,
                              _i64, _i64, _i64, _i64, _i64, _i64, _i, _vp, _sz]),
    "rtp_conv2d_wgrad_workspace_bytes": (_sz, [C.POINTER(ConvGeom), _i64, _i64]),
    "rtp_conv2d_dgrad": (_i, [_vp, _i, _vp, _i64, _i64, _i64, _i64, C.POINTER(ConvGeom), _vp, _i64, _i64, _i64, _i64, _i64,
                              _vp, _i, _vp, _i]),
    "rtp_sgd_step": (_i, [_vp, _i, _vp, _vp, _vp, _i64, _f, _f]),
    "rtp_adam_step": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i64, C.c_double, C.c_double, C.c_double, C.c_double,
                           C.c_double, _i64, _vp, C.c_double]),
    "rtp_adam_step_multi": (_i, [_vp, _i, _vp, _i64, C.c_double, C.c_double, C.c_double, C.c_double, C.c_double, _i64, _vp,
                                 C.c_double, C.c_double]),
    "rtp_sgd_step_multi": (_i, [_vp, _i, _vp, _i64, _f, _f, C.c_double]),
    "rtp_cast": (_i, [_vp, _i, _vp, _i, _vp, _i64]),
    "rtp_profile_enable": (_i, [_i]),
    "rtp_profile_collect": (_i, [C.POINTER(KernelStat), _i, C.POINTER(_i)]),
    "rtp_profile_reset_stamps": (_i, [_vp]),
    "rtp_profile_read": (_i, [C.POINTER(KernelStat), _i, C.POINTER(_i)]),
}

_lib: Optional[C.CDLL] = None
_device_checked = False


def load() -> C.CDLL:
    """dlopen librtp_hip.so (once) and bind every prototype.  Touches no GPU."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RtpError(
                f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
                "(or __graft_entry__.build()); there is no fallback backend")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        if lib.rtp_gemm_desc_size() != C.sizeof(GemmDesc):
            raise RtpError("GemmDesc layout differs from the rtp_gemm_desc this library was built with")
        _lib = lib
    return _lib


def last_error() -> str:
    return load().rtp_last_error().decode("utf-8", "replace")


def check(rc: int) -> None:
    if rc != 0:
        raise RtpError(f"librtp_hip status {rc}: {last_error()}")


def require_device() -> None:
    """Raise unless the current HIP device is gfx950 (checked once per process)."""
    global _device_checked
    if not _device_checked:
        buf = C.create_string_buffer(64)
        check(load().rtp_device_check(buf, 64))
        _device_checked = True


def profile_enable(on) -> None:
    """False / 0: off; True / 1: HIP events around every launch; 2: device time stamps in the GEMM kernels (the mode
    that works for launches recorded into a HIP graph)."""
    check(load().rtp_profile_enable(int(on)))


def profile_reset_stamps(stream: int) -> None:
    check(load().rtp_profile_reset_stamps(stream))


def profile_collect(clear: bool = True):
    """{kernel variant: {launches, total_ms, flops, bytes}} since profiling was enabled; clears the records unless
    clear=False (events recorded into a captured graph stay valid for its later replays)."""
    buf = (KernelStat * 64)()
    n = C.c_int(0)
    lib = load()
    check((lib.rtp_profile_collect if clear else lib.rtp_profile_read)(buf, 64, C.byref(n)))
    return {buf[i].name.decode(): {"launches": buf[i].launches, "total_ms": buf[i].total_ms, "flops": buf[i].flops,
                                   "bytes": buf[i].bytes, "phase_ms": list(buf[i].phase_ms)} for i in range(n.value)}
