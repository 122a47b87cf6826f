"""The C-ABI library loads without a GPU and exports exactly the symbols include/rtp_hip.h declares;
the ctypes prototypes cover the same set.  No compute call is made."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "rtp_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rtp_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_entry_points():
    names = _declared()
    assert "rtp_gemm" in names and "rtp_ring_prefetch" in names and "rtp_embedding_scatter_add_det" in names
    assert len(names) >= 25


def test_library_exports_every_declared_symbol():
    from rtp_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("librtp_hip.so not built (run __graft_entry__.build())")
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared():
        assert hasattr(lib, name), f"{name} declared in rtp_hip.h but not exported"


def test_ctypes_prototypes_cover_the_header():
    from rtp_amd import _lib
    assert sorted(_lib.PROTOTYPES) == _declared()


def test_loader_binds_and_reports_version():
    from rtp_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("librtp_hip.so not built")
    lib = _lib.load()
    assert lib.rtp_abi_version() == 5
    assert isinstance(_lib.last_error(), str)


def test_gemm_desc_matches_c_layout():
    from rtp_amd import _lib
    # 6 pointers + 33 int64 + float + 3 int32, the row-sum pointer and its group stride, the fused update (two
    # pointers and two floats), then the cross-entropy epilogues (two int32, a pointer, an int64, five pointers)
    assert ctypes.sizeof(_lib.GemmDesc) == 6 * 8 + 33 * 8 + 4 + 3 * 4 + 8 + 8 + (8 + 8 + 4 + 4) + (2 * 4 + 8 + 8 + 5 * 8)
    if os.path.exists(_lib.LIB_PATH):
        assert _lib.load().rtp_gemm_desc_size() == ctypes.sizeof(_lib.GemmDesc)


def test_ops_refuse_cpu_tensors():
    """There is no CPU fallback: a CPU tensor is an error, not a slow path."""
    import torch
    from rtp_amd import _lib, ops
    with pytest.raises(_lib.RtpError):
        ops.linear_fwd(torch.zeros(2, 2), torch.zeros(2, 2), torch.zeros(2, 2))
    with pytest.raises(_lib.RtpError):
        ops.embedding_gather(torch.zeros(2, 2), torch.zeros(2, dtype=torch.long), torch.zeros(2, 2))


def test_integration_stub_struct_matches_the_library():
    """The ctypes GemmDesc that the integration notes at the repository root print for a maintainer to paste has the
    layout of rtp_gemm_desc: same size as the library reports and the same field names, order and offsets as the
    package's own binding."""
    from rtp_amd import _lib
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    m = re.search(r"^class GemmDesc\(C\.Structure\):.*?(?=^assert _lib\.rtp_gemm_desc_size)", text, flags=re.S | re.M)
    assert m, "the integration notes no longer hold the GemmDesc stub"
    scope = {"C": ctypes}
    exec(m.group(0), scope)
    stub = scope["GemmDesc"]
    assert ctypes.sizeof(stub) == ctypes.sizeof(_lib.GemmDesc)
    mine = [(n, getattr(_lib.GemmDesc, n).offset, getattr(_lib.GemmDesc, n).size) for n, _ in _lib.GemmDesc._fields_]
    theirs = [(n, getattr(stub, n).offset, getattr(stub, n).size) for n, _ in stub._fields_]
    assert mine == theirs
    if os.path.exists(_lib.LIB_PATH):
        assert _lib.load().rtp_gemm_desc_size() == ctypes.sizeof(stub)
