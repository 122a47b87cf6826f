"""rtp_gate_wgrad_static -- the gate weight gradient with the partial sums in a buffer built into the library, for
callers that cannot allocate -- against rtp_gate_wgrad (caller's workspace) through the C ABI: bit-identical results on
two calls in a row, the second with a smaller input (the buffer keeps the first call's contents), then the size limit."""
import ctypes as C

import pytest
import torch

from gpu_util import DEV

pytestmark = pytest.mark.gpu


def _both(lib, dtype, S, M, E, seed, accumulate):
    from rtp_amd import _lib
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(S, M, generator=gen).to(dtype).to(DEV)
    dl = torch.randn(S, E, generator=gen).to(DEV)
    base = (torch.randn(E, M, generator=gen) * 0.5).to(dtype).to(DEV)
    code = _lib.RTP_F32 if dtype == torch.float32 else _lib.RTP_BF16
    stream = torch.cuda.current_stream().cuda_stream
    nbytes = lib.rtp_gate_wgrad_workspace_bytes(S, M, E)
    ws = torch.empty(nbytes // 4, dtype=torch.float32, device=DEV)
    want = base.clone()
    _lib.check(lib.rtp_gate_wgrad(stream, code, dl.data_ptr(), dl.stride(0), x.data_ptr(), x.stride(0), S, M, E,
                                  want.data_ptr(), want.stride(0), int(accumulate), ws.data_ptr(), nbytes))
    got = base.clone()
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    _lib.check(lib.rtp_gate_wgrad_static(stream, code, dl.data_ptr(), dl.stride(0), x.data_ptr(), x.stride(0), S, M, E,
                                         got.data_ptr(), got.stride(0), int(accumulate)))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    ref = dl.double().T @ x.double() + (base.double() if accumulate else 0)
    assert (got.double() - ref).abs().max() <= (1e-5 if dtype == torch.float32 else 2e-2) * ref.abs().max()
    assert torch.equal(got, want), f"S={S} M={M} E={E} {dtype}: differs from rtp_gate_wgrad"


def test_gate_wgrad_static_matches_workspace_entry_point_twice():
    from rtp_amd import _lib
    _lib.require_device()
    lib = _lib.load()
    # first call fills 64 * 8 * 2048 * 4 B = 4 MiB of the built-in buffer; the second, smaller one must not see it
    _both(lib, torch.bfloat16, 4096, 2048, 8, 1, False)
    _both(lib, torch.bfloat16, 1000, 512, 3, 2, True)
    _both(lib, torch.float32, 777, 64, 16, 3, False)
    _both(lib, torch.float32, 5, 4, 1, 4, True)


def test_gate_wgrad_static_refuses_sizes_beyond_the_buffer():
    from rtp_amd import _lib
    _lib.require_device()
    lib = _lib.load()
    S, M, E = 16384, 2048, 16  # 256 row blocks * 16 * 2048 * 4 B = 32 MiB > 8 MiB
    assert lib.rtp_gate_wgrad_workspace_bytes(S, M, E) > _lib.GATE_WGRAD_STATIC_MAX_BYTES
    x = torch.zeros(S, M, dtype=torch.bfloat16, device=DEV)
    dl = torch.zeros(S, E, device=DEV)
    dw = torch.full((E, M), 3.0, dtype=torch.bfloat16, device=DEV)
    rc = lib.rtp_gate_wgrad_static(torch.cuda.current_stream().cuda_stream, _lib.RTP_BF16, dl.data_ptr(), dl.stride(0),
                                   x.data_ptr(), x.stride(0), S, M, E, dw.data_ptr(), dw.stride(0), 0)
    assert rc < 0 and "exceed" in _lib.last_error()
    torch.cuda.synchronize()
    assert bool((dw == 3.0).all())  # nothing was launched
