"""Helpers shared by the GPU parity tests."""
import torch

DEV = "cuda:0"


def rel_err(a: torch.Tensor, b: torch.Tensor) -> float:
    """max |a-b| / max |b| : error relative to the infinity norm of the oracle's result."""
    a = a.detach().double().cpu()
    b = b.detach().double().cpu()
    denom = b.abs().max().item()
    return (a - b).abs().max().item() / (denom if denom > 0 else 1.0)


# north-star tolerances: 1e-5 relative in fp32, 2e-2 in bf16
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


def assert_close(a, b, dtype, what=""):
    err = rel_err(a, b)
    assert err <= TOL[dtype], f"{what}: relative error {err:.3e} > {TOL[dtype]:.0e}"
