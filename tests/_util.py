"""Shared helpers for the parity tests."""
import torch

# bf16 results are compared with an fp32 reference by the largest absolute deviation relative to
# the largest reference magnitude of the tensor ("max relative error per tensor").
BF16_TOL = 2e-2
F32_TOL = 1e-5


def max_rel(a: torch.Tensor, ref: torch.Tensor) -> float:
    a = a.detach().double().cpu()
    ref = ref.detach().double().cpu()
    assert a.shape == ref.shape, (a.shape, ref.shape)
    denom = ref.abs().max().item()
    if denom == 0.0:
        return a.abs().max().item()
    return (a - ref).abs().max().item() / denom


def assert_close_rel(a, ref, tol, what=""):
    err = max_rel(a, ref)
    assert err <= tol, f"{what}: max relative error {err:.3e} > {tol:.1e}"
    return err
