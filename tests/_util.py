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


#: by how much a gradient that misses BF16_TOL may exceed the error that torch's own bf16 autograd makes on
#: the same tensor (noise of the same kind and size on both sides: the factor absorbs its scatter; the
#: largest ratio seen over the tracked sweep is 1.8)
REF_BF16_SLACK = 2.0


def check_gradients(named, ref_named, run_in_bf16, what="", log=None):
    """Every parameter gradient (``named[name].main_grad``) against the fp32 oracle's (``ref_named``):
    max relative error per tensor within BF16_TOL.  A tensor that misses it must be no further from the
    fp32 result than REF_BF16_SLACK x the reference's own arithmetic is: ``run_in_bf16()`` runs the same
    torch model in bf16 through torch autograd on the CPU and returns its named parameters (it is only
    called if some tensor needs it).  Such tensors are the ones whose gradient is a small difference of
    large terms in any bf16 arithmetic: query / key projections under nearly uniform attention, a key bias
    (no gradient at all in exact arithmetic), sums over all tokens that largely cancel.
    Returns (worst error within tolerance, {name: (error, reference error)} of the tensors that needed the
    clause)."""
    worst, missed = 0.0, {}
    for name, rp in ref_named.items():
        if rp.grad is None:
            assert getattr(named[name], "main_grad", None) is None, name
            continue
        err = max_rel(named[name].main_grad, rp.grad)
        if err <= BF16_TOL:
            worst = max(worst, err)
        else:
            missed[name] = err
    clause = {}
    if missed:
        ref16_named = run_in_bf16()
        assert ref16_named is not None, f"{what}: gradients beyond {BF16_TOL}: {missed}"
        for name, err in missed.items():
            ref_err = max_rel(ref16_named[name].grad.float(), ref_named[name].grad)
            if log is not None:
                log(f"  {name}: {err:.3e} here, {ref_err:.3e} in torch's own bf16 autograd")
            assert err <= REF_BF16_SLACK * ref_err, (
                f"{what}: gradient of {name} is {err:.3e} off the fp32 oracle: beyond {BF16_TOL} and beyond "
                f"{REF_BF16_SLACK} x the {ref_err:.3e} of torch's own bf16 autograd on the same tensor")
            clause[name] = (err, ref_err)
    return worst, clause
