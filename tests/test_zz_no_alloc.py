"""The allocation-free column sum (``pp_colsum_bf16_noalloc``) against ``pp_colsum_bf16``.

The entry point keeps its partial sums in an array the library holds on the GPU instead of a
caller-provided workspace; its results must be bit-identical to the workspace form, also on a second
call with a smaller input (the array then still holds the first call's partial sums) and after the
other tests of the suite have used the GPU.
"""
import ctypes as C

import pytest
import torch

from pippy_amd import _native as N

pytestmark = pytest.mark.gpu


def _colsum_ws(dY, out_dtype):
    M, Nn = dY.shape
    out = torch.empty(Nn, dtype=out_dtype, device=dY.device)
    ws = torch.empty(max(((M + 127) // 128) * Nn, 1), dtype=torch.float32, device=dY.device)
    N.colsum(dY, out, ws)
    return out


def _colsum_noalloc(dY, out_dtype):
    M, Nn = dY.shape
    out = torch.empty(Nn, dtype=out_dtype, device=dY.device)
    rc = N.lib().pp_colsum_bf16_noalloc(dY.data_ptr(), M, Nn, dY.stride(0), out.data_ptr(),
                                        N.PP_F32 if out_dtype == torch.float32 else N.PP_BF16,
                                        N.current_stream())
    N.check(rc, "pp_colsum_bf16_noalloc")
    return out


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_noalloc_colsum_matches_workspace_form_on_two_calls(out_dtype):
    torch.manual_seed(7)
    big = torch.randn(4096, 3072, device="cuda").to(torch.bfloat16)
    small = torch.randn(1000, 768, device="cuda").to(torch.bfloat16)  # ragged last row block
    for dY in (big, small):
        ref = _colsum_ws(dY, out_dtype)
        got = _colsum_noalloc(dY, out_dtype)
        torch.cuda.synchronize()
        assert torch.equal(got, ref)
    # a strided view (leading dimension larger than the width), smaller again
    view = big[:300, 256:512]
    assert torch.equal(_colsum_noalloc(view, out_dtype), _colsum_ws(view, out_dtype))
    # against the definition: an ordered fp32 sum stays within rounding of the fp64 column sums
    exact = small.double().sum(0)
    got = _colsum_noalloc(small, torch.float32).double()
    assert (got - exact).abs().max() <= 1e-5 * small.double().abs().sum(0).max()


def test_noalloc_colsum_rejects_what_does_not_fit():
    limit = N.PP_COLSUM_NOALLOC_MAX_FLOATS
    Nn = 8192
    M = (limit // Nn + 1) * 128  # one row block too many
    dY = torch.zeros(M, Nn, dtype=torch.bfloat16, device="cuda")
    out = torch.empty(Nn, dtype=torch.bfloat16, device="cuda")
    rc = N.lib().pp_colsum_bf16_noalloc(dY.data_ptr(), M, Nn, Nn, out.data_ptr(), N.PP_BF16, N.current_stream())
    assert rc == N.PP_ERR_UNSUPPORTED
    assert b"exceed" in N.lib().pp_last_error()
    # the largest problem that fits still runs
    M_ok = (limit // Nn) * 128
    ok = dY[:M_ok]
    assert torch.equal(_colsum_noalloc(ok, torch.bfloat16), _colsum_ws(ok, torch.bfloat16))


def test_noalloc_colsum_allocates_nothing_on_a_warm_call():
    """What the entry point is for: after the first call on a device (which looks up the address of the
    library's array), a call leaves the device's free memory and torch's allocator untouched."""
    dY = torch.randn(2048, 1024, device="cuda").to(torch.bfloat16)
    out = torch.empty(1024, dtype=torch.bfloat16, device="cuda")

    def call():
        N.check(N.lib().pp_colsum_bf16_noalloc(dY.data_ptr(), 2048, 1024, 1024, out.data_ptr(), N.PP_BF16,
                                               N.current_stream()), "pp_colsum_bf16_noalloc")

    call()                                   # warm: the per-device set-up happens here
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    held0, reserved0 = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    for _ in range(3):
        call()
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert torch.cuda.memory_allocated() == held0 and torch.cuda.memory_reserved() == reserved0
    assert free1 == free0
