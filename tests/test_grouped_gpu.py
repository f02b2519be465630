"""Grouped GEMM launch: several independent problems in one grid must equal separate launches."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.mark.parametrize("fused", [False, True])
def test_grouped_weight_gradient_gemms_equal_single_launches(fused):
    from pippy_amd import _native as N
    N.lib()
    torch.manual_seed(0)
    T = 512
    shapes = [(2304, 768), (768, 768), (3072, 768), (768, 3072), (1024, 256), (8, 8)] * 4  # 24 > one group
    problems, singles = [], []
    for out_f, in_f in shapes:
        dY = torch.randn(T, out_f, device=DEV).to(torch.bfloat16)
        X = torch.randn(T, in_f, device=DEV).to(torch.bfloat16)
        if fused:
            Cg = torch.randn(out_f, in_f, device=DEV)
            Cs = Cg.clone()
            kw = dict(a_trans=True, b_trans=True, epilogue=N.EPI_ACCUM_F32, beta=1)
        else:
            Cg = torch.empty(out_f, in_f, device=DEV, dtype=torch.bfloat16)
            Cs = torch.empty_like(Cg)
            kw = dict(a_trans=True, b_trans=True)
        problems.append((dY, X, Cg, kw))
        singles.append((dY, X, Cs, kw))
    N.gemm_bf16_grouped(problems)
    for dY, X, Cs, kw in singles:
        N.gemm_bf16(dY, X, Cs, **kw)
    torch.cuda.synchronize()
    for (_, _, Cg, _), (_, _, Cs, _) in zip(problems, singles):
        assert torch.equal(Cg, Cs)


def test_grouped_rejects_mixed_configurations():
    from pippy_amd import _native as N
    A = torch.zeros(16, 8, device=DEV, dtype=torch.bfloat16)
    C = torch.zeros(16, 16, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="differs"):
        N.gemm_bf16_grouped([(A, A, C, {}), (A, A, C, dict(epilogue=N.EPI_BIAS_RELU))])
