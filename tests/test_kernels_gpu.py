"""Parity of each HIP kernel, called through the C ABI, against the CPU oracle.

Byte-moving and accumulate kernels must be bit-exact; bf16 arithmetic kernels must stay within
2e-2 max relative error per tensor of the fp32 oracle; fp32 kernels within 1e-5.
"""
import math

import pytest
import torch

from _util import BF16_TOL, F32_TOL, assert_close_rel, max_rel
from oracle import ops as O

pytestmark = pytest.mark.gpu

DEV = "cuda"


def native():
    from pippy_amd import _native
    _native.lib()
    return _native


def note(msg):
    print(msg, flush=True)


# ---- split / merge -------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.uint8, torch.bfloat16, torch.float32, torch.int64])
@pytest.mark.parametrize("shape,dim,n", [
    ((256, 512), 0, 4), ((7, 33, 5), 1, 4), ((3, 10, 17), 2, 3), ((64, 512), 0, 8),
    ((5, 9), 1, 9), ((2, 1024, 50), 1, 8), ((129,), 0, 4),
])
def test_split_merge_bit_exact(dtype, shape, dim, n):
    N = native()
    torch.manual_seed(0)
    if dtype.is_floating_point:
        x = torch.randn(shape, device=DEV).to(dtype)
    else:
        x = torch.randint(0, 127, shape, device=DEV).to(dtype)
    ref = [c.contiguous() for c in torch.tensor_split(x, n, dim)]
    outs = [torch.empty_like(c) for c in ref]
    N.split_copy(x, outs, dim)
    for i, (a, b) in enumerate(zip(outs, ref)):
        assert torch.equal(a, b), f"split chunk {i}"
    merged = torch.empty_like(x)
    N.merge_copy(merged, outs, dim)
    assert torch.equal(merged, x)
    assert torch.equal(merged, torch.cat(ref, dim))


def test_merge_uneven_and_strided_rows():
    N = native()
    torch.manual_seed(1)
    # concatenation of chunks with arbitrary sizes along dim 1
    chunks = [torch.randn(4, d, 6, device=DEV, dtype=torch.bfloat16) for d in (1, 5, 2, 9)]
    ref = torch.cat(chunks, 1)
    out = torch.empty_like(ref)
    N.merge_copy(out, chunks, 1)
    assert torch.equal(out, ref)
    # rows with a padded source stride and an odd row length (vocabulary-like)
    V, ld, rows = 1001, 1008, 37
    src = torch.randn(rows, ld, device=DEV).to(torch.bfloat16)
    dst = torch.empty(rows, V, device=DEV, dtype=torch.bfloat16)
    N.copy_rows([(src.data_ptr(), dst.data_ptr(), rows, V * 2, ld * 2, V * 2)])
    assert torch.equal(dst, src[:, :V])


def test_strided_copy_nd():
    N = native()
    x = torch.arange(2 * 3 * 4 * 5, device=DEV, dtype=torch.float32).reshape(2, 3, 4, 5)
    v = x.permute(2, 0, 3, 1)[1:, :, ::2]
    out = torch.empty(v.shape, device=DEV, dtype=v.dtype)
    N.strided_copy_nd(out, v)
    assert torch.equal(out, v.contiguous())


def test_merge_large_logits_shape():
    """Full-size merge of config 3's logits is checked by a round trip (split then merge)."""
    N = native()
    x = torch.randn(8, 1024, 50257, device=DEV, dtype=torch.bfloat16)  # 0.82 GB
    outs = [torch.empty(2, 1024, 50257, device=DEV, dtype=torch.bfloat16) for _ in range(4)]
    N.split_copy(x, outs, 0)
    back = torch.empty_like(x)
    N.merge_copy(back, outs, 0)
    assert torch.equal(back, x)
    assert torch.equal(outs[3], x[6:8])


# ---- gradient accumulation -------------------------------------------------------------------
@pytest.mark.parametrize("n", [1, 7, 8, 4096 + 3, 768 * 3072, 21_300_000 + 5])
@pytest.mark.parametrize("gdtype", [torch.bfloat16, torch.float32])
def test_grad_accum_bit_exact(n, gdtype):
    N = native()
    torch.manual_seed(n % 97)
    M = 4
    gs = [(torch.randn(n, device=DEV) * (10.0 ** (m - 2))).to(gdtype) for m in range(M)]
    acc = torch.full((n,), float("nan"), device=DEV, dtype=torch.float32)
    for m, g in enumerate(gs):
        N.grad_accum(acc, g, init=(m == 0))
    ref = gs[0].float().clone()
    for g in gs[1:]:
        ref.add_(g.float())
    assert torch.equal(acc, ref)
    # the same on the CPU: the oracle's sequential fp32 adds
    ref_cpu = gs[0].float().cpu().clone()
    for g in gs[1:]:
        ref_cpu.add_(g.float().cpu())
    assert torch.equal(acc.cpu(), ref_cpu)


def test_grad_accum_init_keeps_negative_zero():
    N = native()
    g = torch.tensor([-0.0, 0.0, 1.5, -2.0] * 4, device=DEV, dtype=torch.bfloat16)
    acc = torch.empty(16, device=DEV, dtype=torch.float32)
    N.grad_accum(acc, g, init=True)
    assert torch.equal(acc.view(torch.int32), g.float().view(torch.int32))


def test_fill_bytes():
    N = native()
    t = torch.full((1000003,), 7, device=DEV, dtype=torch.uint8)
    N.fill_bytes(t[3:], 0)
    assert int(t[:3].sum()) == 21 and int(t[3:].sum()) == 0


# ---- GEMM ----------------------------------------------------------------------------------------
def _gemm_ref(A, B, a_trans, b_trans):
    a = A.float().cpu()
    b = B.float().cpu()
    a = a.t() if a_trans else a
    b = b.t() if b_trans else b
    return a @ b.t()


@pytest.mark.parametrize("a_trans,b_trans", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("M,N,K", [(128, 128, 64), (256, 384, 768), (200, 136, 72), (4096, 768, 768),
                                   (1000, 1001, 264), (64, 8, 8), (4088, 2296, 72)])
def test_gemm_bf16_layouts(a_trans, b_trans, M, N, K):
    Nn = native()
    if a_trans and M % 8:
        pytest.skip("transposed A needs M % 8 == 0")
    if b_trans and N % 8:
        pytest.skip("transposed B needs N % 8 == 0")
    torch.manual_seed(M + N + K)
    A = torch.randn((K, M) if a_trans else (M, K), device=DEV).to(torch.bfloat16)
    B = torch.randn((K, N) if b_trans else (N, K), device=DEV).to(torch.bfloat16)
    ldc = (N + 3) // 4 * 4
    Cbuf = torch.full((M, ldc), float("nan"), device=DEV, dtype=torch.bfloat16)
    C = Cbuf[:, :N]
    note(f"gemm {M}x{N}x{K} at={a_trans} bt={b_trans}")
    Nn.gemm_bf16(A, B, C, a_trans=a_trans, b_trans=b_trans)
    torch.cuda.synchronize()
    ref = _gemm_ref(A, B, a_trans, b_trans)
    assert_close_rel(C, ref, BF16_TOL, "gemm")
    # fp32 output is exact up to summation order: much tighter than bf16 rounding
    C32 = torch.empty(M, ldc, device=DEV, dtype=torch.float32)[:, :N]
    Nn.gemm_bf16(A, B, C32, a_trans=a_trans, b_trans=b_trans)
    assert_close_rel(C32, ref, 1e-5, "gemm fp32 out")


def test_gemm_bf16_large_output_takes_256_wide_tiles():
    """Outputs of at least 1024 tiles of 256 x 256 (both operands k-contiguous, no epilogue) run on
    the 256-wide tile variant: edges in M and N, a k tail, and a ragged leading dimension."""
    Nn = native()
    torch.manual_seed(11)
    M, N, K = 8192 - 40, 8192 + 264, 136
    A = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    B = torch.randn(N, K, device=DEV).to(torch.bfloat16)
    Cbuf = torch.full((M, N + 4), float("nan"), device=DEV, dtype=torch.bfloat16)
    C = Cbuf[:, :N]
    Nn.gemm_bf16(A, B, C)
    ref = A.float() @ B.float().t()          # on the GPU in fp32: the CPU would take a minute
    assert_close_rel(C, ref.cpu(), BF16_TOL, "gemm, 256-wide tiles")
    assert bool(torch.isnan(Cbuf[:, N:]).all())


def test_gemm_bf16_output_that_fills_its_rounds_better_takes_256_x_192_tiles():
    """An output whose 256 x 192 tiles fill two rounds of work-groups where 256 x 256 tiles leave the second
    a quarter empty (the shape of a Llama-2-7B q | k | v projection over 2048 tokens) runs on the 192-wide
    tile variant: edges in M and N, a k tail, a ragged leading dimension, and the same bits as the rows
    computed alone on the small tiles (the reduction order does not depend on the tile)."""
    Nn = native()
    torch.manual_seed(12)
    M, N, K = 2048 - 8, 12288 - 8, 200
    A = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    B = torch.randn(N, K, device=DEV).to(torch.bfloat16)
    Cbuf = torch.full((M, N + 4), float("nan"), device=DEV, dtype=torch.bfloat16)
    C = Cbuf[:, :N]
    Nn.gemm_bf16(A, B, C)
    ref = A.float() @ B.float().t()
    assert_close_rel(C, ref.cpu(), BF16_TOL, "gemm, 256 x 192 tiles")
    assert bool(torch.isnan(Cbuf[:, N:]).all())
    part = torch.empty(M, 768, device=DEV, dtype=torch.bfloat16)      # 16 x 8 tiles of 128 x 96: the small path
    Nn.gemm_bf16(A, B[4096:4096 + 768], part)
    assert torch.equal(part, C[:, 4096:4096 + 768])


@pytest.mark.parametrize("M,N,K", [(384, 264, 136), (512, 380, 136), (4096, 768, 264), (4096, 2304, 136)])
def test_gemm_bf16_epilogues(M, N, K):
    """The second and third shapes run on 96-column tiles (they fill more CUs than 128-column ones),
    the last on 192-column tiles (one wave of work-groups instead of one and a bit)."""
    Nn = native()
    torch.manual_seed(5)
    A = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    W = (torch.randn(N, K, device=DEV) * 0.1).to(torch.bfloat16)
    bias = torch.randn(N, device=DEV).to(torch.bfloat16)
    R = torch.randn(M, N, device=DEV).to(torch.bfloat16)
    a, w, b, r = A.float().cpu(), W.float().cpu(), bias.float().cpu(), R.float().cpu()
    lin = a @ w.t()

    C = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    Nn.gemm_bf16(A, W, C, epilogue=Nn.EPI_BIAS, bias=bias)
    assert_close_rel(C, lin + b, BF16_TOL, "bias")

    for epi, fn in ((Nn.EPI_BIAS_GELU_ERF, O.gelu_erf), (Nn.EPI_BIAS_GELU_TANH, O.gelu_tanh)):
        pre = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
        Nn.gemm_bf16(A, W, C, epilogue=epi, bias=bias, aux_out=pre)
        assert_close_rel(pre, lin + b, BF16_TOL, "pre-activation")
        assert_close_rel(C, fn(lin + b), BF16_TOL, "gelu")
        # without saving the pre-activation
        C2 = torch.empty_like(C)
        Nn.gemm_bf16(A, W, C2, epilogue=epi, bias=bias)
        assert torch.equal(C, C2)

    Nn.gemm_bf16(A, W, C, epilogue=Nn.EPI_BIAS_RESIDUAL, bias=bias, aux_in=R)
    assert_close_rel(C, lin + b + r, BF16_TOL, "bias+residual")
    Nn.gemm_bf16(A, W, C, epilogue=Nn.EPI_BIAS_RESIDUAL, aux_in=R)
    assert_close_rel(C, lin + r, BF16_TOL, "residual")

    Nn.gemm_bf16(A, W, C, epilogue=Nn.EPI_BIAS_RELU, bias=bias)
    assert_close_rel(C, torch.relu(lin + b), BF16_TOL, "relu")
    Nn.gemm_bf16(A, W, C, epilogue=Nn.EPI_DRELU, aux_in=R)
    assert_close_rel(C, lin * (r > 0), BF16_TOL, "drelu")

    for epi, fn in ((Nn.EPI_DGELU_ERF, O.gelu_erf), (Nn.EPI_DGELU_TANH, O.gelu_tanh)):
        h = r.clone().requires_grad_(True)
        fn(h).backward(lin)
        Nn.gemm_bf16(A, W, C, epilogue=epi, aux_in=R)
        assert_close_rel(C, h.grad, BF16_TOL, "dgelu")

    acc = torch.randn(M, N, device=DEV, dtype=torch.float32)
    acc0 = acc.cpu().clone()
    Nn.gemm_bf16(A, W, acc, epilogue=Nn.EPI_ACCUM_F32, beta=1)
    assert_close_rel(acc, acc0 + lin, 1e-5, "accumulate")
    Nn.gemm_bf16(A, W, acc, epilogue=Nn.EPI_ACCUM_F32, beta=0)
    assert_close_rel(acc, lin, 1e-5, "accumulate init")


@pytest.mark.parametrize("M,N,K,bt", [(4096, 3072, 264, False), (4096, 768, 136, False), (1000, 376, 136, False),
                                       (384, 264, 136, True), (300, 3072, 72, False)])
def test_gemm_activation_derivative_epilogue_leaves_the_column_sums(M, N, K, bt):
    """With ``colsum`` the epilogue also writes, per band of 32 rows, the column sums of C as stored: C itself
    is unchanged bit for bit, every band's sums are the fp32 sums of the stored bf16 values (at most one
    rounding per addition apart from the ascending-order sum), and pp_colreduce_grouped forms from them the
    bias gradient that the two-pass reduction of C gives.  Shapes cover 192-, 96- and 128-column tiles, ragged
    edges in both directions and a transposed weight."""
    Nn = native()
    torch.manual_seed(51)
    A = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    W = (torch.randn(K, N, device=DEV) * 0.1).to(torch.bfloat16) if bt else \
        (torch.randn(N, K, device=DEV) * 0.1).to(torch.bfloat16)
    R = torch.randn(M, N, device=DEV).to(torch.bfloat16)
    n_part = (M + Nn.GEMM_COLSUM_ROWS - 1) // Nn.GEMM_COLSUM_ROWS
    for epi in (Nn.EPI_DGELU_TANH, Nn.EPI_DGELU_ERF, Nn.EPI_DRELU):
        C0 = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
        C1 = torch.empty_like(C0)
        part = torch.full((n_part, N), float("nan"), device=DEV)
        Nn.gemm_bf16(A, W, C0, b_trans=bt, epilogue=epi, aux_in=R)
        Nn.gemm_bf16(A, W, C1, b_trans=bt, epilogue=epi, aux_in=R, colsum=part)
        assert torch.equal(C0, C1)
        pad = torch.zeros(n_part * 32, N, device=DEV, dtype=torch.float64)
        pad[:M] = C1.double()
        bands = pad.view(n_part, 32, N)
        exact = bands.sum(1)
        assert not bool(torch.isnan(part).any())
        assert (part.double() - exact).abs().max() <= 32 * 2.0 ** -24 * bands.abs().sum(1).max()
        out, ref = torch.empty(N, device=DEV), torch.empty(N, device=DEV)
        Nn.colreduce_grouped([dict(dy=C1, out_sum=out, workspace=part, n_part_ready=n_part)])
        ws = torch.empty(2 * ((M + 127) // 128) * N, device=DEV)
        Nn.colreduce_grouped([dict(dy=C1, out_sum=ref, workspace=ws)])
        assert (out - ref).abs().max() <= 1e-6 * float(C1.float().abs().sum(0).max())
    with pytest.raises(RuntimeError, match="column sums"):
        Nn.gemm_bf16(A, W, C0, b_trans=bt, epilogue=Nn.EPI_NONE, colsum=part)


@pytest.mark.parametrize("M,N,K,at,bt", [(768, 2304, 4096, True, True), (200, 136, 264, True, True),
                                          (50304, 768, 4096, True, True), (11008, 4096, 2048, True, True),
                                          (256, 96, 512, False, False), (4096, 768, 64, False, True)])
def test_gemm_bf16_rounded_accumulate_is_bit_exact(M, N, K, at, bt):
    """PP_EPI_ACCUM_ROUNDED leaves in an fp32 C what a bf16 C followed by the accumulate kernel
    leaves (``acc = float(g)`` when it starts an accumulation, ``acc += float(g)`` after)."""
    Nn = native()
    torch.manual_seed(21)
    A = torch.randn((K, M) if at else (M, K), device=DEV).to(torch.bfloat16)
    B = torch.randn((K, N) if bt else (N, K), device=DEV).to(torch.bfloat16)
    g = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    Nn.gemm_bf16(A, B, g, a_trans=at, b_trans=bt)
    start = torch.randn(M, N, device=DEV)
    want = start.clone()
    Nn.grad_accum(want.view(-1), g.view(-1), init=False)
    got = start.clone()
    Nn.gemm_bf16(A, B, got, a_trans=at, b_trans=bt, epilogue=Nn.EPI_ACCUM_ROUNDED, beta=1)
    assert torch.equal(got, want)
    assert torch.equal(want, start + g.float())
    Nn.gemm_bf16(A, B, got, a_trans=at, b_trans=bt, epilogue=Nn.EPI_ACCUM_ROUNDED, beta=0)
    assert torch.equal(got, g.float())
    # the same through a grouped launch
    got2 = start.clone()
    other = torch.zeros(M, N, device=DEV)
    kw = dict(a_trans=at, b_trans=bt, epilogue=Nn.EPI_ACCUM_ROUNDED, beta=1)
    Nn.gemm_bf16_grouped([(A, B, got2, kw), (A, B, other, kw)])
    assert torch.equal(got2, want) and torch.equal(other, g.float())
    bad = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="fp32 C"):
        Nn.gemm_bf16(A, B, bad, a_trans=at, b_trans=bt, epilogue=Nn.EPI_ACCUM_ROUNDED)


@pytest.mark.parametrize("M,N,K", [(128, 256, 100), (72, 136, 36), (768, 3072, 1001), (64, 64, 7), (256, 128, 65)])
def test_gemm_bf16_transposed_operands_take_any_reduction_length(M, N, K):
    """dW = dY^T X over a number of tokens that is not a multiple of 8 (both operands transposed: k is
    the row index of both, rows past K read as zero), alone, into an accumulator, and in a grouped launch."""
    Nn = native()
    torch.manual_seed(K)
    A = torch.randn(K, M, device=DEV).to(torch.bfloat16)
    B = torch.randn(K, N, device=DEV).to(torch.bfloat16)
    C = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
    note(f"gemm TT {M}x{N}x{K}")
    Nn.gemm_bf16(A, B, C, a_trans=True, b_trans=True)
    torch.cuda.synchronize()
    ref = A.float().cpu().t() @ B.float().cpu()
    assert_close_rel(C, ref, BF16_TOL, "TT gemm, odd K")
    acc, acc2 = torch.ones(M, N, device=DEV), torch.zeros(M, N, device=DEV)
    kw = dict(a_trans=True, b_trans=True, epilogue=Nn.EPI_ACCUM_F32, beta=1)
    Nn.gemm_bf16_grouped([(A, B, acc, kw), (A, B, acc2, kw)])
    torch.cuda.synchronize()
    assert torch.equal(acc2.to(torch.bfloat16), C)
    assert_close_rel(acc - 1.0, ref, BF16_TOL, "TT gemm into an accumulator, odd K")
    with pytest.raises(RuntimeError, match="multiples of 8"):
        Nn.gemm_bf16(A.t().contiguous(), B, torch.empty(M, N, device=DEV, dtype=torch.bfloat16), b_trans=True)


def test_gemm_bf16_rejects_bad_arguments():
    Nn = native()
    A = torch.zeros(16, 12, device=DEV, dtype=torch.bfloat16)
    B = torch.zeros(16, 12, device=DEV, dtype=torch.bfloat16)
    C = torch.zeros(16, 16, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="multiples of 8"):
        Nn.gemm_bf16(A, B, C)


def test_gemm_f32():
    Nn = native()
    torch.manual_seed(6)
    for (M, N, K, at, bt) in [(64, 512, 512, False, False), (64, 10, 256, False, False),
                              (70, 33, 19, False, True), (512, 1024, 64, True, True),
                              (64, 512, 1024, False, True), (1, 1, 1, False, False),
                              (33, 65, 2051, True, False), (256, 10, 64, True, True)]:
        A = torch.randn((K, M) if at else (M, K), device=DEV)
        B = torch.randn((K, N) if bt else (N, K), device=DEV)
        bias = torch.randn(N, device=DEV)
        C = torch.empty(M, N, device=DEV)
        ref = _gemm_ref(A, B, at, bt)
        Nn.gemm_f32(A, B, C, a_trans=at, b_trans=bt)
        assert_close_rel(C, ref, F32_TOL, "gemm_f32")
        Nn.gemm_f32(A, B, C, a_trans=at, b_trans=bt, epilogue=Nn.EPI_BIAS_RELU, bias=bias)
        assert_close_rel(C, torch.relu(ref + bias.cpu()), F32_TOL, "gemm_f32 relu")
        R = torch.randn(M, N, device=DEV)
        Nn.gemm_f32(A, B, C, a_trans=at, b_trans=bt, epilogue=Nn.EPI_DRELU, aux_in=R)
        assert_close_rel(C, ref * (R.cpu() > 0), F32_TOL, "gemm_f32 drelu")
        acc = torch.randn(M, N, device=DEV)
        acc0 = acc.cpu().clone()
        Nn.gemm_f32(A, B, acc, a_trans=at, b_trans=bt, epilogue=Nn.EPI_ACCUM_F32, beta=1)
        assert_close_rel(acc, acc0 + ref, F32_TOL, "gemm_f32 accumulate")


# ---- column sums / LayerNorm ------------------------------------------------------------------
@pytest.mark.parametrize("M,N", [(4096, 768), (100, 264), (1, 8)])
def test_colsum(M, N):
    Nn = native()
    torch.manual_seed(7)
    dY = torch.randn(M, N, device=DEV).to(torch.bfloat16)
    ws = torch.empty(((M + 127) // 128) * N, device=DEV)
    out32 = torch.empty(N, device=DEV)
    Nn.colsum(dY, out32, ws)
    assert_close_rel(out32, dY.float().cpu().sum(0), 1e-5, "colsum fp32")
    out16 = torch.empty(N, device=DEV, dtype=torch.bfloat16)
    Nn.colsum(dY, out16, ws)
    assert_close_rel(out16, dY.float().cpu().sum(0), BF16_TOL, "colsum bf16")


@pytest.mark.parametrize("rows,C", [(4096, 768), (37, 1024), (5, 8), (130, 4096)])
def test_layernorm(rows, C):
    Nn = native()
    torch.manual_seed(8)
    x = (torch.randn(rows, C, device=DEV) * 2 + 0.5).to(torch.bfloat16)
    gamma = (1 + 0.1 * torch.randn(C, device=DEV)).to(torch.bfloat16)
    beta = (0.1 * torch.randn(C, device=DEV)).to(torch.bfloat16)
    dy = torch.randn(rows, C, device=DEV).to(torch.bfloat16)
    dres = torch.randn(rows, C, device=DEV).to(torch.bfloat16)
    y = torch.empty_like(x)
    mean = torch.empty(rows, device=DEV)
    rstd = torch.empty(rows, device=DEV)
    eps = 1e-5
    Nn.layernorm_fwd(x, gamma, beta, y, mean, rstd, eps)

    xr = x.float().cpu().requires_grad_(True)
    gr = gamma.float().cpu().requires_grad_(True)
    br = beta.float().cpu().requires_grad_(True)
    yr = O.layer_norm(xr, gr, br, eps)
    assert_close_rel(y, yr, BF16_TOL, "ln fwd")
    assert_close_rel(mean, xr.detach().mean(-1), 1e-4, "ln mean")
    yr.backward(dy.float().cpu())

    dx = torch.empty_like(x)
    Nn.layernorm_bwd_input(dy, x, gamma, mean, rstd, None, dx)
    assert_close_rel(dx, xr.grad, BF16_TOL, "ln dx")
    Nn.layernorm_bwd_input(dy, x, gamma, mean, rstd, dres, dx)
    assert_close_rel(dx, xr.grad + dres.float().cpu(), BF16_TOL, "ln dx + residual")

    ws = torch.empty(2 * ((rows + 127) // 128) * C, device=DEV)
    dg = torch.empty(C, device=DEV)
    db = torch.empty(C, device=DEV)
    Nn.layernorm_bwd_weight(dy, x, mean, rstd, dg, db, ws)
    assert_close_rel(dg, gr.grad, 1e-3, "ln dgamma")
    assert_close_rel(db, br.grad, 1e-4, "ln dbeta")
    dg16 = torch.empty(C, device=DEV, dtype=torch.bfloat16)
    db16 = torch.empty(C, device=DEV, dtype=torch.bfloat16)
    Nn.layernorm_bwd_weight(dy, x, mean, rstd, dg16, db16, ws)
    assert_close_rel(dg16, gr.grad, BF16_TOL, "ln dgamma bf16")
    assert_close_rel(db16, br.grad, BF16_TOL, "ln dbeta bf16")


@pytest.mark.parametrize("rows,C,rms", [(4096, 768, False), (1000, 768, False), (37, 64, False), (512, 1024, True),
                                        (130, 1024, False)])
def test_layernorm_input_gradient_that_leaves_the_column_sums(rows, C, rms):
    """pp_layernorm_bwd_input_sums: the input gradient bit for bit as pp_layernorm_bwd_input writes it, and
    the final sums that pp_colreduce_grouped forms from its partial sums against the definition (fp64) and
    against the two-pass reductions, for LayerNorm and RMSNorm, with ragged last blocks of rows."""
    Nn = native()
    torch.manual_seed(81)
    x = (torch.randn(rows, C, device=DEV) * 2 + 0.5).to(torch.bfloat16)
    gamma = (1 + 0.1 * torch.randn(C, device=DEV)).to(torch.bfloat16)
    dy = torch.randn(rows, C, device=DEV).to(torch.bfloat16)
    dres = torch.randn(rows, C, device=DEV).to(torch.bfloat16)
    y, rstd = torch.empty_like(x), torch.empty(rows, device=DEV)
    mean = None if rms else torch.empty(rows, device=DEV)
    Nn.layernorm_fwd(x, gamma, None, y, mean, rstd, 1e-5)
    for res in (None, dres):
        dx_ref, dx = torch.empty_like(x), torch.full_like(x, 7.0)
        Nn.layernorm_bwd_input(dy, x, gamma, mean, rstd, res, dx_ref)
        n_part = (rows + Nn.LN_SUM_ROWS - 1) // Nn.LN_SUM_ROWS
        ws_w = torch.full((2 * n_part * C,), float("nan"), device=DEV)
        ws_dx = torch.full((n_part * C,), float("nan"), device=DEV)
        assert Nn.layernorm_bwd_input_sums(dy, x, gamma, mean, rstd, res, dx, ws_w, ws_dx) == n_part
        assert torch.equal(dx, dx_ref)
        # the final sums from the partial sums
        dg, db, dbias = (torch.empty(C, device=DEV) for _ in range(3))
        Nn.colreduce_grouped([
            dict(dy=dy, out_sum=db, out_dot=dg, workspace=ws_w, n_part_ready=n_part),
            dict(dy=dx, out_sum=dbias, workspace=ws_dx, n_part_ready=n_part)])
        xh = (x.double() - (0 if rms else mean.double()[:, None])) * rstd.double()[:, None]
        scale = float(rows) ** 0.5
        assert (dg.double() - (dy.double() * xh).sum(0)).abs().max() <= 1e-5 * scale * 8
        assert (db.double() - dy.double().sum(0)).abs().max() <= 1e-5 * scale * 8
        assert (dbias.double() - dx.double().sum(0)).abs().max() <= 1e-5 * scale * 8
        # and the two-pass reductions over the same tensors: the same sums up to fp32 summation order
        ws2 = torch.empty(2 * ((rows + 127) // 128) * C, device=DEV)
        dg2, db2, dbias2 = (torch.empty(C, device=DEV) for _ in range(3))
        Nn.colreduce_grouped([dict(dy=dy, x=x, mean=mean, rstd=rstd, out_sum=db2, out_dot=dg2, workspace=ws2)])
        Nn.colreduce_grouped([dict(dy=dx, out_sum=dbias2, workspace=ws2)])
        for a, b_ in ((dg, dg2), (db, db2), (dbias, dbias2)):
            assert (a - b_).abs().max() <= 1e-5 * scale * 8
    # only one of the two kinds of sums asked for; bf16 results
    ws_dx = torch.empty(n_part * C, device=DEV)
    dx2 = torch.empty_like(x)
    Nn.layernorm_bwd_input_sums(dy, x, gamma, mean, rstd, dres, dx2, None, ws_dx)
    assert torch.equal(dx2, dx_ref)
    b16 = torch.empty(C, device=DEV, dtype=torch.bfloat16)
    Nn.colreduce_grouped([dict(dy=dx2, out_sum=b16, workspace=ws_dx, n_part_ready=n_part)])
    assert torch.equal(b16, dbias.to(torch.bfloat16))


def test_layernorm_input_gradient_sums_reject_a_wide_row():
    Nn = native()
    C = Nn.LN_SUM_MAX_C + 8
    x = torch.zeros(16, C, device=DEV, dtype=torch.bfloat16)
    ws = torch.empty(2 * C, device=DEV)
    with pytest.raises(RuntimeError, match="exceeds"):
        Nn.layernorm_bwd_input_sums(x, x, x[0], None, torch.ones(16, device=DEV), None, torch.empty_like(x), ws, None)


# ---- embedding / loss ----------------------------------------------------------------------------
def test_embedding():
    Nn = native()
    torch.manual_seed(9)
    vocab, seq, C, B = 1000, 128, 768, 3
    wte = torch.randn(vocab, C, device=DEV).to(torch.bfloat16)
    wpe = torch.randn(seq, C, device=DEV).to(torch.bfloat16)
    ids = torch.randint(0, vocab, (B, seq), device=DEV)
    ids[0, :5] = 7  # repeated ids: one row receives several tokens
    y = torch.empty(B * seq, C, device=DEV, dtype=torch.bfloat16)
    Nn.embed_fwd(ids, wte, wpe, y, seq)
    ref = O.embedding(ids.cpu(), wte.float().cpu(), wpe.float().cpu()).reshape(B * seq, C)
    # a single bf16 rounding of an fp32 sum: identical to torch's bf16 add
    assert torch.equal(y.cpu(), (wte[ids.reshape(-1)] + wpe.repeat(B, 1)).cpu())
    assert_close_rel(y, ref, BF16_TOL, "embed fwd")
    y2 = torch.empty_like(y)
    Nn.embed_fwd(ids, wte, None, y2, seq)
    assert torch.equal(y2, wte[ids.reshape(-1)])

    dy = torch.randn(B * seq, C, device=DEV).to(torch.bfloat16)
    d_wte = torch.zeros(vocab, C, device=DEV)
    d_wpe = torch.zeros(seq, C, device=DEV)
    Nn.embed_bwd(ids, dy, d_wte, d_wpe, seq)
    wr = wte.float().cpu().requires_grad_(True)
    pr = wpe.float().cpu().requires_grad_(True)
    O.embedding(ids.cpu(), wr, pr).reshape(B * seq, C).backward(dy.float().cpu())
    assert_close_rel(d_wte, wr.grad, 1e-5, "d_wte")
    assert_close_rel(d_wpe, pr.grad, 1e-5, "d_wpe")


@pytest.mark.parametrize("B,S,pad", [(3, 128, 1), (2, 37, 0), (5, 200, 7), (1, 1, 1), (4, 64, 3)])
def test_positions_counted_over_real_tokens_and_the_lookup_at_them(B, S, pad):
    """Position indices of an encoder that skips padding tokens (bit-exact against the oracle's loop: rows
    with padding at the front, inside, at the end, everywhere, nowhere) and the embedding sum read at
    those indices (one rounding of the fp32 sum, like the positional form)."""
    Nn = native()
    g = torch.Generator().manual_seed(B * S + pad)
    ids = torch.randint(0, 12, (B, S), generator=g)
    ids[0, : S // 3] = pad
    if B > 1:
        ids[1, S // 2:] = pad
    if B > 2:
        ids[2] = pad
    if B > 3:
        ids[3][ids[3] == pad] = pad + 1
    out = torch.full((B, S), -1, dtype=torch.int64, device=DEV)
    Nn.position_ids_from_padding(ids.to(DEV), out, pad)
    want = O.position_ids_from_padding(ids, pad)
    assert torch.equal(out.cpu(), want)
    C, vocab, n_pos = 256, 12, S + pad + 1
    wte = torch.randn(vocab, C, generator=g).to(torch.bfloat16)
    wpe = torch.randn(n_pos, C, generator=g).to(torch.bfloat16)
    row = torch.randn(C, generator=g).to(torch.bfloat16)
    for extra in (None, row):
        y = torch.full((B * S, C), float("nan"), dtype=torch.bfloat16, device=DEV)
        Nn.embed_fwd_at(ids.to(DEV), out, wte.to(DEV), wpe.to(DEV), y,
                        extra_row=extra.to(DEV) if extra is not None else None)
        ref = O.embedding_at(ids, want, wte.float(), wpe.float(), extra.float() if extra is not None else None)
        assert torch.equal(y.cpu(), ref.reshape(B * S, C).to(torch.bfloat16))


@pytest.mark.parametrize("C,vocab,n_tok,seq", [(768, 50, 1024, 128), (64, 3, 333, 111), (4096, 17, 130, 65),
                                               (1024, 32000, 2048, 1024)])
@pytest.mark.parametrize("rounded", [False, True])
def test_embedding_backward_is_ordered_and_bit_exact(C, vocab, n_tok, seq, rounded):
    """Few distinct ids, so every row of the table receives many tokens: the row sums must equal the
    oracle's one-by-one additions in ascending token order bit for bit, in both accumulation forms
    (unrounded fp32 sums; sums rounded to bf16 first), on top of what the accumulator already holds,
    and again on a second call."""
    import numpy as np
    from oracle import microbatch as OM
    Nn = native()
    g = torch.Generator().manual_seed(C + n_tok)
    ids = torch.randint(0, vocab, (n_tok,), generator=g)
    ids[-1] = ids[0]                      # the first and the last token share a row
    dy = (torch.randn(n_tok, C, generator=g) * 3).to(torch.bfloat16)
    start = torch.randn(vocab, C, generator=g)
    start_p = torch.randn(seq, C, generator=g)
    d_wte, d_wpe = start.to(DEV), start_p.to(DEV)
    bits = dy.view(torch.int16).numpy().view(np.uint16)
    gw = OM.embedding_grad(ids.numpy(), bits, vocab, rounded)
    gp = OM.embedding_grad(np.arange(n_tok) % seq, bits, seq, rounded)
    for call in range(2):
        Nn.embed_bwd(ids.to(DEV), dy.to(DEV), d_wte, d_wpe, seq, round_bf16=rounded)
        start = start + torch.from_numpy(gw)
        start_p = start_p + torch.from_numpy(gp)
        assert torch.equal(d_wte.cpu(), start), f"d_wte, call {call}"
        assert torch.equal(d_wpe.cpu(), start_p), f"d_wpe, call {call}"


def test_embedding_backward_leaves_the_padding_row_alone():
    """``padding_idx``: that row of the table's gradient keeps what it held (here a marker value), however
    many padding tokens the batch has (most of it here), negative indices count from the end of the table
    as in ``nn.Embedding``, and every other row is what the call without a padding row leaves."""
    Nn = native()
    g = torch.Generator().manual_seed(12)
    vocab, C, seq, n_tok = 50, 64, 32, 512
    ids = torch.randint(0, vocab, (n_tok,), generator=g)
    pad = 1
    ids[torch.rand(n_tok, generator=g) < 0.7] = pad
    dy = torch.randn(n_tok, C, generator=g).to(torch.bfloat16)
    for given in (pad, pad - vocab):
        ref = torch.zeros(vocab, C, device=DEV)
        got = torch.zeros(vocab, C, device=DEV)
        got[pad] = 5.0
        Nn.embed_bwd(ids.to(DEV), dy.to(DEV), ref, None, seq)
        Nn.embed_bwd(ids.to(DEV), dy.to(DEV), got, None, seq, padding_idx=given)
        assert bool((got[pad] == 5.0).all())
        keep = torch.arange(vocab) != pad
        assert torch.equal(got[keep], ref[keep])


def test_embedding_and_layernorm_full_size_closed_forms():
    """The embedding and LayerNorm shapes of the GPT-2-small stage (4096 tokens, width 768, 50257
    tokens in the table).  A zero position table makes the embedding an exact gather; rows of the
    form s_r * (+1, -1, +1, ...) have mean 0 and variance s_r^2, so LayerNorm returns +-gamma + beta
    for every row."""
    Nn = native()
    torch.manual_seed(31)
    vocab, seq, C, B = 50257, 1024, 768, 4
    wte = torch.randn(vocab, C, device=DEV).to(torch.bfloat16)
    ids = torch.randint(0, vocab, (B, seq), device=DEV)
    y = torch.full((B * seq, C), float("nan"), device=DEV, dtype=torch.bfloat16)
    Nn.embed_fwd(ids, wte, torch.zeros(seq, C, device=DEV, dtype=torch.bfloat16), y, seq)
    assert torch.equal(y, wte[ids.reshape(-1)])

    rows = B * seq
    sign = torch.ones(C, device=DEV)
    sign[1::2] = -1
    scale = torch.exp2(torch.randint(-6, 7, (rows, 1), device=DEV).float())   # exact in bf16
    x = (scale * sign).to(torch.bfloat16)
    gamma = (1 + 0.1 * torch.randn(C, device=DEV)).to(torch.bfloat16)
    beta = (0.1 * torch.randn(C, device=DEV)).to(torch.bfloat16)
    out = torch.empty_like(x)
    mean = torch.empty(rows, device=DEV)
    rstd = torch.empty(rows, device=DEV)
    Nn.layernorm_fwd(x, gamma, beta, out, mean, rstd, 0.0)
    want = (sign * gamma.float() + beta.float()).to(torch.bfloat16).expand(rows, C)
    assert float(mean.abs().max()) == 0.0
    assert float((rstd * scale.view(-1) - 1).abs().max()) <= 1e-6
    assert torch.equal(out, want)


@pytest.mark.parametrize("rows,V,ld", [(64, 1000, 1000), (33, 1001, 1008), (128, 50257, 50304), (16, 8, 8)])
def test_ce_loss_bf16(rows, V, ld):
    Nn = native()
    torch.manual_seed(10)
    buf = (torch.randn(rows, ld, device=DEV) * 3).to(torch.bfloat16)
    logits = buf[:, :V] if ld != V else buf
    target = torch.randint(0, V, (rows,), device=DEV)
    target[::7] = -100
    loss = torch.empty(1, device=DEV)
    dbuf = torch.full((rows, ld), float("nan"), device=DEV, dtype=torch.bfloat16)
    ws = torch.empty(rows + 2, device=DEV)
    Nn.ce_loss(buf, target, loss, dbuf, ws, V)
    lr = logits.float().cpu().requires_grad_(True)
    ref = O.cross_entropy_mean(lr, target.cpu())
    ref.backward()
    assert_close_rel(loss, ref.detach().reshape(1), 1e-5, "ce loss")
    assert_close_rel(dbuf[:, :V], lr.grad, BF16_TOL, "ce dlogits")
    if ld != V:
        assert float(dbuf[:, V:].float().abs().max()) == 0.0
    # loss only
    loss2 = torch.empty(1, device=DEV)
    Nn.ce_loss(buf, target, loss2, None, ws, V)
    assert torch.equal(loss, loss2)


@pytest.mark.parametrize("rows,V", [(4096, 50257), (2048, 32000)])
def test_ce_loss_bf16_full_size_is_exact_per_element_and_repeatable(rows, V):
    """The logits of a whole microbatch (every CU holds two rows at a time): each gradient element
    against softmax - onehot computed by torch on the GPU in fp32, not only the largest error of the
    tensor, the same bits on every run, and the same bits when the gradient overwrites the logits."""
    Nn = native()
    torch.manual_seed(12)
    ld = (V + 127) // 128 * 128
    buf = torch.zeros(rows, ld, device=DEV, dtype=torch.bfloat16)
    buf[:, :V] = torch.randn(rows, V, device=DEV).to(torch.bfloat16)
    target = torch.randint(0, V, (rows,), device=DEV)
    runs = []
    for _ in range(3):
        loss = torch.empty(1, device=DEV)
        d = torch.full((rows, ld), float("nan"), device=DEV, dtype=torch.bfloat16)
        Nn.ce_loss(buf, target, loss, d, torch.empty(rows + 2, device=DEV), V)
        runs.append((loss, d))
    ref = torch.softmax(buf[:, :V].float(), -1)
    ref[torch.arange(rows, device=DEV), target] -= 1
    ref /= rows
    got = runs[0][1][:, :V].float()
    # bf16 rounding of the result (2^-8 relative) plus that of the stored exponentials
    assert bool(((got - ref).abs() <= 2.0 ** -6 * ref.abs() + 1e-9).all())
    assert bool((runs[0][1][:, V:] == 0).all())
    for loss, d in runs[1:]:
        assert torch.equal(loss, runs[0][0]) and torch.equal(d, runs[0][1])
    inplace = buf.clone()
    Nn.ce_loss(inplace, target, torch.empty(1, device=DEV), inplace, torch.empty(rows + 2, device=DEV), V)
    assert torch.equal(inplace, runs[0][1])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_ce_loss_with_every_row_ignored_is_nan_with_zero_gradient(dtype):
    """The mean over no rows: torch.nn.functional.cross_entropy returns NaN and a zero gradient."""
    Nn = native()
    rows, V = 24, 16
    logits = torch.randn(rows, V, device=DEV).to(dtype)
    target = torch.full((rows,), -100, device=DEV)
    loss = torch.zeros(1, device=DEV)
    dl = torch.full_like(logits, 7.0)
    Nn.ce_loss(logits, target, loss, dl, torch.empty(rows + 2, device=DEV), V)
    lr = logits.float().cpu().requires_grad_(True)
    ref = torch.nn.functional.cross_entropy(lr, target.cpu())
    ref.backward()
    assert torch.isnan(ref) and torch.isnan(loss).all()
    assert float(lr.grad.abs().max()) == 0.0 and float(dl.float().abs().max()) == 0.0


def test_ce_loss_f32():
    Nn = native()
    torch.manual_seed(11)
    rows, V = 64, 10
    logits = torch.randn(rows, V, device=DEV) * 2
    target = torch.randint(0, V, (rows,), device=DEV)
    loss = torch.empty(1, device=DEV)
    dl = torch.empty_like(logits)
    ws = torch.empty(rows + 2, device=DEV)
    Nn.ce_loss(logits, target, loss, dl, ws, V)
    lr = logits.cpu().requires_grad_(True)
    ref = torch.nn.functional.cross_entropy(lr, target.cpu())
    ref.backward()
    assert_close_rel(loss, ref.detach().reshape(1), F32_TOL, "ce f32 loss")
    assert_close_rel(dl, lr.grad, F32_TOL, "ce f32 grad")


# ---- attention -----------------------------------------------------------------------------------
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("B,S,H,D", [(1, 128, 1, 64), (2, 256, 3, 64), (1, 1024, 2, 64),
                                     (1, 128, 1, 128), (2, 256, 3, 128), (1, 2048, 2, 128),
                                     (1, 64, 2, 64), (2, 192, 1, 64), (1, 320, 2, 128), (3, 64, 1, 128),
                                     # few work-groups, head dimension 64: key blocks of 128 on 8 waves, the last
                                     # block half full when S is an odd multiple of 64
                                     (2, 320, 2, 64), (1, 448, 3, 64)])
def test_attention(causal, B, S, H, D):
    Nn = native()
    torch.manual_seed(12 + S)
    qkv = torch.randn(B, S, 3 * H * D, device=DEV).to(torch.bfloat16)
    o = torch.full((B, S, H * D), float("nan"), device=DEV, dtype=torch.bfloat16)
    lse = torch.empty(B, H, S, device=DEV)
    note(f"attention fwd B={B} S={S} H={H} D={D} causal={causal}")
    Nn.attn_fwd(qkv, o, lse, H, causal)
    torch.cuda.synchronize()
    qr = qkv.float().cpu().requires_grad_(True)
    ref = O.attention_fused_qkv(qr, H, causal)
    assert_close_rel(o, ref, BF16_TOL, "attention fwd")

    d_o = torch.randn(B, S, H * D, device=DEV).to(torch.bfloat16)
    dqkv = torch.full_like(qkv, float("nan"))
    delta = torch.empty(B, H, S, device=DEV)
    note(f"attention bwd B={B} S={S} H={H} D={D} causal={causal}")
    Nn.attn_bwd(qkv, o, lse, d_o, dqkv, delta, H, causal)
    torch.cuda.synchronize()
    ref.backward(d_o.float().cpu())
    HD = H * D
    for name, sl in (("dq", slice(0, HD)), ("dk", slice(HD, 2 * HD)), ("dv", slice(2 * HD, 3 * HD))):
        assert_close_rel(dqkv[..., sl], qr.grad[..., sl], BF16_TOL, f"attention {name}")


@pytest.mark.parametrize("causal,exact", [(True, False), (False, True), (False, False)])
@pytest.mark.parametrize("B,S,H,Hkv", [(2, 256, 3, 3), (4, 1024, 12, 12), (1, 64, 2, 2), (2, 192, 4, 2), (1, 320, 6, 1)])
def test_attention_backward_leaves_the_column_sums_of_its_gradients(causal, exact, B, S, H, Hkv):
    """With ``colsum`` (head size 64) the two backward kernels also write, per block of 64 tokens, the column
    sums of dq, dk and dv as stored: the gradients themselves are unchanged bit for bit, every row of sums is
    the fp32 sum of the 64 stored bf16 rows (up to the rounding of the additions), and pp_colreduce_grouped
    forms from them the bias gradient of the fused projection that the two-pass reduction gives.  Multi-head
    and grouped-query layouts, with and without the query-gradient correction."""
    Nn = native()
    torch.manual_seed(3 + S + H)
    D = 64
    width = (H + 2 * Hkv) * D
    qkv = torch.randn(B, S, width, device=DEV).to(torch.bfloat16)
    o = torch.empty(B, S, H * D, device=DEV, dtype=torch.bfloat16)
    lse = torch.empty(B, H, S, device=DEV)
    Nn.attn_fwd(qkv, o, lse, H, causal, n_kv_heads=Hkv)
    d_o = torch.randn(B, S, H * D, device=DEV).to(torch.bfloat16)
    ref, got = torch.full_like(qkv, float("nan")), torch.full_like(qkv, float("nan"))
    delta = torch.empty(B, H, S, device=DEV)
    Nn.attn_bwd(qkv, o, lse, d_o, ref, delta, H, causal, n_kv_heads=Hkv, exact_dq=exact)
    n_part = B * S // 64
    part = torch.full((n_part, width), float("nan"), device=DEV)
    note(f"attention bwd with column sums B={B} S={S} H={H} Hkv={Hkv} causal={causal} exact={exact}")
    Nn.attn_bwd(qkv, o, lse, d_o, got, delta, H, causal, n_kv_heads=Hkv, exact_dq=exact, colsum=part)
    torch.cuda.synchronize()
    assert torch.equal(got, ref)
    blocks = got.double().view(n_part, 64, width)
    assert not bool(torch.isnan(part).any())
    assert (part.double() - blocks.sum(1)).abs().max() <= 64 * 2.0 ** -24 * float(blocks.abs().sum(1).max())
    flat = got.view(B * S, width)
    bias, two_pass = torch.empty(width, device=DEV), torch.empty(width, device=DEV)
    Nn.colreduce_grouped([dict(dy=flat, out_sum=bias, workspace=part, n_part_ready=n_part)])
    ws = torch.empty(2 * ((B * S + 127) // 128) * width, device=DEV)
    Nn.colreduce_grouped([dict(dy=flat, out_sum=two_pass, workspace=ws)])
    assert (bias - two_pass).abs().max() <= 1e-6 * float(flat.float().abs().sum(0).max())


def test_attention_column_sums_are_for_head_size_64():
    Nn = native()
    qkv = torch.zeros(1, 64, 3 * 128, device=DEV, dtype=torch.bfloat16)
    o = torch.zeros(1, 64, 128, device=DEV, dtype=torch.bfloat16)
    lse, delta = torch.zeros(1, 1, 64, device=DEV), torch.zeros(1, 1, 64, device=DEV)
    part = torch.zeros(1, 3 * 128, device=DEV)
    with pytest.raises(RuntimeError, match="head_dim 64"):
        Nn.attn_bwd(qkv, o, lse, o, torch.empty_like(qkv), delta, 1, True, colsum=part)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("D", [64, 128])
def test_attention_backward_where_query_gradients_are_small_differences(causal, D):
    """Nearly uniform attention over keys that share a large common part (an encoder at initialisation):
    the query gradient is a small difference of large terms, and an error of delta = rowsum(dO * O) - the
    forward's output is rounded to bf16 - enters it multiplied by the attention-weighted mean key.
    Checked: (1) after the backward the delta buffer holds the sum of P * dP over the keys as the fp32
    oracle has it, closer than the row sum of the rounded output is; (2) with PP_ATTN_EXACT_DQ dq is within
    tolerance of the oracle and clearly closer to it than without (what remains is the rounding of dS in
    front of the dS K product, which any bf16 path shares); (3) dk and dv are within tolerance either way;
    (4) where the effect is absent (ordinary inputs) the flag changes dq by rounding noise only."""
    Nn = native()
    B, S, H = 2, 256, 2
    HD = H * D
    torch.manual_seed(31 + D)
    qkv = torch.randn(B, S, 3 * HD, device=DEV)
    qkv[..., :HD] *= 0.05                                            # small queries: scores near zero
    qkv[..., HD:2 * HD] = qkv[..., HD:2 * HD] * 0.3 + 1.0 * torch.randn(1, 1, HD, device=DEV)   # keys: common part
    qkv = qkv.to(torch.bfloat16)
    o = torch.empty(B, S, HD, device=DEV, dtype=torch.bfloat16)
    lse = torch.empty(B, H, S, device=DEV)
    Nn.attn_fwd(qkv, o, lse, H, causal)
    d_o = torch.randn(B, S, HD, device=DEV).to(torch.bfloat16)
    qr = qkv.float().cpu().requires_grad_(True)
    ref = O.attention_fused_qkv(qr, H, causal)
    ref.backward(d_o.float().cpu())
    want_delta = (d_o.float().cpu() * ref.detach()).view(B, S, H, D).sum(-1).permute(0, 2, 1)
    from_rounded_o = (d_o.float() * o.float()).view(B, S, H, D).sum(-1).permute(0, 2, 1).cpu()
    got = {}
    for exact in (False, True):
        dqkv = torch.full_like(qkv, float("nan"))
        delta = torch.empty(B, H, S, device=DEV)
        Nn.attn_bwd(qkv, o, lse, d_o, dqkv, delta, H, causal, exact_dq=exact)
        torch.cuda.synchronize()
        got[exact] = (dqkv.float().cpu(), delta.cpu())
    scale = want_delta.abs().max().item()
    e_buf = (got[True][1] - want_delta).abs().max().item() / scale
    e_rounded = (from_rounded_o - want_delta).abs().max().item() / scale
    note(f"delta D={D} causal={causal}: {e_buf:.2e} in the buffer, {e_rounded:.2e} from the rounded output")
    assert e_buf < e_rounded / 4 and e_buf < 2e-4
    assert torch.equal(got[True][1], got[False][1])
    errs = {}
    for name, sl in (("dq", slice(0, HD)), ("dk", slice(HD, 2 * HD)), ("dv", slice(2 * HD, 3 * HD))):
        g = qr.grad[..., sl]
        errs[name] = tuple((got[ex][0][..., sl] - g).abs().max().item() / g.abs().max().item() for ex in (False, True))
        note(f"attention {name} D={D} causal={causal}: {errs[name][0]:.2e} plain, {errs[name][1]:.2e} corrected")
    assert errs["dq"][1] <= BF16_TOL and errs["dq"][1] < 0.8 * errs["dq"][0], errs["dq"]
    for name in ("dk", "dv"):
        assert max(errs[name]) <= BF16_TOL, (name, errs[name])
    # ordinary inputs: the correction is rounding noise
    qkv2 = torch.randn(B, S, 3 * HD, device=DEV).to(torch.bfloat16)
    Nn.attn_fwd(qkv2, o, lse, H, causal)
    a, bq = torch.empty_like(qkv2), torch.empty_like(qkv2)
    Nn.attn_bwd(qkv2, o, lse, d_o, a, torch.empty(B, H, S, device=DEV), H, causal, exact_dq=False)
    Nn.attn_bwd(qkv2, o, lse, d_o, bq, torch.empty(B, H, S, device=DEV), H, causal, exact_dq=True)
    torch.cuda.synchronize()
    assert torch.equal(a[..., HD:], bq[..., HD:])
    assert max_rel(bq[..., :HD], a[..., :HD]) < 1e-2


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("scale,D", [(1.0, 64), (0.05, 128), (0.3, 64)])
def test_attention_with_a_score_factor_of_the_callers(causal, scale, D):
    """The factor on the scores is an argument (models that scale their queries themselves pass 1, some
    pass a constant of their own): forward, log-sum-exp and the three gradients against attention with
    the queries multiplied by scale * sqrt(D) beforehand, which is the same function."""
    Nn = native()
    B, S, H = 2, 192, 3
    torch.manual_seed(int(scale * 100) + D)
    HD = H * D
    qkv = (torch.randn(B, S, 3 * HD, device=DEV) * 0.7).to(torch.bfloat16)
    o = torch.full((B, S, HD), float("nan"), device=DEV, dtype=torch.bfloat16)
    lse = torch.empty(B, H, S, device=DEV)
    Nn.attn_fwd(qkv, o, lse, H, causal, scale=scale)
    d_o = torch.randn(B, S, HD, device=DEV).to(torch.bfloat16)
    dqkv = torch.full_like(qkv, float("nan"))
    delta = torch.empty(B, H, S, device=DEV)
    Nn.attn_bwd(qkv, o, lse, d_o, dqkv, delta, H, causal, scale=scale)
    torch.cuda.synchronize()
    qr = qkv.float().cpu().requires_grad_(True)
    factor = torch.cat([torch.full((HD,), scale * math.sqrt(D)), torch.ones(2 * HD)])
    ref = O.attention_fused_qkv(qr * factor, H, causal)
    assert_close_rel(o, ref, BF16_TOL, "scaled attention fwd")
    ref.backward(d_o.float().cpu())
    for name, sl in (("dq", slice(0, HD)), ("dk", slice(HD, 2 * HD)), ("dv", slice(2 * HD, 3 * HD))):
        assert_close_rel(dqkv[..., sl], qr.grad[..., sl], BF16_TOL, f"scaled attention {name}")


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("B,L,H,Hkv,D", [(2, 100, 2, 2, 64), (1, 40, 3, 3, 64), (2, 193, 2, 1, 128), (1, 330, 4, 2, 64),
                                         (3, 1, 1, 1, 64), (1, 449, 3, 3, 64), (1, 64, 2, 2, 64)])
def test_attention_over_a_padded_sequence_is_attention_over_the_sequence(causal, B, L, H, Hkv, D):
    """A sequence of L tokens handed over in S = the next multiple of 64 rows, the padding rows zero and
    kv_len = L: the first L rows of the output, of the log-sum-exp and (with zero d_o rows in the padding)
    of dq, dk, dv are those of attention over the L tokens."""
    Nn = native()
    torch.manual_seed(7 * L + H)
    S = (L + 63) // 64 * 64
    W = (H + 2 * Hkv) * D
    real = torch.randn(B, L, W).to(torch.bfloat16)
    qkv = torch.zeros(B, S, W, dtype=torch.bfloat16)
    qkv[:, :L] = real
    qkv = qkv.to(DEV)
    o = torch.full((B, S, H * D), float("nan"), device=DEV, dtype=torch.bfloat16)
    lse = torch.empty(B, H, S, device=DEV)
    note(f"padded attention B={B} L={L} S={S} H={H} Hkv={Hkv} D={D} causal={causal}")
    Nn.attn_fwd(qkv, o, lse, H, causal, n_kv_heads=Hkv, kv_len=L)
    torch.cuda.synchronize()
    qr = real.float().requires_grad_(True)
    ref = O.attention_fused_qkv(qr, H, causal, n_kv_heads=Hkv)
    assert_close_rel(o[:, :L], ref, BF16_TOL, "padded attention fwd")
    assert torch.isfinite(o.float()).all() and torch.isfinite(lse).all()
    d_real = torch.randn(B, L, H * D).to(torch.bfloat16)
    d_o = torch.zeros(B, S, H * D, dtype=torch.bfloat16)
    d_o[:, :L] = d_real
    d_o = d_o.to(DEV)
    dqkv = torch.full_like(qkv, float("nan"))
    delta = torch.empty(B, H, S, device=DEV)
    Nn.attn_bwd(qkv, o, lse, d_o, dqkv, delta, H, causal, n_kv_heads=Hkv, kv_len=L)
    torch.cuda.synchronize()
    ref.backward(d_real.float())
    HD, KD = H * D, Hkv * D
    for name, sl in (("dq", slice(0, HD)), ("dk", slice(HD, HD + KD)), ("dv", slice(HD + KD, HD + 2 * KD))):
        assert_close_rel(dqkv[:, :L, sl], qr.grad[..., sl], BF16_TOL, f"padded attention {name}")
    # the padded queries receive no gradient (their d_o rows are zero)
    assert float(dqkv[:, L:, :HD].float().abs().max()) == 0.0 if L < S else True


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("B,S,H,Hkv,D", [(2, 256, 4, 2, 64), (1, 192, 8, 2, 128), (1, 1024, 8, 1, 64),
                                         (2, 128, 6, 3, 64), (1, 64, 16, 8, 64)])
def test_grouped_query_attention(causal, B, S, H, Hkv, D):
    """H query heads on Hkv key / value heads (q | k | v = H, Hkv, Hkv heads of the fused projection):
    the gradients of a key / value head are the sums over its group of query heads."""
    Nn = native()
    torch.manual_seed(S + H + Hkv)
    W = (H + 2 * Hkv) * D
    qkv = torch.randn(B, S, W, device=DEV).to(torch.bfloat16)
    o = torch.full((B, S, H * D), float("nan"), device=DEV, dtype=torch.bfloat16)
    lse = torch.empty(B, H, S, device=DEV)
    note(f"grouped-query attention B={B} S={S} H={H} Hkv={Hkv} D={D} causal={causal}")
    Nn.attn_fwd(qkv, o, lse, H, causal, n_kv_heads=Hkv)
    torch.cuda.synchronize()
    qr = qkv.float().cpu().requires_grad_(True)
    ref = O.attention_fused_qkv(qr, H, causal, n_kv_heads=Hkv)
    assert_close_rel(o, ref, BF16_TOL, "attention fwd")
    d_o = torch.randn(B, S, H * D, device=DEV).to(torch.bfloat16)
    dqkv = torch.full_like(qkv, float("nan"))
    delta = torch.empty(B, H, S, device=DEV)
    Nn.attn_bwd(qkv, o, lse, d_o, dqkv, delta, H, causal, n_kv_heads=Hkv)
    torch.cuda.synchronize()
    ref.backward(d_o.float().cpu())
    HD, KD = H * D, Hkv * D
    for name, sl in (("dq", slice(0, HD)), ("dk", slice(HD, HD + KD)), ("dv", slice(HD + KD, HD + 2 * KD))):
        assert_close_rel(dqkv[..., sl], qr.grad[..., sl], BF16_TOL, f"attention {name}")
    # one key / value head per query head written out by hand gives the same bits as the grouping:
    # the grouped form only shares the loads
    if H <= 8:
        G = H // Hkv
        k_rep = qkv[..., HD:HD + KD].view(B, S, Hkv, D).repeat_interleave(G, dim=2).reshape(B, S, HD)
        v_rep = qkv[..., HD + KD:].view(B, S, Hkv, D).repeat_interleave(G, dim=2).reshape(B, S, HD)
        full = torch.cat([qkv[..., :HD], k_rep, v_rep], dim=-1).contiguous()
        o2 = torch.empty_like(o)
        lse2 = torch.empty_like(lse)
        Nn.attn_fwd(full, o2, lse2, H, causal)
        assert torch.equal(o2, o) and torch.equal(lse2, lse)


def test_grouped_query_attention_rejects_a_group_that_does_not_divide_the_heads():
    Nn = native()
    qkv = torch.zeros(1, 64, (6 + 2 * 4) * 64, device=DEV, dtype=torch.bfloat16)
    o = torch.zeros(1, 64, 6 * 64, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(AssertionError):
        Nn.attn_fwd(qkv, o, torch.zeros(1, 6, 64, device=DEV), 6, True, n_kv_heads=4)


@pytest.mark.parametrize("B,S,H,D,causal", [(4, 1024, 12, 64, True), (8, 512, 12, 64, False),
                                           (1, 2048, 32, 128, True)])
def test_attention_full_size_with_equal_keys_is_a_running_mean(B, S, H, D, causal):
    """The attention shapes of the full-size configurations.  When all keys of a head are the same
    vector every allowed score is equal, so row i of the output is the mean of the values 0..i
    (causal) or of all values, whatever the queries are, and the log-sum-exp is that score plus
    log(count): closed forms computed with cumsum, no O(S^2) reference.  Backward: dQ vanishes and
    dV is a (reversed) cumulative sum of dO / count."""
    Nn = native()
    torch.manual_seed(S + D)
    HD = H * D
    qkv = torch.randn(B, S, 3 * HD, device=DEV).to(torch.bfloat16)
    key = torch.randn(B, 1, HD, device=DEV).to(torch.bfloat16)
    qkv[..., HD:2 * HD] = key                    # one key vector per (batch, head)
    o = torch.full((B, S, HD), float("nan"), device=DEV, dtype=torch.bfloat16)
    lse = torch.empty(B, H, S, device=DEV)
    Nn.attn_fwd(qkv, o, lse, H, causal)
    v = qkv[..., 2 * HD:].float()
    count = torch.arange(1, S + 1, device=DEV, dtype=torch.float32) if causal else \
        torch.full((S,), float(S), device=DEV)
    want = v.cumsum(1) / count.view(1, S, 1) if causal else v.mean(1, keepdim=True).expand(B, S, HD)
    # probabilities are rounded to bf16 before the second product: 2^-9 relative per term
    assert float((o.float() - want).abs().max()) <= 2e-2 * float(want.abs().max())
    q = qkv[..., :HD].float().view(B, S, H, D)
    score = (q * key.float().view(B, 1, H, D)).sum(-1) / math.sqrt(D)          # [B, S, H]
    want_lse = score.permute(0, 2, 1) + torch.log(count).view(1, 1, S)
    assert float((lse - want_lse).abs().max()) <= 1e-2 * max(1.0, float(want_lse.abs().max()))
    # backward: uniform probabilities do not depend on the queries, so dQ = 0, and
    # dV[j] = sum over the rows i that see key j of dO[i] / count[i] (a reversed cumsum when causal)
    d_o = torch.randn(B, S, HD, device=DEV).to(torch.bfloat16)
    dqkv = torch.full_like(qkv, float("nan"))
    delta = torch.empty(B, H, S, device=DEV)
    Nn.attn_bwd(qkv, o, lse, d_o, dqkv, delta, H, causal)
    w = d_o.float() / count.view(1, S, 1)
    want_dv = w.flip(1).cumsum(1).flip(1) if causal else w.sum(1, keepdim=True).expand(B, S, HD)
    got_dv = dqkv[..., 2 * HD:].float()
    assert float((got_dv - want_dv).abs().max()) <= 2e-2 * float(want_dv.abs().max())
    # dQ is a sum of terms that cancel: compare with the size of the terms, |dO| |V| |K| / sqrt(D)
    term = float(d_o.float().abs().max() * v.abs().max() * key.float().abs().max()) / math.sqrt(D)
    assert float(dqkv[..., :HD].float().abs().max()) <= 2e-2 * term
    assert bool(torch.isfinite(dqkv.float()).all())


@pytest.mark.parametrize("M,N,K,at,bt", [(4096, 768, 768, False, False), (4096, 2304, 768, False, False),
                                         (4096, 50304, 768, False, False), (4096, 768, 50304, False, False),
                                         (3072, 768, 4096, True, True), (2048, 11008, 4096, False, False)])
def test_gemm_bf16_full_size_selects_rows_exactly(M, N, K, at, bt):
    """GEMM shapes of the full-size configurations (every tile shape the dispatcher picks).  With
    one-hot rows in A the product is a row selection of B: C[m, :] = B[:, k_m], which bf16
    reproduces exactly, so every element of C checks the indexing of its tile bit for bit."""
    Nn = native()
    g = torch.Generator(device=DEV).manual_seed(M + N + K)
    pick = torch.randint(0, K, (M,), device=DEV, generator=g)
    A = torch.zeros(M, K, device=DEV, dtype=torch.bfloat16)
    A[torch.arange(M, device=DEV), pick] = 1
    Bm = torch.randn(N, K, device=DEV, generator=g).to(torch.bfloat16)
    want = Bm[:, pick].t().contiguous()
    Aop = A.t().contiguous() if at else A
    Bop = Bm.t().contiguous() if bt else Bm
    C = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
    Nn.gemm_bf16(Aop, Bop, C, a_trans=at, b_trans=bt)
    assert torch.equal(C, want)


@pytest.mark.parametrize("M,N,K", [(4096, 768, 50304), (512, 256, 16384), (300, 200, 9000), (4096, 768, 768)])
def test_gemm_bf16_split_along_k(M, N, K):
    """pp_gemm_bf16_splitk: a long reduction into a small output runs as several k-splits on
    256 x 256 tiles whose fp32 partial results are added in split order; problems it is not meant
    for (the last case) fall back to the ordinary kernel.  One-hot rows in A make the exact answer
    a row selection of B; random operands are compared with the fp32 product, and two runs agree."""
    Nn = native()
    g = torch.Generator(device=DEV).manual_seed(M + K)
    ws = torch.empty(8 * M * N, device=DEV, dtype=torch.float32)
    pick = torch.randint(0, K, (M,), device=DEV, generator=g)
    A = torch.zeros(M, K, device=DEV, dtype=torch.bfloat16)
    A[torch.arange(M, device=DEV), pick] = 1
    Bm = torch.randn(N, K, device=DEV, generator=g).to(torch.bfloat16)
    C = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
    Nn.gemm_bf16_splitk(A, Bm, C, ws)
    assert torch.equal(C, Bm[:, pick].t().contiguous())
    A = (torch.randn(M, K, device=DEV, generator=g) * 0.5).to(torch.bfloat16)
    runs = []
    for _ in range(2):
        C = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
        ws.fill_(float("nan"))
        Nn.gemm_bf16_splitk(A, Bm, C, ws)
        runs.append(C)
    assert torch.equal(runs[0], runs[1])
    ref = A.float() @ Bm.float().t()
    assert_close_rel(runs[0], ref.cpu(), BF16_TOL, "split-K GEMM")
    small = torch.empty(M * N, device=DEV, dtype=torch.float32)     # room for one copy only: no split
    Nn.gemm_bf16_splitk(A, Bm, C, small)
    assert_close_rel(C, ref.cpu(), BF16_TOL, "split-K GEMM without room to split")


# ---- launch list ---------------------------------------------------------------------------------
def test_run_ops_matches_direct_calls():
    import ctypes as C
    Nn = native()
    torch.manual_seed(13)
    M, N, K = 256, 128, 64
    A = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    W = torch.randn(N, K, device=DEV).to(torch.bfloat16)
    bias = torch.randn(N, device=DEV).to(torch.bfloat16)
    C1 = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    C2 = torch.empty_like(C1)
    acc1 = torch.zeros(M * N, device=DEV)
    acc2 = torch.zeros(M * N, device=DEV)
    Nn.gemm_bf16(A, W, C1, epilogue=Nn.EPI_BIAS, bias=bias)
    Nn.grad_accum(acc1, C1.reshape(-1), init=True)
    ops = (Nn.Op * 2)()
    g = ops[0]
    g.kind = Nn.OP_GEMM_BF16
    g.p[0], g.p[1], g.p[2], g.p[3] = A.data_ptr(), W.data_ptr(), C2.data_ptr(), bias.data_ptr()
    g.i[0], g.i[1], g.i[2], g.i[3], g.i[4], g.i[5] = M, N, K, K, K, N
    g.j[2], g.j[3] = Nn.EPI_BIAS, Nn.PP_BF16
    a = ops[1]
    a.kind = Nn.OP_ACCUM_BF16
    a.p[0], a.p[1] = acc2.data_ptr(), C2.data_ptr()
    a.i[0] = M * N
    a.j[0] = 1
    Nn.run_ops(ops, 2)
    assert torch.equal(C1, C2) and torch.equal(acc1, acc2)
    ops[1].kind = 999
    with pytest.raises(RuntimeError, match="op 1"):
        Nn.run_ops(ops, 2)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, F32_TOL), (torch.bfloat16, BF16_TOL)])
@pytest.mark.parametrize("act", ["relu", "gelu_erf", "gelu_tanh"])
def test_activation_bwd(dtype, tol, act):
    Nn = native()
    torch.manual_seed(14)
    n = 64 * 512 + 5
    aux = torch.randn(n, device=DEV).to(dtype)
    dy = torch.randn(n, device=DEV).to(dtype)
    dz = torch.empty_like(dy)
    kind = {"relu": Nn.ACT_RELU, "gelu_erf": Nn.ACT_GELU_ERF, "gelu_tanh": Nn.ACT_GELU_TANH}[act]
    Nn.activation_bwd(dy, aux, dz, kind)
    a = aux.float().cpu().requires_grad_(True)
    fn = {"relu": torch.relu, "gelu_erf": O.gelu_erf, "gelu_tanh": O.gelu_tanh}[act]
    fn(a).backward(dy.float().cpu())
    assert_close_rel(dz, a.grad, tol, f"activation bwd {act}")


def test_erf_gelu_derivative_over_its_whole_range():
    """The erf form of GELU is computed through a rational-exponential form of erfc (absolute error below
    1.5e-7) instead of the library's erff: its derivative Phi(x) + x phi(x), taken by the stand-alone kernel in
    fp32 on a grid over [-9, 9], stays within 1e-6 of the fp64 value everywhere, and the tail towards -inf keeps
    its sign and decays (no cancellation 1 - (1 - tiny))."""
    Nn = native()
    x = torch.linspace(-9.0, 9.0, 360001, device=DEV)
    dz = torch.empty_like(x)
    Nn.activation_bwd(torch.ones_like(x), x, dz, Nn.ACT_GELU_ERF)
    xd = x.double().cpu()
    exact = 0.5 * (1.0 + torch.erf(xd / 2.0 ** 0.5)) + xd * torch.exp(-0.5 * xd * xd) / (2.0 * torch.pi) ** 0.5
    assert (dz.double().cpu() - exact).abs().max() <= 1e-6
    tail = dz[x < -6.0]
    assert bool((tail <= 0).all()) and bool((tail.abs() <= 1e-7).all())


# ---- optimizer step on the fp32 accumulators -----------------------------------------------------
from oracle import optim as OO
import numpy as np


def _bf16_ulp_diff(a: torch.Tensor, b: torch.Tensor) -> int:
    ia = a.view(torch.int16).to(torch.int32)
    ib = b.view(torch.int16).to(torch.int32)
    return int((ia - ib).abs().max())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("momentum,dampening,wd,nesterov", [(0.0, 0.0, 0.0, False), (0.9, 0.0, 0.01, False),
                                                            (0.9, 0.0, 0.0, True), (0.8, 0.2, 0.1, False)])
@pytest.mark.parametrize("master", [False, True])
def test_sgd_step_matches_oracle(dtype, momentum, dampening, wd, nesterov, master):
    if master and dtype != torch.bfloat16:
        pytest.skip("a master copy goes with bf16 parameters")
    N = native()
    n = 4 * 1000 + 4
    g0 = torch.Generator().manual_seed(11)
    p_host = torch.randn(n, generator=g0).to(dtype)
    p = p_host.cuda()
    mst = p.float() if master else None
    buf = torch.zeros(n, device="cuda") if momentum else None
    p_o = p_host.float().numpy().copy()
    buf_o = None
    for step in range(3):
        grad = torch.randn(n, generator=g0)
        N.sgd_step(p, grad.cuda(), buf, master=mst, lr=0.05, momentum=momentum, dampening=dampening,
                   weight_decay=wd, nesterov=nesterov, first_step=step == 0)
        p_o, buf_o = OO.sgd_step(p_o, grad.numpy(), buf_o, lr=0.05, momentum=momentum, dampening=dampening,
                                 weight_decay=wd, nesterov=nesterov, first_step=step == 0)
        if dtype == torch.float32:
            assert_close_rel(p.cpu(), torch.from_numpy(p_o), 2e-6, "sgd fp32 parameters")
        elif master:
            assert_close_rel(mst.cpu(), torch.from_numpy(p_o), 2e-6, "sgd master copy")
            assert _bf16_ulp_diff(p.cpu(), torch.from_numpy(OO.round_bf16(p_o)).to(torch.bfloat16)) <= 1
        else:
            # the parameter is re-rounded to bf16 every step; the oracle does the same
            p_o = OO.round_bf16(p_o)
            assert _bf16_ulp_diff(p.cpu(), torch.from_numpy(p_o).to(torch.bfloat16)) <= 1
            p_o = p.cpu().float().numpy().copy()  # continue from the device value so 1-ulp ties do not compound
        if momentum:
            assert_close_rel(buf.cpu(), torch.from_numpy(buf_o), 2e-6, "sgd momentum buffer")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,master", [(torch.float32, False), (torch.bfloat16, False), (torch.bfloat16, True)])
@pytest.mark.parametrize("wd", [0.0, 0.1])
def test_adamw_step_matches_oracle(dtype, master, wd):
    N = native()
    n = 4 * 777
    g0 = torch.Generator().manual_seed(13)
    p_host = torch.randn(n, generator=g0).to(dtype)
    p = p_host.cuda()
    mst = p.float() if master else None
    m = torch.zeros(n, device="cuda")
    v = torch.zeros(n, device="cuda")
    p_o = p_host.float().numpy().copy()
    m_o = np.zeros(n, np.float32)
    v_o = np.zeros(n, np.float32)
    lr, b1, b2, eps = 1e-2, 0.9, 0.95, 1e-8
    for step in range(1, 4):
        grad = torch.randn(n, generator=g0)
        N.adamw_step(p, grad.cuda(), m, v, master=mst, lr=lr, beta1=b1, beta2=b2, eps=eps, weight_decay=wd,
                     bias_correction1=1 - b1 ** step, bias_correction2_sqrt=math.sqrt(1 - b2 ** step))
        p_o, m_o, v_o = OO.adamw_step(p_o, grad.numpy(), m_o, v_o, lr=lr, beta1=b1, beta2=b2, eps=eps,
                                      weight_decay=wd, step=step)
        assert_close_rel(m.cpu(), torch.from_numpy(m_o), 2e-6, "adamw exp_avg")
        assert_close_rel(v.cpu(), torch.from_numpy(v_o), 2e-6, "adamw exp_avg_sq")
        if dtype == torch.float32:
            assert_close_rel(p.cpu(), torch.from_numpy(p_o), 3e-6, "adamw fp32 parameters")
        elif master:
            assert_close_rel(mst.cpu(), torch.from_numpy(p_o), 3e-6, "adamw master copy")
            assert _bf16_ulp_diff(p.cpu(), torch.from_numpy(OO.round_bf16(p_o)).to(torch.bfloat16)) <= 1
        else:
            assert _bf16_ulp_diff(p.cpu(), torch.from_numpy(OO.round_bf16(p_o)).to(torch.bfloat16)) <= 1
            p_o = p.cpu().float().numpy().copy()


@pytest.mark.gpu
def test_optimizer_steps_reject_bad_arguments():
    N = native()
    p = torch.zeros(6, device="cuda")
    g = torch.zeros(6, device="cuda")
    with pytest.raises(RuntimeError, match="multiple of 4"):
        N.sgd_step(p, g, None, lr=0.1)
    p = torch.zeros(8, device="cuda")
    g = torch.zeros(8, device="cuda")
    with pytest.raises(RuntimeError, match="momentum needs"):
        N.sgd_step(p, g, None, lr=0.1, momentum=0.9)
    with pytest.raises(RuntimeError, match="master copy goes with bf16"):
        N.sgd_step(p, g, None, master=torch.zeros(8, device="cuda"), lr=0.1)


# ---- RMSNorm, SwiGLU, RoPE ----------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("rows,C", [(64, 4096), (37, 1024), (5, 128)])
def test_rmsnorm_matches_oracle(rows, C):
    N = native()
    g0 = torch.Generator().manual_seed(rows)
    x = (torch.randn(rows, C, generator=g0) * 2).to(torch.bfloat16)
    w = (1 + 0.1 * torch.randn(C, generator=g0)).to(torch.bfloat16)
    dy = torch.randn(rows, C, generator=g0).to(torch.bfloat16)
    dres = torch.randn(rows, C, generator=g0).to(torch.bfloat16)
    xd, wd, dyd, dresd = x.cuda(), w.cuda(), dy.cuda(), dres.cuda()
    y = torch.empty_like(xd)
    rstd = torch.empty(rows, device="cuda")
    N.layernorm_fwd(xd, wd, None, y, None, rstd, 1e-5)
    xr = x.float().requires_grad_(True)
    wr = w.float().requires_grad_(True)
    yr = O.rms_norm(xr, wr, 1e-5)
    assert_close_rel(y, yr.detach(), BF16_TOL, "rmsnorm forward")
    yr.backward(dy.float())
    dx = torch.empty_like(xd)
    N.layernorm_bwd_input(dyd, xd, wd, None, rstd, dresd, dx)
    assert_close_rel(dx, xr.grad + dres.float(), BF16_TOL, "rmsnorm input gradient (+ residual)")
    dgamma = torch.empty(C, device="cuda")
    ws = torch.empty(2 * ((rows + 127) // 128) * C, device="cuda")
    N.layernorm_bwd_weight(dyd, xd, None, rstd, dgamma, None, ws)
    assert_close_rel(dgamma, wr.grad, 1e-3, "rmsnorm weight gradient")


@pytest.mark.gpu
@pytest.mark.parametrize("n", [8, 2048 * 11008, 1000 * 8])
def test_swiglu_matches_oracle(n):
    N = native()
    g0 = torch.Generator().manual_seed(n % 97)
    g = (torch.randn(n, generator=g0) * 2).to(torch.bfloat16)
    u = torch.randn(n, generator=g0).to(torch.bfloat16)
    dh = torch.randn(n, generator=g0).to(torch.bfloat16)
    gd, ud, dhd = g.cuda(), u.cuda(), dh.cuda()
    h = torch.empty_like(gd)
    N.swiglu_fwd(gd, ud, h)
    gr, ur = g.float().requires_grad_(True), u.float().requires_grad_(True)
    hr = O.swiglu(gr, ur)
    assert_close_rel(h, hr.detach(), BF16_TOL, "swiglu forward")
    hr.backward(dh.float())
    dg, du = torch.empty_like(gd), torch.empty_like(gd)
    N.swiglu_bwd(gd, ud, dhd, dg, du)
    assert_close_rel(dg, gr.grad, BF16_TOL, "swiglu gate gradient")
    assert_close_rel(du, ur.grad, BF16_TOL, "swiglu up gradient")


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,F", [(4096, 1024, 2816), (130, 72, 200), (1, 8, 8), (257, 4096, 344),
                                   # outputs that fill the CUs with 256-row tiles on 8 waves: forward 256 x 256,
                                   # backward 256 x 192 (first) and 256 x 256 (the other two), the second with ragged edges
                                   (2048, 264, 11008), (2050, 72, 11016), (2048, 136, 8192)])
def test_gemm_fused_swiglu_equals_the_separate_kernels_and_the_oracle(M, K, F):
    """The gate / up GEMM that applies SwiGLU in its epilogue, and the down projection's input-gradient
    GEMM that applies its derivative, leave the bits of the GEMMs followed by the element-wise kernels
    (values are rounded to bf16 at the same points); the oracle's fp32 feed-forward pins both."""
    N = native()
    g0 = torch.Generator().manual_seed(M + F)
    x = torch.randn(M, K, generator=g0).to(torch.bfloat16)
    wg = (torch.randn(F, K, generator=g0) / K ** 0.5 * 2).to(torch.bfloat16)
    wu = (torch.randn(F, K, generator=g0) / K ** 0.5).to(torch.bfloat16)
    wd = (torch.randn(K, F, generator=g0) / F ** 0.5).to(torch.bfloat16)   # down projection [out=K, in=F]
    dy = torch.randn(M, K, generator=g0).to(torch.bfloat16)
    xd, wgd, wud, dyd = x.cuda(), wg.cuda(), wu.cuda(), dy.cuda()
    wdt = wd.t().contiguous().cuda()                                       # [F, K]
    # separate kernels
    g = torch.empty(M, F, device="cuda", dtype=torch.bfloat16)
    u, h, dh, dg, du = (torch.empty_like(g) for _ in range(5))
    N.gemm_bf16(xd, wgd, g)
    N.gemm_bf16(xd, wud, u)
    N.swiglu_fwd(g, u, h)
    N.gemm_bf16(dyd, wdt, dh)
    N.swiglu_bwd(g, u, dh, dg, du)
    # fused, into buffers with a recognisable fill so that stray writes show
    gu = torch.full((M, 2 * F), 7.0, device="cuda", dtype=torch.bfloat16)
    hf = torch.full((M, F), 7.0, device="cuda", dtype=torch.bfloat16)
    dgu = torch.full((M, 2 * F), 7.0, device="cuda", dtype=torch.bfloat16)
    N.gemm_swiglu(xd, wgd, wud, gu, hf)
    N.gemm_dswiglu(dyd, wdt, gu, dgu)
    torch.cuda.synchronize()
    assert torch.equal(gu[:, :F], g) and torch.equal(gu[:, F:], u), "gate / up products"
    assert torch.equal(hf, h), "activation"
    assert torch.equal(dgu[:, :F], dg) and torch.equal(dgu[:, F:], du), "gate / up gradients"
    # oracle: fp32 feed-forward and its autograd gradients
    gr = (x.float() @ wg.float().t()).requires_grad_(True)
    ur = (x.float() @ wu.float().t()).requires_grad_(True)
    hr = O.swiglu(gr, ur)
    assert_close_rel(hf, hr.detach(), BF16_TOL, "fused swiglu forward")
    hr.backward(dy.float() @ wd.float())
    assert_close_rel(dgu[:, :F], gr.grad, 2 * BF16_TOL, "fused gate gradient")
    assert_close_rel(dgu[:, F:], ur.grad, 2 * BF16_TOL, "fused up gradient")


@pytest.mark.gpu
def test_gemm_fused_swiglu_rejects_bad_arguments():
    N = native()
    x = torch.zeros(16, 8, device="cuda", dtype=torch.bfloat16)
    w = torch.zeros(12, 8, device="cuda", dtype=torch.bfloat16)   # N = 12 is not a multiple of 8
    gu = torch.zeros(16, 24, device="cuda", dtype=torch.bfloat16)
    h = torch.zeros(16, 12, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        N.gemm_swiglu(x, w, w, gu, h)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        N.gemm_dswiglu(x, w, gu, gu.clone())
    seg = torch.tensor([0, 16], dtype=torch.int32, device="cuda")
    ptr = torch.tensor([w.data_ptr()], dtype=torch.int64, device="cuda")
    with pytest.raises(RuntimeError, match="multiple of 8"):
        N.gemm_segmented_swiglu(x, ptr, ptr, seg, gu, h)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        N.gemm_segmented_dswiglu(x, ptr, seg, gu, gu.clone())


@pytest.mark.gpu
@pytest.mark.parametrize("B,S,H,D", [(2, 64, 3, 64), (1, 2048, 4, 128), (3, 16, 2, 32)])
def test_rope_matches_oracle_and_inverts(B, S, H, D):
    N = native()
    g0 = torch.Generator().manual_seed(S + D)
    qkv = torch.randn(B * S, 3 * H * D, generator=g0).to(torch.bfloat16)
    cos, sin = O.rope_tables(S, D)
    x = qkv.cuda()
    N.rope(x, cos.cuda(), sin.cuda(), S, 2 * H, D)
    ref = qkv.float().view(B, S, 3, H, D).clone()
    ref[:, :, 0] = O.rope(ref[:, :, 0].transpose(1, 2), cos, sin).transpose(1, 2)
    ref[:, :, 1] = O.rope(ref[:, :, 1].transpose(1, 2), cos, sin).transpose(1, 2)
    assert_close_rel(x, ref.view(B * S, 3 * H * D), BF16_TOL, "rope on the q and k heads")
    # the v third of every row is untouched, bit for bit
    assert torch.equal(x.view(B * S, 3, H * D)[:, 2].cpu(), qkv.view(B * S, 3, H * D)[:, 2])
    # the inverse rotation brings q and k back (two bf16 roundings away)
    N.rope(x, cos.cuda(), sin.cuda(), S, 2 * H, D, inverse=True)
    assert_close_rel(x, qkv.float(), BF16_TOL, "rope followed by its transpose")


# ---- mixture-of-experts routing and segmented GEMMs ---------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("T,E", [(2048, 8), (77, 3), (1000, 64)])
def test_moe_router_top2_matches_oracle(T, E):
    N = native()
    torch.manual_seed(0)
    logits = (torch.randn(T, E) * 0.6).to(torch.bfloat16)     # bf16 values: ties do occur
    logits[0] = 1.0                                            # a row of equal logits
    idx = torch.empty(T, 2, dtype=torch.int32, device=DEV)
    gate = torch.empty(T, 2, dtype=torch.float32, device=DEV)
    N.moe_router_top2(logits.to(DEV), idx, gate)
    ref_idx, ref_gate = O.moe_route_top2(logits.float())
    assert torch.equal(idx.cpu().long(), ref_idx)
    assert (gate.cpu() - ref_gate).abs().max() <= 1e-6
    # where the three largest values are distinct the selection is torch.topk's
    top3 = torch.topk(logits.float(), min(3, E), -1).values
    clean = (top3[:, 0] != top3[:, 1]) & ((top3[:, 1] != top3[:, 2]) if E > 2 else True)
    assert clean.sum() > T // 2
    assert torch.equal(idx.cpu().long()[clean], torch.topk(logits.float(), 2, -1).indices[clean])


@pytest.mark.gpu
@pytest.mark.parametrize("n,E", [(4096, 8), (5001, 3), (10, 64), (0, 4)])
def test_moe_permute_bit_exact(n, E):
    N = native()
    torch.manual_seed(1)
    slots = torch.randint(0, E, (n,), dtype=torch.int32)
    if n > 100:
        slots[slots == 1] = 0                                  # an expert without tokens
    seg = torch.full((E + 1,), -7, dtype=torch.int32, device=DEV)
    row_src = torch.full((n,), -7, dtype=torch.int32, device=DEV)
    pos = torch.full((n,), -7, dtype=torch.int32, device=DEV)
    N.moe_permute(slots.to(DEV), E, seg, row_src, pos)
    ref_seg, ref_rows, ref_pos = O.moe_permutation(slots, E)
    assert torch.equal(seg.cpu().long(), ref_seg)
    assert torch.equal(row_src.cpu().long(), ref_rows)
    assert torch.equal(pos.cpu().long(), ref_pos)


@pytest.mark.gpu
def test_moe_permute_drops_slots_with_an_invalid_expert():
    N = native()
    slots = torch.tensor([2, 9, 0, -1, 2, 1], dtype=torch.int32)
    seg = torch.empty(4, dtype=torch.int32, device=DEV)
    row_src = torch.full((6,), -7, dtype=torch.int32, device=DEV)
    pos = torch.empty(6, dtype=torch.int32, device=DEV)
    N.moe_permute(slots.to(DEV), 3, seg, row_src, pos)
    assert seg.tolist() == [0, 1, 2, 4]
    assert row_src.tolist()[:4] == [2, 5, 0, 4]
    assert pos.tolist() == [2, -1, 0, -1, 3, 1]


@pytest.mark.gpu
def test_moe_gather_and_combine():
    N = native()
    torch.manual_seed(2)
    T, Cc, K, E = 300, 256, 2, 8
    x = torch.randn(T, Cc).to(torch.bfloat16)
    slots = torch.randint(0, E, (T * K,), dtype=torch.int32)
    _, row_src, pos = O.moe_permutation(slots, E)
    gate = torch.rand(T * K)
    xd, rows_d, pos_d, gate_d = x.to(DEV), row_src.int().to(DEV), pos.int().to(DEV), gate.to(DEV)
    out = torch.empty(T * K, Cc, dtype=torch.bfloat16, device=DEV)
    N.moe_gather(xd, rows_d, K, out)
    assert torch.equal(out.cpu(), x[row_src // K])               # a plain gather moves bytes
    N.moe_gather(xd, rows_d, K, out, scale=gate_d)
    ref = (gate[row_src, None] * x[row_src // K].float())
    assert torch.equal(out.cpu(), ref.to(torch.bfloat16))        # one product, one rounding
    # only the first *n_rows rows are written
    out.fill_(7)
    n_rows = torch.tensor([10], dtype=torch.int32, device=DEV)
    N.moe_gather(xd, rows_d, K, out, n_rows=n_rows)
    assert torch.equal(out[:10].cpu(), x[row_src[:10] // K]) and bool((out[10:] == 7).all())
    # combine: resid + sum_k gate * y[pos]
    y = torch.randn(T * K, Cc).to(torch.bfloat16)
    resid = torch.randn(T, Cc).to(torch.bfloat16)
    res = torch.empty(T, Cc, dtype=torch.bfloat16, device=DEV)
    N.moe_combine(y.to(DEV), pos_d, K, res, gate=gate_d, resid=resid.to(DEV))
    ref = resid.float() + (gate.view(T, K, 1) * y.float()[pos].view(T, K, Cc)).sum(1)
    assert_close_rel(res, ref, 4e-3, "combine")                  # one bf16 rounding of an fp32 sum
    N.moe_combine(y.to(DEV), pos_d, K, res)
    assert_close_rel(res, y.float()[pos].view(T, K, Cc).sum(1), 4e-3, "unweighted combine")


@pytest.mark.gpu
@pytest.mark.parametrize("E", [8, 5, 12, 64])
def test_moe_gate_bwd_matches_autograd(E):
    N = native()
    torch.manual_seed(3)
    T, Cc, K = 200, 128, 2
    logits = (torch.randn(T, E) * 0.6).to(torch.bfloat16)
    idx, gate = O.moe_route_top2(logits.float())
    _, row_src, pos = O.moe_permutation(idx, E)
    y = torch.randn(T * K, Cc).to(torch.bfloat16)
    dout = (torch.randn(T, Cc) * 0.1).to(torch.bfloat16)
    # autograd through softmax -> gather -> renormalise -> weighted sum of the expert rows
    lg = logits.float().requires_grad_()
    top = torch.softmax(lg, -1).gather(-1, idx)
    g = top / top.sum(-1, keepdim=True)
    out = (g.unsqueeze(-1) * y.float()[pos].view(T, K, Cc)).sum(1)
    out.backward(dout.float())
    Ep = (E + 7) // 8 * 8                                   # logits are stored padded to a multiple of 8
    dl = torch.full((T, Ep), 7.0, dtype=torch.bfloat16, device=DEV)
    N.moe_gate_bwd(dout.to(DEV), y.to(DEV), pos.int().to(DEV), idx.int().to(DEV), gate.to(DEV), E, dl)
    assert_close_rel(dl[:, :E], lg.grad, BF16_TOL, "router logit gradient")
    unselected = torch.ones(T, E, dtype=torch.bool).scatter(1, idx, False)
    assert bool((dl.cpu()[:, :E][unselected] == 0).all())
    assert float(dl[:, E:].float().abs().sum()) == 0.0      # the padding columns come back as zeros


def _segments(R, E, seed):
    g = torch.Generator().manual_seed(seed)
    cuts = torch.sort(torch.randint(0, R + 1, (E - 1,), generator=g)).values
    seg = torch.cat([torch.zeros(1, dtype=torch.long), cuts, torch.tensor([R])])
    return seg


@pytest.mark.gpu
@pytest.mark.parametrize("R,K,Nn,E", [(4096, 1024, 512, 8), (1000, 256, 384, 5), (130, 64, 128, 3),
                                      (3000, 64, 136, 63), (3000, 64, 136, 64), (2000, 64, 128, 130)])
def test_segmented_gemm_rows_mode(R, K, Nn, E):
    N = native()
    torch.manual_seed(4)
    seg = _segments(R, E, R)
    seg[2] = seg[1]                                              # an empty segment
    A = (torch.randn(R, K) * 0.5).to(torch.bfloat16)
    W = (torch.randn(E, Nn, K) * 0.05).to(torch.bfloat16)
    aux = torch.randn(R, Nn).to(torch.bfloat16)
    Ad, Wd, auxd = A.to(DEV), W.to(DEV), aux.to(DEV)
    ptrs = torch.tensor([Wd[e].data_ptr() for e in range(E)], dtype=torch.int64, device=DEV)
    segd = seg.int().to(DEV)
    ref = torch.empty(R, Nn)
    for e in range(E):
        r0, r1 = int(seg[e]), int(seg[e + 1])
        ref[r0:r1] = A[r0:r1].float() @ W[e].float().T
    Cm = torch.full((R, Nn), 3.0, dtype=torch.bfloat16, device=DEV)
    N.gemm_bf16_segmented(Ad, ptrs, Cm, segd, N.SEG_ROWS)
    assert_close_rel(Cm, ref, BF16_TOL, "segmented rows")
    N.gemm_bf16_segmented(Ad, ptrs, Cm, segd, N.SEG_ROWS, epilogue=N.EPI_BIAS_RESIDUAL, aux_in=auxd)
    assert_close_rel(Cm, ref + aux.float(), BF16_TOL, "segmented rows + residual")


@pytest.mark.gpu
@pytest.mark.parametrize("R,K,F,E", [(4096, 1024, 512, 8), (1000, 256, 384, 5), (130, 64, 128, 3),
                                     (3000, 64, 136, 63), (2000, 64, 128, 130)])
def test_segmented_gemms_with_swiglu_inside_leave_the_bits_of_the_separate_kernels(R, K, F, E):
    """The expert feed-forward's gate / up GEMM with SwiGLU in its epilogue, and the down projection's
    input-gradient GEMM with its derivative, over ragged row segments with a weight each (one of them
    empty): the bits of the segmented GEMMs followed by the element-wise kernels; rows and columns that
    belong to no tile of a segment keep their fill."""
    N = native()
    torch.manual_seed(R + F)
    seg = _segments(R, E, R + 1)
    seg[2] = seg[1]
    x = (torch.randn(R, K) * 0.5).to(torch.bfloat16).to(DEV)
    dy = (torch.randn(R, K) * 0.5).to(torch.bfloat16).to(DEV)
    wg = (torch.randn(E, F, K) * 0.1).to(torch.bfloat16).to(DEV)
    wu = (torch.randn(E, F, K) * 0.05).to(torch.bfloat16).to(DEV)
    wdt = (torch.randn(E, F, K) * 0.05).to(torch.bfloat16).to(DEV)
    ptrs = lambda w: torch.tensor([w[e].data_ptr() for e in range(E)], dtype=torch.int64, device=DEV)
    pg, pu, pd = ptrs(wg), ptrs(wu), ptrs(wdt)
    segd = seg.int().to(DEV)
    g = torch.empty(R, F, dtype=torch.bfloat16, device=DEV)
    u, h, dh, dg, du = (torch.empty_like(g) for _ in range(5))
    N.gemm_bf16_segmented(x, pg, g, segd, N.SEG_ROWS)
    N.gemm_bf16_segmented(x, pu, u, segd, N.SEG_ROWS)
    N.swiglu_fwd(g, u, h)
    N.gemm_bf16_segmented(dy, pd, dh, segd, N.SEG_ROWS)
    N.swiglu_bwd(g, u, dh, dg, du)
    gu = torch.full((R, 2 * F + 8), 7.0, dtype=torch.bfloat16, device=DEV)      # a leading dimension beyond 2 F
    hf = torch.full((R, F), 7.0, dtype=torch.bfloat16, device=DEV)
    dgu = torch.full((R, 2 * F + 8), 7.0, dtype=torch.bfloat16, device=DEV)
    N.gemm_segmented_swiglu(x, pg, pu, segd, gu[:, :2 * F], hf)
    N.gemm_segmented_dswiglu(dy, pd, segd, gu[:, :2 * F], dgu[:, :2 * F])
    torch.cuda.synchronize()
    assert torch.equal(gu[:, :F], g) and torch.equal(gu[:, F:2 * F], u), "gate / up products"
    assert torch.equal(hf, h), "activation"
    assert torch.equal(dgu[:, :F], dg) and torch.equal(dgu[:, F:2 * F], du), "gate / up gradients"
    assert bool((gu[:, 2 * F:] == 7.0).all()) and bool((dgu[:, 2 * F:] == 7.0).all()), "stray writes"
    # fp32 statement of one non-empty segment
    e = int(torch.argmax(seg[1:] - seg[:-1]))
    r0, r1 = int(seg[e]), int(seg[e + 1])
    gr = x[r0:r1].float() @ wg[e].float().T
    ur = x[r0:r1].float() @ wu[e].float().T
    assert_close_rel(hf[r0:r1], torch.nn.functional.silu(gr) * ur, BF16_TOL, "segment of h")


@pytest.mark.gpu
def test_segmented_gemms_full_size_equal_one_dense_gemm_per_expert():
    """The expert GEMMs of the Mixtral-style configuration (4096 permuted rows, 8 ragged segments,
    1024 -> 4096): the segmented kernels run the dense kernel's tile code, so rows mode must give
    the bits of one dense GEMM per expert, k mode those of one transposed dense GEMM per expert
    (also through the rounded accumulation), and a second run the same bits again."""
    N = native()
    torch.manual_seed(41)
    R, K, Nn, E = 4096, 1024, 4096, 8
    bounds = [0, 450, 1010, 1500, 1500, 2560, 3100, 3620, 4096]     # one empty segment
    seg = torch.tensor(bounds, dtype=torch.int32, device=DEV)
    A = (torch.randn(R, K, device=DEV) * 0.5).to(torch.bfloat16)
    W = (torch.randn(E, Nn, K, device=DEV) * 0.05).to(torch.bfloat16)
    ptrs = torch.tensor([W[e].data_ptr() for e in range(E)], dtype=torch.int64, device=DEV)
    want = torch.zeros(R, Nn, device=DEV, dtype=torch.bfloat16)
    for e in range(E):
        r0, r1 = bounds[e], bounds[e + 1]
        if r1 > r0:
            N.gemm_bf16(A[r0:r1], W[e], want[r0:r1])
    for _ in range(2):
        got = torch.full((R, Nn), float("nan"), device=DEV, dtype=torch.bfloat16)
        N.gemm_bf16_segmented(A, ptrs, got, seg, N.SEG_ROWS)
        assert torch.equal(got, want)
    # k mode: dW_e = dY[r0:r1]^T X[r0:r1], accumulated on top of earlier sums
    dY = (torch.randn(R, Nn, device=DEV) * 0.5).to(torch.bfloat16)
    start = torch.randn(E, Nn, K, device=DEV)
    want_acc = start.clone()
    g = torch.empty(Nn, K, device=DEV, dtype=torch.bfloat16)
    for e in range(E):
        r0, r1 = bounds[e], bounds[e + 1]
        if r1 > r0:
            rows = (r1 - r0 + 7) // 8 * 8          # the dense entry point wants K in multiples of 8
            dYp = torch.zeros(rows, Nn, device=DEV, dtype=torch.bfloat16)
            Xp = torch.zeros(rows, K, device=DEV, dtype=torch.bfloat16)
            dYp[:r1 - r0], Xp[:r1 - r0] = dY[r0:r1], A[r0:r1]
            N.gemm_bf16(dYp, Xp, g, a_trans=True, b_trans=True)
            want_acc[e] += g.float()
    for _ in range(2):
        acc = start.clone()
        aptrs = torch.tensor([acc[e].data_ptr() for e in range(E)], dtype=torch.int64, device=DEV)
        N.gemm_bf16_segmented(dY, aptrs, None, seg, N.SEG_K, other=A, epilogue=N.EPI_ACCUM_ROUNDED, beta=1,
                              c_dtype=torch.float32)
        assert torch.equal(acc, want_acc)


@pytest.mark.gpu
@pytest.mark.parametrize("R,M,Nn,E", [(4096, 512, 1024, 8), (1000, 128, 136, 4), (50, 8, 64, 3)])
def test_segmented_gemm_k_mode(R, M, Nn, E):
    N = native()
    torch.manual_seed(5)
    seg = _segments(R, E, R + 1)
    seg[2] = seg[1]
    dY = (torch.randn(R, M) * 0.5).to(torch.bfloat16)
    X = (torch.randn(R, Nn) * 0.5).to(torch.bfloat16)
    ref = torch.stack([dY[int(seg[e]):int(seg[e + 1])].float().T @ X[int(seg[e]):int(seg[e + 1])].float()
                       for e in range(E)])
    segd = seg.int().to(DEV)
    out = torch.full((E, M, Nn), 3.0, dtype=torch.bfloat16, device=DEV)
    ptrs = torch.tensor([out[e].data_ptr() for e in range(E)], dtype=torch.int64, device=DEV)
    N.gemm_bf16_segmented(dY.to(DEV), ptrs, None, segd, N.SEG_K, other=X.to(DEV))
    assert_close_rel(out, ref, BF16_TOL, "segmented k")
    assert bool((out[1] == 0).all())                             # the empty segment writes zeros
    acc = torch.ones(E, M, Nn, dtype=torch.float32, device=DEV)
    ptrs = torch.tensor([acc[e].data_ptr() for e in range(E)], dtype=torch.int64, device=DEV)
    N.gemm_bf16_segmented(dY.to(DEV), ptrs, None, segd, N.SEG_K, other=X.to(DEV), epilogue=N.EPI_ACCUM_F32,
                          beta=1, c_dtype=torch.float32)
    assert_close_rel(acc, ref + 1.0, 1e-3, "segmented k, fp32 accumulate")
    # rounded accumulation: the bits of the bf16 result added by the accumulate kernel
    start = torch.randn(E, M, Nn, device=DEV)
    rounded = start.clone()
    ptrs = torch.tensor([rounded[e].data_ptr() for e in range(E)], dtype=torch.int64, device=DEV)
    N.gemm_bf16_segmented(dY.to(DEV), ptrs, None, segd, N.SEG_K, other=X.to(DEV), epilogue=N.EPI_ACCUM_ROUNDED,
                          beta=1, c_dtype=torch.float32)
    assert torch.equal(rounded, start + out.float())


@pytest.mark.gpu
def test_moe_and_segmented_entry_points_reject_bad_arguments():
    Nn = native()
    seg = torch.tensor([0, 4, 8], dtype=torch.int32, device=DEV)
    A = torch.zeros(8, 64, device=DEV, dtype=torch.bfloat16)
    W = torch.zeros(2, 16, 64, device=DEV, dtype=torch.bfloat16)
    ptrs = torch.tensor([W[0].data_ptr(), W[1].data_ptr()], dtype=torch.int64, device=DEV)
    Cm = torch.zeros(8, 16, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="rows mode epilogue"):
        Nn.gemm_bf16_segmented(A, ptrs, Cm, seg, Nn.SEG_ROWS, epilogue=Nn.EPI_BIAS_RELU)
    with pytest.raises(ValueError, match="unknown mode"):
        Nn.gemm_bf16_segmented(A, ptrs, Cm, seg, 7)
    with pytest.raises(RuntimeError, match="multiples of 8"):
        Nn.gemm_bf16_segmented(A[:, :60], ptrs, Cm, seg, Nn.SEG_ROWS)
    logits = torch.zeros(4, 1, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="pp_moe_router_top2"):
        Nn.moe_router_top2(logits, torch.zeros(4, 2, dtype=torch.int32, device=DEV),
                           torch.zeros(4, 2, device=DEV))
    slots = torch.zeros(4, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="at most 64 experts"):
        Nn.moe_permute(slots, 65, torch.zeros(66, dtype=torch.int32, device=DEV), slots.clone(), slots.clone())
    x = torch.zeros(4, 12, device=DEV, dtype=torch.bfloat16)       # width not a multiple of 8
    with pytest.raises(RuntimeError, match="pp_moe_gather"):
        Nn.moe_gather(x, slots, 1, torch.zeros(4, 12, device=DEV, dtype=torch.bfloat16))


@pytest.mark.gpu
def test_launch_timer_counts_the_algorithmic_work_of_each_gemm_kind():
    """The per-launch timer behind the bench's roofline figures must attribute 2 M N K flops to a GEMM
    (4 M N K to the kernel that forms the gate and up products together): a slip here would scale every
    reported MFMA fraction."""
    from pippy_amd import _program as P
    N = native()
    M, K, F = 256, 128, 192
    x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    w = torch.randn(F, K, device="cuda").to(torch.bfloat16)
    wt = torch.randn(F, K, device="cuda").to(torch.bfloat16)
    y = torch.empty(M, F, device="cuda", dtype=torch.bfloat16)
    gu = torch.empty(M, 2 * F, device="cuda", dtype=torch.bfloat16)
    dgu = torch.empty_like(gu)
    ops = P.OpList()
    ops.append(P.op_gemm(x, w, y))
    ops.append(P.op_gemm(x, w, y))
    ops.append(P.op_gemm_swiglu(x, w, w, gu, y))
    ops.append(P.op_gemm_dswiglu(x, wt, gu, dgu))
    N.profile_start(64)
    ops.run()
    torch.cuda.synchronize()
    N.profile_stop()
    for kind, want_work, want_count in ((N.OP_GEMM_BF16, 2 * 2.0 * M * F * K, 2), (N.OP_GEMM_SWIGLU, 4.0 * M * F * K, 1),
                                        (N.OP_GEMM_DSWIGLU, 2.0 * M * F * K, 1)):
        ms, work, cnt = N.profile_read(kind)
        assert cnt == want_count and work == want_work and ms > 0, (kind, ms, work, cnt)
