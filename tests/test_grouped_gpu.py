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
    At = torch.zeros(8, 16, device=DEV, dtype=torch.bfloat16)
    C = torch.zeros(16, 16, device=DEV, dtype=torch.bfloat16)
    Cf = torch.zeros(16, 16, device=DEV)
    with pytest.raises(RuntimeError, match="differs in layout"):
        N.gemm_bf16_grouped([(A, A, C, {}), (At, A, C, dict(a_trans=True))])
    with pytest.raises(RuntimeError, match="differs in layout or output dtype"):
        N.gemm_bf16_grouped([(A, A, C, {}), (A, A, Cf, {})])
    with pytest.raises(RuntimeError, match="mixes plain and accumulating"):
        N.gemm_bf16_grouped([(A, A, Cf, {}), (A, A, Cf, dict(epilogue=N.EPI_ACCUM_F32, beta=1))])
    with pytest.raises(RuntimeError, match="with bf16 C"):
        N.gemm_bf16_grouped([(A, A, C, {}), (A, A, C, dict(epilogue=N.EPI_ACCUM_F32))])


@pytest.mark.parametrize("M,K", [(4096, 768), (200, 136)])
def test_grouped_problems_with_different_epilogues_equal_single_launches(M, K):
    """The GEMMs that several stages reach at the same point of their passes go out as one launch in
    which every problem brings its own epilogue; each must leave the bits of its own single launch
    (the reduction order over k does not depend on the tile shape or on the neighbours in the grid)."""
    from pippy_amd import _native as N
    torch.manual_seed(3)

    def problem(Nn, epi):
        A = torch.randn(M, K, device=DEV).to(torch.bfloat16)
        B = (torch.randn(Nn, K, device=DEV) * 0.05).to(torch.bfloat16)
        kw = dict(epilogue=epi)
        if epi in (N.EPI_BIAS, N.EPI_BIAS_GELU_TANH, N.EPI_BIAS_GELU_ERF, N.EPI_BIAS_RESIDUAL, N.EPI_BIAS_RELU):
            kw["bias"] = torch.randn(Nn, device=DEV).to(torch.bfloat16)
        if epi in (N.EPI_BIAS_RESIDUAL, N.EPI_DGELU_TANH, N.EPI_DGELU_ERF, N.EPI_DRELU):
            kw["aux_in"] = torch.randn(M, Nn, device=DEV).to(torch.bfloat16)
        return A, B, kw

    specs = [(768, N.EPI_BIAS_RESIDUAL), (2304, N.EPI_BIAS), (3072, N.EPI_BIAS_GELU_TANH), (768, N.EPI_NONE),
             (3072, N.EPI_DGELU_TANH), (264, N.EPI_BIAS_GELU_ERF), (136, N.EPI_DGELU_ERF), (520, N.EPI_BIAS_RELU),
             (392, N.EPI_DRELU)]
    group, singles = [], []
    for Nn, epi in specs:
        A, B, kw = problem(Nn, epi)
        outs = []
        for _ in range(2):
            C = torch.full((M, Nn), 7.0, device=DEV, dtype=torch.bfloat16)
            k2 = dict(kw)
            if epi in (N.EPI_BIAS_GELU_TANH, N.EPI_BIAS_GELU_ERF):
                k2["aux_out"] = torch.full((M, Nn), 7.0, device=DEV, dtype=torch.bfloat16)
            outs.append((C, k2))
        group.append((A, B, outs[0][0], outs[0][1]))
        singles.append((A, B, outs[1][0], outs[1][1]))
    N.gemm_bf16_grouped(group)
    for A, B, C, kw in singles:
        N.gemm_bf16(A, B, C, **kw)
    torch.cuda.synchronize()
    for (Nn, epi), g, s_ in zip(specs, group, singles):
        assert torch.equal(g[2], s_[2]), f"C of N={Nn} epilogue {epi}"
        if "aux_out" in g[3]:
            assert torch.equal(g[3]["aux_out"], s_[3]["aux_out"]), f"saved pre-activation of N={Nn} epilogue {epi}"


def test_grouped_column_reductions_equal_single_calls():
    from pippy_amd import _native as N
    torch.manual_seed(1)
    items, refs = [], []
    for k, (rows, C, with_x, f32) in enumerate([(4096, 768, True, False), (4096, 2304, False, False),
                                                 (300, 264, True, True), (1, 8, False, True)] * 8):
        dy = torch.randn(rows, C, device=DEV).to(torch.bfloat16)
        odt = torch.float32 if f32 else torch.bfloat16
        n_part = (rows + 127) // 128
        it = {"dy": dy, "out_sum": torch.empty(C, device=DEV, dtype=odt),
              "workspace": torch.empty(2 * n_part * C, device=DEV)}
        ref_sum = torch.empty(C, device=DEV, dtype=odt)
        ref_dot = None
        ws = torch.empty(2 * n_part * C, device=DEV)
        if with_x:
            x = torch.randn(rows, C, device=DEV).to(torch.bfloat16)
            mean = x.float().mean(-1)
            rstd = 1.0 / torch.sqrt(x.float().var(-1, unbiased=False) + 1e-5)
            it.update(x=x, mean=mean, rstd=rstd, out_dot=torch.empty(C, device=DEV, dtype=odt))
            ref_dot = torch.empty(C, device=DEV, dtype=odt)
            N.layernorm_bwd_weight(dy, x, mean, rstd, ref_dot, ref_sum, ws)
        else:
            N.colsum(dy, ref_sum, ws)
        items.append(it)
        refs.append((ref_sum, ref_dot))
    N.colreduce_grouped(items)
    torch.cuda.synchronize()
    for it, (ref_sum, ref_dot) in zip(items, refs):
        assert torch.equal(it["out_sum"], ref_sum)
        if ref_dot is not None:
            assert torch.equal(it["out_dot"], ref_dot)


def test_transpose_and_weight_refresh_after_optimizer_step():
    """The transposed weight copies used by the input-gradient GEMMs follow parameter updates."""
    import copy
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    from pippy_amd import _native as N
    x = torch.randn(130, 77, device=DEV).to(torch.bfloat16)
    t = torch.empty(77, 130, device=DEV, dtype=torch.bfloat16)
    N.transpose_bf16(x, t)
    assert torch.equal(t, x.t())

    import pippy_amd as pp
    from oracle import pipeline as OP
    from test_pipeline_gpu import _build_decoder, _ce
    from _util import BF16_TOL, max_rel
    M = 2
    model, ref, stages, ref_stages, ids = _build_decoder(2, n_layers=2, M=M)
    target = torch.randint(0, 1000, ids.shape)
    sched = pp.Schedule1F1B(stages, M, loss_fn=pp.CrossEntropyLoss())
    sched.step(ids.to(DEV), target=target.to(DEV))
    # "optimizer step": perturb every parameter in place on both sides, then compare a fresh step
    torch.manual_seed(7)
    with torch.no_grad():
        for (n, p), (_, rp) in zip(model.named_parameters(), ref.named_parameters()):
            d = (torch.randn(rp.shape) * 0.02).to(torch.bfloat16)
            p.add_(d.to(DEV))
            rp.copy_(p.detach().float().cpu())
    sched.zero_grad()
    sched.step(ids.to(DEV), target=target.to(DEV))
    for p in ref.parameters():
        p.grad = None
    OP.step(ref_stages, ids, target, M, _ce)
    named = dict(model.named_parameters())
    for name, rp in ref.named_parameters():
        assert max_rel(named[name].main_grad, rp.grad) <= BF16_TOL, name


@pytest.mark.parametrize("dtype,V,ld,rows", [(torch.bfloat16, 50257, 50304, 64), (torch.uint8, 4099, 4112, 33),
                                              (torch.float32, 1027, 1030, 17), (torch.bfloat16, 1025, 1025, 9)])
def test_copy_rows_with_unaligned_rows_is_bit_exact(dtype, V, ld, rows):
    """Rows that do not start on 16-byte boundaries take the head / aligned body / tail path."""
    from pippy_amd import _native as N
    torch.manual_seed(2)
    es = torch.empty(0, dtype=dtype).element_size()
    src = (torch.randn(rows, ld, device=DEV) * 100).to(dtype)
    dst = torch.zeros(rows * V + 16, device=DEV, dtype=dtype)
    for shift in (0, 1, 3):   # destination start misaligned by `shift` elements
        dst.zero_()
        N.copy_rows([(src.data_ptr(), dst.data_ptr() + shift * es, rows, V * es, ld * es, V * es)])
        got = dst[shift:shift + rows * V].view(rows, V)
        assert torch.equal(got, src[:, :V])
        assert float(dst[:shift].float().abs().sum()) == 0 and float(dst[shift + rows * V:].float().abs().sum()) == 0


@pytest.mark.parametrize("epi_name", ["rounded", "f32"])
@pytest.mark.parametrize("beta", [0, 1])
def test_weight_gradients_of_several_microbatches_in_one_launch_equal_one_launch_each(epi_name, beta):
    """``pp_gemm_bf16_grouped_kseg``: C = (beta ? C : 0) + g_0 + g_1 + ... added in microbatch order must
    leave the bits that one accumulating launch per microbatch leaves (fp32 addition is not associative,
    so the order and the per-microbatch rounding both show), for ragged shapes too."""
    from pippy_amd import _native as N
    N.lib()
    torch.manual_seed(5)
    epi = N.EPI_ACCUM_ROUNDED if epi_name == "rounded" else N.EPI_ACCUM_F32
    n_seg, T = 5, 392                      # a token count that is no multiple of the k-tile
    shapes = [(2304, 768), (768, 768), (136, 200), (8, 8), (3072, 256)]
    problems, want = [], []
    for out_f, in_f in shapes:
        dYs = [torch.randn(T, out_f, device=DEV).to(torch.bfloat16) for _ in range(n_seg)]
        Xs = [torch.randn(T, in_f, device=DEV).to(torch.bfloat16) for _ in range(n_seg)]
        C0 = torch.randn(out_f, in_f, device=DEV) * 30
        ref = C0.clone()
        for s in range(n_seg):
            N.gemm_bf16(dYs[s], Xs[s], ref, a_trans=True, b_trans=True, epilogue=epi, beta=1 if (s or beta) else 0)
        got = C0.clone()
        problems.append((dYs, Xs, got, dict(epilogue=epi, beta=beta)))
        want.append(ref)
    keep = []
    N.gemm_bf16_grouped_kseg(problems, keep)
    torch.cuda.synchronize()
    for (_, _, got, _), ref in zip(problems, want):
        assert torch.equal(got, ref)
    # the sum is not the sum of a different order: adding the microbatches backwards differs somewhere
    dYs, Xs, _, kw = problems[0]
    back = (torch.zeros_like(want[0]) if not beta else None)
    if back is not None:
        N.gemm_bf16_grouped_kseg([(dYs[::-1], Xs[::-1], back, kw)], keep)
        torch.cuda.synchronize()
        assert not torch.equal(back, want[0])
        assert torch.allclose(back, want[0], rtol=1e-3, atol=1e-2)


def test_kseg_rejects_what_it_does_not_compute():
    from pippy_amd import _native as N
    A = torch.zeros(16, 16, device=DEV, dtype=torch.bfloat16)
    Cb = torch.zeros(16, 16, device=DEV, dtype=torch.bfloat16)
    Cf = torch.zeros(16, 16, device=DEV)
    with pytest.raises(RuntimeError, match="accumulated into an fp32 C"):
        N.gemm_bf16_grouped_kseg([([A], [A], Cb, {})], [])
    with pytest.raises(RuntimeError, match="accumulated into an fp32 C"):
        N.gemm_bf16_grouped_kseg([([A], [A], Cf, {})], [])      # epilogue NONE does not accumulate


@pytest.mark.parametrize("epi_name,beta", [("rounded", 0), ("rounded", 1), ("f32", 1)])
def test_expert_weight_gradients_of_several_microbatches_in_one_launch(epi_name, beta):
    """``pp_gemm_bf16_segmented_kseg``: every expert's C_e = (beta ? C_e : 0) + its product over each
    microbatch's rows of that expert, added in microbatch order, against one accumulating k-mode launch per
    microbatch (bit for bit); every microbatch has its own row partition, with empty and ragged segments."""
    import ctypes as C
    from pippy_amd import _native as N
    N.lib()
    torch.manual_seed(9)
    epi = N.EPI_ACCUM_ROUNDED if epi_name == "rounded" else N.EPI_ACCUM_F32
    E, n_mb, Mo, Ni = 5, 3, 256, 136
    rows = [[70, 0, 131, 8, 47], [0, 0, 256, 0, 0], [33, 64, 1, 100, 58]]
    As, Bs, segs = [], [], []
    for m in range(n_mb):
        R = sum(rows[m])
        As.append(torch.randn(R, Mo, device=DEV).to(torch.bfloat16))
        Bs.append(torch.randn(R, Ni, device=DEV).to(torch.bfloat16))
        segs.append(torch.tensor([0] + list(torch.tensor(rows[m]).cumsum(0)), dtype=torch.int32, device=DEV))
    C0 = [torch.randn(Mo, Ni, device=DEV) * 20 for _ in range(E)]
    want = [c.clone() for c in C0]
    want_ptrs = torch.tensor([c.data_ptr() for c in want], dtype=torch.int64, device=DEV)
    for m in range(n_mb):
        N.gemm_bf16_segmented(As[m], want_ptrs, None, segs[m], N.SEG_K, other=Bs[m], ld=Ni, epilogue=epi,
                              beta=1 if (m or beta) else 0, c_dtype=torch.float32)
    got = [c.clone() for c in C0]
    got_ptrs = torch.tensor([c.data_ptr() for c in got], dtype=torch.int64, device=DEV)
    a_of = torch.tensor([a.data_ptr() for a in As], dtype=torch.int64, device=DEV)
    b_of = torch.tensor([b.data_ptr() for b in Bs], dtype=torch.int64, device=DEV)
    s_of = torch.tensor([s.data_ptr() for s in segs], dtype=torch.int64, device=DEV)
    d = N.GemmDesc()
    d.M, d.N, d.K = Mo, Ni, max(sum(r) for r in rows)
    d.lda, d.ldb, d.ldc = Mo, Ni, Ni
    d.a_trans = d.b_trans = 1
    d.c_dtype, d.epilogue, d.beta = N.PP_F32, epi, beta
    N.check(N.lib().pp_gemm_bf16_segmented_kseg(C.byref(d), a_of.data_ptr(), b_of.data_ptr(), s_of.data_ptr(),
                                                got_ptrs.data_ptr(), E, n_mb, N.current_stream()),
            "pp_gemm_bf16_segmented_kseg")
    torch.cuda.synchronize()
    for e in range(E):
        assert torch.equal(got[e], want[e]), f"expert {e}"
    if not beta:
        assert float(got[1].abs().max()) > 0          # expert 1 has rows in the last microbatch only
