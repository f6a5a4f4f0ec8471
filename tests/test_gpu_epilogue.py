"""GPU tests of the decode kernels' epilogues (nf4hip_gemv_epilogue), called through the C ABI by
``functional.matmul_nf4_epilogue``.

What an epilogue does to a finished sum is element-wise arithmetic on bf16 values, so wherever the two-step route
(nf4hip_gemv, then the step as a kernel of its own) computes the same thing the bits must agree: SiLU * up on pairs of
outputs, the new residual, the next norm's input times its weight.  The row scale (1 / rms applied to the finished
sums instead of to every element of x) is floating-point work in another order: held to the matmul's bar,
rtol = atol = 2e-2 against float64 on the same inputs.
"""

import importlib

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda"
TOL = dict(rtol=2e-2, atol=2e-2)


def _randn(shape, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g, dtype=torch.float32) * std).to(torch.bfloat16)


@pytest.fixture(scope="module")
def F(ta):
    return ta.functional


@pytest.fixture(scope="module")
def glue():
    return importlib.import_module("lightning-thunder_amd.glue")


def _quantized(ta, N, K, seed):
    qw, absmax, code = ta.quantize_nf4(_randn((N, K), seed, 0.02).to(DEV))
    return qw, absmax, code


def _bits(t):
    return t.contiguous().view(torch.int16)


# (N, K): small, the Llama-3-8B gate-up and down shapes, K in the fp16-code-book range, ragged sizes
PAIR_SHAPES = [(1024, 512), (28672, 4096), (2048, 14336), (272, 2080)]


def _served(F, M, N, K, **which):
    """K % 32 == 0 up to four rows of x, K % 512 == 0 beyond, K within one workgroup's reach with one row of x; the residual
    epilogue of the tile kernel (nine and more rows of x, or a large weight) leaves one partial sum per 16 weight rows,
    at most 512 of them."""
    return F.epilogue_served(M, (N, K), **which)


@pytest.mark.parametrize("M", [1, 2, 3, 4, 8, 16])
@pytest.mark.parametrize("shape", PAIR_SHAPES)
def test_silu_pairs_gives_the_two_step_bits(ta, F, glue, M, shape):
    N, K = shape
    if not _served(F, M, N, K, silu_pairs=True):
        pytest.skip("not a shape the kernels take with an epilogue (K % 512 beyond four rows of x, K within one workgroup with one row of x)")
    print(f"epilogue silu_pairs M={M} N={N} K={K}", flush=True)
    qw, absmax, code = _quantized(ta, N, K, seed=N + K)
    x = _randn((M, K), seed=3 * N + M).to(DEV)
    bias = _randn((N,), seed=N, std=0.5).to(DEV) if N == 272 else None
    two_step = glue.silu_mul(F.matmul_nf4(x, qw, bias, absmax, code, 64, torch.bfloat16, (N, K)), pairs=True)
    out = F.matmul_nf4_epilogue(x, qw, bias, absmax, code, 64, torch.bfloat16, (N, K), silu_pairs=True)
    torch.cuda.synchronize()
    assert out is not None and out.shape == (M, N // 2)
    assert torch.equal(_bits(out), _bits(two_step))


# (N, K): Llama-3-8B output and down projections, ragged, the longest K one workgroup holds
RESID_SHAPES = [(4096, 4096), (4096, 14336), (517, 1056), (256, 16384), (8192, 8192), (1000, 28672)]


@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 8, 16])
@pytest.mark.parametrize("shape", RESID_SHAPES)
def test_resid_norm_epilogue(ta, F, M, shape):
    N, K = shape
    if not _served(F, M, N, K, resid_norm=True):
        pytest.skip("not a shape the kernels take with an epilogue (K % 512 beyond four rows of x, K within one workgroup with one row of x)")
    print(f"epilogue resid_norm M={M} N={N} K={K}", flush=True)
    qw, absmax, code = _quantized(ta, N, K, seed=N + K + 1)
    x = _randn((M, K), seed=5 * N + M).to(DEV)
    resid = _randn((M, N), seed=7 * N + M, std=2.0).to(DEV)
    nw = (1.0 + _randn((N,), seed=N, std=0.1).float()).to(torch.bfloat16).to(DEV)
    bias = _randn((N,), seed=N + 1, std=0.5).to(DEV) if N == 517 else None
    resid_before = resid.clone()
    got = F.matmul_nf4_epilogue(x, qw, bias, absmax, code, 64, torch.bfloat16, (N, K), resid_norm=(resid, nw))
    assert got is not None
    r, xnext, sumsq = got
    # the plain call's bf16 output: a shape's plain product and its residual epilogue are served by the same kernel (where
    # the LDS-staged kernel takes the product and has no such epilogue, the epilogue is refused instead)
    delta = F.matmul_nf4(x, qw, bias, absmax, code, 64, torch.bfloat16, (N, K))
    torch.cuda.synchronize()
    r_ref = (resid_before.float() + delta.float()).to(torch.bfloat16)
    assert torch.equal(resid, resid_before)
    assert torch.equal(_bits(r), _bits(r_ref)), "resid_out is not bf16(resid + bf16(linear))"
    assert torch.equal(_bits(xnext), _bits((r_ref.float() * nw.float()).to(torch.bfloat16))), "xnext is not bf16(r * norm_weight)"
    assert sumsq.shape == (M, ta._lib.load().nf4hip_gemv_norm_parts(M, N, K))
    torch.testing.assert_close(sumsq.double().sum(-1), r_ref.double().pow(2).sum(-1), rtol=1e-5, atol=0)


@pytest.mark.parametrize("M", [1, 7, 16])
@pytest.mark.parametrize("shape", [(520, 8192), (1032, 14336), (256, 16384), (4096, 8192)])
def test_resid_norm_epilogue_of_the_staged_kernel(ta, F, M, shape):
    """The LDS-staged kernel forced (``nf4hip_gemv_prefer_staged(1)``) on shapes whose K it splits over workgroups: the
    workgroup that adds the K ranges does the residual step -- bit for bit what the plain call of the same kernel and
    the step by itself store, one partial sum of squares per row range."""
    N, K = shape
    lib = ta._lib.load()
    print(f"staged resid_norm M={M} N={N} K={K}", flush=True)
    qw, absmax, code = _quantized(ta, N, K, seed=N + K + 2)
    x = _randn((M, K), seed=3 * N + M).to(DEV)
    resid = _randn((M, N), seed=5 * N + M, std=2.0).to(DEV)
    nw = (1.0 + _randn((N,), seed=N + 3, std=0.1).float()).to(torch.bfloat16).to(DEV)
    bias = _randn((N,), seed=N + 4, std=0.5).to(DEV) if N == 520 else None
    assert lib.nf4hip_gemv_prefer_staged(1) == 0
    try:
        assert _served(F, M, N, K, resid_norm=True)
        got = F.matmul_nf4_epilogue(x, qw, bias, absmax, code, 64, torch.bfloat16, (N, K), resid_norm=(resid, nw))
        delta = F.matmul_nf4(x, qw, bias, absmax, code, 64, torch.bfloat16, (N, K))
        parts = lib.nf4hip_gemv_norm_parts(M, N, K)
    finally:
        assert lib.nf4hip_gemv_prefer_staged(-1) == 0
    assert got is not None
    r, xnext, sumsq = got
    r_ref = (resid.float() + delta.float()).to(torch.bfloat16)
    assert torch.equal(_bits(r), _bits(r_ref)) and torch.equal(_bits(xnext), _bits((r_ref.float() * nw.float()).to(torch.bfloat16)))
    assert sumsq.shape == (M, parts) and parts > 0
    torch.testing.assert_close(sumsq.double().sum(-1), r_ref.double().pow(2).sum(-1), rtol=1e-5, atol=0)


@pytest.mark.parametrize("M,shape", [(1, (4096, 4096)), (9, (4096, 4096)), (16, (4096, 4096)), (16, (14336, 4096)), (8, (28672, 4096)),
                                     (16, (1000, 2048)), (5, (8, 512)), (16, (2040, 4096))])
def test_resid_norm_epilogue_of_the_staged_kernel_one_k_range(ta, F, M, shape):
    """The same where one workgroup covers K: the finishing waves do the residual step on a residual and norm weight
    staged in LDS -- few rows per workgroup, (M + 1) rows of values in all -- and leave one partial sum of squares per
    workgroup.  With sixteen rows of x the output projection of the decode step takes this route by the dispatcher's
    own rule."""
    N, K = shape
    lib = ta._lib.load()
    print(f"staged resid_norm, one K range M={M} N={N} K={K}", flush=True)
    qw, absmax, code = _quantized(ta, N, K, seed=N + K + 5)
    x = _randn((M, K), seed=3 * N + M + 1).to(DEV)
    resid = _randn((M, N), seed=5 * N + M + 1, std=2.0).to(DEV)
    nw = (1.0 + _randn((N,), seed=N + 6, std=0.1).float()).to(torch.bfloat16).to(DEV)
    bias = _randn((N,), seed=N + 7, std=0.5).to(DEV) if N in (1000, 14336) else None
    assert lib.nf4hip_gemv_prefer_staged(1) == 0
    try:
        import ctypes

        plan = (ctypes.c_int * 4)()
        assert lib.nf4hip_gemv_plan(M, N, K, 64, 0, ctypes.byref(plan)) == 0 and plan[0] == 5, "the staged kernel serves the plain product"
        assert _served(F, M, N, K, resid_norm=True)
        got = F.matmul_nf4_epilogue(x, qw, bias, absmax, code, 64, torch.bfloat16, (N, K), resid_norm=(resid, nw))
        delta = F.matmul_nf4(x, qw, bias, absmax, code, 64, torch.bfloat16, (N, K))
        parts = lib.nf4hip_gemv_norm_parts(M, N, K)
    finally:
        assert lib.nf4hip_gemv_prefer_staged(-1) == 0
    assert got is not None
    r, xnext, sumsq = got
    r_ref = (resid.float() + delta.float()).to(torch.bfloat16)
    assert torch.equal(_bits(r), _bits(r_ref)) and torch.equal(_bits(xnext), _bits((r_ref.float() * nw.float()).to(torch.bfloat16)))
    assert sumsq.shape == (M, parts) and parts > 0
    torch.testing.assert_close(sumsq.double().sum(-1), r_ref.double().pow(2).sum(-1), rtol=1e-5, atol=0)
    # the same call again on the same buffers: the same bits (nothing depends on which workgroup finishes first)
    assert lib.nf4hip_gemv_prefer_staged(1) == 0
    try:
        again = F.matmul_nf4_epilogue(x, qw, bias, absmax, code, 64, torch.bfloat16, (N, K), resid_norm=(resid, nw))
    finally:
        assert lib.nf4hip_gemv_prefer_staged(-1) == 0
    assert all(torch.equal(a_.view(torch.int16) if a_.dtype == torch.bfloat16 else a_, b_.view(torch.int16) if b_.dtype == torch.bfloat16 else b_)
               for a_, b_ in zip(again, got))


def test_resid_norm_epilogue_too_many_rows_for_the_staging(ta, F):
    """[28672, 4096] with sixteen rows of x: 112 weight rows per workgroup times seventeen rows of values do not fit
    the staging area; the staged kernel serves the plain product, so the epilogue form is refused (the caller's
    two-step route adds to the same sums)."""
    lib = ta._lib.load()
    assert lib.nf4hip_gemv_norm_parts(16, 28672, 4096) == 0
    assert not _served(F, 16, 28672, 4096, resid_norm=True)


def _deq(oracle, qw, absmax, code, shape):
    return oracle.dequantize_4bit_eager(qw.cpu(), absmax.cpu(), code.cpu(), 64, torch.bfloat16, shape).double()


_last_weight = {}


def _quantized_with_reference(ta, oracle, N, K, seed):
    """``_quantized`` plus the oracle's dequantised weight (CPU, bf16 values); the last one is kept, so that the cases
    of one shape (the lm_head takes the CPU half a minute) dequantise once."""
    key = (N, K, seed)
    if _last_weight.get("key") != key:
        qw, absmax, code = _quantized(ta, N, K, seed)
        w = oracle.dequantize_4bit_eager(qw.cpu(), absmax.cpu(), code.cpu(), 64, torch.bfloat16, (N, K))
        _last_weight.clear()
        _last_weight.update(key=key, value=(qw, absmax, code, w))
    return _last_weight["value"]


@pytest.mark.parametrize("M", [1, 2, 4, 7, 8, 16])
@pytest.mark.parametrize("silu", [False, True])
@pytest.mark.parametrize("shape", [(6144, 4096), (1024, 512), (28672, 4096), (128256, 4096), (304, 8192)])  # outermost: cases of a shape run back to back
def test_rowscale_epilogue_against_float64(ta, F, glue, oracle, M, silu, shape):
    """A producer's (xnext, sumsq) made by hand from a residual r: the consumer must give linear(rms_norm(r) * w)."""
    N, K = shape
    if N == 128256 and silu:
        pytest.skip("the lm_head has no (gate, up) pairs")
    if not _served(F, M, N, K, rowscale_parts=37, silu_pairs=silu):
        pytest.skip("not a shape the kernels take with an epilogue (K % 512 beyond four rows of x, K within one workgroup with one row of x)")
    print(f"epilogue rowscale M={M} N={N} K={K} silu={silu}", flush=True)
    qw, absmax, code, w_ref = _quantized_with_reference(ta, oracle, N, K, seed=N + K + 2)
    r = _randn((M, K), seed=11 * N + M, std=3.0)
    nw = (1.0 + _randn((K,), seed=K, std=0.1).float()).to(torch.bfloat16)
    eps = 1e-5
    xnext = (r.float() * nw.float()).to(torch.bfloat16)
    parts = 37  # any split of the sum of squares into partial sums will do
    sq = r.double().pow(2)
    sumsq = torch.stack([c.sum(-1) for c in sq.chunk(parts, dim=-1)], dim=-1).float().contiguous()
    out = F.matmul_nf4_epilogue(xnext.to(DEV), qw, None, absmax, code, 64, torch.bfloat16, (N, K), rowscale=(sumsq.to(DEV), eps))
    torch.cuda.synchronize()
    assert out is not None
    h = r.double() * torch.rsqrt(sq.mean(-1, keepdim=True) + eps) * nw.double()
    # the float64 product of the oracle's weight (a textbook matmul), in slabs of rows so that the lm_head's 525 M
    # weights never exist as float64 at once
    y = torch.cat([h @ w_ref[n0:n0 + 16384].double().t() for n0 in range(0, N, 16384)], dim=-1)
    torch.testing.assert_close(out.cpu().double(), y, **TOL)
    if silu:  # SiLU * up on the scaled sums: the bits of the element-wise kernel on the scaled output above
        both = F.matmul_nf4_epilogue(xnext.to(DEV), qw, None, absmax, code, 64, torch.bfloat16, (N, K), rowscale=(sumsq.to(DEV), eps),
                                     silu_pairs=True)
        assert both is not None and torch.equal(_bits(both), _bits(glue.silu_mul(out, pairs=True)))


def test_chain_of_epilogues_is_a_decoder_layer_tail(ta, F, oracle):
    """o_proj (residual add, next norm's input) -> gate-up (row scale, SiLU * up) -> down (residual add) against the same
    arithmetic in float64 with bf16 roundings only where tensors are stored."""
    d, dff, M = 1024, 2048, 2
    print("epilogue chain", flush=True)
    qo, ao, code = _quantized(ta, d, d, seed=1)
    qg, ag, _ = _quantized(ta, 2 * dff, d, seed=2)
    qd, ad, _ = _quantized(ta, d, dff, seed=3)
    y = _randn((M, d), 4)
    r0 = _randn((M, d), 5, 2.0)
    w2 = (1.0 + _randn((d,), 6, 0.1).float()).to(torch.bfloat16)
    w1 = (1.0 + _randn((d,), 7, 0.1).float()).to(torch.bfloat16)
    eps = 1e-5
    r1, xn, ss = F.matmul_nf4_epilogue(y.to(DEV), qo, None, ao, code, 64, torch.bfloat16, (d, d), resid_norm=(r0.to(DEV), w2.to(DEV)))
    h = F.matmul_nf4_epilogue(xn, qg, None, ag, code, 64, torch.bfloat16, (2 * dff, d), rowscale=(ss, eps), silu_pairs=True)
    r2, xn2, ss2 = F.matmul_nf4_epilogue(h, qd, None, ad, code, 64, torch.bfloat16, (d, dff), resid_norm=(r1, w1.to(DEV)))
    torch.cuda.synchronize()

    Wo, Wg, Wd = _deq(oracle, qo, ao, code, (d, d)), _deq(oracle, qg, ag, code, (2 * dff, d)), _deq(oracle, qd, ad, code, (d, dff))
    bf = lambda t: t.to(torch.bfloat16).double()
    r1_ref = bf(r0.double() + bf(y.double() @ Wo.t()))
    hn = r1_ref * torch.rsqrt(r1_ref.pow(2).mean(-1, keepdim=True) + eps) * w2.double()
    gu = hn @ Wg.t()
    h_ref = bf(torch.nn.functional.silu(gu[:, 0::2]) * gu[:, 1::2])
    r2_ref = bf(r1_ref + bf(h_ref @ Wd.t()))
    torch.testing.assert_close(r1.cpu().double(), r1_ref, **TOL)
    torch.testing.assert_close(h.cpu().double(), h_ref, rtol=4e-2, atol=4e-2)  # a product of two linear outputs
    torch.testing.assert_close(r2.cpu().double(), r2_ref, rtol=4e-2, atol=4e-2)  # two linears deep
    torch.testing.assert_close(ss2.double().sum(-1), r2.double().pow(2).sum(-1), rtol=1e-5, atol=0)
    assert torch.equal(_bits(xn2), _bits((r2.float() * w1.to(DEV).float()).to(torch.bfloat16)))


@pytest.mark.parametrize("M,shape", [(1, (64, 20480)), (1, (64, 32768))])
def test_cases_the_kernels_do_not_serve_return_none(ta, F, M, shape):
    """A K that one workgroup of the row kernel does not hold: the library answers NF4HIP_E_SHAPE before it launches
    anything, and the host function hands None to its caller, which takes the two-step route."""
    N, K = shape
    qw, absmax, code = _quantized(ta, N, K, seed=N + K + 3)
    x = _randn((M, K), seed=1).to(DEV)
    resid = _randn((M, N), seed=2).to(DEV)
    nw = torch.ones(N, dtype=torch.bfloat16, device=DEV)
    assert not F.epilogue_served(M, (N, K), resid_norm=True) and not F.epilogue_served(M, (N, K), silu_pairs=True)
    assert F.matmul_nf4_epilogue(x, qw, None, absmax, code, 64, torch.bfloat16, (N, K), resid_norm=(resid, nw)) is None
    assert F.matmul_nf4_epilogue(x, qw, None, absmax, code, 64, torch.bfloat16, (N, K), silu_pairs=True) is None
    ss = torch.ones(M, 8, device=DEV)
    assert F.matmul_nf4_epilogue(x, qw, None, absmax, code, 64, torch.bfloat16, (N, K), rowscale=(ss, 1e-5)) is None


def test_residual_epilogue_of_the_tile_kernel_needs_at_most_512_tiles(ta, F):
    """Sixteen rows of x on [16384, 4096]: the tile kernel serves it, 1024 tiles of 16 weight rows are more partial
    sums than a consumer's workgroup has threads -- refused for the residual epilogue, served for the others."""
    N, K, M = 16384, 4096, 16
    qw, absmax, code = _quantized(ta, N, K, seed=77)
    x = _randn((M, K), seed=1).to(DEV)
    assert not F.epilogue_served(M, (N, K), resid_norm=True) and F.epilogue_served(M, (N, K), silu_pairs=True)
    resid = _randn((M, N), seed=2).to(DEV)
    nw = torch.ones(N, dtype=torch.bfloat16, device=DEV)
    assert F.matmul_nf4_epilogue(x, qw, None, absmax, code, 64, torch.bfloat16, (N, K), resid_norm=(resid, nw)) is None
    out = F.matmul_nf4_epilogue(x, qw, None, absmax, code, 64, torch.bfloat16, (N, K), silu_pairs=True)
    two_step = importlib.import_module("lightning-thunder_amd.glue").silu_mul(
        F.matmul_nf4(x, qw, None, absmax, code, 64, torch.bfloat16, (N, K)), pairs=True)
    assert out is not None and torch.equal(_bits(out), _bits(two_step))


@pytest.mark.parametrize("batch", [1, 2, 3, 8, 16])
def test_decode_step_with_linear_epilogues(ta, glue, monkeypatch, batch):
    """The single-token step with the epilogues (five launches per layer) against the step with the glue kernels of
    their own and against the plain-PyTorch step of the same quantized model; graph replay equals the eager loop."""
    D = importlib.import_module("lightning-thunder_amd.decode")
    print(f"decode with linear epilogues batch={batch}", flush=True)
    dev = torch.device(DEV)
    cfg = D.LlamaConfig.tiny(fused_projections=True, gate_up_interleaved=True, hip_glue=True)
    model = D.build_llama(cfg, device=dev, seed=5)
    jm = ta.jit(model, transforms=[ta.BitsAndBytesLinearQuant4bit()])
    g = torch.Generator(device=dev).manual_seed(2)
    prompt = torch.randint(0, cfg.vocab, (batch, 16), generator=g, device=dev)
    eager, s0 = D.greedy_decode(jm, cfg, prompt, n_new=12, use_graph=False)
    graph, s1 = D.greedy_decode(jm, cfg, prompt, n_new=12, use_graph=True)
    assert s1["graph"] and torch.equal(eager, graph)

    caches = [D.new_caches(cfg, batch, dev) for _ in range(3)]
    pos = torch.arange(16, device=dev)
    first = jm(prompt, pos, *caches[0]).argmax(-1, keepdim=True)
    for kc, vc in caches[1:]:
        jm(prompt, pos, kc, vc)
    p1 = torch.full((1,), 16, device=dev, dtype=torch.long)
    calls = {"silu": 0}
    real = glue.silu_mul
    monkeypatch.setattr(glue, "silu_mul", lambda *a, **k: (calls.__setitem__("silu", calls["silu"] + 1), real(*a, **k))[1])
    a = jm(first, p1, *caches[0]).float()
    # every linear of this small model is served by a kernel with epilogues at these batch sizes: the gate-up kernel
    # applies SiLU * up itself
    assert calls["silu"] == 0
    cfg.linear_epilogues = False
    b = jm(first, p1, *caches[1]).float()
    cfg.hip_glue = False
    c = jm(first, p1, *caches[2]).float()
    torch.testing.assert_close(a, b, rtol=3e-2, atol=3e-2)
    torch.testing.assert_close(a, c, rtol=3e-2, atol=3e-2)
    for kc, vc in caches[1:]:
        torch.testing.assert_close(caches[0][0][:, :, :, :17].float(), kc[:, :, :, :17].float(), rtol=2e-2, atol=2e-2)
        torch.testing.assert_close(caches[0][1][:, :, :, :17].float(), vc[:, :, :, :17].float(), rtol=2e-2, atol=2e-2)


def test_epilogues_hold_over_many_launches_with_k_split_over_workgroups(ta, F):
    """A producer / consumer pair whose kernels split K over workgroups (eight rows of x on [4096, 14336]: the quad
    kernel's last-arriving workgroup runs the residual epilogue; sixteen rows on [6144, 4096]: the tile kernel's
    reducing wave applies the row scale), 600 times on the stream's one workspace: every result must equal the first
    bit for bit, whichever workgroup arrived last.  The comparison runs on the device; the host looks every 100."""
    print("epilogues with split K, 600 launches", flush=True)
    lib = ta._lib.load()
    M8, M16 = 8, 16
    qd, ad, code = _quantized(ta, 4096, 14336, seed=21)
    qq, aq, _ = _quantized(ta, 6144, 4096, seed=22)
    assert lib.nf4hip_gemv_workspace_bytes(M8, 4096, 14336) > 65536 * 4 and lib.nf4hip_gemv_workspace_bytes(M16, 6144, 4096) > 65536 * 4
    x8 = _randn((M8, 14336), seed=23).to(DEV)
    r8 = _randn((M8, 4096), seed=24, std=2.0).to(DEV)
    nw = (1.0 + _randn((4096,), seed=25, std=0.1).float()).to(torch.bfloat16).to(DEV)
    xn16 = _randn((M16, 4096), seed=26, std=2.0).to(DEV)
    ss16 = (torch.rand(M16, 256, device=DEV) * 100.0).contiguous()

    def once():
        r, xn, ss = F.matmul_nf4_epilogue(x8, qd, None, ad, code, 64, torch.bfloat16, (4096, 14336), resid_norm=(r8, nw))
        q = F.matmul_nf4_epilogue(xn16, qq, None, aq, code, 64, torch.bfloat16, (6144, 4096), rowscale=(ss16, 1e-5))
        return r, xn, ss, q

    first = once()
    bad = torch.zeros((), dtype=torch.bool, device=DEV)
    for it in range(600):
        got = once()
        for a, b in zip(got, first):
            bad |= (a.view(torch.int32 if a.dtype == torch.float32 else torch.int16) !=
                    b.view(torch.int32 if b.dtype == torch.float32 else torch.int16)).any()
        if it % 100 == 99:
            assert not bool(bad), f"a result changed between launches {it - 99} and {it}"


@pytest.mark.parametrize("M,shape", [(2, (4096, 4096)), (16, (4096, 14336)), (1, (64, 20480)), (32, (512, 1024))])
def test_epilogue_operator_returns_what_its_meta_describes(ta, F, M, shape):
    """The operator registered on the executor: its meta function takes the number of partial sums from the library
    (the serving kernel's launch plan), and where the kernels refuse a case (one row of x with K = 20480, 32 rows of x)
    the operator computes the step itself instead of returning None -- same shapes, same stored roundings."""
    import types

    Q = importlib.import_module("lightning-thunder_amd.transforms.quantization")
    N, K = shape
    print(f"epilogue operator M={M} N={N} K={K}", flush=True)
    qw, absmax, code = _quantized(ta, N, K, seed=N + K + 9)
    x = _randn((M, K), seed=1).to(DEV)
    resid = _randn((M, N), seed=2, std=2.0).to(DEV)
    nw = (1.0 + _randn((N,), seed=3, std=0.1).float()).to(torch.bfloat16).to(DEV)
    proxy = types.SimpleNamespace(shape=(M, K), dtype=torch.bfloat16, device=x.device, requires_grad=False)
    meta = Q.hip_matmul_nf4_epilogue_meta(proxy, None, None, None, None, 64, torch.bfloat16, (N, K), resid_norm=(None, None))
    r, xn, ss = Q.hip_matmul_nf4_epilogue_impl(x, qw, None, absmax, code, 64, torch.bfloat16, (N, K), resid_norm=(resid, nw))
    assert [tuple(t.shape) for t in meta] == [tuple(r.shape), tuple(xn.shape), tuple(ss.shape)]
    delta = F.matmul_nf4(x, qw, None, absmax, code, 64, torch.bfloat16, (N, K))
    r_ref = (resid.float() + delta.float()).to(torch.bfloat16)
    assert torch.equal(_bits(r), _bits(r_ref)) and torch.equal(_bits(xn), _bits((r_ref.float() * nw.float()).to(torch.bfloat16)))
    torch.testing.assert_close(ss.double().sum(-1), r_ref.double().pow(2).sum(-1), rtol=1e-5, atol=0)
    # row scale + SiLU pairs through the operator against the two-step arithmetic
    ss_in = (torch.rand(M, 5, device=DEV) * K).contiguous()
    out = Q.hip_matmul_nf4_epilogue_impl(x, qw, None, absmax, code, 64, torch.bfloat16, (N, K), rowscale=(ss_in, 1e-5), silu_pairs=True)
    meta2 = Q.hip_matmul_nf4_epilogue_meta(proxy, None, None, None, None, 64, torch.bfloat16, (N, K), rowscale=(None, 1e-5), silu_pairs=True)
    assert tuple(out.shape) == tuple(meta2.shape) == (M, N // 2)
    y = (delta.float() * torch.rsqrt(ss_in.sum(-1, keepdim=True) / K + 1e-5))
    ref = torch.nn.functional.silu(y[:, 0::2]) * y[:, 1::2]
    torch.testing.assert_close(out.float(), ref, rtol=4e-2, atol=4e-2)
