"""The dense bf16 GEMM that follows nf4hip_dequantize on the dequantize + linear route (csrc/nf4_gemm_dense.hip,
``nf4hip_linear``), called through the C ABI with guard bands around the output and the workspace, against the product of
the same bf16 operands in float64 (rtol = atol = 2e-2, the matmul's bar, and no worse than twice the error of a float32
product rounded to bf16), bit for bit against itself over repeated launches (tiles cut in two along K meet in the
workspace in whichever order the workgroups arrive), and end to end behind ``matmul_nf4`` against the CPU oracle."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda"
SENTINEL = 0xA5
GUARD = 4096


def _guarded(nbytes, fill=None):
    raw = torch.full((GUARD + nbytes + (-nbytes) % 256 + GUARD,), SENTINEL, dtype=torch.uint8, device=DEV)
    body = raw[GUARD:GUARD + nbytes]
    if fill is not None:
        body.fill_(fill)
    return raw, body


def _intact(raw, nbytes):
    return bool((raw[:GUARD] == SENTINEL).all()) and bool((raw[GUARD + nbytes:] == SENTINEL).all())


def _operands(M, N, K, seed, bias):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) / K ** 0.5).to(torch.bfloat16)
    b = torch.randn(N, generator=g).to(torch.bfloat16) if bias else None
    return x, w, b


def _reference(x, w, b, rows=None):
    xs = x if rows is None else x[rows]
    ref = xs.double() @ w.double().t()
    return ref + b.double() if b is not None else ref


def _call(ta, x, w, b, reps=1):
    """nf4hip_linear through the C ABI on guarded buffers; returns the outputs of ``reps`` launches."""
    L, lib = ta._lib, ta._lib.load()
    M, K = x.shape
    N = w.shape[0]
    xd, wd = x.to(DEV), w.to(DEV)
    bd = None if b is None else b.to(DEV)
    need = lib.nf4hip_linear_workspace_bytes(M, N, K)
    ws_raw, ws = _guarded(max(need, 16), fill=0)
    outs = []
    for _ in range(reps):
        out_raw, out = _guarded(2 * M * N)
        rc = lib.nf4hip_linear(xd.data_ptr(), L.BF16, M, wd.data_ptr(), None if bd is None else bd.data_ptr(), N, K, out.data_ptr(),
                               ws.data_ptr() if need else None, ws.numel() if need else 0, torch.cuda.current_stream().cuda_stream)
        L.check(rc)
        torch.cuda.synchronize()
        assert _intact(out_raw, 2 * M * N), "write outside the output"
        outs.append(out.view(torch.bfloat16).reshape(M, N).clone())
    assert _intact(ws_raw, max(need, 16)), "write outside the workspace"
    if need:
        assert not bool(ws[: 4 * 2 * 128].any()), "the tile counters are not back at zero"
    return outs


# (M, N, K): one tile; ragged rows of x and of w; the shortest k loops (2 and 3 steps); odd N (scalar stores); tiles cut
# in two along K (<= 128 tiles, K >= 2048), also with ragged edges and an odd number of k steps; several rounds of tiles
SHAPES = [
    (256, 256, 128), (256, 256, 192), (1, 8, 128), (300, 520, 192), (255, 257, 4096), (17, 1000, 320), (513, 77, 2048 + 64),
    (512, 1000, 2048), (777, 1024, 4096), (2048, 4096, 4096), (1024, 2048, 14336), (2304, 7168, 512), (64, 33000, 1024),
]


@pytest.mark.parametrize("M,N,K", SHAPES)
@pytest.mark.parametrize("bias", [False, True])
def test_linear_equals_the_float64_product(ta, M, N, K, bias):
    print(f"nf4hip_linear M={M} N={N} K={K} bias={bias}", flush=True)
    x, w, b = _operands(M, N, K, seed=M + N + K, bias=bias)
    (out,) = _call(ta, x, w, b)
    rows = None if M * N * K <= 1 << 33 else torch.arange(0, M, max(1, M // 256))
    ref = _reference(x, w, b, rows)
    got = (out.cpu() if rows is None else out.cpu()[rows]).double()
    torch.testing.assert_close(got, ref, rtol=2e-2, atol=2e-2)
    rounded = ref.float().to(torch.bfloat16).double()  # what an exact product leaves after the one rounding to bf16
    assert (got - ref).abs().max() <= 2 * (rounded - ref).abs().max() + 1e-6


@pytest.mark.parametrize("M,N,K", [(512, 1000, 2048), (2048, 4096, 4096), (300, 520, 2048 + 64)])
def test_pieces_meet_in_any_order_with_the_same_bits(ta, M, N, K):
    print(f"nf4hip_linear repeats M={M} N={N} K={K}", flush=True)
    lib = ta._lib.load()
    plan = (ctypes.c_int * 4)()
    assert lib.nf4hip_linear_plan(M, N, K, ctypes.byref(plan)) == 0 and plan[2] == 2 and plan[3] == 2 * plan[1]
    x, w, b = _operands(M, N, K, seed=7, bias=True)
    outs = _call(ta, x, w, b, reps=40)
    assert all(torch.equal(o, outs[0]) for o in outs[1:])


def test_linear_matches_the_library_on_a_prefill_shape(ta):
    """[14336, 4096] with 2048 rows of x (BASELINE config 3): same fp32 accumulation, one rounding -- the hand-written
    kernel and torch.nn.functional.linear may differ by an ulp of bf16 where the sums differ in their last bits."""
    M, N, K = 2048, 14336, 4096
    print(f"nf4hip_linear vs library M={M} N={N} K={K}", flush=True)
    x, w, b = _operands(M, N, K, seed=11, bias=False)
    out = ta.functional.linear_bf16(x.to(DEV), w.to(DEV))
    lib = torch.nn.functional.linear(x.to(DEV), w.to(DEV))
    torch.testing.assert_close(out.float(), lib.float(), rtol=2 ** -7, atol=2 ** -7)


@pytest.mark.parametrize("M,N,K", [(512, 4096, 4096), (4096, 1024, 4096)])
def test_dense_route_of_matmul_nf4_runs_the_hand_written_kernel(ta, oracle, monkeypatch, M, N, K):
    print(f"matmul_nf4 dequant+gemm M={M} N={N} K={K}", flush=True)
    F = ta.functional
    g = torch.Generator().manual_seed(M + N)
    w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    bias = torch.randn(N, generator=g).to(torch.bfloat16)
    qw, absmax, code = ta.quantize_nf4(w.to(DEV))
    ref = oracle.matmul_4bit_f64(x, qw.cpu(), bias, absmax.cpu(), oracle.nf4_lut(), 64, torch.bfloat16, (N, K))
    called = []
    real = F.linear_bf16
    monkeypatch.setattr(F, "linear_bf16", lambda *a: (called.append(1), real(*a))[1])
    monkeypatch.setattr(torch.nn.functional, "linear", lambda *a, **k: pytest.fail("the library GEMM ran on the dequant+gemm route"))
    y = F._matmul_nf4_on(x.to(DEV), qw, bias.to(DEV), absmax, code, 64, torch.bfloat16, (N, K), "dequant+gemm")
    assert called == [1]
    torch.testing.assert_close(y.cpu().float(), ref.float(), rtol=2e-2, atol=2e-2)


def test_linear_refuses_what_it_does_not_serve(ta):
    F = ta.functional
    x = torch.zeros(4, 96, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(8, 96, dtype=torch.bfloat16, device=DEV)
    assert not F.linear_possible(x, w)
    with pytest.raises(ValueError):
        F.linear_bf16(x, w)
    with pytest.raises(ValueError):
        F.linear_bf16(torch.zeros(4, 128, dtype=torch.float16, device=DEV), torch.zeros(8, 128, dtype=torch.float16, device=DEV))
