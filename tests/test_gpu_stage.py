"""The decode kernel that stages codes and absmax through LDS (csrc/nf4_gemv_stage.hip), forced through the C ABI
(``nf4hip_gemv_prefer_staged(1)``) on shapes chosen to hit its corners, against the CPU oracle's dequantised weights
multiplied in float64 (rtol = atol = 2e-2, the matmul's bar), with guard bands around the output and the workspace,
and bit for bit against itself over repeated launches."""

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda"
SENTINEL = 0xA5
GUARD = 4096


@pytest.fixture()
def staged(ta):
    lib = ta._lib.load()
    assert lib.nf4hip_gemv_prefer_staged(1) == 0
    yield lib
    assert lib.nf4hip_gemv_prefer_staged(-1) == 0


def _guarded(nbytes, fill=None):
    raw = torch.full((GUARD + nbytes + (-nbytes) % 256 + GUARD,), SENTINEL, dtype=torch.uint8, device=DEV)
    body = raw[GUARD:GUARD + nbytes]
    if fill is not None:
        body.fill_(fill)
    return raw, body


def _intact(raw, nbytes):
    return bool((raw[:GUARD] == SENTINEL).all()) and bool((raw[GUARD + nbytes:] == SENTINEL).all())


def _run(ta, lib, oracle, M, N, K, seed, bias=False, reps=1, bias_shift=0):
    L = ta._lib
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    b = (torch.randn(N, generator=g) * 0.5).to(torch.bfloat16) if bias else None
    qw, absmax, code = ta.quantize_nf4(w.to(DEV))
    xd = x.to(DEV)
    # (bias_shift = 1: the bias starts two bytes into its allocation, i.e. at an address that is not a multiple of four)
    bd = torch.cat([torch.zeros(bias_shift, dtype=torch.bfloat16), b]).to(DEV)[bias_shift:] if bias else None
    need = lib.nf4hip_gemv_workspace_bytes(M, N, K)
    ws_raw, ws = _guarded(max(need, 256), fill=0)
    out_raw, out = _guarded(M * N * 2)
    stream = torch.cuda.current_stream().cuda_stream
    results = []
    for _ in range(reps):
        out.fill_(0xFF)
        L.check(lib.nf4hip_gemv(xd.data_ptr(), L.BF16, M, qw.data_ptr(), absmax.data_ptr(), code.data_ptr(),
                                None if bd is None else bd.data_ptr(), N, K, 64, out.data_ptr(), ws.data_ptr(), ws.numel(), stream))
        torch.cuda.synchronize()
        results.append(out.view(torch.bfloat16).view(M, N).clone())
    assert _intact(out_raw, M * N * 2), "bytes written outside the output"
    assert _intact(ws_raw, max(need, 256)), "bytes written outside the workspace"
    deq = oracle.C().dequantize(qw.cpu(), absmax.cpu(), oracle.nf4_lut(), 64, torch.bfloat16, (N, K)).double()
    ref = x.double() @ deq.t()
    if bias:
        ref = ref + b.double()
    torch.testing.assert_close(results[0].cpu().double(), ref, rtol=2e-2, atol=2e-2)
    for r in results[1:]:
        assert torch.equal(r.view(torch.int16), results[0].view(torch.int16)), "a repeated launch gave other bits"


# K = 4096: sixteen slices, one K range.  N: one half tile, a last tile that is half filled (N % 16 == 8), more rows than
# one round of workgroups
@pytest.mark.parametrize("M", [1, 2, 4, 5, 8, 9, 13, 16])
@pytest.mark.parametrize("N,K", [(8, 4096), (1000, 4096), (4096, 4096), (6152, 4096)])
def test_staged_kernel_one_k_range(ta, oracle, staged, M, N, K):
    print(f"staged gemv M={M} N={N} K={K}", flush=True)
    _run(ta, staged, oracle, M, N, K, seed=M + N, bias=(N == 1000))


# fewer than sixteen slices (waves without a slice), and K beyond 4096: two to four K ranges meeting in the workspace,
# in fp16 arithmetic beyond 8192
@pytest.mark.parametrize("M", [1, 7, 16])
@pytest.mark.parametrize("N,K", [(520, 512), (2048, 1024), (1024, 2560), (4096, 8192), (1160, 6144), (304, 7168),
                                 (1032, 14336), (4096, 16384), (640, 9216), (2048, 12288)])
def test_staged_kernel_short_and_split_k(ta, oracle, staged, M, N, K):
    print(f"staged gemv M={M} N={N} K={K}", flush=True)
    _run(ta, staged, oracle, M, N, K, seed=3 * M + N + K, bias=(K == 6144), reps=3)


# nested (8-bit) absmax: against the same kernel on the reconstructed fp32 absmax, bit for bit (the reconstruction is the
# same two roundings either way), and against the oracle like every other case
@pytest.mark.parametrize("M", [1, 6, 16])
@pytest.mark.parametrize("N,K", [(1000, 4096), (2048, 1024), (4096, 8192), (1032, 14336), (640, 9216)])
def test_staged_kernel_nested_absmax(ta, oracle, staged, M, N, K):
    import ctypes

    print(f"staged gemv, nested absmax M={M} N={N} K={K}", flush=True)
    plan = (ctypes.c_int * 4)()
    assert staged.nf4hip_gemv_plan(M, N, K, 64, 1, ctypes.byref(plan)) == 0 and plan[0] == 5
    g = torch.Generator().manual_seed(11 * M + N + K)
    # rows of very different magnitude, so that the second-level absmax matters
    w = (torch.randn(N, K, generator=g) * 0.02 * torch.logspace(-2, 0, N).unsqueeze(1)).to(torch.bfloat16)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    qw, absmax, code = ta.quantize_nf4(w.to(DEV))
    nested = ta.compress_absmax(absmax)
    rec = ta.reconstruct_absmax(nested)
    y = ta.matmul_nf4(x.to(DEV), qw, None, nested, code, 64, torch.bfloat16, (N, K))
    y_rec = ta.matmul_nf4(x.to(DEV), qw, None, rec, code, 64, torch.bfloat16, (N, K))
    assert torch.equal(y.view(torch.int16), y_rec.view(torch.int16))
    deq = oracle.C().dequantize(qw.cpu(), rec.cpu(), oracle.nf4_lut(), 64, torch.bfloat16, (N, K)).double()
    torch.testing.assert_close(y.cpu().double(), x.double() @ deq.t(), rtol=2e-2, atol=2e-2)


def _random_cases(count, seed):
    import random

    rnd = random.Random(seed)
    cases = []
    for _ in range(count):
        K = 256 * rnd.choice([1, 2, 3, 5, 8, 15, 16, 17, 20, 24, 31, 32, 33, 40, 47, 48, 49, 56, 63, 64])
        N = 8 * rnd.randint(1, 160 if K <= 8192 else 80)
        cases.append((rnd.randint(1, 16), N, K, rnd.random() < 0.4, rnd.random() < 0.3))
    return cases


@pytest.mark.parametrize("M,N,K,nested,bias", _random_cases(36, 20240611))
def test_staged_kernel_random_shapes(ta, oracle, staged, M, N, K, nested, bias):
    """Random (M, N, K) inside the kernel's rules -- every number of K ranges (1..4), last ranges with fewer slices than the
    others, row ranges that end in a half tile, fp32 and nested absmax, with and without bias -- against the oracle."""
    print(f"staged gemv, random case M={M} N={N} K={K} nested={nested} bias={bias}", flush=True)
    g = torch.Generator().manual_seed(M * 7 + N * 3 + K)
    w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    b = (torch.randn(N, generator=g) * 0.5).to(torch.bfloat16) if bias else None
    qw, absmax, code = ta.quantize_nf4(w.to(DEV))
    state = ta.compress_absmax(absmax) if nested else absmax
    rec = ta.reconstruct_absmax(state) if nested else absmax
    y = ta.matmul_nf4(x.to(DEV), qw, None if b is None else b.to(DEV), state, code, 64, torch.bfloat16, (N, K))
    deq = oracle.C().dequantize(qw.cpu(), rec.cpu(), oracle.nf4_lut(), 64, torch.bfloat16, (N, K)).double()
    ref = x.double() @ deq.t()
    if bias:
        ref = ref + b.double()
    torch.testing.assert_close(y.cpu().double(), ref, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("M", [1, 16])
def test_staged_kernel_bias(ta, oracle, staged, M):
    """The bias of a workgroup's rows is staged in LDS, 128 rows per wave: workgroups with one, two and eight waves' worth
    of rows, a last workgroup that ends inside a wave's 128 rows, and K split over workgroups (the bias is added by
    the workgroup that adds the K ranges).  A bias at an address that is no multiple of four, or more than 1024 rows
    per workgroup, is left to the other kernels: same result contract."""
    for (N, K, shift) in [(4096, 4096, 0), (40000, 512, 0), (262144 - 8, 512, 0), (1000, 8192, 0), (4096, 4096, 1), (262144 + 4096, 512, 0)]:
        print(f"staged gemv with bias M={M} N={N} K={K} shift={shift}", flush=True)
        _run(ta, staged, oracle, M, N, K, seed=N + K + M, bias=True, bias_shift=shift)


def test_staged_kernel_many_launches_are_bit_stable(ta, oracle, staged):
    """[4096, 8192] and [4096, 14336], sixteen rows of x: K is split over two / four workgroups per row range, whichever
    arrives last adds the partial sums in range order -- 200 launches on one workspace must give one result."""
    print("staged gemv, 200 launches with K split", flush=True)
    _run(ta, staged, oracle, 16, 4096, 8192, seed=99, reps=200)
    _run(ta, staged, oracle, 16, 4096, 14336, seed=98, reps=200)


def test_staged_kernel_is_refused_where_it_does_not_apply(ta, oracle, staged):
    """K not a multiple of 256 or beyond 16384, N not a multiple of 8: nf4hip_gemv falls back to its other kernels (same
    result contract)."""
    print("staged gemv, shapes it leaves to the other kernels", flush=True)
    _run(ta, staged, oracle, 4, 512, 4096 + 512 + 32, seed=5)
    _run(ta, staged, oracle, 16, 512, 16384 + 512, seed=6)
    _run(ta, staged, oracle, 3, 1004, 4096, seed=7)
