"""nf4hip_gemv_static (the entry point that allocates nothing: split-K counters and partial sums in an
array inside the library's device image) against nf4hip_gemv with a caller's workspace, through the C
ABI.  Same kernels, same arithmetic, same order of the partial sums: the outputs must be bit-identical.
Two calls in a row per case, the second with a smaller input, so that what the first left in the array
(partial sums of a larger problem, counters back at zero) is what the second starts from.
"""

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _case(ta, M, N, K, seed):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(N, K, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16).to(DEV)
    x = torch.randn(M, K, generator=g, dtype=torch.float32).to(torch.bfloat16).to(DEV)
    bias = torch.randn(N, generator=g, dtype=torch.float32).to(torch.bfloat16).to(DEV)
    qw, absmax, code = ta.quantize_nf4(w)
    return x, qw, absmax, code, bias


def _both(ta, M, N, K, seed, with_bias, check_memory=False):
    L, lib = ta._lib, ta._lib.load()
    x, qw, absmax, code, bias = _case(ta, M, N, K, seed)
    bptr = bias.data_ptr() if with_bias else None
    stream = torch.cuda.current_stream().cuda_stream
    need = lib.nf4hip_gemv_workspace_bytes(M, N, K)
    assert need <= L.STATIC_SCRATCH_BYTES
    ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
    ref = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    L.check(lib.nf4hip_gemv(x.data_ptr(), L.BF16, M, qw.data_ptr(), absmax.data_ptr(), code.data_ptr(), bptr, N, K, 64,
                            ref.data_ptr(), ws.data_ptr(), ws.numel(), stream))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0] if check_memory else None
    L.check(lib.nf4hip_gemv_static(x.data_ptr(), L.BF16, M, qw.data_ptr(), absmax.data_ptr(), code.data_ptr(), bptr, N, K,
                                   64, out.data_ptr(), stream))
    torch.cuda.synchronize()
    if check_memory:  # what the entry point exists for: the device's free memory is the same after the call
        assert torch.cuda.mem_get_info()[0] == free_before, "nf4hip_gemv_static changed the device's free memory"
    assert not torch.isnan(ref.float()).any()
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), f"M={M} N={N} K={K}: static scratch differs"
    return need


# (first call, second call with a smaller input); every pair splits K over workgroups at least once, so
# the scratch array is really used: M = 16 on short weights (MFMA tile kernel), M = 4 / 2 on a long K
# (quad and row-streaming kernels)
PAIRS = [
    ((16, 6144, 4096), (16, 2048, 4096 + 512)),
    ((16, 4096, 14336), (9, 1000, 4096)),
    ((4, 8192, 28672), (2, 512, 28672)),
    ((8, 4096, 14336), (1, 4096, 4096)),
]


@pytest.mark.parametrize("first,second", PAIRS)
def test_static_scratch_matches_workspace_entry(ta, first, second):
    print(f"gemv_static {first} then {second}", flush=True)
    n1 = _both(ta, *first, seed=11, with_bias=False)
    n2 = _both(ta, *second, seed=12, with_bias=True, check_memory=True)  # (the first call on a device sets the array up)
    assert max(n1, n2) > 65536 * 4, "neither call of the pair used partial sums"


def test_static_scratch_refuses_oversized_shape(ta):
    print("gemv_static oversized", flush=True)
    L, lib = ta._lib, ta._lib.load()
    t = torch.zeros(64, dtype=torch.uint8, device=DEV)
    p = t.data_ptr()
    rc = lib.nf4hip_gemv_static(p, L.BF16, 16, p, p, p, None, 8192, 1 << 20, 64, p, None)
    assert rc == L.E_WORKSPACE
    with pytest.raises(L.NF4HipError, match="scratch"):
        L.check(rc)


def test_static_scratch_under_graph_capture(ta):
    """After one eager call on the device (which resolves the array), the entry point may be recorded into a HIP graph:
    every replay, with eager calls of other shapes on the same array in between, gives the bits of nf4hip_gemv."""
    print("gemv_static in a graph", flush=True)
    L, lib = ta._lib, ta._lib.load()
    M, N, K = 16, 6144, 4096  # K split over workgroups: counters and partial sums in use
    x, qw, absmax, code, _ = _case(ta, M, N, K, seed=21)
    need = lib.nf4hip_gemv_workspace_bytes(M, N, K)
    assert 65536 * 4 < need <= L.STATIC_SCRATCH_BYTES
    ws = torch.zeros(need, dtype=torch.uint8, device=DEV)
    ref = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    L.check(lib.nf4hip_gemv(x.data_ptr(), L.BF16, M, qw.data_ptr(), absmax.data_ptr(), code.data_ptr(), None, N, K, 64,
                            ref.data_ptr(), ws.data_ptr(), ws.numel(), stream))
    L.check(lib.nf4hip_gemv_static(x.data_ptr(), L.BF16, M, qw.data_ptr(), absmax.data_ptr(), code.data_ptr(), None, N, K,
                                   64, out.data_ptr(), stream))  # warm-up: outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            L.check(lib.nf4hip_gemv_static(x.data_ptr(), L.BF16, M, qw.data_ptr(), absmax.data_ptr(), code.data_ptr(), None,
                                           N, K, 64, out.data_ptr(), side.cuda_stream))
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(4):
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), f"replay {rep} differs"
        _both(ta, 8, 4096, 14336, seed=30 + rep, with_bias=False)  # eager work on the same array between the replays
