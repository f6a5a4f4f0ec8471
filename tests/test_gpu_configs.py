"""GPU parity at the full sizes of the benchmark configurations, through the C ABI, with guard bands.

* decode shapes: the five Llama-3-8B projection shapes, blocksize 64, fp32 absmax, M in {1, 4, 16};
* prefill shapes: the same weights, M in {512, 2048, 8192}, on the route the router picks and on the fused
  kernel forced;
* Llama-3-70B shapes with nested (double-quantised) absmax, M in {1, 16, 2048}.

Reference: float64 accumulation of x against weights dequantised by the CPU ORACLE (not by the kernels under test),
over every row of x and, per weight, three complete 256-row tiles (first, middle, last) plus 64 scattered rows --
a defect confined to one tile of the grid cannot hide between samples.  Tolerance rtol = atol = 2e-2 (bf16 output,
fp32 accumulation).  The decode cases are also compared over ALL outputs against x @ dequantize(w) computed with
the HIP dequantize kernel, which is itself pinned bit-exact at small sizes.

Every output the kernels write (out, packed codes, absmax, workspace) sits between guard bands filled with a
sentinel; the bands must be untouched after the call.
"""

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda"
GUARD = 4096  # bytes on either side
SENTINEL = 0xA5

LLAMA_8B = [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336), (128256, 4096)]
LLAMA_70B = [(8192, 8192), (1024, 8192), (28672, 8192), (8192, 28672)]


class Guarded:
    """A device buffer of ``nbytes`` between two sentinel-filled bands."""

    def __init__(self, nbytes: int, fill=None):
        pad = (-nbytes) % 256
        self.raw = torch.full((GUARD + nbytes + pad + GUARD,), SENTINEL, dtype=torch.uint8, device=DEV)
        self.nbytes = nbytes
        self.body = self.raw[GUARD : GUARD + nbytes]
        if fill is not None:
            self.body.fill_(fill)
        assert self.body.data_ptr() % 256 == 0

    def ptr(self) -> int:
        return self.body.data_ptr()

    def view(self, dtype, shape):
        return self.body.view(dtype).view(shape)

    def check(self, what: str):
        head = self.raw[:GUARD]
        tail = self.raw[GUARD + self.nbytes :]
        assert bool((head == SENTINEL).all()), f"{what}: bytes written BEFORE the buffer"
        assert bool((tail == SENTINEL).all()), f"{what}: bytes written PAST the buffer"


def _cpu_weight(N, K, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(N, K, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16)


def _cpu_acts(M, K, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(M, K, generator=g, dtype=torch.float32).to(torch.bfloat16)


class QuantizedWeight:
    """One benchmark weight, quantised once through nf4hip_quantize into guarded buffers (seeded on the CPU)."""

    def __init__(self, ta, N, K, seed, nested=False):
        L, lib = ta._lib, ta._lib.load()
        self.N, self.K = N, K
        n = N * K
        w_cpu = _cpu_weight(N, K, seed)
        w = w_cpu.to(DEV)
        self.packed_g = Guarded(n // 2)
        self.absmax_g = Guarded(n // 64 * 4)
        L.check(lib.nf4hip_quantize(w.data_ptr(), L.BF16, n, 64, self.packed_g.ptr(), self.absmax_g.ptr(),
                                    torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        self.packed_g.check("nf4hip_quantize packed")
        self.absmax_g.check("nf4hip_quantize absmax")
        del w
        self.packed = self.packed_g.view(torch.uint8, (n // 2, 1))
        self.absmax = self.absmax_g.view(torch.float32, (n // 64,))
        self.code = ta.nf4_code(DEV)
        self.nested = ta.compress_absmax(self.absmax) if nested else None
        # what the matmul kernels are given / what the reference uses for absmax
        self.absmax_arg = self.nested if nested else self.absmax
        self.absmax_ref = ta.reconstruct_absmax(self.nested) if nested else self.absmax
        g = torch.Generator().manual_seed(seed + 7)
        tiles = sorted({0, (N // 256) // 2 * 256, max(N - 256, 0)})
        rows = torch.cat([torch.arange(t, min(t + 256, N)) for t in tiles] + [torch.randint(0, N, (64,), generator=g)])
        self.rows = torch.unique(rows)
        self.w_rows = w_cpu[self.rows].clone()  # the sampled rows of the bf16 weight, for the oracle's own quantisation
        del w_cpu

    def oracle_rows(self, oracle):
        """fp64 [len(rows), K] on the GPU: the sampled weight rows dequantised by the CPU oracle."""
        K = self.K
        rows = self.rows.to(DEV)
        packed = self.packed.view(self.N, K // 2)[rows].cpu().reshape(-1, 1)
        absmax = self.absmax_ref.view(self.N, K // 64)[rows].cpu().reshape(-1)
        deq = oracle.C().dequantize(packed, absmax, oracle.nf4_lut(), 64, torch.bfloat16, (len(rows), K))
        return deq.to(DEV).double()


@pytest.fixture(scope="module")
def weights(ta):
    cache = {}

    def get(N, K, seed, nested=False):
        key = (N, K, seed, nested)
        if key not in cache:
            if len(cache) >= 2:  # the lm_head weight alone is 0.3 GB packed; keep the fixture small
                cache.pop(next(iter(cache)))
            cache[key] = QuantizedWeight(ta, N, K, seed, nested)
        return cache[key]

    yield get
    cache.clear()


@pytest.mark.parametrize("shape,seed", [(s, 2000 + i) for i, s in enumerate(LLAMA_8B)] + [(s, 5000 + i) for i, s in enumerate(LLAMA_70B)])
def test_full_size_quantize_equals_the_oracle_on_sampled_rows(ta, oracle, weights, shape, seed):
    """nf4hip_quantize ran over the whole benchmark weight; its codes and absmax of three complete 256-row tiles (first,
    middle, last) and 64 scattered rows must be the CPU oracle's for the same bf16 rows, bit for bit (K is a multiple of
    the blocksize, so a row's blocks depend on that row alone)."""
    N, K = shape
    print(f"full-size quantize vs oracle [{N},{K}]", flush=True)
    qw = weights(N, K, seed, nested=shape in LLAMA_70B)
    rows = qw.rows.to(DEV)
    packed = qw.packed.view(N, K // 2)[rows].cpu()
    absmax = qw.absmax.view(N, K // 64)[rows].cpu()
    packed_o, absmax_o = oracle.C().quantize(qw.w_rows, 64)
    assert torch.equal(packed.reshape(-1, 1), packed_o), "packed codes differ from the oracle's"
    assert torch.equal(absmax.reshape(-1).view(torch.int32), absmax_o.view(torch.int32)), "absmax differs from the oracle's"


def _check_against_oracle(out, x, qw, oracle, what):
    ref = x.double() @ qw.oracle_rows(oracle).T  # [M, rows]
    got = out[:, qw.rows.to(DEV)].double()
    torch.testing.assert_close(got, ref, rtol=2e-2, atol=2e-2, msg=lambda m: f"{what}: {m}")


def _call_matmul(ta, kind, x, qw, out_g, M):
    """nf4hip_gemv / nf4hip_gemm (or their nested-absmax forms) through the C ABI into a guarded output, with a
    guarded workspace."""
    L, lib = ta._lib, ta._lib.load()
    N, K = qw.N, qw.K
    need = (lib.nf4hip_gemv_workspace_bytes if kind == "gemv" else lib.nf4hip_gemm_workspace_bytes)(M, N, K)
    ws = Guarded(max(need, 256), fill=0)
    stream = torch.cuda.current_stream().cuda_stream
    if qw.nested is None:
        fn = lib.nf4hip_gemv if kind == "gemv" else lib.nf4hip_gemm
        L.check(fn(x.data_ptr(), L.BF16, M, qw.packed.data_ptr(), qw.absmax.data_ptr(), qw.code.data_ptr(), None, N, K, 64,
                   out_g.ptr(), ws.ptr(), ws.nbytes, stream))
    else:
        nq = qw.nested
        fn = lib.nf4hip_gemv_dq if kind == "gemv" else lib.nf4hip_gemm_dq
        L.check(fn(x.data_ptr(), L.BF16, M, qw.packed.data_ptr(), nq.q.data_ptr(), nq.absmax2.data_ptr(), nq.map256.data_ptr(),
                   float(nq.offset), int(nq.blocksize), qw.code.data_ptr(), None, N, K, 64, out_g.ptr(), ws.ptr(), ws.nbytes, stream))
    torch.cuda.synchronize()
    out_g.check(f"nf4hip_{kind} out")
    ws.check(f"nf4hip_{kind} workspace")
    if need > 65536 * 4:
        assert not bool(ws.body[: 65536 * 4].any()), f"nf4hip_{kind}: arrival counters not back at zero"


# ------------------------------------------------------------------------------------------------
# decode regime, Llama-3-8B shapes, M in {1, 4, 16}
# ------------------------------------------------------------------------------------------------


@pytest.mark.parametrize("M", [1, 4, 16])
@pytest.mark.parametrize("shape_index", range(len(LLAMA_8B)))
def test_decode_shapes_full_size(ta, oracle, weights, shape_index, M):
    N, K = LLAMA_8B[shape_index]
    print(f"config 2 [{N},{K}] M={M}", flush=True)
    qw = weights(N, K, 2000 + shape_index)
    x = _cpu_acts(M, K, 200000 + 100 * shape_index + [1, 4, 16].index(M)).to(DEV)
    out_g = Guarded(M * N * 2)
    _call_matmul(ta, "gemv", x, qw, out_g, M)
    out = out_g.view(torch.bfloat16, (M, N))
    _check_against_oracle(out, x, qw, oracle, f"gemv [{N},{K}] M={M}")
    # every output, against x @ dequantize(w) with the HIP dequantize kernel (pinned bit-exact elsewhere)
    ref = torch.empty(M, N, dtype=torch.float64, device=DEV)
    step = max(1, (1 << 26) // K)
    for n0 in range(0, N, step):
        n1 = min(N, n0 + step)
        wd = ta.dequantize_nf4(qw.packed[n0 * K // 2 : n1 * K // 2], qw.absmax[n0 * K // 64 : n1 * K // 64], qw.code, 64,
                               torch.bfloat16, (n1 - n0, K))
        ref[:, n0:n1] = x.double() @ wd.double().T
    torch.testing.assert_close(out.double(), ref, rtol=2e-2, atol=2e-2)
    # the product op takes the same route and gives the same bits
    y = ta.matmul_nf4(x, qw.packed, None, qw.absmax, qw.code, 64, torch.bfloat16, (N, K))
    assert ta.functional.fused_route(x, None, 64, torch.bfloat16, (N, K)) == "gemv"
    assert torch.equal(y.view(torch.int16), out.view(torch.int16))


# ------------------------------------------------------------------------------------------------
# prefill regime, the same weights, M in {512, 2048, 8192}
# ------------------------------------------------------------------------------------------------


@pytest.mark.parametrize("M", [512, 2048, 8192])
@pytest.mark.parametrize("shape_index", range(len(LLAMA_8B)))
def test_prefill_shapes_full_size(ta, oracle, weights, shape_index, M):
    N, K = LLAMA_8B[shape_index]
    qw = weights(N, K, 2000 + shape_index)
    x = _cpu_acts(M, K, 300000 + 100 * shape_index + [512, 2048, 8192].index(M)).to(DEV)
    route = ta.functional.fused_route(x, None, 64, torch.bfloat16, (N, K))
    print(f"config 3 [{N},{K}] M={M} router -> {route}", flush=True)
    assert route in ("gemm", "dequant+gemm")
    # the route the router picks
    y = ta.matmul_nf4(x, qw.packed, None, qw.absmax, qw.code, 64, torch.bfloat16, (N, K))
    assert y.shape == (M, N) and y.dtype == torch.bfloat16
    _check_against_oracle(y, x, qw, oracle, f"{route} [{N},{K}] M={M}")
    del y
    # the hand-written fused kernel, forced, through the C ABI
    out_g = Guarded(M * N * 2)
    _call_matmul(ta, "gemm", x, qw, out_g, M)
    _check_against_oracle(out_g.view(torch.bfloat16, (M, N)), x, qw, oracle, f"nf4hip_gemm [{N},{K}] M={M}")


@pytest.mark.parametrize("M", [512, 1024])
def test_lm_head_router_takes_fused_kernel(ta, oracle, weights, M):
    N, K = LLAMA_8B[4]
    print(f"lm_head M={M} through the router", flush=True)
    qw = weights(N, K, 2004)
    x = _cpu_acts(M, K, 310000 + M).to(DEV)
    assert ta.functional.fused_route(x, None, 64, torch.bfloat16, (N, K)) == "gemm"
    y = ta.matmul_nf4(x, qw.packed, None, qw.absmax, qw.code, 64, torch.bfloat16, (N, K))
    _check_against_oracle(y, x, qw, oracle, f"router gemm lm_head M={M}")


# Calls with fewer tiles than CUs cut every tile into 2..8 pieces along k that meet in the workspace (two pieces: the
# later one adds the other's partial to its registers; more: the last to publish adds all of them from memory in k
# order).  Both tile heights, ragged M and N, nested absmax; every case is also repeated on one workspace and must
# give the same bits every time (the sum order does not depend on which workgroup finishes last).
@pytest.mark.parametrize("M,N,K,nested", [
    (300, 1000, 2048, False),    # 128-row tile, 12 tiles x 2 pieces, ragged M and N
    (512, 4096, 4096, False),    # 128-row tile, 64 tiles x 4 pieces
    (256, 1024, 8192, False),    # 128-row tile, 8 tiles x 8 pieces
    (1024, 4096, 4096, True),    # 128-row tile, 128 tiles x 2 pieces, nested absmax
    (2048, 4096, 14336, False),  # 256-row tile, 128 tiles x 2 pieces
    (512, 8192, 28672, False),   # 256-row tile, 64 tiles x 4 pieces
    (130, 264, 2048 + 64, False),  # 33 k steps: one quantum per k step
])
def test_fused_gemm_cut_up_tiles(ta, oracle, M, N, K, nested):
    print(f"cut-up tiles M={M} [{N},{K}] nested={nested}", flush=True)
    lib = ta._lib.load()
    assert lib.nf4hip_gemm_workspace_bytes(M, N, K) > 65536 * 4, "this shape is expected to cut its tiles"
    qw = QuantizedWeight(ta, N, K, 4242 + M, nested=nested)
    x = _cpu_acts(M, K, 4243 + N).to(DEV)
    out_g = Guarded(M * N * 2)
    _call_matmul(ta, "gemm", x, qw, out_g, M)
    first = out_g.view(torch.int16, (M, N)).clone()
    _check_against_oracle(out_g.view(torch.bfloat16, (M, N)), x, qw, oracle, f"nf4hip_gemm cut up [{N},{K}] M={M}")
    # the ABI insists on the workspace it asked for
    L = ta._lib
    if not nested:
        rc = lib.nf4hip_gemm(x.data_ptr(), L.BF16, M, qw.packed.data_ptr(), qw.absmax.data_ptr(), qw.code.data_ptr(), None, N, K, 64,
                             out_g.ptr(), None, 0, torch.cuda.current_stream().cuda_stream)
        assert rc == L.E_WORKSPACE
    for rep in range(4):
        out_g.body.fill_(0)
        _call_matmul(ta, "gemm", x, qw, out_g, M)
        assert torch.equal(out_g.view(torch.int16, (M, N)), first), f"repeat {rep} differs"


# ------------------------------------------------------------------------------------------------
# Llama-3-70B shapes, nested absmax, M in {1, 16, 2048}
# ------------------------------------------------------------------------------------------------


@pytest.mark.parametrize("M", [1, 16, 2048])
@pytest.mark.parametrize("shape_index", range(len(LLAMA_70B)))
def test_llama70b_shapes_nested_full_size(ta, oracle, weights, shape_index, M):
    N, K = LLAMA_70B[shape_index]
    print(f"config 5 [{N},{K}] M={M} nested absmax", flush=True)
    qw = weights(N, K, 5000 + shape_index, nested=True)
    x = _cpu_acts(M, K, 500000 + 100 * shape_index + [1, 16, 2048].index(M)).to(DEV)
    out_g = Guarded(M * N * 2)
    kind = "gemv" if M <= 16 else "gemm"
    _call_matmul(ta, kind, x, qw, out_g, M)
    out = out_g.view(torch.bfloat16, (M, N))
    _check_against_oracle(out, x, qw, oracle, f"nf4hip_{kind}_dq [{N},{K}] M={M}")
    # the product op (router's choice) on the nested form
    y = ta.matmul_nf4(x, qw.packed, None, qw.nested, qw.code, 64, torch.bfloat16, (N, K))
    _check_against_oracle(y, x, qw, oracle, f"matmul_nf4 nested [{N},{K}] M={M}")


# ------------------------------------------------------------------------------------------------
# ragged shapes: guard bands around every output of every entry point
# ------------------------------------------------------------------------------------------------


@pytest.mark.parametrize("M,N,K", [(1, 1000, 4096), (3, 17, 1376 - 32), (4, 130, 2048), (7, 1000, 4096), (16, 4100, 4096),
                                   (13, 77, 512), (40, 300, 576), (100, 1000, 1344), (129, 257, 4096), (300, 513, 1024),
                                   (257, 4097, 128)])
def test_ragged_shapes_guard_bands(ta, oracle, M, N, K):
    print(f"guards M={M} N={N} K={K}", flush=True)
    qw = QuantizedWeight(ta, N, K, seed=N + K)
    x = _cpu_acts(M, K, M + N).to(DEV)
    out_g = Guarded(M * N * 2)
    kind = "gemv" if M <= 16 and (K % 512 == 0 or M <= 4) else "gemm"
    _call_matmul(ta, kind, x, qw, out_g, M)
    ref = x.double() @ qw.oracle_rows(oracle).T
    torch.testing.assert_close(out_g.view(torch.bfloat16, (M, N))[:, qw.rows.to(DEV)].double(), ref, rtol=2e-2, atol=2e-2)
    # dequantize into a guarded buffer, all three output dtypes
    L, lib = ta._lib, ta._lib.load()
    n = N * K
    for dtype, code, size in ((torch.bfloat16, L.BF16, 2), (torch.float16, L.F16, 2), (torch.float32, L.F32, 4)):
        deq_g = Guarded(n * size)
        L.check(lib.nf4hip_dequantize(qw.packed.data_ptr(), qw.absmax.data_ptr(), qw.code.data_ptr(), n, 64, deq_g.ptr(), code,
                                      torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        deq_g.check(f"nf4hip_dequantize {dtype}")
        want = oracle.C().dequantize(qw.packed.cpu(), qw.absmax.cpu(), oracle.nf4_lut(), 64, dtype, (N, K))
        assert torch.equal(deq_g.view(dtype, (N, K)).cpu().view(torch.uint8), want.view(torch.uint8))


@pytest.mark.parametrize("n", [2, 64, 66, 4096 + 2, 64 * 1000 + 34, 2048 * 33])
@pytest.mark.parametrize("blocksize", [64, 256, 4096])
def test_quantize_guard_bands(ta, oracle, n, blocksize):
    print(f"guards quantize n={n} blocksize={blocksize}", flush=True)
    L, lib = ta._lib, ta._lib.load()
    w = _cpu_weight(1, n, n + blocksize)
    wd = w.to(DEV)
    nblocks = (n + blocksize - 1) // blocksize
    packed_g, absmax_g = Guarded((n + 1) // 2), Guarded(nblocks * 4)
    L.check(lib.nf4hip_quantize(wd.data_ptr(), L.BF16, n, blocksize, packed_g.ptr(), absmax_g.ptr(),
                                torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    packed_g.check("quantize packed")
    absmax_g.check("quantize absmax")
    qw_o, absmax_o = oracle.C().quantize(w, blocksize)
    assert torch.equal(packed_g.view(torch.uint8, ((n + 1) // 2, 1)).cpu(), qw_o)
    assert torch.equal(absmax_g.view(torch.float32, (nblocks,)).cpu(), absmax_o)


# ------------------------------------------------------------------------------------------------
# double quantisation through the product API: jit(model, transforms=[BitsAndBytesLinearQuant4bit(double_quant=True)])
# ------------------------------------------------------------------------------------------------


@pytest.mark.parametrize("N,K", [(1024, 8192), (8192, 8192)])
def test_double_quant_linear_through_jit(ta, oracle, N, K):
    print(f"double_quant through jit [{N},{K}]", flush=True)
    lin = torch.nn.Linear(K, N, bias=False, dtype=torch.bfloat16)
    with torch.no_grad():
        lin.weight.copy_(_cpu_weight(N, K, 5100 + N // 1024))
    w_cpu = lin.weight.detach().clone()
    lin = lin.to(DEV).eval().requires_grad_(False)
    jm = ta.jit(lin, transforms=[ta.BitsAndBytesLinearQuant4bit(double_quant=True)], executors=(ta.get_hip_nf4_executor(),))
    sd = {k: v.cpu() for k, v in jm.state_dict().items()}
    assert set(sd) == {"weight", "weight.absmax", "weight.code", "weight.nested_absmax", "weight.nested_quant_map", "weight.nested_offset"}
    # every stored tensor is what the CPU oracle computes from the same weight
    qw_o, absmax_o = oracle.C().quantize(w_cpu, 64)
    D = oracle.create_dynamic_map()
    off = oracle.C().dq_offset(absmax_o)
    q_o, a2_o = oracle.C().dq_compress(absmax_o, D, off)
    assert torch.equal(sd["weight"], qw_o) and torch.equal(sd["weight.absmax"], q_o) and torch.equal(sd["weight.nested_absmax"], a2_o)
    assert torch.equal(sd["weight.nested_quant_map"], D) and sd["weight.nested_offset"].tolist() == [off]
    absmax_ref = oracle.C().dq_reconstruct(q_o, a2_o, D, off)
    g = torch.Generator().manual_seed(N + K)
    rows = torch.unique(torch.cat([torch.arange(0, 256), torch.arange(N - 256, N), torch.randint(0, N, (64,), generator=g)]))
    deq = oracle.C().dequantize(qw_o.view(N, K // 2)[rows].reshape(-1, 1), absmax_ref.view(N, K // 64)[rows].reshape(-1), oracle.nf4_lut(),
                                64, torch.bfloat16, (len(rows), K)).to(DEV).double()
    for M in (1, 16, 2048):
        x = _cpu_acts(M, K, 510000 + M).to(DEV)
        y = jm(x)
        assert y.shape == (M, N) and y.dtype == torch.bfloat16
        torch.testing.assert_close(y[:, rows.to(DEV)].double(), x.double() @ deq.T, rtol=2e-2, atol=2e-2)
    calls = [b.sym.name for b in ta.last_traces(jm)[-1].bound_symbols if b.sym.executor is not None]
    assert calls == ["hip_matmul_nf4_dq"]
