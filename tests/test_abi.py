"""The C-ABI library without a GPU: it loads, exports every symbol include/nf4hip.h declares, and
every argument error is reported before any HIP call is made."""

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "nf4hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nf4hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol(ta):
    lib = ta._lib.load()
    declared = _declared_symbols()
    assert len(declared) >= 13
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/nf4hip.h but not exported"
    assert sorted(ta._lib.SYMBOLS) == declared, "ctypes prototypes out of sync with the header"
    assert lib.nf4hip_abi_version() == ta._lib.ABI_VERSION == 6


def test_probe_library_loads_and_validates(ta):
    """libnf4hip_probe.so (bench.py's read-only kernel) is built next to the path's library and refuses bad arguments
    before it launches anything."""
    import ctypes
    import os

    path = os.path.join(os.path.dirname(ta.__file__), "libnf4hip_probe.so")
    assert os.path.exists(path), "run __graft_entry__.build()"
    probe = ctypes.CDLL(path)
    fn = probe.nf4hip_probe_stream_read
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]
    assert fn(None, 1024, None, 0, None, None) != 0
    assert fn(4096, 1000, None, 0, None, None) != 0  # not a multiple of 16
    assert fn(4096, 1024, None, 16, None, None) != 0  # bytes of b without b


def test_missing_library_fails_loudly(ta, tmp_path):
    with pytest.raises(RuntimeError, match="not found"):
        ta._lib.load(str(tmp_path / "libnf4hip.so"))


def _err(ta):
    return ta._lib.load().nf4hip_last_error().decode()


def test_gemv_plan_names_the_kernel(ta):
    """nf4hip_gemv_plan: which decode kernel a call goes to, without a GPU; it follows nf4hip_gemv_prefer_staged."""
    import ctypes

    L, lib = ta._lib, ta._lib.load()
    plan = (ctypes.c_int * 4)()

    def kernel(M, N, K, nested=0):
        assert lib.nf4hip_gemv_plan(M, N, K, 64, nested, ctypes.byref(plan)) == 0
        return plan[0], plan[1]

    assert lib.nf4hip_gemv_prefer_staged(-1) == 0
    assert kernel(1, 4096, 4096) == (1, 0) and kernel(4, 4096, 4096) == (2, 0) and kernel(16, 1024, 4096) == (3, 0)
    assert kernel(1, 128256, 4096) == (5, 0) and kernel(16, 14336, 4096) == (5, 0) and kernel(4, 14336, 4096) == (2, 0)
    # K beyond one workgroup's sixteen slices: the staged kernel splits K over workgroups, from 5 rows of x on (in fp16
    # arithmetic beyond K = 8192)
    assert kernel(1, 4096, 14336) == (1, 1) and kernel(4, 4096, 14336)[0] == 2 and kernel(5, 4096, 14336) == (5, 1)
    assert kernel(16, 4096, 14336) == (5, 1)
    assert kernel(1, 28672, 8192) == (1, 0) and kernel(4, 28672, 8192)[0] != 5 and kernel(5, 28672, 8192) == (5, 0)
    assert kernel(16, 4096, 16384 + 512)[0] == 4
    assert kernel(1, 128256, 4096, nested=1)[0] == 5 and kernel(5, 28672, 8192, nested=1) == (5, 0)  # nested absmax too
    assert lib.nf4hip_gemv_prefer_staged(0) == 0
    assert kernel(1, 128256, 4096)[0] == 1
    assert lib.nf4hip_gemv_prefer_staged(-1) == 0
    assert lib.nf4hip_gemv_plan(17, 4096, 4096, 64, 0, ctypes.byref(plan)) == L.E_SHAPE
    assert lib.nf4hip_gemv_plan(8, 4096, 4096 + 64, 64, 0, ctypes.byref(plan)) == L.E_SHAPE
    assert lib.nf4hip_gemv_plan(1, 4096, 4096, 48, 0, ctypes.byref(plan)) == L.E_BLOCKSIZE
    assert lib.nf4hip_gemv_plan(1, 4096, 4096, 64, 0, None) == L.E_NULL


def test_linear_argument_errors_and_plan(ta):
    """nf4hip_linear validates before its first HIP call; its plan and workspace queries need no GPU."""
    import ctypes

    L, lib = ta._lib, ta._lib.load()
    A = 4096
    assert lib.nf4hip_linear(None, L.BF16, 4, A, None, 8, 128, A, None, 0, None) == L.E_NULL
    assert lib.nf4hip_linear(A, L.F16, 4, A, None, 8, 128, A, None, 0, None) == L.E_DTYPE
    assert lib.nf4hip_linear(A, L.BF16, 0, A, None, 8, 128, A, None, 0, None) == L.E_SHAPE
    assert lib.nf4hip_linear(A, L.BF16, 4, A, None, 8, 96, A, None, 0, None) == L.E_SHAPE and "64" in _err(ta)
    assert lib.nf4hip_linear(A, L.BF16, 4, A, None, 8, 64, A, None, 0, None) == L.E_SHAPE  # one k step: not served
    assert lib.nf4hip_linear(A + 2, L.BF16, 4, A, None, 8, 128, A, None, 0, None) == L.E_ALIGN
    assert lib.nf4hip_linear(A, L.BF16, 4, A, A + 1, 8, 128, A, None, 0, None) == L.E_ALIGN
    # [4096, 14336] with 2048 rows of x: 128 tiles cut in two along K -> two partial tiles each and the counter region
    need = lib.nf4hip_linear_workspace_bytes(2048, 4096, 14336)
    assert need == 65536 * 4 + 128 * 2 * 256 * 256 * 4
    assert lib.nf4hip_linear(A, L.BF16, 2048, A, None, 4096, 14336, A, None, 0, None) == L.E_WORKSPACE
    assert lib.nf4hip_linear(A, L.BF16, 2048, A, None, 4096, 14336, A, A, need - 1, None) == L.E_WORKSPACE
    assert lib.nf4hip_linear_workspace_bytes(2048, 14336, 4096) == 0  # 448 tiles: taken whole
    assert lib.nf4hip_linear_workspace_bytes(2048, 4096, 1024) == 0  # too few k steps to cut
    assert lib.nf4hip_linear_workspace_bytes(4, 8, 96) == 0
    plan = (ctypes.c_int * 4)()
    assert lib.nf4hip_linear_plan(2048, 4096, 14336, ctypes.byref(plan)) == 0 and list(plan) == [256, 128, 2, 256]
    assert lib.nf4hip_linear_plan(2048, 14336, 4096, ctypes.byref(plan)) == 0 and list(plan) == [256, 448, 1, 448]
    assert lib.nf4hip_linear_plan(300, 520, 192, ctypes.byref(plan)) == 0 and list(plan) == [256, 6, 1, 6]
    assert lib.nf4hip_linear_plan(2048, 4096, 96, ctypes.byref(plan)) == L.E_SHAPE
    assert lib.nf4hip_linear_plan(2048, 4096, 128, None) == L.E_NULL


A = 4096  # any non-null, 16-byte aligned fake device address: validation never dereferences


def test_quantize_dequantize_argument_errors(ta):
    L, lib = ta._lib, ta._lib.load()
    assert lib.nf4hip_quantize(None, L.BF16, 128, 64, A, A, None) == L.E_NULL
    assert lib.nf4hip_quantize(A, 7, 128, 64, A, A, None) == L.E_DTYPE
    assert lib.nf4hip_quantize(A, L.BF16, 128, 48, A, A, None) == L.E_BLOCKSIZE
    assert "48" in _err(ta)
    assert lib.nf4hip_quantize(A, L.BF16, -1, 64, A, A, None) == L.E_SHAPE
    assert lib.nf4hip_quantize(A + 2, L.BF16, 128, 64, A, A, None) == L.E_ALIGN
    assert lib.nf4hip_quantize(None, L.BF16, 0, 64, None, None, None) == 0  # empty input is a no-op
    assert lib.nf4hip_dequantize(A, A, None, 128, 64, A, L.BF16, None) == L.E_NULL
    assert lib.nf4hip_dequantize(A, A, A, 128, 64, A, 3, None) == L.E_DTYPE
    assert lib.nf4hip_dequantize(A, A, A, 128, 100, A, L.F16, None) == L.E_BLOCKSIZE
    assert lib.nf4hip_dequantize(A, A, A, 128, 64, A + 8, L.F32, None) == L.E_ALIGN
    assert lib.nf4hip_dequantize(None, None, None, 0, 64, None, L.BF16, None) == 0
    assert lib.nf4hip_dequantize_dq(A, None, A, A, 0.0, 256, A, 128, 64, A, L.BF16, None) == L.E_NULL
    assert lib.nf4hip_dequantize_dq(A, A, A, A, 0.0, 100, A, 128, 64, A, L.BF16, None) == L.E_BLOCKSIZE
    assert lib.nf4hip_dq_compress(A, 10, 256, None, 0.0, A, A, None) == L.E_NULL
    assert lib.nf4hip_dq_compress(A, -1, 256, A, 0.0, A, A, None) == L.E_SHAPE
    assert lib.nf4hip_dq_reconstruct(A, A, A, 0.0, 10, 3, A, None) == L.E_BLOCKSIZE


def test_matmul_argument_errors(ta):
    L, lib = ta._lib, ta._lib.load()
    ws = 1 << 30

    def gemv(x=A, dt=L.BF16, M=1, packed=A, absmax=A, lut=A, bias=None, N=64, K=4096, bs=64, out=A, w=A, wb=ws):
        return lib.nf4hip_gemv(x, dt, M, packed, absmax, lut, bias, N, K, bs, out, w, wb, None)

    def gemm(x=A, dt=L.BF16, M=64, packed=A, absmax=A, lut=A, bias=None, N=64, K=4096, bs=64, out=A, w=None, wb=0):
        return lib.nf4hip_gemm(x, dt, M, packed, absmax, lut, bias, N, K, bs, out, w, wb, None)

    assert gemv(x=None) == L.E_NULL and gemv(absmax=None) == L.E_NULL and gemm(out=None) == L.E_NULL
    assert gemv(dt=L.F16) == L.E_DTYPE and gemm(dt=L.F32) == L.E_DTYPE  # only bf16 x is fused
    assert gemv(bs=96) == L.E_BLOCKSIZE
    assert gemv(M=0) == L.E_SHAPE and gemv(M=17) == L.E_SHAPE and gemv(N=-5) == L.E_SHAPE
    assert gemv(M=1, K=48) == L.E_SHAPE      # row-streaming kernel: K % 32
    assert gemv(M=8, K=1376) == L.E_SHAPE    # tile kernel: K % 512
    assert "512" in _err(ta)
    assert gemm(K=100) == L.E_SHAPE and gemm(K=192, bs=128) == L.E_SHAPE
    assert gemv(x=A + 4) == L.E_ALIGN and gemm(packed=A + 1) == L.E_ALIGN and gemv(bias=A + 1) == L.E_ALIGN
    assert gemv(lut=A + 2) == L.E_ALIGN
    # the small tables need their natural alignment only: these calls get past the alignment check (and stop at the next one)
    assert gemv(lut=A + 4, w=None) == L.E_WORKSPACE and gemv(bias=A + 2, w=None) == L.E_WORKSPACE
    assert lib.nf4hip_dq_compress(A + 4, 512, 256, A, 0.0, A, A, None) == L.E_ALIGN
    assert lib.nf4hip_dq_reconstruct(A, A + 8, A, 0.0, 512, 256, A, None) == L.E_ALIGN
    assert lib.nf4hip_dq_compress(A, 512, 256, A + 2, 0.0, A, A, None) == L.E_ALIGN
    assert gemv(w=None) == L.E_WORKSPACE and gemv(wb=16) == L.E_WORKSPACE
    assert "workspace" in _err(ta)
    # the entry point that brings its own scratch: same checks, and a shape whose partial sums exceed the
    # built-in array is refused before any HIP call
    assert lib.nf4hip_gemv_static(A, L.BF16, 1, A, A, None, None, 64, 4096, 64, A, None) == L.E_NULL
    assert lib.nf4hip_gemv_static(A, L.BF16, 17, A, A, A, None, 64, 4096, 64, A, None) == L.E_SHAPE
    assert lib.nf4hip_gemv_static(A, L.BF16, 16, A + 4, A, A, None, 64, 4096, 64, A, None) == L.E_ALIGN
    assert lib.nf4hip_gemv_workspace_bytes(16, 8192, 1 << 20) > L.STATIC_SCRATCH_BYTES
    assert lib.nf4hip_gemv_static(A, L.BF16, 16, A, A, A, None, 8192, 1 << 20, 64, A, None) == L.E_WORKSPACE
    assert "scratch" in _err(ta)
    assert lib.nf4hip_gemv_dq(A, L.BF16, 1, A, None, A, A, 0.0, 256, A, None, 64, 4096, 64, A, A, ws, None) == L.E_NULL
    assert lib.nf4hip_gemm_dq(A, L.BF16, 64, A, A, A, A, 0.0, 7, A, None, 64, 4096, 64, A, None, 0, None) == L.E_BLOCKSIZE
    # workspace sizing is pure arithmetic: split-K arrival counters (65536 x 4 bytes), then partial sums
    COUNTERS = 65536 * 4
    assert lib.nf4hip_gemv_workspace_bytes(16, 128256, 4096) == COUNTERS                  # big N: K is not split
    assert lib.nf4hip_gemv_workspace_bytes(1, 4096, 4096) == COUNTERS
    assert lib.nf4hip_gemv_workspace_bytes(4, 8192, 28672) == COUNTERS + 4 * 4 * 8192 * 4  # K split over 4 workgroups
    assert lib.nf4hip_gemv_workspace_bytes(16, 1024, 4096) == COUNTERS                       # small weight: quad kernel on two halves of x
    assert lib.nf4hip_gemv_workspace_bytes(16, 6144, 4096) > COUNTERS                        # tile kernel splits K
    assert lib.nf4hip_gemm_workspace_bytes(2048, 4096, 4096) == 0


def test_python_wrappers_refuse_cpu_tensors(ta):
    import torch

    w = torch.zeros(4, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        ta.quantize_nf4(w)
    with pytest.raises(ValueError):
        ta.quantize_nf4(w, blocksize=100)
    with pytest.raises(RuntimeError, match="GPU"):
        ta.matmul_nf4(torch.zeros(1, 64, dtype=torch.bfloat16), torch.zeros(128, 1, dtype=torch.uint8), None,
                      torch.zeros(4), ta.nf4_code(), 64, torch.bfloat16, (4, 64))


def test_check_raises_with_message(ta):
    lib = ta._lib.load()
    rc = lib.nf4hip_quantize(A, 9, 1, 64, A, A, None)
    with pytest.raises(ta._lib.NF4HipError, match="NF4HIP_E_DTYPE") as e:
        ta._lib.check(rc)
    assert e.value.code == ta._lib.E_DTYPE


def test_fused_route_rules(ta):
    import torch

    F = ta.functional
    bf = torch.bfloat16

    def route(M, N, K, dtype=bf, xdtype=bf, bs=64, bias=None):
        return F.fused_route(torch.empty(M, K, dtype=xdtype), bias, bs, dtype, (N, K))

    assert route(1, 4096, 4096) == "gemv" and route(4, 64, 1376) == "gemv" and route(16, 4096, 4096) == "gemv"
    assert route(5, 64, 1376) == "dequant+linear"        # tile kernel needs K % 512, gemm K % 64
    assert route(8, 64, 1344) == "gemm"                   # fused GEMM kernel below DENSE_ROUTE_MIN_M rows
    # 17..128 rows: one launch of the fused GEMM (64- or 128-row tile, K split over workgroups) wherever it is
    # modelled faster than the dense route's dequantize pass -- every projection shape of the Llama models
    assert route(17, 4096, 4096) == "gemm" and route(128, 4096, 4096) == "gemm"
    assert route(64, 1024, 4096) == "gemm" and route(65, 1024, 4096) == "dequant+gemm"
    # 17..32 rows of x on a weight of 40 M elements and more: two passes of the decode kernel (the LDS-staged one at these
    # shapes) beat the fused GEMM; three do not
    assert route(17, 14336, 4096) == "gemv-chunks" and route(32, 28672, 4096) == "gemv-chunks" and route(32, 128256, 4096) == "gemv-chunks"
    assert route(33, 14336, 4096) == "gemm" and route(48, 28672, 4096) == "gemm" and route(128, 14336, 4096) == "gemm"
    assert route(17, 6144, 4096) == "gemm" and route(32, 4096, 4096) == "gemm"  # below 40 M weights never
    assert route(128, 4096, 14336) == "gemm"
    assert route(17, 8192, 28672) == "gemm"               # exact at any K
    assert route(17, 28672, 4096 + 64) == "gemm"          # the tile kernel needs K % 512, the fused GEMM K % 64
    assert route(17, 128, 64) == "gemm"                   # tiny: one launch instead of two
    # more than 128 rows: the fused kernel of nf4_gemm_wide.hip (calls with fewer tiles than CUs cut their tiles
    # along k) up to 1024 rows on every Llama projection shape but the smallest, and at 2048 rows where the models
    # put it within 3 % of dequantize + library GEMM; the library GEMM's higher rate wins beyond
    # (measured crossovers, see functional._fused_gemm_wins)
    for N, K in [(4096, 4096), (6144, 4096), (14336, 4096), (4096, 14336), (28672, 4096), (128256, 4096), (8192, 8192),
                 (28672, 8192), (8192, 28672)]:
        for M in (129, 256, 512, 1024):
            assert route(M, N, K) == "gemm", (M, N, K)
        assert route(8192, N, K) == "dequant+gemm", (N, K)
    assert route(2048, 4096, 4096) == "gemm" and route(2048, 4096, 14336) == "gemm" and route(2048, 128256, 4096) == "gemm"
    assert route(2048, 28672, 4096) == "dequant+gemm" and route(2048, 28672, 8192) == "dequant+gemm"
    assert route(129, 1024, 4096) == "dequant+gemm" and route(512, 1024, 4096) == "gemm" and route(8192, 1024, 4096) == "dequant+gemm"
    # a few more than 16 rows on a short, very wide weight: the decode kernel once per 16 rows
    assert route(17, 2048, 20480) == "gemv-chunks" and route(32, 2048, 20480) == "gemv-chunks" and route(33, 2048, 20480) == "gemm"
    assert route(32, 1536, 28672) == "gemv-chunks" and route(33, 1536, 28672) == "dequant+gemm"
    assert route(17, 2048, 20480 + 64) == "dequant+gemm"  # the decode kernels need K % 512; 321 k steps do not split
    assert route(16, 8192, 28672) == "gemv"              # K > 8192: the tile kernel's exact-weights variant
    assert route(1, 8192, 28672) == "gemv"               # row-streaming kernel has an exact variant
    assert route(1, 64, 4096, dtype=torch.float32) == "dequant+linear"
    assert route(1, 64, 4096, xdtype=torch.float16, dtype=torch.float16) == "dequant+linear"
    assert route(1, 2, 2) == "dequant+linear"
    assert route(1, 64, 4096, bias=torch.zeros(64)) == "dequant+linear"  # fp32 bias with bf16 x
    _ = ctypes  # (imported for readers who want to poke at the library by hand)


def test_epilogue_argument_errors(ta):
    """nf4hip_gemv_epilogue validates its struct before any HIP call; what the kernels do not serve is E_SHAPE."""
    import ctypes

    L = ta._lib
    lib = L.load()
    A = 1 << 20  # fake, aligned device address: validation dereferences nothing
    ws = lib.nf4hip_gemv_workspace_bytes(1, 64, 4096)
    args = (A, L.BF16, 1, A, A, A, None, 64, 4096, 64, A, A, ws)
    err = lambda: lib.nf4hip_last_error().decode()
    call = lambda e, a=args: lib.nf4hip_gemv_epilogue(*a, ctypes.byref(e), None)
    assert lib.nf4hip_gemv_epilogue(*args, None, None) == L.E_NULL
    assert call(L.Epilogue(8)) == L.E_SHAPE and "flags" in err()
    assert call(L.Epilogue(L.EPI_RESID_NORM | L.EPI_ROWSCALE)) == L.E_SHAPE and "stands alone" in err()
    assert call(L.Epilogue(L.EPI_ROWSCALE)) == L.E_NULL and "in_sumsq" in err()
    assert call(L.Epilogue(L.EPI_ROWSCALE, 1e-5, A + 2, 8)) == L.E_ALIGN
    assert call(L.Epilogue(L.EPI_RESID_NORM, 0.0, None, 0, A, A, A, None, A)) == L.E_NULL and "xnext_out" in err()
    assert call(L.Epilogue(L.EPI_RESID_NORM, 0.0, None, 0, A, A, A + 1, A, A)) == L.E_ALIGN
    tiles = (A, L.BF16, 16, A, A, A, None, 16384, 4096, 64, A, A, 1 << 30)  # tile kernel: 1024 tiles of 16 weight rows
    assert call(L.Epilogue(L.EPI_RESID_NORM, 0.0, None, 0, A, A, A, A, A), tiles) == L.E_SHAPE and "not served" in err()
    odd = (A, L.BF16, 3, A, A, A, None, 63, 4096, 64, A, A, 1 << 30)
    assert call(L.Epilogue(L.EPI_SILU_PAIRS), odd) == L.E_SHAPE and "not served" in err()  # pairs need an even N
    long_k = (A, L.BF16, 1, A, A, A, None, 64, 20480, 64, A, A, 1 << 30)
    assert call(L.Epilogue(L.EPI_SILU_PAIRS), long_k) == L.E_SHAPE and "not served" in err()
    assert call(L.Epilogue(L.EPI_ROWSCALE, 1e-5, A, 513)) == L.E_SHAPE  # more partial sums than a workgroup has threads
    assert lib.nf4hip_gemv_norm_parts(16, 16384, 4096) == 0 and lib.nf4hip_gemv_norm_parts(1, 64, 20480) == 0
    assert lib.nf4hip_gemv_norm_parts(4, 8192, 28672) > 0
    assert lib.nf4hip_gemv_norm_parts(8, 8192, 8192) == 128  # staged kernel, K split two ways: 128 row ranges
    # the product alone goes to the staged kernel, one K range: its residual epilogue holds (M + 1) x rows per workgroup
    # values in LDS, at most 1024 -- 17 x 32 here, one partial sum per workgroup; 17 x 64 on twice the rows is too many
    assert lib.nf4hip_gemv_norm_parts(16, 8192, 4096) == 256
    assert lib.nf4hip_gemv_norm_parts(16, 16384, 4096) == 0 and lib.nf4hip_gemv_norm_parts(9, 16384, 4096) == 256
    assert lib.nf4hip_gemv_norm_parts(3, 64, 4096) > 0
    assert lib.nf4hip_gemv_norm_parts(8, 4096, 14336) == 64  # staged kernel, K split four ways: one partial sum per row range


def test_gemm_plan_is_the_launchers_and_agrees_with_the_workspace(ta):
    """nf4hip_gemm_plan is what the host-side time models read instead of restating the launchers' rules: over a sweep of
    shapes its answer must account for nf4hip_gemm_workspace_bytes exactly (counter region + one fp32 partial tile of
    `rows x 256` per piece wherever tiles are cut along K, nothing otherwise), and the Python helpers must pass it on."""
    import torch  # noqa: F401

    F, L = ta.functional, ta._lib
    lib = L.load()
    counter_region = 65536 * 4
    seen_cut = seen_whole = 0
    for M in (17, 64, 65, 128, 129, 256, 512, 1000, 2048, 4096, 8192):
        for N in (64, 1000, 1024, 4096, 6144, 14336, 28672, 128256):
            for K in (64, 1344, 4096, 8192, 14336, 28672):
                rows, tiles, pieces, wgs = F._gemm_plan(M, N, K)
                n_tiles = (N + 255) // 256
                assert rows in (64, 128, 256) and tiles == ((M + rows - 1) // rows) * n_tiles
                assert 1 <= pieces <= 8 and wgs <= max(256, tiles)
                need = lib.nf4hip_gemm_workspace_bytes(M, N, K)
                if pieces == 1:
                    assert need == 0 and wgs == tiles
                    seen_whole += 1
                else:
                    cut = tiles if M <= 128 else tiles % 256  # beyond 128 rows of x only a call without a full round is cut
                    assert wgs == (tiles - cut) + cut * pieces and (K // 64) >= pieces
                    assert need == counter_region + cut * pieces * rows * 256 * 4
                    seen_cut += 1
                assert F._gemm_splits(M, N, K) == (pieces if M <= 128 else 1)
                if M > 128:
                    assert F._wide_schedule(M, N, K) == (rows, tiles, pieces)
    assert seen_cut > 50 and seen_whole > 50
    plan = (ctypes.c_int * 4)()
    assert lib.nf4hip_gemm_plan(0, 64, 64, ctypes.byref(plan)) == L.E_SHAPE
    assert lib.nf4hip_gemm_plan(64, 64, 100, ctypes.byref(plan)) == L.E_SHAPE
    assert lib.nf4hip_gemm_plan(64, 64, 64, None) == L.E_NULL
