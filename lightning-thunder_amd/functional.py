"""Tensor-level NF4 ops on PyTorch-ROCm tensors, backed by ``libnf4hip.so``.

These are the functions the executor registers as operators.  They mirror what the reference
gets from bitsandbytes at thunder/transforms/quantization.py:35-39,63:

* :func:`quantize_nf4`      -- ``bitsandbytes.functional.quantize_4bit(w, quant_type="nf4")``
* :func:`dequantize_nf4`    -- ``bitsandbytes.functional.dequantize_4bit``
* :func:`matmul_nf4`        -- ``bitsandbytes.matmul_4bit(x, qweight.t(), bias, quant_state)``

All tensors must live on the GPU (``device.type == "cuda"`` on ROCm builds of torch); kernels are
queued on ``torch.cuda.current_stream()`` and nothing synchronises.
"""

from __future__ import annotations

import ctypes
import math
import os
from dataclasses import dataclass

import torch

from . import _lib
from ._workspace import WorkspacePool

SUPPORTED_BLOCKSIZES = (64, 128, 256, 512, 1024, 2048, 4096)

# Beyond this K the decode kernels round every weight exactly like the reference's dequantisation
# (the cheaper "scale the partial sum" arithmetic drifts from it like sqrt(K)); the 5..16-row tile
# kernel has no such variant, so those calls go to the prefill kernel, which is exact by construction.
EXACT_K = 8192
# K beyond which a call that no model above claims goes to dequantize + dense GEMM even for a few rows of x
LONG_K = 16384
# From this many rows of x on, HIP dequantize followed by the dense library GEMM is a candidate
# (the fused GEMM kernels re-expand the weight tile once per 256 rows of x and reach 1.0-1.15
# PFLOP/s, the library GEMM 1.1-1.5 PFLOP/s and the dequantize kernel runs at HBM speed); see
# _fused_gemm_wins for which of the two serves a shape.  Raise it to force the fused, allocation-free
# kernels everywhere.
DENSE_ROUTE_MIN_M = 17

_DTYPE_CODE = {torch.bfloat16: _lib.BF16, torch.float16: _lib.F16, torch.float32: _lib.F32}

# fp32 NF4 code values (QLoRA), index = 4-bit code; the table bitsandbytes stores as QuantState.code
NF4_CODE = (
    -1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453,
    -0.28444138169288635, -0.18477343022823334, -0.09105003625154495, 0.0,
    0.07958029955625534, 0.16093020141124725, 0.24611230194568634, 0.33791524171829224,
    0.44070982933044434, 0.5626170039176941, 0.7229568362236023, 1.0,
)  # fmt: skip


_code_masters: dict[tuple[str, torch.dtype], torch.Tensor] = {}


def nf4_code(device=None, dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """The 16-entry code book as a new tensor (``quant_map`` / ``QuantState.code``).  One master copy
    per device is kept and cloned, so that only the first call on a device pays a host-to-device
    copy (which synchronises the stream)."""
    dev = torch.device(device) if device is not None else torch.device("cpu")
    if dev.type == "cuda" and dev.index is None:
        dev = torch.device("cuda", torch.cuda.current_device())
    key = (str(dev), dtype)
    master = _code_masters.get(key)
    if master is None:
        master = torch.tensor(NF4_CODE, dtype=torch.float32, device=dev).to(dtype)
        _code_masters[key] = master
    return master.clone()


def dynamic_map(device=None) -> torch.Tensor:
    """The 256-entry signed "dynamic" 8-bit code bitsandbytes uses for nested absmax quantisation
    (``create_dynamic_map(signed=True, max_exponent_bits=7, total_bits=8)``)."""
    data: list[float] = []
    for i in range(7):
        boundaries = torch.linspace(0.1, 1, 2**i + 1)
        means = (boundaries[:-1] + boundaries[1:]) / 2.0
        scale = 10 ** (-6 + i)
        data += (scale * means).tolist()
        data += (-scale * means).tolist()
    data += [0.0, 1.0]
    assert len(data) == 256
    data.sort()
    return torch.tensor(data, dtype=torch.float32, device=device)


@dataclass
class NestedAbsmax:
    """absmax in nested ("double quantised") form: ``map256[q] * absmax2[i // blocksize] + offset``."""

    q: torch.Tensor  # uint8 [nblocks]
    absmax2: torch.Tensor  # fp32 [ceil(nblocks / blocksize)]
    map256: torch.Tensor  # fp32 [256]
    offset: float
    blocksize: int = 256


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """hipStream_t of the current stream of the current device (the raw query where this torch has
    it: it skips building a Stream object, a third of the host time of a small call)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


class _on_device:
    """``torch.cuda.device(dev)`` that does nothing when ``dev`` is already current."""

    def __init__(self, device: torch.device):
        idx = device.index
        self._ctx = None if idx is None or idx == torch.cuda.current_device() else torch.cuda.device(idx)

    def __enter__(self):
        if self._ctx is not None:
            self._ctx.__enter__()

    def __exit__(self, *exc):
        if self._ctx is not None:
            return self._ctx.__exit__(*exc)


def _require_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and t.device.type != "cuda":
            raise RuntimeError(f"NF4 HIP ops need GPU tensors, got a tensor on {t.device}")


def _aligned(t: torch.Tensor) -> torch.Tensor:
    """Contiguous and 16-byte aligned view or copy of ``t``."""
    t = t.contiguous()
    if t.data_ptr() % 16:
        t = t.clone(memory_format=torch.contiguous_format)
    return t


def _check_blocksize(blocksize: int) -> None:
    if blocksize not in SUPPORTED_BLOCKSIZES:
        raise ValueError(f"blocksize must be one of {SUPPORTED_BLOCKSIZES}, got {blocksize}")


# ------------------------------------------------------------------------------------------------
# quantize / dequantize
# ------------------------------------------------------------------------------------------------


def quantize_nf4(w: torch.Tensor, blocksize: int = 64):
    """Blockwise NF4 quantisation of ``w`` (bf16/f16/f32, any shape, flattened row-major).

    Returns ``(qweight uint8 [(n+1)//2, 1], absmax fp32 [ceil(n/blocksize)], code fp32 [16])``,
    the tensors the reference stores as ``<w>``, ``<w>.absmax`` and ``<w>.code``
    (thunder/transforms/quantization.py:87-89).
    """
    _check_blocksize(blocksize)
    _require_gpu(w)
    if w.dtype not in _DTYPE_CODE:
        raise TypeError(f"cannot quantize dtype {w.dtype}")
    lib = _lib.load()
    w = _aligned(w.detach())
    n = w.numel()
    with _on_device(w.device):
        packed = torch.empty(((n + 1) // 2, 1), dtype=torch.uint8, device=w.device)
        absmax = torch.empty(((n + blocksize - 1) // blocksize,), dtype=torch.float32, device=w.device)
        _lib.check(lib.nf4hip_quantize(w.data_ptr(), _DTYPE_CODE[w.dtype], n, blocksize, packed.data_ptr(), absmax.data_ptr(), _stream()))
    return packed, absmax, nf4_code(w.device)


def dequantize_nf4(qweight, absmax, quant_map, blocksize, dtype, shape) -> torch.Tensor:
    """``cast(quant_map[code] * absmax[block])`` reshaped to ``shape``; ``absmax`` is an fp32
    tensor or a :class:`NestedAbsmax`."""
    _check_blocksize(blocksize)
    if dtype not in _DTYPE_CODE:
        raise TypeError(f"cannot dequantize to dtype {dtype}")
    shape = tuple(int(s) for s in shape)
    n = math.prod(shape)
    lib = _lib.load()
    _require_gpu(qweight, quant_map)
    qweight = _aligned(qweight)
    if qweight.numel() < (n + 1) // 2:
        raise ValueError(f"qweight holds {qweight.numel()} bytes, shape {shape} needs {(n + 1) // 2}")
    quant_map = _aligned(quant_map.to(torch.float32))
    nblocks = (n + blocksize - 1) // blocksize
    with _on_device(qweight.device):
        out = torch.empty(shape, dtype=dtype, device=qweight.device)
        if isinstance(absmax, NestedAbsmax):
            nq = _nested_args(absmax, nblocks)
            _lib.check(
                lib.nf4hip_dequantize_dq(qweight.data_ptr(), nq[0].data_ptr(), nq[1].data_ptr(), nq[2].data_ptr(), nq[3], nq[4],
                                         quant_map.data_ptr(), n, blocksize, out.data_ptr(), _DTYPE_CODE[dtype], _stream())
            )  # fmt: skip
        else:
            _require_gpu(absmax)
            absmax = _aligned(absmax.to(torch.float32))
            if absmax.numel() < nblocks:
                raise ValueError(f"absmax holds {absmax.numel()} entries, need {nblocks}")
            _lib.check(
                lib.nf4hip_dequantize(qweight.data_ptr(), absmax.data_ptr(), quant_map.data_ptr(), n, blocksize,
                                      out.data_ptr(), _DTYPE_CODE[dtype], _stream())
            )  # fmt: skip
    return out


# ------------------------------------------------------------------------------------------------
# nested (double) quantisation of absmax
# ------------------------------------------------------------------------------------------------


def _nested_args(nq: NestedAbsmax, nblocks: int):
    _require_gpu(nq.q, nq.absmax2, nq.map256)
    if nq.q.numel() < nblocks:
        raise ValueError(f"nested absmax holds {nq.q.numel()} codes, need {nblocks}")
    return (_aligned(nq.q), _aligned(nq.absmax2.to(torch.float32)), _aligned(nq.map256.to(torch.float32)), float(nq.offset), int(nq.blocksize))


def compress_absmax(absmax: torch.Tensor, nested_blocksize: int = 256, map256: torch.Tensor | None = None) -> NestedAbsmax:
    """bitsandbytes' ``compress_statistics=True``: subtract the mean, then 8-bit blockwise quantise.
    The mean is taken in float64 and rounded to fp32 once, so it does not depend on reduction order."""
    _check_blocksize(nested_blocksize)
    _require_gpu(absmax)
    lib = _lib.load()
    absmax = _aligned(absmax.to(torch.float32))
    nb = absmax.numel()
    offset = float(absmax.double().mean().to(torch.float32)) if nb else 0.0
    with _on_device(absmax.device):
        if map256 is None:
            map256 = dynamic_map(absmax.device)
        map256 = _aligned(map256.to(torch.float32))
        q = torch.empty(nb, dtype=torch.uint8, device=absmax.device)
        absmax2 = torch.empty(((nb + nested_blocksize - 1) // nested_blocksize,), dtype=torch.float32, device=absmax.device)
        _lib.check(lib.nf4hip_dq_compress(absmax.data_ptr(), nb, nested_blocksize, map256.data_ptr(), offset, q.data_ptr(), absmax2.data_ptr(), _stream()))
    return NestedAbsmax(q, absmax2, map256, offset, nested_blocksize)


def reconstruct_absmax(nq: NestedAbsmax) -> torch.Tensor:
    lib = _lib.load()
    nb = nq.q.numel()
    q, a2, m, off, bs = _nested_args(nq, nb)
    with _on_device(q.device):
        out = torch.empty(nb, dtype=torch.float32, device=q.device)
        _lib.check(lib.nf4hip_dq_reconstruct(q.data_ptr(), a2.data_ptr(), m.data_ptr(), off, nb, bs, out.data_ptr(), _stream()))
    return out


# Nested state as plain tensors (what a state dict can hold): absmax_q uint8 [nblocks], nested_absmax fp32
# [ceil(nblocks / nested_blocksize)], nested_quant_map fp32 [256], nested_offset fp32 [1].  The C ABI takes the
# offset by value; reading it back from the device costs a synchronisation, so it is read once per tensor and
# again only after the tensor was written to (torch bumps ``_version`` on every in-place write) or rebound to other
# storage.  The value is kept ON the tensor object: it dies with it, so a new tensor that happens to get a dead one's
# id and address (CPython reuses ids, the caching allocator reuses addresses) can never see a stale value.
_OFFSET_ATTR = "_nf4hip_offset_value"


def _remember_offset(nested_offset: torch.Tensor, value: float) -> None:
    setattr(nested_offset, _OFFSET_ATTR, (nested_offset.data_ptr(), nested_offset._version, value))


def _offset_value(nested_offset) -> float:
    if not isinstance(nested_offset, torch.Tensor):
        return float(nested_offset)
    hit = getattr(nested_offset, _OFFSET_ATTR, None)
    if hit is not None and hit[0] == nested_offset.data_ptr() and hit[1] == nested_offset._version:
        return hit[2]
    value = float(nested_offset.reshape(-1)[0].item())
    _remember_offset(nested_offset, value)
    return value


def nested_state(absmax_q, nested_absmax, nested_quant_map, nested_offset, nested_blocksize: int = 256) -> NestedAbsmax:
    return NestedAbsmax(absmax_q, nested_absmax, nested_quant_map, _offset_value(nested_offset), int(nested_blocksize))


def quantize_nf4_dq(w: torch.Tensor, blocksize: int = 64, nested_blocksize: int = 256):
    """NF4 quantisation with double-quantised statistics (bitsandbytes' ``compress_statistics=True``).  Returns
    ``(qweight, absmax_q, nested_absmax, nested_quant_map, nested_offset, code)``; ``nested_offset`` is a one-element
    fp32 tensor so that it can live in a state dict."""
    qw, absmax, code = quantize_nf4(w, blocksize)
    nq = compress_absmax(absmax, nested_blocksize)
    offset = torch.tensor([nq.offset], dtype=torch.float32, device=qw.device)
    _remember_offset(offset, float(nq.offset))
    return qw, nq.q, nq.absmax2, nq.map256, offset, code


def dequantize_nf4_dq(qweight, absmax_q, nested_absmax, nested_quant_map, nested_offset, quant_map, blocksize, nested_blocksize,
                      dtype, shape) -> torch.Tensor:
    nq = nested_state(absmax_q, nested_absmax, nested_quant_map, nested_offset, nested_blocksize)
    return dequantize_nf4(qweight, nq, quant_map, blocksize, dtype, shape)


def matmul_nf4_dq(x, qweight, bias, absmax_q, nested_absmax, nested_quant_map, nested_offset, quant_map, blocksize,
                  nested_blocksize, dtype, shape) -> torch.Tensor:
    """:func:`matmul_nf4` on double-quantised statistics given as tensors: ``absmax`` is replaced by ``(absmax_q,
    nested_absmax, nested_quant_map, nested_offset)`` and ``nested_blocksize`` follows ``blocksize``."""
    nq = nested_state(absmax_q, nested_absmax, nested_quant_map, nested_offset, nested_blocksize)
    return matmul_nf4(x, qweight, bias, nq, quant_map, blocksize, dtype, shape)


# ------------------------------------------------------------------------------------------------
# matmul
# ------------------------------------------------------------------------------------------------

# 40 MiB covers every Llama-3-8B / 70B projection shape on both fused routes (the largest need is the fused
# GEMM's 33 MB of partial tiles at [16384, 8192], M = 128), so a stream's buffer is normally allocated once.
_workspace_pool = WorkspacePool(65 << 20, "NF4 matmul")  # 256 partial tiles of 256 x 256 floats + the counter region


def _gemv_workspace(device: torch.device, nbytes: int, stream: int | None = None) -> torch.Tensor:
    """Zero-initialised scratch of the split-K kernels for (device, stream); the kernels leave their
    counters zeroed, so it is reused without clearing.  Raises instead of allocating under capture."""
    return _workspace_pool.get(device, nbytes, stream)


def reserve_workspace(device=None, nbytes: int | None = None) -> int:
    """Give the current stream of ``device`` its matmul workspace now (for example before capturing a
    graph on a stream that has not run an NF4 matmul yet).  Returns the buffer's size in bytes."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    with _on_device(dev):
        return _workspace_pool.reserve(dev, nbytes)


def _gemm_plan(M: int, N: int, K: int) -> tuple[int, int, int, int]:
    """``(rows of x per tile, tiles, pieces per tile along K, workgroups)`` of the fused GEMM for this shape: the
    library's own answer (``nf4hip_gemm_plan``), so that the time models below never restate a launcher's rules."""
    plan = (ctypes.c_int * 4)()
    _lib.check(_lib.load().nf4hip_gemm_plan(M, N, K, ctypes.byref(plan)))
    return plan[0], plan[1], plan[2], plan[3]


def _gemm_splits(M: int, N: int, K: int) -> int:
    """K splits of the fused GEMM kernel for up to 128 rows of x (1 beyond)."""
    return _gemm_plan(M, N, K)[2] if M <= 128 else 1


def _fused_gemm_us(M: int, N: int, K: int) -> float:
    """Model of the fused GEMM kernel's time for up to 128 rows of x (one tile of x rows): tiles of
    256 weight rows x K splits run in rounds of 256 workgroups (one per CU), K / 64 / splits steps
    each; a step takes 0.6 us (64-row tile, M <= 64) or 0.8 us (128-row tile) on a sparsely filled chip
    and 0.35 / 0.5 us more on a full one; merging the splits adds 9 / 16 us, a launch 3 (measured,
    M = 64 / 128: [4096, 4096] 19 / 30, [6144, 4096] 20 / 30, [4096, 14336] 31 / 45, [14336, 4096] 26 / 35,
    [16384, 8192] 40 / 56, [28672, 4096] 37 / 52, lm_head [128256, 4096] 121 / 167 us)."""
    splits = _gemm_splits(M, N, K)
    wgs = (N + 255) // 256 * splits
    rounds = (wgs + 255) // 256
    fill = min(1.0, wgs / rounds / 256.0)
    step = 0.6 + 0.35 * fill if M <= 64 else 0.8 + 0.5 * fill
    merge = 0.0 if splits == 1 else 9.0 if M <= 64 else 16.0
    return 3.0 + rounds * (K // 64 // splits) * step + merge


def _dense_route_us(N: int, K: int) -> float:
    """Model of the dense route before its GEMM: the dequantize kernel writes 2 bytes per weight at HBM
    speed, 20 + 0.62 W us for W million weights (measured with the GEMM of 64 rows of x: [14336, 4096]
    56, [28672, 4096] 108, [16384, 8192] 115, lm_head [128256, 4096] 428 us)."""
    return 20.0 + 0.62 * N * K / 1e6


def _wide_schedule(M: int, N: int, K: int) -> tuple[int, int, int]:
    """(rows of x per tile, tiles, pieces per tile) of the fused GEMM kernel for more than 128 rows of x: the 256-row
    tile from 160 tiles on or when tiles x k steps >= 28672, else the 128-row tile; a call with fewer tiles than the 256
    CUs cuts every tile into up to 8 equal pieces along k that meet in the workspace."""
    bm, tiles, pieces, _ = _gemm_plan(M, N, K)
    return bm, tiles, pieces


def _wide_gemm_us(M: int, N: int, K: int) -> float:
    """Model of the fused GEMM kernel for more than 128 rows of x (csrc/nf4_gemm_wide.hip): workgroups (one per tile
    or piece of a tile) run in rounds of 256, K / 64 / pieces steps each; a step of the 256-row tile takes 1.85 us
    on a full chip, of the 128-row tile 1.0 us, up to 40 % less on a sparsely filled one; 12 us of launch, prologue
    and epilogue; pieces that meet in the workspace add 6 us (128-row tile) or 12 us.  Measured / modelled, us:
    [4096, 4096] M = 256 / 512 / 1024 / 2048: 30 / 36 / 53 / 75 vs 29 / 37 / 53 / 76; [1024, 4096] M = 256 / 2048: 25 / 34
    vs 27 / 37; [4096, 14336] M = 256 / 512 / 2048: 52 / 77 / 229 vs 49 / 77 / 233; [8192, 28672] M = 512: 230 vs 233;
    [14336, 4096] M = 512 / 1024 / 2048: 69 / 113 / 220 vs 68 / 124 / 237; lm_head [128256, 4096] M = 2048: 1940 vs 1890."""
    bm, tiles, pieces = _wide_schedule(M, N, K)
    wgs = tiles * pieces
    rounds = (wgs + 255) // 256
    fill = wgs / (rounds * 256.0)
    step = (1.85 if bm == 256 else 1.0) * (0.6 + 0.4 * fill)
    merge = 0.0 if pieces == 1 else 6.0 if bm == 128 else 12.0
    return 12.0 + rounds * (K // 64 // pieces) * step + merge


def _dense_gemm_us(M: int, N: int, K: int) -> float:
    """Model of the dense route for more than 128 rows of x, kernel time: the dequantize pass (10 us with the gap to the
    GEMM + 0.45 us per million weights) plus the library GEMM, 3 us + flops / rate with 1 / rate = 1 / cap(M) + 85 / t in s per PFLOP: cap
    is the rate the library reaches for M rows of x on a full, power-limited chip (1.0 PFLOP/s at 256 rows, 1.3
    at 512, 1.4 at 1024, 1.5 at 2048, 1.6 at 4096, 1.68 beyond, times K / (K + 512) for the start and end of the
    k loop) and t the number of 128 x 128 output tiles (few
    tiles leave CUs idle).  Measured (kernel trace) / modelled, us: [4096, 4096] M = 512 / 2048 / 8192: 42 / 74 / 217 vs
    45 / 74 / 214; [1024, 4096] M = 512 / 8192: 25 / 72 vs 30 / 68; [14336, 4096] M = 512 / 2048 / 8192: 89 / 236 / 676 vs 99 /
    227 / 684; [4096, 14336] M = 512 / 2048: 110 / 250 vs 136 / 232; lm_head M = 512 / 2048 / 8192: 788 / 1850 / 6191 vs 735 /
    1868 / 6005."""
    cap = 1.0 if M <= 256 else 1.3 if M <= 512 else 1.4 if M <= 1024 else 1.5 if M <= 2048 else 1.6 if M <= 4096 else 1.68
    cap *= K / (K + 512.0)
    t = ((M + 127) // 128) * ((N + 127) // 128)
    per_pflop = 1.0 / cap + 85.0 / t
    return 10.0 + 0.45 * N * K / 1e6 + 3.0 + 2.0 * M * N * K * per_pflop / 1e9


def _fused_gemm_wins(M: int, N: int, K: int, nested: bool = False) -> bool:
    """Is the fused GEMM kernel faster than dequantize + dense GEMM?  Both sides are modelled from
    measurements on MI355X.  Up to 128 rows of x (one tile of x rows, K split over workgroups) the fused kernel's
    time hardly depends on N while the chip is not full, the dense route's grows with the weight (M = 64, us:
    [4096, 4096] 19 vs 34, [14336, 4096] 26 vs 55, [4096, 14336] 31 vs 64, [28672, 4096] 37 vs 107).  Beyond that the fused kernel
    runs at 1.0-1.15 PFLOP/s, the library GEMM at up to 1.5, but the dense route first writes the bf16 weight: the
    two cross near 1024 rows of x wherever the fused kernel has a workgroup for most CUs (fused vs dense, us, M =
    512 / 1024 / 2048: [14336, 4096] 71 / 117 / 232 vs 84 / 118 / 198; [28672, 4096] 127 / 239 / 473 vs 155 / 238 / 405; [28672, 8192] 226 /
    442 / 881 vs 291 / 466 / 789; lm_head [128256, 4096] 497 / 978 / 1938 vs 741 / 1099 / 1831; short weights leave the chip
    empty: [4096, 14336] 164 / 174 / 255 vs 107 / 142 / 216, [4096, 4096] 54 / 58 / 79 vs 42 / 52 / 75).  A tie goes to the fused kernel,
    which needs no transient bf16 weight."""
    if M <= 128:
        return _fused_gemm_us(M, N, K) < _dense_route_us(N, K)
    # nested absmax: the fp32 absmax is written out ahead of the fused kernel (_matmul_nf4_on), 2-7 % on top; the
    # dequantize pass of the dense route resolves the codes itself at no measurable cost
    return _wide_gemm_us(M, N, K) * (1.05 if nested else 1.0) <= 1.03 * _dense_gemm_us(M, N, K)


def _gemv_pass_us(N: int, K: int, nested: bool = False) -> float:
    """Model of one 16-row pass of the decode kernels over a weight of W million elements, from measurements on MI355X
    (us): the LDS-staged kernel 7.6 + 0.09 W while one workgroup covers K ([14336, 4096] 12.9, [28672, 4096] 17.6,
    [32000, 4096] 18.5, lm_head [128256, 4096] 54.7) and 9.5 + 0.108 W with K split over workgroups ([4096, 14336] 16.8,
    [10240, 8192] 17.0, [28672, 8192] 33.8, [57344, 8192] 60.3); the other decode kernels 12 + 0.105 W.  Which kernel it is, the
    library says (nf4hip_gemv_plan, no GPU needed)."""
    w = N * K / 1e6
    plan = (ctypes.c_int * 4)()
    if _lib.load().nf4hip_gemv_plan(16, N, K, 64, 1 if nested else 0, ctypes.byref(plan)) == 0 and plan[0] == 5:
        return 7.6 + 0.09 * w if K <= 4096 else 9.5 + 0.108 * w
    return 12.0 + 0.105 * w


def _chunked_gemv_wins(M: int, N: int, K: int, nested: bool = False) -> bool:
    """For a few more than 16 rows of x: are ceil(M / 16) passes of the decode kernel over the NF4
    weight cheaper than the alternatives?  All sides modelled from measurements on MI355X
    (microseconds, W = weights in millions): a 16-row pass takes _gemv_pass_us; the dense route
    20 + 0.62 W before its GEMM, and the passes must beat that by 20 %; the fused GEMM kernel, where
    it applies, _fused_gemm_us.  Measured, passes vs fused GEMM, M = 32 / 48: [28672, 4096] 34.8 / 51.6 vs 43.6 / 40.2;
    lm_head [128256, 4096] 115.7 / 166.5 vs 124.5 / 126.9; [4096, 14336] 32.6 / 47.4 vs 34.2 / 34.3; [14336, 4096] 24.6 / 36.6 vs
    26.5 / 26.8; [28672, 8192] 66.4 / 98.1 vs 68.1 / 67.6; [6144, 4096] 18.6 / 27.3 vs 19.4 / 19.8: two passes win, three do not;
    below 40 M weights never."""
    n_weights = N * K
    if M <= 16 or n_weights < 40_000_000:
        return False
    passes = (M + 15) // 16
    t = passes * _gemv_pass_us(N, K, nested)
    if _fused_gemm_wins(M, N, K) and t >= _fused_gemm_us(M, N, K):
        return False
    return t < 0.8 * _dense_route_us(N, K)


# Many rows of x: the fused GEMM and dequantize + dense GEMM are within a few per cent of each other over a wide range
# of shapes, and which one leads moves with the board (clocks under a power limit, the library's GEMM heuristics).  The
# time models above are the answer where nothing can be measured (on the CPU, under stream capture); otherwise the
# first call of a shape on a device times both routes once -- a few launches each -- and every later call takes the
# faster one.  NF4HIP_CALIBRATE=0 switches the measurement off.
CALIBRATE_MIN_M = 129
_route_measured: dict[tuple, str] = {}


def _route_key(device: torch.device, M: int, N: int, K: int, blocksize: int, nested: bool, has_bias: bool) -> tuple:
    index = device.index if device.index is not None else (torch.cuda.current_device() if device.type == "cuda" else -1)
    return (device.type, index, M, N, K, blocksize, nested, has_bias)


def _calibration_enabled() -> bool:
    return os.environ.get("NF4HIP_CALIBRATE", "1") != "0"


def _library_gemm_allowed() -> bool:
    """Is dequantize + the vendor library's GEMM ("dequant+libgemm") one of the routes that are timed against each
    other?  Yes unless NF4HIP_LIBRARY_GEMM=0, which keeps every fused-eligible call on this package's own kernels.  It
    is only ever chosen by measurement, and only when it beats both hand-written routes by more than 3 %."""
    return os.environ.get("NF4HIP_LIBRARY_GEMM", "1") != "0"


def _measure_route(key: tuple, candidates: dict, launches: int = 3) -> str:
    """Time every candidate (a callable per route name) on the current stream: one untimed call, then ``launches``
    calls between two events; remember and return the fastest.  The vendor library's GEMM ("dequant+libgemm") has to
    beat the best hand-written route by more than 3 %; a candidate within 2 % of the best that needs no transient
    bf16 weight ("gemm") is preferred."""
    times = {}
    for name, fn in candidates.items():
        fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(launches):
            fn()
        e1.record()
        e1.synchronize()
        times[name] = e0.elapsed_time(e1)
    best = min(times, key=times.get)
    own = {name: t for name, t in times.items() if name != "dequant+libgemm"}
    if best == "dequant+libgemm" and own and min(own.values()) <= 1.03 * times[best]:
        best = min(own, key=own.get)
    if "gemm" in times and times["gemm"] <= 1.02 * times[best]:
        best = "gemm"
    _route_measured[key] = best
    return best


def fused_route(x: torch.Tensor, bias, blocksize: int, dtype: torch.dtype, shape, nested: bool = False) -> str:
    """Which kernel serves this call: ``"gemv"``, ``"gemv-chunks"`` (the decode kernel once per 16
    rows of x), ``"gemm"`` (fused), ``"dequant+gemm"`` (HIP dequantize, then the hand-written dense MFMA kernel
    ``nf4hip_linear``, because that is the faster of the two for many rows of x), ``"dequant+libgemm"`` (HIP
    dequantize, then the vendor library's GEMM; only when NF4HIP_LIBRARY_GEMM=1 and measured faster) or
    ``"dequant+linear"`` (dequantize + ``torch.nn.functional.linear``, for dtypes and shapes no kernel here takes).

    Mirrors bitsandbytes.matmul_4bit: the fused single-row kernel when the shape allows, else
    dequantize followed by a dense matmul.
    """
    N, K = shape
    M = x.numel() // K if K else 0
    fused = (
        x.dtype == torch.bfloat16
        and dtype == torch.bfloat16
        and (bias is None or bias.dtype == torch.bfloat16)
        and blocksize in SUPPORTED_BLOCKSIZES
        and M > 0
        and N > 0
        and (N * K) % 2 == 0
    )
    if not fused:
        return "dequant+linear"
    if M <= 4 and K % 32 == 0:
        return "gemv"  # row-streaming kernel: blocks may straddle rows
    if K % 64 or K % blocksize:
        return "dequant+linear"
    if M <= 16 and K % 512 == 0:
        return "gemv"  # MFMA tile kernel (its exact-weights variant beyond EXACT_K)
    if K % 512 == 0 and _chunked_gemv_wins(M, N, K, nested):
        return "gemv-chunks"  # a few 16-row passes over the 4-bit weights beat writing them out as bf16
    measured = _route_measured.get(_route_key(x.device, M, N, K, blocksize, nested, bias is not None))
    if measured is not None:
        return measured  # both routes were timed on this device for this shape (_measure_route)
    if _fused_gemm_wins(M, N, K, nested):
        return "gemm"  # expanding the weight tiles in registers beats writing the bf16 weight out
    # the fused GEMM kernel streams K sequentially per tile: beyond LONG_K even a few rows of x are
    # served faster by dequantize + dense GEMM
    return "dequant+gemm" if M >= DENSE_ROUTE_MIN_M or K > LONG_K else "gemm"


def matmul_nf4(x, qweight, bias, absmax, quant_map, blocksize, dtype, shape) -> torch.Tensor:
    """``x @ dequantize(qweight).T + bias`` with the signature of the reference operator
    ``bnb_matmul_nf4`` (thunder/transforms/quantization.py:34).  ``absmax`` may be a
    :class:`NestedAbsmax`."""
    shape = tuple(int(s) for s in shape)
    assert len(shape) == 2
    N, K = shape
    assert x.shape[-1] == K, f"{x.shape=}, rhs {shape=}"
    _require_gpu(x, qweight, quant_map, bias)
    nested = isinstance(absmax, NestedAbsmax)
    route = fused_route(x, bias, blocksize, dtype, shape, nested)
    M = x.numel() // K
    if (route in ("gemm", "dequant+gemm") and M >= CALIBRATE_MIN_M and _calibration_enabled()
            and not torch.cuda.is_current_stream_capturing()):
        key = _route_key(x.device, M, N, K, blocksize, nested, bias is not None)
        if key not in _route_measured:
            with _on_device(x.device):
                names = ["gemm", "dequant+gemm"] + (["dequant+libgemm"] if _library_gemm_allowed() else [])
                route = _measure_route(key, {
                    name: (lambda name=name: _matmul_nf4_on(x, qweight, bias, absmax, quant_map, blocksize, dtype, shape, name))
                    for name in names
                })
    return _matmul_nf4_on(x, qweight, bias, absmax, quant_map, blocksize, dtype, shape, route)


# nested absmax, fused GEMM: beyond this many rows of x the fp32 absmax is written out first (measured, us, nested kernel /
# reconstruct + fp32 kernel / fp32 kernel alone: [8192, 8192] M = 256 64 / 58 / 53, M = 512 107 / 91 / 85, M = 2048 255 / 242 / 235;
# [28672, 8192] M = 512 242 / 226 / 213, M = 2048 930 / 854 / 837; [8192, 28672] M = 1024 481 / 439 / 425; [1024, 8192] M = 512 38 / 37 / 34)
NESTED_RECONSTRUCT_MIN_M = 128


def _matmul_nf4_on(x, qweight, bias, absmax, quant_map, blocksize, dtype, shape, route: str) -> torch.Tensor:
    """:func:`matmul_nf4` on a given route (one of ``fused_route``'s answers)."""
    N, K = shape
    if route in ("dequant+linear", "dequant+gemm", "dequant+libgemm"):
        w = dequantize_nf4(qweight, absmax, quant_map, blocksize, dtype, shape).to(x.dtype)
        if route == "dequant+gemm":
            return linear_bf16(x, w, bias)  # the hand-written dense kernel
        return torch.nn.functional.linear(x, w, bias)

    lib = _lib.load()
    x2 = _aligned(x.reshape(-1, K))
    M = x2.shape[0]
    qweight = _aligned(qweight)
    if qweight.numel() < N * K // 2:
        raise ValueError(f"qweight holds {qweight.numel()} bytes, shape {shape} needs {N * K // 2}")
    quant_map = _aligned(quant_map.to(torch.float32))
    b = None if bias is None else bias.contiguous()
    nblocks = N * K // blocksize
    with _on_device(x.device):
        out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
        stream = _stream()
        if route in ("gemv", "gemv-chunks"):
            need = lib.nf4hip_gemv_workspace_bytes(min(M, 16), N, K)
            ws = _gemv_workspace(x.device, need, stream)
            ws_ptr, ws_bytes = ws.data_ptr(), ws.numel()
            fn, fn_dq = lib.nf4hip_gemv, lib.nf4hip_gemv_dq
        else:
            need = lib.nf4hip_gemm_workspace_bytes(M, N, K)  # K split over workgroups: partial tiles and counters
            ws = _gemv_workspace(x.device, need, stream) if need else None
            ws_ptr, ws_bytes = (None, 0) if ws is None else (ws.data_ptr(), ws.numel())
            fn, fn_dq = lib.nf4hip_gemm, lib.nf4hip_gemm_dq
        bptr = None if b is None else b.data_ptr()
        # row chunks of x and out: one call, or 16 rows at a time (rows are contiguous, K and N even,
        # so every chunk starts 16-byte aligned when the whole does and K, N are multiples of 8)
        step = 16 if route == "gemv-chunks" else M
        if isinstance(absmax, NestedAbsmax) and route == "gemm" and M > NESTED_RECONSTRUCT_MIN_M:
            # Many rows of x on nested absmax: the fused GEMM resolves an 8-bit code through two more loads per block and
            # k step and runs 5-27 % longer than on fp32 absmax; writing the fp32 absmax out first (nf4hip_dq_reconstruct,
            # 4 bytes per block into a transient buffer, 4-15 us) costs 2-7 %.  Same two roundings, same bits.
            absmax = reconstruct_absmax(absmax)
        if isinstance(absmax, NestedAbsmax):
            q, a2, m256, off, nbs = _nested_args(absmax, nblocks)
            for m0 in range(0, M, step):
                mc = min(step, M - m0)
                _lib.check(fn_dq(x2.data_ptr() + 2 * m0 * K, _lib.BF16, mc, qweight.data_ptr(), q.data_ptr(), a2.data_ptr(), m256.data_ptr(), off, nbs,
                                 quant_map.data_ptr(), bptr, N, K, blocksize, out.data_ptr() + 2 * m0 * N, ws_ptr, ws_bytes, stream))  # fmt: skip
        else:
            _require_gpu(absmax)
            absmax = _aligned(absmax.to(torch.float32))
            if absmax.numel() < nblocks:
                raise ValueError(f"absmax holds {absmax.numel()} entries, need {nblocks}")
            for m0 in range(0, M, step):
                mc = min(step, M - m0)
                _lib.check(fn(x2.data_ptr() + 2 * m0 * K, _lib.BF16, mc, qweight.data_ptr(), absmax.data_ptr(), quant_map.data_ptr(), bptr,
                              N, K, blocksize, out.data_ptr() + 2 * m0 * N, ws_ptr, ws_bytes, stream))  # fmt: skip
    return out.reshape(*x.shape[:-1], N)


def linear_possible(x: torch.Tensor, w: torch.Tensor, bias=None) -> bool:
    """Does ``linear_bf16`` take these operands (bf16, K a multiple of 64 and at least 128)?"""
    K = w.shape[-1]
    return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and (bias is None or bias.dtype == torch.bfloat16)
            and w.dim() == 2 and x.shape[-1] == K and K % 64 == 0 and K >= 128 and x.numel() > 0 and w.numel() > 0)


def linear_bf16(x: torch.Tensor, w: torch.Tensor, bias=None) -> torch.Tensor:
    """``torch.nn.functional.linear(x, w, bias)`` for bf16 operands on the hand-written dense MFMA kernel
    (``nf4hip_linear``): the GEMM that follows ``dequantize_nf4`` on the dequantize + linear route of
    bitsandbytes.matmul_4bit (MatMul4Bit.forward, reached from thunder/transforms/quantization.py:39).  ``w`` is [N, K]."""
    if not linear_possible(x, w, bias):
        raise ValueError(f"linear_bf16: bf16 operands with K a multiple of 64 (>= 128) only, got x {tuple(x.shape)} {x.dtype}, "
                         f"w {tuple(w.shape)} {w.dtype}")
    _require_gpu(x, w, bias)
    lib = _lib.load()
    N, K = w.shape
    x2 = _aligned(x.reshape(-1, K))
    w = _aligned(w)
    M = x2.shape[0]
    b = None if bias is None else bias.contiguous()
    with _on_device(x.device):
        out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
        stream = _stream()
        need = lib.nf4hip_linear_workspace_bytes(M, N, K)
        ws = _gemv_workspace(x.device, need, stream) if need else None
        ws_ptr, ws_bytes = (None, 0) if ws is None else (ws.data_ptr(), ws.numel())
        _lib.check(lib.nf4hip_linear(x2.data_ptr(), _lib.BF16, M, w.data_ptr(), None if b is None else b.data_ptr(), N, K,
                                     out.data_ptr(), ws_ptr, ws_bytes, stream))
    return out.reshape(*x.shape[:-1], N)


# ---- the decode kernels with an epilogue ---------------------------------------------------------------------


def epilogue_served(rows: int, shape, blocksize: int = 64, dtype: torch.dtype = torch.bfloat16, nested: bool = False, *,
                    rowscale_parts: int = 0, silu_pairs: bool = False, resid_norm: bool = False) -> bool:
    """Will ``matmul_nf4_epilogue`` serve ``rows`` rows of bf16 x on an [N, K] weight with this epilogue
    (``rowscale_parts``: the number of partial sums a row scale would be given, 0 for none)?  The library's own answer
    for the current device; for callers that must know before they launch the first kernel of a chain."""
    N, K = (int(s) for s in shape)
    if nested or dtype != torch.bfloat16 or blocksize not in SUPPORTED_BLOCKSIZES:
        return False
    flags = (_lib.EPI_ROWSCALE if rowscale_parts else 0) | (_lib.EPI_SILU_PAIRS if silu_pairs else 0) | (_lib.EPI_RESID_NORM if resid_norm else 0)
    return bool(_lib.load().nf4hip_gemv_epilogue_served(rows, N, K, blocksize, flags, rowscale_parts))


def matmul_nf4_epilogue(x, qweight, bias, absmax, quant_map, blocksize, dtype, shape, *, rowscale=None, silu_pairs=False,
                        resid_norm=None):
    """``matmul_nf4`` at decode shapes with the step that follows (or precedes) the linear in a decoder layer done by
    the thread that finishes each output (``nf4hip_gemv_epilogue``), one launch instead of two:

    * ``resid_norm=(resid, norm_weight)``: ``r = resid + linear(x)``; returns ``(r, xnext, sumsq)`` with
      ``xnext = r * norm_weight`` (not yet divided by the rms) and ``sumsq`` [rows, parts] partial sums of ``r**2``.
    * ``rowscale=(sumsq, eps)``: ``x`` is such an ``xnext``; the sums are multiplied by ``rsqrt(sumsq.sum(-1) / K + eps)``,
      which makes the result ``linear(rms_norm(r) * norm_weight)``.
    * ``silu_pairs``: weight rows 2j / 2j+1 are gate row j / up row j; returns ``silu(gate) * up`` [rows, N/2].

    Returns None where the library does not serve the case (more than sixteen rows of x, nested absmax, other dtypes,
    one row of x with K > 16384, ...; ``epilogue_served`` answers beforehand): the caller then runs
    ``matmul_nf4`` and the step by itself."""
    N, K = (int(s) for s in shape)
    x2 = x.reshape(-1, K)
    M = x2.shape[0]
    if isinstance(absmax, NestedAbsmax) or M > 16 or not x2.is_cuda:
        return None
    if fused_route(x2, bias, blocksize, dtype, (N, K)) != "gemv":
        return None
    lib = _lib.load()
    _require_gpu(x2, qweight, quant_map, bias, absmax)
    x2, qweight = _aligned(x2), _aligned(qweight)
    quant_map, absmax = _aligned(quant_map.to(torch.float32)), _aligned(absmax.to(torch.float32))
    if qweight.numel() < N * K // 2 or absmax.numel() < N * K // blocksize:
        raise ValueError(f"qweight / absmax hold {qweight.numel()} / {absmax.numel()} entries, too few for {shape}")
    b = None if bias is None else bias.contiguous()
    epi = _lib.Epilogue()
    keep = []  # tensors whose addresses the struct holds
    with _on_device(x2.device):
        out = None
        if rowscale is not None:
            sumsq, eps = rowscale
            if sumsq.dtype != torch.float32 or sumsq.dim() != 2 or sumsq.shape[0] != M or not sumsq.is_contiguous():
                raise ValueError(f"rowscale: sumsq must be a contiguous fp32 [rows, parts] tensor, got {sumsq.dtype} {tuple(sumsq.shape)}")
            epi.flags |= _lib.EPI_ROWSCALE
            epi.eps, epi.in_sumsq, epi.in_parts = float(eps), sumsq.data_ptr(), sumsq.shape[1]
            keep.append(sumsq)
        if silu_pairs:
            if N % 2:
                return None
            epi.flags |= _lib.EPI_SILU_PAIRS
        if resid_norm is not None:
            resid, norm_weight = resid_norm
            if resid.shape != (M, N) or resid.dtype != torch.bfloat16 or norm_weight.shape != (N,) or norm_weight.dtype != torch.bfloat16:
                raise ValueError(f"resid_norm: need bf16 resid [{M}, {N}] and norm_weight [{N}], got {tuple(resid.shape)} {resid.dtype}, "
                                 f"{tuple(norm_weight.shape)} {norm_weight.dtype}")
            parts = lib.nf4hip_gemv_norm_parts(M, N, K)
            if parts <= 0:
                return None
            resid, norm_weight = resid.contiguous(), norm_weight.contiguous()
            r_out, xnext = torch.empty_like(resid), torch.empty_like(resid)
            out_sumsq = torch.empty((M, parts), dtype=torch.float32, device=x2.device)
            epi.flags |= _lib.EPI_RESID_NORM
            epi.resid_in, epi.norm_weight = resid.data_ptr(), norm_weight.data_ptr()
            epi.resid_out, epi.xnext_out, epi.out_sumsq = r_out.data_ptr(), xnext.data_ptr(), out_sumsq.data_ptr()
            keep += [resid, norm_weight]
        else:
            out = torch.empty((M, N // 2 if silu_pairs else N), dtype=torch.bfloat16, device=x2.device)
        stream = _stream()
        ws = _gemv_workspace(x2.device, lib.nf4hip_gemv_workspace_bytes(M, N, K), stream)
        rc = lib.nf4hip_gemv_epilogue(x2.data_ptr(), _lib.BF16, M, qweight.data_ptr(), absmax.data_ptr(), quant_map.data_ptr(),
                                      None if b is None else b.data_ptr(), N, K, blocksize, None if out is None else out.data_ptr(),
                                      ws.data_ptr(), ws.numel(), ctypes.byref(epi), stream)
    if rc == _lib.E_SHAPE:
        return None
    _lib.check(rc)
    if resid_norm is not None:
        return r_out, xnext, out_sumsq
    return out.reshape(*x.shape[:-1], out.shape[-1])
