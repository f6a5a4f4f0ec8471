"""Decode-step glue: ctypes binding of ``libnf4hip_decode.so`` (C ABI in ``include/nf4hip_decode.h``).

Three kernels for the work between the 4-bit linears of a Llama decode step -- residual add +
RMSNorm, rotary embedding + KV-cache update + grouped-query attention, SiLU(gate) * up -- and a row
argmax for greedy sampling, used by ``decode.Llama`` / ``decode.greedy_decode`` when ``LlamaConfig.hip_glue`` is set.  The reference leaves this work to its other
executors (thunder/executors/sdpaex.py, nvFuser / torch.compile fusions); it is not part of the
bitsandbytes path.  There is no CPU fallback: without the built library these functions raise.
"""

from __future__ import annotations

import ctypes
import os
import threading

import torch

from ._workspace import WorkspacePool

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libnf4hip_decode.so")

_vp, _i32, _i64, _f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
# every symbol include/nf4hip_decode.h declares: name -> (restype, argtypes)
SYMBOLS = {
    "nf4hip_decode_last_error": (ctypes.c_char_p, []),
    "nf4hip_decode_add_rmsnorm": (_i32, [_vp, _vp, _vp, _f32, _i64, _i64, _vp, _vp]),
    "nf4hip_decode_attention_workspace_bytes": (ctypes.c_size_t, [_i64, _i32, _i32]),
    "nf4hip_decode_attention": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _i64, _vp, _vp, ctypes.c_size_t, _vp]),
    "nf4hip_decode_silu_mul": (_i32, [_vp, _i64, _i64, _vp, _vp]),
    "nf4hip_decode_silu_mul_pairs": (_i32, [_vp, _i64, _i64, _vp, _vp]),
    "nf4hip_decode_argmax": (_i32, [_vp, _i64, _i64, _vp, _vp, _vp]),
}

_lib = None
_lock = threading.Lock()
_workspace_pool = WorkspacePool(1 << 20, "decode attention")  # split-key partials and counters


def _workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    """Zero-initialised scratch of the attention kernel for (device, current stream); the kernel leaves
    its counters zeroed, so the buffer is reused without clearing.  Raises instead of allocating under
    capture."""
    return _workspace_pool.get(device, nbytes)


def load(path: str | None = None) -> ctypes.CDLL:
    """Load (once) and return the shared library; raises if it has not been built."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    with _lock:
        if _lib is not None and path is None:
            return _lib
        p = path or LIB_PATH
        if not os.path.exists(p):
            raise RuntimeError(
                f"{p} not found: the HIP extension has not been built "
                "(run `python -c 'import __graft_entry__ as g; g.build()'` or `make -C lightning-thunder_amd/csrc`). "
                "There is no CPU fallback."
            )
        lib = ctypes.CDLL(p)
        for name, (restype, argtypes) in SYMBOLS.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = restype, argtypes
        if path is None:
            _lib = lib
        return lib


def _check(lib, rc: int) -> None:
    if rc != 0:
        raise RuntimeError(lib.nf4hip_decode_last_error().decode())


def _bf16_cuda(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if not (t.is_cuda and t.dtype == torch.bfloat16 and t.is_contiguous()):
            raise ValueError(f"expected a contiguous bf16 tensor on the GPU, got {t.dtype} {t.device} contiguous={t.is_contiguous()}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor) -> int:
    idx = t.device.index if t.device.index is not None else torch.cuda.current_device()
    if _raw_stream is not None:
        return _raw_stream(idx)
    return torch.cuda.current_stream(t.device).cuda_stream


def add_rmsnorm(x: torch.Tensor, delta: torch.Tensor | None, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``x += delta`` in place (skipped when ``delta`` is None), then returns ``rms_norm(x) * weight``.
    ``x``, ``delta`` [rows, d], ``weight`` [d]."""
    lib = load()
    _bf16_cuda(x, weight, *(() if delta is None else (delta,)))
    rows, d = x.shape
    if delta is not None and delta.shape != x.shape:
        raise ValueError(f"{delta.shape=} != {x.shape=}")
    y = torch.empty_like(x)
    with torch.cuda.device(x.device):
        _check(lib, lib.nf4hip_decode_add_rmsnorm(x.data_ptr(), None if delta is None else delta.data_ptr(), weight.data_ptr(),
                                                  float(eps), rows, d, y.data_ptr(), _stream(x)))
    return y


def attention_decode(qkv: torch.Tensor, pos: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, kcache: torch.Tensor,
                     vcache: torch.Tensor, n_head: int, n_kv_head: int) -> torch.Tensor:
    """One new token per sequence: rotary embedding of the q and k heads in ``qkv`` [B, (H + 2 Hkv) hd],
    the new k / v rows written into ``kcache`` / ``vcache`` [B, Hkv, max_seq, hd] at position ``pos``
    (a one-element int64 tensor on the GPU), attention over rows 0..pos.  Returns [B, H hd]."""
    lib = load()
    _bf16_cuda(qkv, kcache, vcache)
    B, Hkv, max_seq, hd = kcache.shape
    if Hkv != n_kv_head or qkv.shape != (B, (n_head + 2 * n_kv_head) * hd) or vcache.shape != kcache.shape:
        raise ValueError(f"{qkv.shape=} {kcache.shape=} {vcache.shape=} do not fit {n_head=} {n_kv_head=}")
    if not (pos.is_cuda and pos.dtype == torch.int64 and pos.numel() == 1):
        raise ValueError("pos must be a one-element int64 tensor on the GPU")
    for t in (cos, sin):
        if not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.shape == (max_seq, hd)):
            raise ValueError(f"rotary tables must be contiguous fp32 [{max_seq}, {hd}] on the GPU")
    out = torch.empty((B, n_head * hd), dtype=torch.bfloat16, device=qkv.device)
    with torch.cuda.device(qkv.device):
        need = lib.nf4hip_decode_attention_workspace_bytes(B, n_head, hd)
        ws = _workspace(qkv.device, need) if need else None
        _check(lib, lib.nf4hip_decode_attention(qkv.data_ptr(), pos.data_ptr(), cos.data_ptr(), sin.data_ptr(), kcache.data_ptr(),
                                                vcache.data_ptr(), B, n_head, n_kv_head, hd, max_seq, out.data_ptr(),
                                                None if ws is None else ws.data_ptr(), 0 if ws is None else ws.numel(), _stream(qkv)))
    return out


def silu_mul(gate_up: torch.Tensor, pairs: bool = False) -> torch.Tensor:
    """``silu(gate) * up`` for ``gate_up`` [rows, 2 dff] = (gate | up), or with ``pairs`` gate and up interleaved
    (column 2j = gate j, column 2j + 1 = up j).  Returns [rows, dff]."""
    lib = load()
    _bf16_cuda(gate_up)
    rows, two = gate_up.shape
    dff = two // 2
    out = torch.empty((rows, dff), dtype=torch.bfloat16, device=gate_up.device)
    fn = lib.nf4hip_decode_silu_mul_pairs if pairs else lib.nf4hip_decode_silu_mul
    with torch.cuda.device(gate_up.device):
        _check(lib, fn(gate_up.data_ptr(), rows, dff, out.data_ptr(), _stream(gate_up)))
    return out


def argmax_into(logits: torch.Tensor, out: torch.Tensor, pos: torch.Tensor | None = None) -> None:
    """``out[r] = logits[r].argmax()`` for ``logits`` [rows, vocab] bf16 and ``out`` int64 with ``rows`` elements;
    ``pos`` (a one-element int64 tensor on the GPU), when given, is advanced by one in the same launch."""
    lib = load()
    _bf16_cuda(logits)
    rows, vocab = logits.shape
    if not (out.is_cuda and out.dtype == torch.int64 and out.is_contiguous() and out.numel() == rows):
        raise ValueError(f"out must be a contiguous int64 GPU tensor of {rows} elements, got {out.dtype} {tuple(out.shape)}")
    if pos is not None and not (pos.is_cuda and pos.dtype == torch.int64 and pos.numel() == 1):
        raise ValueError("pos must be a one-element int64 tensor on the GPU")
    with torch.cuda.device(logits.device):
        _check(lib, lib.nf4hip_decode_argmax(logits.data_ptr(), rows, vocab, out.data_ptr(), None if pos is None else pos.data_ptr(),
                                             _stream(logits)))
