"""CPU oracle for the NF4 weight-only linear path.  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may import
this module; the shipped package never does.

Two independent restatements live here and are cross-checked by the tests:

* ``C``  -- ctypes bindings of ``oracle/nf4_oracle.c`` (scalar C, one element at a time);
* ``*_eager`` functions -- a vectorised torch-eager restatement.  It doubles as the reference's
  CPU-side semantics (bitsandbytes' ``MatMul4Bit`` route: ``dequantize_4bit(...).to(x.dtype)``
  followed by ``torch.nn.functional.linear``, reached from
  thunder/transforms/quantization.py:39) and is what ``bench.py`` times as ``cpu_baseline``.

The arithmetic is bitsandbytes==0.48.0's (requirements/test.txt:20), which is not vendored in
the reference; call sites: thunder/transforms/quantization.py:63 (``quantize_4bit``) and
thunder/transforms/quantization.py:34-39 (``matmul_4bit``).

Parity unpinned (no import of bitsandbytes is possible, nothing in the reference's tests covers
them): exact-threshold ties, the pad nibble for odd ``n``, NaN/Inf inputs and the whole nested
("double") quantisation of absmax, which the reference transform never calls
(thunder/transforms/quantization.py:84 ``# TODO: double quant support``).
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libnf4oracle.so")

DTYPE_CODE = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}

# fp32 NF4 code values, index = 4-bit code (bitsandbytes functional.get_4bit_type("nf4")).
NF4_LUT = (
    -1.0,
    -0.6961928009986877,
    -0.5250730514526367,
    -0.39491748809814453,
    -0.28444138169288635,
    -0.18477343022823334,
    -0.09105003625154495,
    0.0,
    0.07958029955625534,
    0.16093020141124725,
    0.24611230194568634,
    0.33791524171829224,
    0.44070982933044434,
    0.5626170039176941,
    0.7229568362236023,
    1.0,
)

# double midpoints of adjacent code values; compared as fp32 (bitsandbytes dQuantizeNF4 literals).
NF4_THRESHOLDS = (
    -0.8480964004993439,
    -0.6106329262256622,
    -0.4599952697753906,
    -0.33967943489551544,
    -0.23460740596055984,
    -0.13791173323988914,
    -0.045525018125772476,
    0.03979014977812767,
    0.1202552504837513,
    0.2035212516784668,
    0.2920137718319893,
    0.3893125355243683,
    0.5016634166240692,
    0.6427869200706482,
    0.8614784181118011,
)


# The same 15 thresholds as the fp32 values a C compiler produces for the literals
# ``-0.8480964004993439f`` ... ``0.8614784181118011f`` (correct rounding of the DECIMAL text; four
# of the midpoints are exact fp32 ties, so rounding the double instead would move them by 1 ulp).
NF4_THRESHOLD_BITS = (
    0xBF591CD9, 0xBF1C5270, 0xBEEB8480, 0xBEADEA76, 0xBE703CEC, 0xBE0D38BC, 0xBD3A7871, 0x3D22FAFF,
    0x3DF64863, 0x3E5067E0, 0x3E9582D4, 0x3EC753F9, 0x3F006D03, 0x3F248DAF, 0x3F5C89D9,
)


def nf4_thresholds_f32() -> torch.Tensor:
    return torch.from_numpy(np.array(NF4_THRESHOLD_BITS, dtype=np.uint32).view(np.float32).copy())


def build_c_oracle(force: bool = False) -> str:
    """Compile ``nf4_oracle.c`` into ``libnf4oracle.so`` (gcc, a few hundred ms)."""
    src = os.path.join(_HERE, "nf4_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libnf4oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


class _COracle:
    """ctypes view of the scalar C restatement; tensors are CPU, contiguous."""

    def __init__(self):
        path = _LIB_PATH if os.path.exists(_LIB_PATH) else build_c_oracle()
        L = ctypes.CDLL(path)
        i64, i32, vp, f32 = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_float
        L.nf4o_quantize.argtypes = [vp, i32, i64, i32, vp, vp]
        L.nf4o_dequantize.argtypes = [vp, vp, vp, i64, i32, vp, i32]
        L.nf4o_matmul.argtypes = [vp, i32, i64, vp, vp, vp, vp, i64, i64, i32, i32, vp]
        L.nf4o_dq_offset.argtypes = [vp, i64]
        L.nf4o_dq_offset.restype = f32
        L.nf4o_dq_compress.argtypes = [vp, i64, i32, vp, f32, vp, vp]
        L.nf4o_dq_reconstruct.argtypes = [vp, vp, vp, f32, i64, i32, vp]
        L.nf4o_lut16.argtypes = [vp]
        L.nf4o_thresholds.argtypes = [vp]
        L.nf4o_code_of.argtypes = [f32]
        L.nf4o_f32_to_bf16.argtypes = [f32]
        L.nf4o_f32_to_bf16.restype = ctypes.c_uint16
        L.nf4o_f32_to_f16.argtypes = [f32]
        L.nf4o_f32_to_f16.restype = ctypes.c_uint16
        L.nf4o_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.nf4o_f16_to_f32.restype = f32
        self.L = L

    @staticmethod
    def _chk(rc):
        if rc != 0:
            raise RuntimeError(f"nf4 oracle returned {rc}")

    def lut16(self) -> torch.Tensor:
        out = torch.empty(16, dtype=torch.float32)
        self.L.nf4o_lut16(out.data_ptr())
        return out

    def thresholds(self) -> torch.Tensor:
        out = torch.empty(15, dtype=torch.float32)
        self.L.nf4o_thresholds(out.data_ptr())
        return out

    def quantize(self, w: torch.Tensor, blocksize: int = 64):
        w = w.detach().contiguous().cpu()
        n = w.numel()
        packed = torch.empty(((n + 1) // 2, 1), dtype=torch.uint8)
        absmax = torch.empty(((n + blocksize - 1) // blocksize,), dtype=torch.float32)
        self._chk(self.L.nf4o_quantize(w.data_ptr(), DTYPE_CODE[w.dtype], n, blocksize, packed.data_ptr(), absmax.data_ptr()))
        return packed, absmax

    def dequantize(self, packed, absmax, lut16, blocksize, dtype, shape) -> torch.Tensor:
        n = int(np.prod(shape))
        packed = packed.contiguous().cpu()
        absmax = absmax.contiguous().cpu().float()
        lut16 = lut16.contiguous().cpu().float()
        out = torch.empty(n, dtype=dtype)
        self._chk(
            self.L.nf4o_dequantize(packed.data_ptr(), absmax.data_ptr(), lut16.data_ptr(), n, blocksize, out.data_ptr(), DTYPE_CODE[dtype])
        )
        return out.reshape(tuple(shape))

    def matmul(self, x, packed, bias, absmax, lut16, blocksize, w_dtype, shape) -> torch.Tensor:
        N, K = shape
        x2 = x.detach().contiguous().cpu().reshape(-1, K)
        M = x2.shape[0]
        packed = packed.contiguous().cpu()
        absmax = absmax.contiguous().cpu().float()
        lut16 = lut16.contiguous().cpu().float()
        b = None if bias is None else bias.detach().contiguous().cpu().to(x2.dtype)
        out = torch.empty((M, N), dtype=x2.dtype)
        self._chk(
            self.L.nf4o_matmul(
                x2.data_ptr(), DTYPE_CODE[x2.dtype], M, packed.data_ptr(), absmax.data_ptr(), lut16.data_ptr(),
                None if b is None else b.data_ptr(), N, K, blocksize, DTYPE_CODE[w_dtype], out.data_ptr(),
            )
        )
        return out.reshape(*x.shape[:-1], N)

    def dq_offset(self, absmax) -> float:
        absmax = absmax.contiguous().cpu().float()
        return float(self.L.nf4o_dq_offset(absmax.data_ptr(), absmax.numel()))

    def dq_compress(self, absmax, map256, offset, nested_blocksize: int = 256):
        absmax = absmax.contiguous().cpu().float()
        map256 = map256.contiguous().cpu().float()
        nb = absmax.numel()
        q = torch.empty(nb, dtype=torch.uint8)
        absmax2 = torch.empty(((nb + nested_blocksize - 1) // nested_blocksize,), dtype=torch.float32)
        self._chk(self.L.nf4o_dq_compress(absmax.data_ptr(), nb, nested_blocksize, map256.data_ptr(), offset, q.data_ptr(), absmax2.data_ptr()))
        return q, absmax2

    def dq_reconstruct(self, q, absmax2, map256, offset, nested_blocksize: int = 256) -> torch.Tensor:
        q = q.contiguous().cpu()
        absmax2 = absmax2.contiguous().cpu().float()
        map256 = map256.contiguous().cpu().float()
        out = torch.empty(q.numel(), dtype=torch.float32)
        self._chk(self.L.nf4o_dq_reconstruct(q.data_ptr(), absmax2.data_ptr(), map256.data_ptr(), offset, q.numel(), nested_blocksize, out.data_ptr()))
        return out


_C = None


def C() -> _COracle:
    global _C
    if _C is None:
        _C = _COracle()
    return _C


# --------------------------------------------------------------------------------------------
# torch-eager restatement
# --------------------------------------------------------------------------------------------


def nf4_lut(dtype=torch.float32) -> torch.Tensor:
    return torch.tensor(NF4_LUT, dtype=torch.float32).to(dtype)


def create_normal_map_closed_form() -> torch.Tensor:
    """QLoRA construction of the NF4 code values (bitsandbytes functional.create_normal_map,
    offset=0.9677083, use_extra_value=True): 8 positive quantiles, 0, 7 negative quantiles of
    N(0,1), normalised by the largest."""
    from scipy.stats import norm

    offset = 0.9677083
    v1 = norm.ppf(torch.linspace(offset, 0.5, 9)[:-1]).tolist()
    v3 = (-norm.ppf(torch.linspace(offset, 0.5, 8)[:-1])).tolist()
    v = torch.tensor(v1 + [0.0] + v3, dtype=torch.float64).sort().values
    v = v / v.max()
    return v.to(torch.float32)


def create_dynamic_map(signed: bool = True, max_exponent_bits: int = 7, total_bits: int = 8) -> torch.Tensor:
    """The 256-entry "dynamic" 8-bit code used for nested absmax quantisation
    (bitsandbytes functional.create_dynamic_map)."""
    data = []
    non_sign_bits = total_bits - 1
    additional_items = 2 ** (non_sign_bits - max_exponent_bits) - 1
    for i in range(max_exponent_bits):
        fraction_items = int(2 ** (i + non_sign_bits - max_exponent_bits) + 1 if signed else 2 ** (i + non_sign_bits - max_exponent_bits + 1) + 1)
        boundaries = torch.linspace(0.1, 1, fraction_items)
        means = (boundaries[:-1] + boundaries[1:]) / 2.0
        data += ((10 ** (-(max_exponent_bits - 1) + i)) * means).tolist()
        if signed:
            data += (-(10 ** (-(max_exponent_bits - 1) + i)) * means).tolist()
    if additional_items > 0:
        boundaries = torch.linspace(0.1, 1, additional_items + 1)
        means = (boundaries[:-1] + boundaries[1:]) / 2.0
        data += ((10 ** (-(max_exponent_bits - 1) + i)) * means).tolist()
        if signed:
            data += (-(10 ** (-(max_exponent_bits - 1) + i)) * means).tolist()
    data.append(0)
    data.append(1.0)
    assert len(data) == 2**total_bits
    data.sort()
    return torch.tensor(data, dtype=torch.float32)


def quantize_4bit_eager(w: torch.Tensor, blocksize: int = 64, rule: str = "threshold"):
    """Blockwise NF4 quantisation.  ``rule="threshold"`` counts thresholds strictly below the
    scaled value (the CUDA kernel's decision tree); ``rule="argmin"`` is nearest neighbour over
    the code values (the eager backend).  Returns (packed uint8 [(n+1)//2, 1], absmax fp32)."""
    w = w.detach().cpu()
    n = w.numel()
    flat = w.reshape(-1).to(torch.float32)
    nblocks = (n + blocksize - 1) // blocksize
    pad = nblocks * blocksize - n
    if pad:
        flat = torch.cat([flat, torch.zeros(pad, dtype=torch.float32)])
    blocks = flat.view(nblocks, blocksize)
    absmax = blocks.abs().max(dim=1).values
    inv = 1.0 / absmax  # IEEE fp32 division
    scaled = blocks * inv.view(-1, 1)
    if rule == "threshold":
        thr = nf4_thresholds_f32()
        codes = (scaled.unsqueeze(-1) > thr).sum(dim=-1)
    elif rule == "argmin":
        lut = nf4_lut()
        s = torch.nan_to_num(scaled.clamp(-1, 1), nan=-1.0)
        codes = torch.argmin((s.unsqueeze(-1) - lut).abs(), dim=-1)
        codes = torch.where(torch.isnan(scaled), torch.zeros_like(codes), codes)
    else:
        raise ValueError(rule)
    codes = codes.reshape(-1).to(torch.uint8)
    n_even = (n + 1) // 2 * 2
    codes = codes[:n_even] if codes.numel() >= n_even else torch.cat([codes, torch.full((n_even - codes.numel(),), 7, dtype=torch.uint8)])
    packed = (codes[0::2] << 4) | codes[1::2]
    return packed.reshape(-1, 1).contiguous(), absmax.contiguous()


def unpack_codes(packed: torch.Tensor, n: int) -> torch.Tensor:
    p = packed.reshape(-1).cpu()
    codes = torch.stack([p >> 4, p & 15], dim=1).reshape(-1)
    return codes[:n].long()


def dequantize_4bit_eager(packed, absmax, lut16, blocksize, dtype, shape) -> torch.Tensor:
    """``cast(lut16[code] * absmax[block])``: one fp32 multiply, one rounding to ``dtype``."""
    n = int(np.prod(shape))
    codes = unpack_codes(packed, n)
    lut16 = lut16.detach().cpu().to(torch.float32)
    scale = absmax.detach().cpu().to(torch.float32).repeat_interleave(blocksize)[:n]
    return (lut16[codes] * scale).to(dtype).reshape(tuple(shape))


def matmul_4bit_eager(x, packed, bias, absmax, lut16, blocksize, w_dtype, shape) -> torch.Tensor:
    """The reference's CPU-side route: dequantize, convert to x's dtype, ``F.linear``."""
    w = dequantize_4bit_eager(packed, absmax, lut16, blocksize, w_dtype, shape).to(x.dtype)
    return torch.nn.functional.linear(x.cpu(), w, None if bias is None else bias.cpu())


def matmul_4bit_f64(x, packed, bias, absmax, lut16, blocksize, w_dtype, shape) -> torch.Tensor:
    """Same contraction accumulated in float64 and rounded once: the centre of the tolerance band."""
    w = dequantize_4bit_eager(packed, absmax, lut16, blocksize, w_dtype, shape).to(x.dtype).double()
    y = x.cpu().double() @ w.t()
    if bias is not None:
        y = y + bias.cpu().double()
    return y.to(x.dtype)


def dq_compress_eager(absmax: torch.Tensor, map256: torch.Tensor, nested_blocksize: int = 256):
    """Nested quantisation of absmax.  Returns (q uint8, absmax2 fp32, offset float)."""
    absmax = absmax.detach().cpu().to(torch.float32)
    offset = float(absmax.double().mean().to(torch.float32)) if absmax.numel() else 0.0
    r = absmax - torch.tensor(offset, dtype=torch.float32)
    nb = r.numel()
    nnb = (nb + nested_blocksize - 1) // nested_blocksize
    pad = nnb * nested_blocksize - nb
    rp = torch.cat([r, torch.zeros(pad)]) if pad else r
    blocks = rp.view(nnb, nested_blocksize)
    absmax2 = blocks.abs().max(dim=1).values
    inv = 1.0 / absmax2
    s = blocks * inv.view(-1, 1)
    d = (s.unsqueeze(-1) - map256.cpu().float()).abs()
    q = torch.argmin(torch.nan_to_num(d, nan=float("inf")), dim=-1)
    zero_code = int((map256 == 0).nonzero()[0])
    q = torch.where((absmax2 == 0).view(-1, 1), torch.full_like(q, zero_code), q)
    return q.reshape(-1)[:nb].to(torch.uint8), absmax2, offset


def dq_reconstruct_eager(q, absmax2, map256, offset, nested_blocksize: int = 256) -> torch.Tensor:
    m = map256.cpu().float()[q.cpu().long()]
    s = absmax2.cpu().float().repeat_interleave(nested_blocksize)[: q.numel()]
    return m * s + torch.tensor(offset, dtype=torch.float32)
