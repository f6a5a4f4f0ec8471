"""CPU stand-in for libnf4hip.so, for tests of the HOST logic only (executor registration, module
surgery, state dicts, planning).  It swaps the tensor-level ops (quantize, dequantize, matmul, absmax compression) for the oracle and lets the
transform quantise on the CPU.  Nothing in the shipped package can reach this; a GPU run never
uses it (the same tests run there against the real kernels)."""

import contextlib

import torch

from oracle import nf4_oracle as O


@contextlib.contextmanager
def installed(ta):
    F = ta.functional
    Q = ta.transforms.quantization
    saved = (F.quantize_nf4, F.dequantize_nf4, F.matmul_nf4, Q.WORK_DEVICE, F.compress_absmax)

    def plain(absmax):
        """fp32 absmax from either form of the statistics."""
        if isinstance(absmax, F.NestedAbsmax):
            return O.C().dq_reconstruct(absmax.q, absmax.absmax2, absmax.map256, absmax.offset, absmax.blocksize)
        return absmax

    def compress_absmax(absmax, nested_blocksize=256, map256=None):
        D = O.create_dynamic_map() if map256 is None else map256
        offset = O.C().dq_offset(absmax)
        q, a2 = O.C().dq_compress(absmax, D, offset, nested_blocksize)
        return F.NestedAbsmax(q, a2, D, offset, nested_blocksize)

    def quantize_nf4(w, blocksize=64):
        qw, absmax = O.C().quantize(w, blocksize)
        return qw, absmax, O.nf4_lut()

    def dequantize_nf4(qweight, absmax, quant_map, blocksize, dtype, shape):
        return O.C().dequantize(qweight, plain(absmax), quant_map, blocksize, dtype, tuple(shape))

    def matmul_nf4(x, qweight, bias, absmax, quant_map, blocksize, dtype, shape):
        assert len(shape) == 2 and x.shape[-1] == shape[1]
        return O.matmul_4bit_eager(x, qweight, bias, plain(absmax), quant_map, blocksize, dtype, tuple(shape))

    F.quantize_nf4, F.dequantize_nf4, F.matmul_nf4, Q.WORK_DEVICE, F.compress_absmax = quantize_nf4, dequantize_nf4, matmul_nf4, "cpu", compress_absmax
    try:
        yield
    finally:
        F.quantize_nf4, F.dequantize_nf4, F.matmul_nf4, Q.WORK_DEVICE, F.compress_absmax = saved
