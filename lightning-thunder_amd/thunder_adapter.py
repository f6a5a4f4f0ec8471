"""The HIP NF4 path on a REAL Thunder installation (import-guarded: nothing here runs unless
``thunder`` itself is importable, which it is not in this build's environment).

``install()`` registers ``hip_matmul_nf4`` on a ``thunder.extend.OperatorExecutor`` the way the
reference registers ``bnb_matmul_nf4`` (thunder/transforms/quantization.py:19-44) and returns a
subclass of the reference's own ``BitsAndBytesLinearQuant4bit`` whose two bitsandbytes touch
points are replaced:

* ``quantize_weight`` (quantization.py:53-63) calls ``functional.quantize_nf4`` and returns the
  ``(qweight, state)`` pair the rest of the class reads (``absmax, code, dtype, shape, blocksize``);
* ``transform_traces_pre_prologue`` (quantization.py:128-293) is the reference's, run with the module
  global ``bnb_matmul_nf4`` pointing at the HIP symbol for the duration of the call, so the bound
  symbol it creates (quantization.py:262-266) already belongs to this executor and the dispatch pass
  keeps it (thunder/executors/passes.py:80-83).

Usage: ``T = install(); jm = thunder.jit(model, transforms=[T()], executors=(T.executor,))``.
"""

from __future__ import annotations

from collections.abc import Sequence
from types import SimpleNamespace

import torch

from . import functional
from .transforms import quantization

EXECUTOR_NAME = "quant_hip_nf4"


def install():
    try:
        import thunder
        import thunder.transforms.quantization as ref
    except ImportError as e:  # pragma: no cover - exercised only where Thunder is absent
        raise ImportError("thunder_adapter.install() needs an importable lightning-thunder installation") from e

    ex = thunder.extend.get_executor(EXECUTOR_NAME)
    if ex is None:
        ex = thunder.extend.OperatorExecutor(EXECUTOR_NAME, version=0.1)

        def hip_matmul_nf4_meta(x, qweight, bias, absmax, quant_map, blocksize, dtype, shape):
            assert isinstance(shape, Sequence) and len(shape) == 2
            assert x.shape[-1] == shape[1], f"{x.shape=}, rhs {shape=}"
            return thunder.TensorProxy(like=x, shape=(*x.shape[:-1], shape[0]))

        # resolved at call time, so that whoever replaces functional.matmul_nf4 (a test's stand-in) is honoured
        ex.register_operator("hip_matmul_nf4", meta=hip_matmul_nf4_meta, fn=lambda *args: functional.matmul_nf4(*args))
        thunder.extend.register_executor(ex)
    hip_matmul_nf4 = ex.opmap["hip_matmul_nf4"]

    class HipLinearQuant4bit(ref.BitsAndBytesLinearQuant4bit):
        executor = ex

        def __init__(self, blocksize: int = 64):
            # the reference's __init__ imports bitsandbytes; only its two attributes are needed
            self.quant_states = {}
            self.quantized_submodule_names = set()
            self.blocksize = blocksize

        def quantize_weight(self, w):
            # the reference's device policy (quantization.py:53-63): meta stands for zeros on the GPU, a weight
            # elsewhere is copied there, a GPU weight is used where it is
            work = torch.device(quantization.WORK_DEVICE)
            if w.device.type == "meta":
                w_work = torch.zeros_like(w, device=work)
            elif w.device.type != work.type:
                with torch.no_grad():
                    w_work = w.to(work)
            else:
                w_work = w
            qw, absmax, code = functional.quantize_nf4(w_work, self.blocksize)
            state = SimpleNamespace(absmax=absmax, code=code, dtype=w.dtype, shape=tuple(w.shape), blocksize=self.blocksize)
            return qw, state

        def transform_traces_pre_prologue(self, prologue_trace, computation_trace, epilogue_trace, **kwargs):
            missing = object()
            saved = getattr(ref, "bnb_matmul_nf4", missing)
            ref.bnb_matmul_nf4 = hip_matmul_nf4
            try:
                return super().transform_traces_pre_prologue(prologue_trace, computation_trace, epilogue_trace, **kwargs)
            finally:
                if saved is missing:
                    del ref.bnb_matmul_nf4
                else:
                    ref.bnb_matmul_nf4 = saved

    return HipLinearQuant4bit
