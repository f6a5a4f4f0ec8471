"""``BitsAndBytesLinearQuant4bit`` with the HIP executor behind it.

Mirror of thunder/transforms/quantization.py: same class name, hooks, ``quant_states`` layout,
override keys (``<w>``, ``<w>.absmax``, ``<w>.code``) and operator signature.  The executor is
``quant_hip_nf4`` instead of ``quant_bnb`` and its operator ``hip_matmul_nf4`` calls the gfx950
kernels of libnf4hip.so instead of bitsandbytes.
"""

from __future__ import annotations

from collections.abc import Sequence

import torch

from .. import extend, functional
from ..trace import (
    STATIC_MEMORY_LOCATION,
    TensorProxy,
    add_trace_output,
    check_tensor_shape_and_metadata,
    get_checks,
    python_return,
    trace_with_replaced_proxy_metadata,
    unpack_trivial,
)
from ..transform_common import Transform

hip_nf4_executor: extend.OperatorExecutor | None = None
hip_matmul_nf4: extend.Symbol | None = None
hip_quantize_nf4: extend.Symbol | None = None
hip_dequantize_nf4: extend.Symbol | None = None


def hip_matmul_nf4_meta(x, qweight, bias, absmax, quant_map, blocksize, dtype, shape):
    """Shape/dtype inference of the operator (thunder/transforms/quantization.py:29-32)."""
    assert isinstance(shape, Sequence) and len(shape) == 2
    assert x.shape[-1] == shape[1], f"{x.shape=}, rhs {shape=}"
    return TensorProxy(like=x, shape=(*x.shape[:-1], shape[0]))


def hip_matmul_nf4_impl(x, qweight, bias, absmax, quant_map, blocksize, dtype, shape):
    """``x @ dequantize(qweight).T + bias`` (thunder/transforms/quantization.py:34-39)."""
    return functional.matmul_nf4(x, qweight, bias, absmax, quant_map, blocksize, dtype, shape)


def hip_quantize_nf4_impl(w, blocksize=64):
    return functional.quantize_nf4(w, blocksize)


def hip_dequantize_nf4_impl(qweight, absmax, quant_map, blocksize, dtype, shape):
    return functional.dequantize_nf4(qweight, absmax, quant_map, blocksize, dtype, shape)


# Device on which weights are quantised.  The reference hard-codes "cuda" (quantization.py:53-63);
# ROCm builds of torch use the same device name.
WORK_DEVICE = "cuda"


def _quantize_meta(w, blocksize=64):
    n = 1
    for s in w.shape:
        n *= s
    return (
        TensorProxy(like=w, shape=((n + 1) // 2, 1), dtype=torch.uint8, requires_grad=False),
        TensorProxy(like=w, shape=((n + blocksize - 1) // blocksize,), dtype=torch.float32, requires_grad=False),
        TensorProxy(like=w, shape=(16,), dtype=torch.float32, requires_grad=False),
    )


def _dequantize_meta(qweight, absmax, quant_map, blocksize, dtype, shape):
    return TensorProxy(like=qweight, shape=tuple(shape), dtype=dtype, requires_grad=False)


def get_hip_nf4_executor() -> extend.OperatorExecutor:
    """The singleton executor ``quant_hip_nf4`` with its operators registered; idempotent
    (thunder/transforms/quantization.py:19-44).  Loading the HIP library is part of it: a missing
    or mismatching ``libnf4hip.so`` fails here, not at the first forward."""
    global hip_nf4_executor, hip_matmul_nf4, hip_quantize_nf4, hip_dequantize_nf4
    if hip_nf4_executor is None:
        from .. import _lib

        _lib.load()
        ex = extend.OperatorExecutor("quant_hip_nf4", version=0.1)
        hip_matmul_nf4 = ex.register_operator("hip_matmul_nf4", meta=hip_matmul_nf4_meta, fn=hip_matmul_nf4_impl)
        hip_quantize_nf4 = ex.register_operator("hip_quantize_nf4", meta=_quantize_meta, fn=hip_quantize_nf4_impl)
        hip_dequantize_nf4 = ex.register_operator("hip_dequantize_nf4", meta=_dequantize_meta, fn=hip_dequantize_nf4_impl)
        extend.register_executor(ex)
        hip_nf4_executor = ex
    return hip_nf4_executor


# the reference's spelling, so that code written against it keeps working
get_bitsandbytes_executor = get_hip_nf4_executor


class BitsAndBytesLinearQuant4bit(Transform):
    """Quantise the weight of every ``nn.Linear`` to NF4 and route its matmul to the HIP operator.

    ``BitsAndBytesLinearQuant4bit()`` behaves like the reference (blocksize 64, fp32 absmax).
    ``lut_rounding="dtype"`` stores the code book pre-rounded to the weight dtype, which reproduces
    bitsandbytes' eager (non-CUDA) dequantisation instead of its CUDA kernel's.
    """

    def __init__(self, *, blocksize: int = 64, lut_rounding: str = "none"):
        assert lut_rounding in ("none", "dtype")
        self.quant_states: dict[str, dict] = {}
        self.quantized_submodule_names: set[str] = set()
        self.blocksize = blocksize
        self.lut_rounding = lut_rounding
        get_hip_nf4_executor()

    def quantize_weight(self, w: torch.Tensor):
        """Device policy of the reference (quantization.py:53-63): meta -> zeros on the GPU, anything
        not on the GPU is moved there; then the quantise kernel.  Returns (qweight, absmax, code)."""
        work = torch.device(WORK_DEVICE)
        if w.device.type == "meta":
            w_work = torch.zeros_like(w, device=work)
        elif w.device.type != work.type:
            with torch.no_grad():
                w_work = w.to(work)
        else:
            w_work = w
        qw, absmax, code = hip_quantize_nf4(w_work.detach(), self.blocksize)
        if self.lut_rounding == "dtype":
            code = code.to(w.dtype).to(torch.float32)
        return qw, absmax, code

    def transform_module(self, model) -> None:
        self.thunder_module = model
        shared_names = model._get_shared_names()
        processed: set[str] = set()

        def convert_linear_submodule(tm, name: str) -> None:
            self.quantized_submodule_names.add(name)
            weight_name = f"{name}.weight" if name else "weight"
            done_copies = shared_names[weight_name] & processed
            if done_copies:  # tied weight: share the already quantised tensors
                copy_name = next(iter(done_copies))
                self.quant_states[weight_name] = self.quant_states[copy_name]
                for suffix in ("", ".absmax", ".code"):
                    tm._overrides_parameters[weight_name + suffix] = tm._overrides_parameters[copy_name + suffix]
                processed.add(weight_name)
                return
            w = tm.get_parameter(weight_name)
            qw, absmax, code = self.quantize_weight(w)
            tm._overrides_parameters[weight_name] = qw.to(w.device)
            tm._overrides_parameters[f"{weight_name}.absmax"] = absmax.to(w.device)
            tm._overrides_parameters[f"{weight_name}.code"] = code.to(w.device)
            self.quant_states[weight_name] = {
                "dtype": w.dtype,
                "shape": tuple(w.shape),
                "blocksize": self.blocksize,
                "qweight.dtype": qw.dtype,
                "qweight.shape": tuple(qw.shape),
                "absmax.dtype": absmax.dtype,
                "absmax.shape": tuple(absmax.shape),
                "code.dtype": code.dtype,
                "code.shape": tuple(code.shape),
                "device": getattr(w, "_thunder_device", w.device),
            }
            processed.add(weight_name)

        for n, submodule in model._model.named_modules():
            if isinstance(submodule, torch.nn.Linear):
                convert_linear_submodule(model, n)

    def transform_state_dict_for_submodule(self, model, submodule_name: str, state_dict: dict) -> dict:
        """Quantise an incoming original weight; keys carry no submodule prefix (quantization.py:108-126)."""
        if submodule_name not in self.quantized_submodule_names:
            return state_dict
        weight_name_full = f"{submodule_name}.weight" if submodule_name else "weight"
        qs = self.quant_states[weight_name_full]
        w = state_dict["weight"]
        assert w.dtype == qs["dtype"]
        assert tuple(w.shape) == tuple(qs["shape"])
        qw, absmax, code = self.quantize_weight(w)
        state_dict = state_dict.copy()
        state_dict["weight"] = qw.to(w.device)
        state_dict["weight.absmax"] = absmax.to(w.device)
        state_dict["weight.code"] = code.to(w.device)
        return state_dict

    def reverse_transform_state_dict_for_submodule(self, model, submodule_name: str, state_dict: dict) -> dict:
        """Dequantise back to the original dtype and shape.  (The reference has no reverse; its
        ``original_state_dict()`` of a quantised module returns the packed tensors.)"""
        if submodule_name not in self.quantized_submodule_names or "weight.absmax" not in state_dict:
            return state_dict
        qs = self.quant_states[f"{submodule_name}.weight" if submodule_name else "weight"]
        sd = {k: v for k, v in state_dict.items() if k not in ("weight.absmax", "weight.code")}
        qw, absmax, code = state_dict["weight"], state_dict["weight.absmax"], state_dict["weight.code"]
        dev = qw.device
        w = hip_dequantize_nf4(qw.to(WORK_DEVICE), absmax.to(WORK_DEVICE), code.to(WORK_DEVICE), qs["blocksize"], qs["dtype"], qs["shape"])
        sd["weight"] = w.to(dev)
        return sd

    def transform_traces_pre_prologue(self, prologue_trace, computation_trace, epilogue_trace, **kwargs):
        """Rewrite the plan of a call (quantization.py:128-293): the checks of quantised weights expect
        the packed tensor; absmax and code become extra prologue outputs / computation inputs; every
        ``linear`` on a quantised weight becomes ``hip_matmul_nf4(x, qweight, bias, absmax, code,
        blocksize, dtype, shape)``; nothing else changes."""
        tm = self.thunder_module
        checks = get_checks(prologue_trace)
        prologue_proxy_map = {
            get_param.output.name: dict(shape=self.quant_states[n]["qweight.shape"], dtype=self.quant_states[n]["qweight.dtype"])
            for n, (check, get_param) in checks.items()
            if n in self.quant_states
        }
        prologue_trace = trace_with_replaced_proxy_metadata(prologue_trace, prologue_proxy_map)
        checks = get_checks(prologue_trace)
        output_idxes = {o.name: i for i, o in enumerate(prologue_trace.output[0])}

        quantized_proxies: dict[str, str] = {}  # proxy name -> parameter name
        additional_proxies: dict[str, TensorProxy] = {}  # parameter name.(absmax|code) -> proxy
        new_bsyms, new_compute_inputs = [], []
        for n, qs in self.quant_states.items():
            for key in (n, f"{n}.absmax", f"{n}.code"):
                tm.get_parameter(key)  # must exist
            check, get_param = checks[n]
            quantized_proxies[get_param.output.name] = n
            proxy, _, device, _, _ = check.args
            check.args = (proxy, qs["qweight.shape"], device, qs["qweight.dtype"], False)
            proxy.requires_grad = False
            if get_param.output.name not in output_idxes:
                continue
            for suffix in ("absmax", "code"):
                p = TensorProxy(f"{get_param.output.name}_{suffix}", shape=qs[f"{suffix}.shape"], dtype=qs[f"{suffix}.dtype"],
                                device=device, requires_grad=False, tags={STATIC_MEMORY_LOCATION})
                new_bsyms.append(get_param.sym.bind(get_param.args[0], f"{n}.{suffix}", output=p))
                add_trace_output(prologue_trace, p, subindex=0)
                new_compute_inputs.append(p)
                new_bsyms.append(check_tensor_shape_and_metadata.bind(p, qs[f"{suffix}.shape"], device, qs[f"{suffix}.dtype"], False, output=None))
                additional_proxies[f"{n}.{suffix}"] = p
        prologue_trace.bound_symbols[-1:-1] = new_bsyms

        computation_trace.args = (*computation_trace.args, *new_compute_inputs)
        computation_trace.names.update(i.name for i in new_compute_inputs)
        insert_idx = 0
        for i, bsym in enumerate(computation_trace.bound_symbols):
            if bsym.sym is unpack_trivial:
                insert_idx = i + 1
        computation_trace.bound_symbols[insert_idx:insert_idx] = [
            unpack_trivial.bind(i, output=i, name=i.name) for i in new_compute_inputs
        ]

        new_bound_symbols = []
        for bsym in computation_trace.bound_symbols:
            if bsym.sym is extend.linear and isinstance(bsym.args[1], TensorProxy) and bsym.args[1].name in quantized_proxies:
                assert len(bsym.args) == 3  # linear(input, weight, bias)
                n = quantized_proxies[bsym.args[1].name]
                qs = self.quant_states[n]
                new_args = (*bsym.args[:3], additional_proxies[f"{n}.absmax"], additional_proxies[f"{n}.code"],
                            qs["blocksize"], qs["dtype"], qs["shape"])
                new_bound_symbols.append(bsym.from_bsym(sym=hip_matmul_nf4, subsymbols=(), args=new_args))
            elif bsym.sym is python_return:
                ret = dict(bsym.args[0])
                ret["flat_args"] = list(computation_trace.args)
                new_bound_symbols.append(bsym.from_bsym(args=(ret,)))
            else:
                new_bound_symbols.append(bsym)
        computation_trace.bound_symbols = new_bound_symbols
        computation_trace.set_provenance("quant pass")
        return prologue_trace, computation_trace, epilogue_trace
