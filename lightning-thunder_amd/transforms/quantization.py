"""``BitsAndBytesLinearQuant4bit`` with the HIP executor behind it.

Same class name, hooks, ``quant_states`` layout, override keys (``<w>``, ``<w>.absmax``, ``<w>.code``) and
operator signature as thunder/transforms/quantization.py; the executor is ``quant_hip_nf4`` instead of
``quant_bnb`` and its operator ``hip_matmul_nf4`` runs the gfx950 kernels of libnf4hip.so instead of
bitsandbytes.

Beyond the reference (which leaves it as a TODO, thunder/transforms/quantization.py:84):
``BitsAndBytesLinearQuant4bit(double_quant=True)`` also quantises the per-block absmax to 8 bits
(bitsandbytes' ``compress_statistics=True``).  ``<w>.absmax`` then holds the uint8 codes and three more
entries appear next to it -- ``<w>.nested_absmax``, ``<w>.nested_quant_map``, ``<w>.nested_offset`` -- and the
linears run ``hip_matmul_nf4_dq``, whose arguments are those tensors in place of ``absmax``.
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
hip_matmul_nf4_dq: extend.Symbol | None = None
# hip_matmul_nf4 with an epilogue: the residual add / RMSNorm / SiLU * up next to the linear done by the decode kernel
# (no counterpart in the reference, whose other executors fuse those steps around bnb_matmul_nf4)
hip_matmul_nf4_epilogue: extend.Symbol | None = None
hip_quantize_nf4_dq: extend.Symbol | None = None
hip_dequantize_nf4_dq: extend.Symbol | None = None

# Device on which weights are quantised.  The reference hard-codes "cuda" (quantization.py:53-63);
# ROCm builds of torch use the same device name.
WORK_DEVICE = "cuda"


# ---- operators: meta (shape / dtype inference on proxies) and implementation --------------------------


def _numel(shape) -> int:
    n = 1
    for s in shape:
        n *= int(s)
    return n


def _check_matmul_shapes(x, shape) -> None:
    assert isinstance(shape, Sequence) and len(shape) == 2
    assert x.shape[-1] == shape[1], f"{x.shape=}, rhs {shape=}"


def hip_matmul_nf4_meta(x, qweight, bias, absmax, quant_map, blocksize, dtype, shape):
    """Shape/dtype inference of the operator (thunder/transforms/quantization.py:29-32)."""
    _check_matmul_shapes(x, shape)
    return TensorProxy(like=x, shape=(*x.shape[:-1], shape[0]))


def hip_matmul_nf4_impl(x, qweight, bias, absmax, quant_map, blocksize, dtype, shape):
    """``x @ dequantize(qweight).T + bias`` (thunder/transforms/quantization.py:34-39)."""
    return functional.matmul_nf4(x, qweight, bias, absmax, quant_map, blocksize, dtype, shape)


def hip_matmul_nf4_dq_meta(x, qweight, bias, absmax_q, nested_absmax, nested_quant_map, nested_offset, quant_map, blocksize,
                           nested_blocksize, dtype, shape):
    _check_matmul_shapes(x, shape)
    return TensorProxy(like=x, shape=(*x.shape[:-1], shape[0]))


def hip_matmul_nf4_dq_impl(x, qweight, bias, absmax_q, nested_absmax, nested_quant_map, nested_offset, quant_map, blocksize,
                           nested_blocksize, dtype, shape):
    return functional.matmul_nf4_dq(x, qweight, bias, absmax_q, nested_absmax, nested_quant_map, nested_offset, quant_map,
                                    blocksize, nested_blocksize, dtype, shape)


def _norm_parts(rows: int, shape) -> int:
    """Partial sums of squares per row of x that the residual epilogue leaves for this shape on the current device (the
    band or tile count of the serving kernel's launch plan, asked of the library); 1 where the kernels do not serve the
    case and the operator computes the step itself."""
    from .. import _lib

    parts = _lib.load().nf4hip_gemv_norm_parts(rows, int(shape[0]), int(shape[1])) if 0 < rows <= 16 else 0
    return parts if parts > 0 else 1


def hip_matmul_nf4_epilogue_meta(x, qweight, bias, absmax, quant_map, blocksize, dtype, shape, rowscale=None, silu_pairs=False,
                                 resid_norm=None):
    _check_matmul_shapes(x, shape)
    n = shape[0] // 2 if silu_pairs else shape[0]
    out = TensorProxy(like=x, shape=(*x.shape[:-1], n))
    if resid_norm is None:
        return out
    rows = _numel(x.shape[:-1])
    return out, TensorProxy(like=x, shape=(*x.shape[:-1], n)), _plain(x, (rows, _norm_parts(rows, shape)), torch.float32)


def hip_matmul_nf4_epilogue_impl(x, qweight, bias, absmax, quant_map, blocksize, dtype, shape, rowscale=None, silu_pairs=False,
                                 resid_norm=None):
    """``hip_matmul_nf4`` with the decoder layer's neighbouring step done in the kernel's epilogue
    (``functional.matmul_nf4_epilogue``).  Where the kernels do not serve the case (more than sixteen rows of x, nested
    absmax, a shape outside their rules) the operator runs ``hip_matmul_nf4`` and the step by itself, with the same
    roundings of stored tensors, so that it always returns what its meta function describes."""
    got = functional.matmul_nf4_epilogue(x, qweight, bias, absmax, quant_map, blocksize, dtype, shape, rowscale=rowscale,
                                         silu_pairs=silu_pairs, resid_norm=resid_norm)
    if got is not None:
        return got
    N, K = (int(v) for v in shape)
    if rowscale is not None:
        sumsq, eps = rowscale
        rstd = torch.rsqrt(sumsq.float().sum(-1, keepdim=True) / K + eps)
        sums = functional.matmul_nf4(x, qweight, None, absmax, quant_map, blocksize, dtype, shape).float() * rstd.reshape(*x.shape[:-1], 1)
        if bias is not None:
            sums = sums + bias.float()
        y = sums.to(x.dtype)
    else:
        y = functional.matmul_nf4(x, qweight, bias, absmax, quant_map, blocksize, dtype, shape)
    if silu_pairs:
        gate, up = y[..., 0::2].float(), y[..., 1::2].float()
        return (torch.nn.functional.silu(gate).to(x.dtype).float() * up).to(x.dtype)
    if resid_norm is not None:
        resid, norm_weight = resid_norm
        r = (resid.float() + y.float()).to(x.dtype)
        xnext = (r.float() * norm_weight.float()).to(x.dtype)
        return r, xnext, r.float().pow(2).sum(-1, keepdim=True).reshape(-1, 1)
    return y


def hip_quantize_nf4_impl(w, blocksize=64):
    return functional.quantize_nf4(w, blocksize)


def hip_dequantize_nf4_impl(qweight, absmax, quant_map, blocksize, dtype, shape):
    return functional.dequantize_nf4(qweight, absmax, quant_map, blocksize, dtype, shape)


def _plain(like, shape, dtype) -> TensorProxy:
    return TensorProxy(like=like, shape=tuple(shape), dtype=dtype, requires_grad=False)


def _quantize_meta(w, blocksize=64):
    n = _numel(w.shape)
    return (_plain(w, ((n + 1) // 2, 1), torch.uint8), _plain(w, (-(-n // blocksize),), torch.float32), _plain(w, (16,), torch.float32))


def _dequantize_meta(qweight, absmax, quant_map, blocksize, dtype, shape):
    return _plain(qweight, shape, dtype)


def _quantize_dq_meta(w, blocksize=64, nested_blocksize=256):
    n = _numel(w.shape)
    nblocks = -(-n // blocksize)
    return (_plain(w, ((n + 1) // 2, 1), torch.uint8), _plain(w, (nblocks,), torch.uint8),
            _plain(w, (-(-nblocks // nested_blocksize),), torch.float32), _plain(w, (256,), torch.float32),
            _plain(w, (1,), torch.float32), _plain(w, (16,), torch.float32))


def _dequantize_dq_meta(qweight, absmax_q, nested_absmax, nested_quant_map, nested_offset, quant_map, blocksize, nested_blocksize,
                        dtype, shape):
    return _plain(qweight, shape, dtype)


def get_hip_nf4_executor() -> extend.OperatorExecutor:
    """The singleton executor ``quant_hip_nf4`` with its operators registered; idempotent
    (thunder/transforms/quantization.py:19-44).  Loading the HIP library is part of it: a missing
    or mismatching ``libnf4hip.so`` fails here, not at the first forward."""
    global hip_nf4_executor, hip_matmul_nf4, hip_quantize_nf4, hip_dequantize_nf4
    global hip_matmul_nf4_dq, hip_quantize_nf4_dq, hip_dequantize_nf4_dq, hip_matmul_nf4_epilogue
    if hip_nf4_executor is None:
        from .. import _lib

        _lib.load()
        ex = extend.OperatorExecutor("quant_hip_nf4", version=0.1)
        hip_matmul_nf4 = ex.register_operator("hip_matmul_nf4", meta=hip_matmul_nf4_meta, fn=hip_matmul_nf4_impl)
        hip_matmul_nf4_epilogue = ex.register_operator("hip_matmul_nf4_epilogue", meta=hip_matmul_nf4_epilogue_meta,
                                                       fn=hip_matmul_nf4_epilogue_impl)
        hip_quantize_nf4 = ex.register_operator("hip_quantize_nf4", meta=_quantize_meta, fn=hip_quantize_nf4_impl)
        hip_dequantize_nf4 = ex.register_operator("hip_dequantize_nf4", meta=_dequantize_meta, fn=hip_dequantize_nf4_impl)
        hip_matmul_nf4_dq = ex.register_operator("hip_matmul_nf4_dq", meta=hip_matmul_nf4_dq_meta, fn=hip_matmul_nf4_dq_impl)
        hip_quantize_nf4_dq = ex.register_operator("hip_quantize_nf4_dq", meta=_quantize_dq_meta,
                                                   fn=lambda w, blocksize=64, nested_blocksize=256: functional.quantize_nf4_dq(w, blocksize, nested_blocksize))
        hip_dequantize_nf4_dq = ex.register_operator("hip_dequantize_nf4_dq", meta=_dequantize_dq_meta,
                                                     fn=lambda *a: functional.dequantize_nf4_dq(*a))
        extend.register_executor(ex)
        hip_nf4_executor = ex
    return hip_nf4_executor


# the reference's spelling, so that code written against it keeps working
get_bitsandbytes_executor = get_hip_nf4_executor


# ---- the transform -------------------------------------------------------------------------------------

# What a quantised weight brings along besides the packed tensor, as suffixes of the weight's name, in the order
# in which the entries are installed, appear in state dicts and are appended to the computation's inputs.
_PLAIN_EXTRAS = ("absmax", "code")
_NESTED_EXTRAS = ("absmax", "code", "nested_absmax", "nested_quant_map", "nested_offset")


class BitsAndBytesLinearQuant4bit(Transform):
    """Quantise the weight of every ``nn.Linear`` to NF4 and route its matmul to the HIP operator.

    ``BitsAndBytesLinearQuant4bit()`` behaves like the reference (blocksize 64, fp32 absmax).
    ``lut_rounding="dtype"`` stores the code book pre-rounded to the weight dtype, which reproduces
    bitsandbytes' eager (non-CUDA) dequantisation instead of its CUDA kernel's.  ``double_quant=True`` stores the
    absmax statistics in 8 bits (nested blocks of ``nested_blocksize``) next to an fp32 offset.
    """

    def __init__(self, *, blocksize: int = 64, lut_rounding: str = "none", double_quant: bool = False, nested_blocksize: int = 256):
        assert lut_rounding in ("none", "dtype")
        self.quant_states: dict[str, dict] = {}
        self.quantized_submodule_names: set[str] = set()
        self.blocksize = blocksize
        self.lut_rounding = lut_rounding
        self.double_quant = bool(double_quant)
        self.nested_blocksize = nested_blocksize
        get_hip_nf4_executor()

    @property
    def _extras(self) -> tuple[str, ...]:
        return _NESTED_EXTRAS if self.double_quant else _PLAIN_EXTRAS

    # ---- quantising one weight ---------------------------------------------------------------------
    @staticmethod
    def _on_work_device(w: torch.Tensor) -> torch.Tensor:
        """Device policy of the reference (quantization.py:53-63): a meta weight stands for zeros on the GPU,
        a weight anywhere else is copied to the GPU, a GPU weight is used where it is."""
        work = torch.device(WORK_DEVICE)
        if w.device.type == "meta":
            return torch.zeros_like(w, device=work)
        if w.device.type == work.type:
            return w.detach()
        with torch.no_grad():
            return w.to(work).detach()

    def _quantized_tensors(self, w: torch.Tensor) -> dict[str, torch.Tensor]:
        """suffix -> tensor for one weight: ``""`` is the packed weight, the others are this transform's extras."""
        src = self._on_work_device(w)
        if self.double_quant:
            qw, absmax_q, nested_absmax, nested_map, nested_offset, code = hip_quantize_nf4_dq(src, self.blocksize, self.nested_blocksize)
            out = {"": qw, "absmax": absmax_q, "code": code, "nested_absmax": nested_absmax, "nested_quant_map": nested_map,
                   "nested_offset": nested_offset}
        else:
            qw, absmax, code = hip_quantize_nf4(src, self.blocksize)
            out = {"": qw, "absmax": absmax, "code": code}
        if self.lut_rounding == "dtype":
            out["code"] = out["code"].to(w.dtype).to(torch.float32)
        return out

    def quantize_weight(self, w: torch.Tensor):
        """``(qweight, absmax, code)`` of ``w`` like the reference's method of the same name; with ``double_quant``
        ``absmax`` is a :class:`functional.NestedAbsmax`."""
        t = self._quantized_tensors(w)
        if not self.double_quant:
            return t[""], t["absmax"], t["code"]
        nested = functional.nested_state(t["absmax"], t["nested_absmax"], t["nested_quant_map"], t["nested_offset"], self.nested_blocksize)
        return t[""], nested, t["code"]

    def _state_record(self, w: torch.Tensor, tensors: dict[str, torch.Tensor]) -> dict:
        qw = tensors[""]
        record = {"dtype": w.dtype, "shape": tuple(w.shape), "blocksize": self.blocksize,
                  "qweight.dtype": qw.dtype, "qweight.shape": tuple(qw.shape)}
        for suffix in self._extras:
            record[f"{suffix}.dtype"] = tensors[suffix].dtype
            record[f"{suffix}.shape"] = tuple(tensors[suffix].shape)
        record["device"] = getattr(w, "_thunder_device", w.device)
        if self.double_quant:
            record["nested_blocksize"] = self.nested_blocksize
        return record

    # ---- hooks --------------------------------------------------------------------------------------
    def transform_module(self, model) -> None:
        """Quantise every ``nn.Linear`` weight of the wrapped module, in ``named_modules()`` order, into the
        wrapper's parameter overrides.  Tied weights are quantised once and keep sharing their tensors."""
        self.thunder_module = model
        table = model._overrides_parameters
        tied = model._get_shared_names()
        for module_name, submodule in model._model.named_modules():
            if not isinstance(submodule, torch.nn.Linear):
                continue
            self.quantized_submodule_names.add(module_name)
            weight_name = f"{module_name}.weight" if module_name else "weight"
            twin = next((other for other in sorted(tied[weight_name]) if other != weight_name and other in self.quant_states), None)
            if twin is not None:
                self.quant_states[weight_name] = self.quant_states[twin]
                for suffix in ("", *self._extras):
                    dot = "." if suffix else ""
                    table[f"{weight_name}{dot}{suffix}"] = table[f"{twin}{dot}{suffix}"]
                continue
            w = model.get_parameter(weight_name)
            tensors = self._quantized_tensors(w)
            table[weight_name] = tensors[""].to(w.device)
            for suffix in self._extras:
                table[f"{weight_name}.{suffix}"] = tensors[suffix].to(w.device)
            self.quant_states[weight_name] = self._state_record(w, tensors)

    def transform_state_dict_for_submodule(self, model, submodule_name: str, state_dict: dict) -> dict:
        """An incoming ORIGINAL weight of a quantised submodule is replaced by its packed form plus extras; keys
        carry no submodule prefix (quantization.py:108-126)."""
        if submodule_name not in self.quantized_submodule_names:
            return state_dict
        record = self.quant_states[f"{submodule_name}.weight" if submodule_name else "weight"]
        w = state_dict["weight"]
        assert w.dtype == record["dtype"], f"{submodule_name}.weight: dtype {w.dtype}, quantised as {record['dtype']}"
        assert tuple(w.shape) == tuple(record["shape"]), f"{submodule_name}.weight: shape {tuple(w.shape)}, quantised as {record['shape']}"
        tensors = self._quantized_tensors(w)
        out = dict(state_dict)
        out["weight"] = tensors[""].to(w.device)
        for suffix in self._extras:
            out[f"weight.{suffix}"] = tensors[suffix].to(w.device)
        return out

    def reverse_transform_state_dict_for_submodule(self, model, submodule_name: str, state_dict: dict) -> dict:
        """Dequantise back to the original dtype and shape.  (The reference has no reverse; its
        ``original_state_dict()`` of a quantised module returns the packed tensors.)"""
        if submodule_name not in self.quantized_submodule_names or "weight.absmax" not in state_dict:
            return state_dict
        record = self.quant_states[f"{submodule_name}.weight" if submodule_name else "weight"]
        extra_keys = {f"weight.{suffix}" for suffix in self._extras}
        out = {k: v for k, v in state_dict.items() if k not in extra_keys}
        home = state_dict["weight"].device
        on_gpu = {k: state_dict[k].to(WORK_DEVICE) for k in ("weight", *sorted(extra_keys))}
        if self.double_quant:
            w = hip_dequantize_nf4_dq(on_gpu["weight"], on_gpu["weight.absmax"], on_gpu["weight.nested_absmax"],
                                      on_gpu["weight.nested_quant_map"], on_gpu["weight.nested_offset"], on_gpu["weight.code"],
                                      record["blocksize"], record["nested_blocksize"], record["dtype"], record["shape"])
        else:
            w = hip_dequantize_nf4(on_gpu["weight"], on_gpu["weight.absmax"], on_gpu["weight.code"], record["blocksize"],
                                   record["dtype"], record["shape"])
        out["weight"] = w.to(home)
        return out

    # ---- the plan of a call -------------------------------------------------------------------------
    def _operator_call(self, bsym, record: dict, extras: dict[str, TensorProxy]):
        """``linear(x, w, b)`` on a quantised weight as a call of this executor's operator."""
        x, w, b = bsym.args
        if self.double_quant:
            args = (x, w, b, extras["absmax"], extras["nested_absmax"], extras["nested_quant_map"], extras["nested_offset"],
                    extras["code"], record["blocksize"], record["nested_blocksize"], record["dtype"], record["shape"])
            return bsym.from_bsym(sym=hip_matmul_nf4_dq, subsymbols=(), args=args)
        args = (x, w, b, extras["absmax"], extras["code"], record["blocksize"], record["dtype"], record["shape"])
        return bsym.from_bsym(sym=hip_matmul_nf4, subsymbols=(), args=args)

    def transform_traces_pre_prologue(self, prologue_trace, computation_trace, epilogue_trace, **kwargs):
        """Rewrite the plan of a call (what quantization.py:128-293 does to Thunder's traces):

        * the prologue's check of every quantised weight expects the packed tensor (uint8, ``[n/2, 1]``, no grad);
        * the weight's extras are fetched and checked in the prologue too, become prologue outputs and -- tagged as
          static memory -- inputs of the computation, after the existing ones;
        * every ``linear`` on a quantised weight becomes ``hip_matmul_nf4(x, qweight, bias, absmax, code, blocksize,
          dtype, shape)`` (or its ``_dq`` form); nothing else in the computation changes."""
        model = self.thunder_module
        packed_meta = {}
        for name, (check, unpack) in get_checks(prologue_trace).items():
            if name in self.quant_states:
                record = self.quant_states[name]
                packed_meta[unpack.output.name] = {"shape": record["qweight.shape"], "dtype": record["qweight.dtype"]}
        prologue_trace = trace_with_replaced_proxy_metadata(prologue_trace, packed_meta)
        checks = get_checks(prologue_trace)
        returned = {proxy.name for proxy in prologue_trace.output[0]}

        weight_of_proxy: dict[str, str] = {}           # proxy of a packed weight -> parameter name
        extras_of: dict[str, dict[str, TensorProxy]] = {}  # parameter name -> suffix -> proxy
        fetches, new_inputs = [], []
        for name, record in self.quant_states.items():
            for suffix in ("", *self._extras):
                model.get_parameter(f"{name}.{suffix}" if suffix else name)  # the overrides must be in place
            check, unpack = checks[name]
            weight_proxy, _, device, _, _ = check.args
            check.args = (weight_proxy, record["qweight.shape"], device, record["qweight.dtype"], False)
            weight_proxy.requires_grad = False
            weight_of_proxy[unpack.output.name] = name
            if unpack.output.name not in returned:
                continue  # the computation never sees this weight
            owner = unpack.args[0]
            extras_of[name] = {}
            for suffix in self._extras:
                shape, dtype = record[f"{suffix}.shape"], record[f"{suffix}.dtype"]
                proxy = TensorProxy(f"{unpack.output.name}_{suffix}", shape=shape, dtype=dtype, device=device, requires_grad=False,
                                    tags={STATIC_MEMORY_LOCATION})
                fetches.append(unpack.sym.bind(owner, f"{name}.{suffix}", output=proxy))
                fetches.append(check_tensor_shape_and_metadata.bind(proxy, shape, device, dtype, False, output=None))
                add_trace_output(prologue_trace, proxy, subindex=0)
                extras_of[name][suffix] = proxy
                new_inputs.append(proxy)
        at_return = len(prologue_trace.bound_symbols) - 1
        prologue_trace.bound_symbols[at_return:at_return] = fetches

        computation_trace.args = (*computation_trace.args, *new_inputs)
        computation_trace.names |= {p.name for p in new_inputs}
        body = computation_trace.bound_symbols
        after_unpacks = max((i + 1 for i, b in enumerate(body) if b.sym is unpack_trivial), default=0)
        body[after_unpacks:after_unpacks] = [unpack_trivial.bind(p, output=p, name=p.name) for p in new_inputs]

        rewritten = []
        for bsym in body:
            weight = bsym.args[1] if bsym.sym is extend.linear and len(bsym.args) > 1 else None
            if isinstance(weight, TensorProxy) and weight.name in weight_of_proxy:
                assert len(bsym.args) == 3, "linear(input, weight, bias)"
                name = weight_of_proxy[weight.name]
                rewritten.append(self._operator_call(bsym, self.quant_states[name], extras_of[name]))
            elif bsym.sym is python_return:
                returned_dict = dict(bsym.args[0])
                returned_dict["flat_args"] = list(computation_trace.args)
                rewritten.append(bsym.from_bsym(args=(returned_dict,)))
            else:
                rewritten.append(bsym)
        computation_trace.bound_symbols = rewritten
        computation_trace.set_provenance("quant pass")
        return prologue_trace, computation_trace, epilogue_trace
