"""A small symbolic model of the prologue / computation traces that Thunder hands to
``Transform.transform_traces_pre_prologue`` (thunder/__init__.py:507-527).

There is no program acquisition here: the traces are derived from the module tree.  The prologue
holds, per parameter/buffer, an ``unpack_parameter`` and a ``check_tensor_shape_and_metadata``
bound symbol (thunder/core/jit_ext.py:1746-1780, thunder/core/prims.py:499-515, 1061-1099); the
computation holds one ``linear(x, w, b)`` bound symbol per ``nn.Linear`` plus the return.  That is
exactly the surface the quantisation transform inspects and rewrites
(thunder/transforms/quantization.py:128-293), so the transform can be written the way the
reference writes it, and its *effect* -- which operator runs for which weight, with which
arguments -- is what the runtime executes.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import torch

from .extend import BoundSymbol, Symbol, TensorProxy, linear  # noqa: F401

STATIC_MEMORY_LOCATION = "STATIC_MEMORY_LOCATION"  # cf. ProxyTag.STATIC_MEMORY_LOCATION

# prims the prologue is made of
unpack_parameter = Symbol("unpack_parameter", None, id="prims.unpack_parameter", is_prim=True)
unpack_buffer = Symbol("unpack_buffer", None, id="prims.unpack_buffer", is_prim=True)
check_tensor_shape_and_metadata = Symbol("check_tensor_shape_and_metadata", None, id="prims.check_tensor_shape_and_metadata", is_prim=True)
unpack_trivial = Symbol("unpack_trivial", None, id="prims.unpack_trivial", is_prim=True)
python_return = Symbol("python_return", None, id="prims.python_return", is_prim=True)


def proxy_name(param_name: str) -> str:
    return "t_" + param_name.replace(".", "_")


@dataclass
class Trace:
    """Ordered bound symbols plus the signature (``args``) and, for the prologue, ``output``."""

    bound_symbols: list = field(default_factory=list)
    args: tuple = ()
    output: tuple = ()
    names: set = field(default_factory=set)
    provenance: str | None = None

    def set_provenance(self, p: str) -> None:
        self.provenance = p

    def __str__(self) -> str:
        head = f"# {self.provenance}\n" if self.provenance else ""
        sig = ", ".join(getattr(a, "name", str(a)) for a in self.args)
        body = "\n".join(f"  {b.output.name + ' = ' if isinstance(b.output, TensorProxy) else ''}{b!r}" for b in self.bound_symbols)
        return f"{head}def trace({sig}):\n{body}"


def check_tensor(t: torch.Tensor, shape, device, dtype, requires_grad) -> None:
    """Runtime form of ``check_tensor_shape_and_metadata`` (thunder/executors/pythonex.py:41-53):
    an ``AssertionError`` here means the cached plan no longer matches the module."""
    assert isinstance(t, torch.Tensor), f"expected a tensor, got {type(t)}"
    assert tuple(t.shape) == tuple(shape), f"shape {tuple(t.shape)} != {tuple(shape)}"
    assert t.dtype == dtype, f"dtype {t.dtype} != {dtype}"
    assert torch.device(device).type == t.device.type and (
        torch.device(device).index is None or t.device.index is None or torch.device(device).index == t.device.index
    ), f"device {t.device} != {device}"
    assert bool(t.requires_grad) == bool(requires_grad), f"requires_grad {t.requires_grad} != {requires_grad}"


def build_initial_traces(tmodule) -> tuple[Trace, Trace, Trace]:
    """What acquisition would produce for the wrapped module: it sees the ORIGINAL parameters
    (thunder/__init__.py:439-460 runs on ``model``, not on the overrides)."""
    model = tmodule._model
    pro, comp, epi = Trace(provenance="prologue"), Trace(provenance="computation"), Trace(provenance="epilogue")
    outs: list[TensorProxy] = []
    by_name: dict[str, TensorProxy] = {}

    def add(name: str, t: torch.Tensor, sym: Symbol) -> None:
        device = getattr(t, "_thunder_device", t.device)
        p = TensorProxy(proxy_name(name), shape=tuple(t.shape), dtype=t.dtype, device=device, requires_grad=t.requires_grad)
        mod_name, _, leaf = name.rpartition(".")
        pro.bound_symbols.append(sym.bind(mod_name, name, output=p))
        pro.bound_symbols.append(check_tensor_shape_and_metadata.bind(p, p.shape, p.device, p.dtype, p.requires_grad, output=None))
        outs.append(p)
        by_name[name] = p

    for name, t in model.named_parameters(remove_duplicate=False):
        add(name, t, unpack_parameter)
    for name, t in model.named_buffers(remove_duplicate=False):
        add(name, t, unpack_buffer)
    pro.output = (tuple(outs), ())
    pro.bound_symbols.append(python_return.bind(pro.output, output=None))

    comp.args = tuple(outs)
    comp.names = {p.name for p in outs}
    for p in outs:
        comp.bound_symbols.append(unpack_trivial.bind(p, output=p, name=p.name))
    for mod_name, sub in model.named_modules():
        if isinstance(sub, torch.nn.Linear):
            prefix = f"{mod_name}." if mod_name else ""
            w = by_name[f"{prefix}weight"]
            b = by_name.get(f"{prefix}bias") if sub.bias is not None else None
            x = TensorProxy(f"{proxy_name(mod_name or 'root')}_input", shape=(w.shape[1],), dtype=w.dtype, device=w.device)
            out = TensorProxy(f"{proxy_name(mod_name or 'root')}_output", shape=(w.shape[0],), dtype=w.dtype, device=w.device)
            comp.bound_symbols.append(linear.bind(x, w, b, output=out))
    comp.bound_symbols.append(python_return.bind({"output": None, "flat_args": list(comp.args)}, output=None))
    return pro, comp, epi


# ---- helpers of thunder/transforms/utils.py:8-76 ------------------------------------------------


def get_checks(prologue: Trace) -> dict[str, tuple[BoundSymbol, BoundSymbol]]:
    """parameter name -> (check bound symbol, unpack bound symbol); exactly one check per name."""
    unpack_by_proxy: dict[str, BoundSymbol] = {}
    for b in prologue.bound_symbols:
        if b.sym in (unpack_parameter, unpack_buffer):
            unpack_by_proxy[b.output.name] = b
    checks: dict[str, tuple[BoundSymbol, BoundSymbol]] = {}
    for b in prologue.bound_symbols:
        if b.sym is check_tensor_shape_and_metadata:
            u = unpack_by_proxy.get(b.args[0].name)
            if u is None:
                continue
            name = u.args[1]
            assert name not in checks, f"duplicate check for {name}"
            checks[name] = (b, u)
    return checks


def add_trace_output(trace: Trace, output: TensorProxy, subindex: int | None = None) -> None:
    if subindex is None:
        trace.output = (*trace.output, output)
    else:
        out = list(trace.output)
        out[subindex] = (*out[subindex], output)
        trace.output = tuple(out)
    ret = trace.bound_symbols[-1]
    assert ret.sym is python_return
    ret.args = (trace.output,)


def trace_with_replaced_proxy_metadata(trace: Trace, proxy_replacement_metadata: dict[str, dict]) -> Trace:
    """Copy of ``trace`` in which the named proxies carry new shape/dtype (every use is updated,
    because uses share the proxy object)."""
    for bsym in trace.bound_symbols:
        leaves = list(bsym.args) + ([bsym.output] if bsym.output is not None else [])
        for a in leaves:
            if isinstance(a, TensorProxy) and a.name in proxy_replacement_metadata:
                meta = proxy_replacement_metadata[a.name]
                a.shape = tuple(meta.get("shape", a.shape))
                a.dtype = meta.get("dtype", a.dtype)
    return trace
