"""``jit`` / ``compile`` for ``nn.Module``s (thunder/__init__.py:274-327, 881-919).

What is reproduced is the CONTRACT the 4-bit path relies on, not a compiler:

* ``jit(model, transforms=[...], executors=[...])`` wraps the module in a :class:`ThunderModule`
  and calls every transform's ``transform_module`` in order;
* the first call (and any call after the parameter overrides were rebound) plans the forward pass:
  initial prologue/computation traces -> every transform's ``transform_traces_pre_prologue`` ->
  dispatch, where a bound symbol that already belongs to an executor is kept as is
  (thunder/executors/passes.py:80-83) and ``linear`` falls to PyTorch;
* each call runs the prologue (fetch every parameter, check shape/dtype/device/requires_grad; an
  ``AssertionError`` means re-plan, thunder/__init__.py:725-728) and then the computation: the wrapped
  module's own ``forward`` over the overridden parameters, with every planned ``linear`` on a
  quantised weight executed by the operator's ``fn``.
"""

from __future__ import annotations

from collections.abc import Sequence
from typing import Any

import torch

from . import extend
from .module import ThunderModule
from .plugins import Plugin, PluginPolicy, get_plugin
from .trace import (
    TensorProxy,
    build_initial_traces,
    check_tensor,
    check_tensor_shape_and_metadata,
    unpack_buffer,
    unpack_parameter,
)


class CompileStats:
    """Counters and the last traces (thunder/common.py:65-173)."""

    def __init__(self):
        self.calls = 0
        self.cache_hits = 0
        self.cache_misses = 0
        self.last_traces: list = []
        self.last_prologue_traces: list = []


class CompileData:
    def __init__(self, fn, executors_list, transforms, compile_options):
        self.fn = fn
        self.executors_list = executors_list
        self.transforms = transforms
        self.compile_options = compile_options
        self.is_module = isinstance(fn, torch.nn.Module)


class _QuantWeight(torch.Tensor):
    """The packed weight as the shadow module sees it.  ``F.linear(x, <this>, b)`` -- whoever calls
    it, ``nn.Linear.forward`` or user code -- is routed to the planned operator; any other use
    sees the plain uint8 tensor."""

    @staticmethod
    def __new__(cls, packed: torch.Tensor, call, operator=None):
        t = packed.detach().as_subclass(cls)
        t._planned_call = call
        # (operator name, packed weight, the operator's arguments after bias): for callers that run a variant of the
        # planned operator on this weight (the decode step's linears with an epilogue)
        t._planned_operator = operator
        return t

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        if func is torch.nn.functional.linear:
            x = args[0] if args else kwargs["input"]
            w = args[1] if len(args) > 1 else kwargs["weight"]
            b = args[2] if len(args) > 2 else kwargs.get("bias")
            if isinstance(w, _QuantWeight) and not isinstance(x, _QuantWeight):
                return w._planned_call(x, b)
        with torch._C.DisableTorchFunctionSubclass():
            return func(*args, **kwargs)


class _Plan:
    """One cache entry: transformed traces, the prologue as a list of runtime checks, and the
    shadow module that executes the computation."""

    def __init__(self):
        self.prologue_trace = None
        self.computation_trace = None
        self.epilogue_trace = None
        self.checks: list[tuple[str, bool, tuple]] = []  # (name, is_buffer, (shape, device, dtype, requires_grad))
        self.shadow: torch.nn.Module | None = None
        self.call = None  # what a forward call runs: the shadow module, possibly behind a graph runner
        self.versions = (-1, -1)


def _plan_call(tm: ThunderModule, cd: CompileData, cs: CompileStats) -> _Plan:
    plan = _Plan()
    pro, comp, epi = build_initial_traces(tm)
    cs.last_prologue_traces = [pro]
    cs.last_traces = [comp]
    for t in cd.transforms:
        pro, comp, epi = t.transform_traces_pre_prologue(pro, comp, epi, executors_list=cd.executors_list)
    # dispatch (thunder/executors/passes.py:32-104): operator-executor symbols are kept, `linear`
    # is claimed by PyTorch, everything else in these traces is bookkeeping
    proxy_to_param: dict[str, tuple[str, bool]] = {}
    for b in pro.bound_symbols:
        if b.sym in (unpack_parameter, unpack_buffer):
            proxy_to_param[b.output.name] = (b.args[1], b.sym is unpack_buffer)
    for b in pro.bound_symbols:
        if b.sym is check_tensor_shape_and_metadata:
            name, is_buffer = proxy_to_param[b.args[0].name]
            plan.checks.append((name, is_buffer, tuple(b.args[1:])))

    wrappers: dict[str, Any] = {}
    for b in comp.bound_symbols:
        if b.sym.executor is None:
            continue  # linear / prims: executed by the module's own forward under PyTorch
        # an operator call planned for a weight: args = (x, w, bias, *rest)
        w_proxy = b.args[1]
        w_name, _ = proxy_to_param[w_proxy.name]

        def resolve(a):
            if isinstance(a, TensorProxy):
                pname, is_buffer = proxy_to_param[a.name]
                return tm.get_buffer(pname) if is_buffer else tm.get_parameter(pname)
            return a

        packed = resolve(w_proxy)
        rest = tuple(resolve(a) for a in b.args[3:])

        def call(x, bias, _b=b, _packed=packed, _rest=rest):
            return _b(x, _packed, bias, *_rest)

        wrappers[w_name] = _QuantWeight(packed, call, (b.sym.name, packed, rest))
    for t in cd.transforms:
        comp = t.transform_trace_post_optimization(comp, executors_list=cd.executors_list)
    plan.prologue_trace, plan.computation_trace, plan.epilogue_trace = pro, comp, epi
    cs.last_prologue_traces.append(pro)
    cs.last_traces.append(comp)
    plan.shadow = tm._build_shadow(wrappers)
    plan.call = plan.shadow
    for t in cd.transforms:
        if hasattr(t, "wrap_callable"):
            plan.call = t.wrap_callable(plan.call)
    plan.versions = (tm._overrides_parameters.version, tm._overrides_buffers.version)
    return plan


def _run_prologue(tm: ThunderModule, plan: _Plan) -> None:
    for name, is_buffer, (shape, device, dtype, requires_grad) in plan.checks:
        t = tm.get_buffer(name) if is_buffer else tm.get_parameter(name)
        check_tensor(t, shape, device, dtype, requires_grad)


def jit(fn, /, *, langctx=None, executors: Sequence | None = None, sharp_edges=None, cache=None,
        disable_torch_autograd: bool = False, transforms: list | None = None, debug_options=None, **compile_options):
    """Wrap ``fn`` (an ``nn.Module``) so that the given transforms and executors apply
    (signature of thunder.jit, thunder/__init__.py:315-327).

    ``check_prologue="always"`` re-validates every parameter on every call like the reference does;
    the default ``"on_change"`` validates when a plan is made and whenever an override is rebound.
    """
    if not isinstance(fn, torch.nn.Module):
        raise NotImplementedError("this build wraps nn.Modules only: the 4-bit path is a module transform")
    transforms = list(transforms) if transforms is not None else []
    executors_list = extend.resolve_executors(executors)
    check_mode = compile_options.get("check_prologue", "on_change")
    assert check_mode in ("always", "on_change")
    cd = CompileData(fn, executors_list, transforms, compile_options)
    cs = CompileStats()
    state: dict[str, Any] = {"plan": None}

    def fn_(*args, **kwargs):
        cs.calls += 1
        tm: ThunderModule = state["tm"]
        plan: _Plan | None = state["plan"]
        versions = (tm._overrides_parameters.version, tm._overrides_buffers.version)
        if plan is not None and plan.versions == versions:
            if check_mode == "always":
                try:
                    _run_prologue(tm, plan)
                except AssertionError:
                    plan = None
        else:
            plan = None
        if plan is None:
            cs.cache_misses += 1
            plan = _plan_call(tm, cd, cs)
            _run_prologue(tm, plan)  # a failure here is a real error: the transforms disagree with the module
            state["plan"] = plan
        else:
            cs.cache_hits += 1
        if kwargs or plan.call is plan.shadow:
            return plan.shadow(*args, **kwargs)
        return plan.call(*args)

    tm = ThunderModule(fn, fn_)
    tm._lc_cd = cd
    tm._lc_cs = cs
    tm._lc_transforms = transforms
    state["tm"] = tm
    for t in transforms:
        t.transform_module(tm)
    return tm


def compile(fn, recipe=None, plugins=None, *, transforms: list | None = None, executors: Sequence | None = None):
    """``compile(model, plugins="quantize-int4")`` (thunder/__init__.py:274-311 with the plugin
    handling of thunder/core/recipe.py:115-183).  ``transforms=`` / ``executors=`` are accepted as a
    convenience and are applied after the plugins' own."""
    if recipe not in (None, "auto"):
        raise NotImplementedError("recipes other than the default are outside this build")
    if plugins is None:
        plugins = []
    elif not isinstance(plugins, (list, tuple)):
        plugins = [plugins]
    resolved: list[Plugin] = []
    for p in plugins:
        if isinstance(p, str):
            cls = get_plugin(p)
            if cls is None:
                raise ValueError(f"Plugin {p} not recognized")
            resolved.append(cls())
        elif isinstance(p, Plugin):
            resolved.append(p)
        else:
            raise ValueError(f"expected a Plugin or a plugin name, got {type(p)}")
    all_transforms, all_executors = [], []
    for policy in (PluginPolicy.PRE, PluginPolicy.POST):
        for p in resolved:
            if p.policy is policy:
                all_transforms += p.setup_transforms() or []
                all_executors += p.setup_executors() or []
    all_transforms += list(transforms or [])
    all_executors += list(executors or [])
    return jit(fn, transforms=all_transforms, executors=all_executors)


def compile_data(fn) -> CompileData | None:
    return getattr(fn, "_lc_cd", None)


def compile_stats(fn) -> CompileStats | None:
    return getattr(fn, "_lc_cs", None)


def last_traces(fn) -> list:
    cs = compile_stats(fn)
    if cs is None:
        raise TypeError(f"{fn} doesn't seem to be a thunder compiled function.")
    if not cs.last_traces:
        raise TypeError(f"{fn} doesn't seem to have been called yet.")
    return cs.last_traces


def last_prologue_traces(fn) -> list:
    cs = compile_stats(fn)
    if cs is None:
        raise TypeError(f"{fn} doesn't seem to be a thunder compiled function.")
    if not cs.last_prologue_traces:
        raise TypeError(f"{fn} doesn't seem to have been called yet.")
    return cs.last_prologue_traces


def cache_hits(fn) -> int:
    return compile_stats(fn).cache_hits


def cache_misses(fn) -> int:
    return compile_stats(fn).cache_misses
