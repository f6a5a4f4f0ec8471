"""Executor / operator registration, mirroring the part of ``thunder.extend`` that the 4-bit path
sits behind (thunder/extend/__init__.py:53-198, 260-281, 459-651).

Only what the NF4 path needs is modelled: an executor owns named operator *symbols*; a symbol has
a ``meta`` function (shape/dtype inference on proxies) and an implementation ``fn``; binding a
symbol to arguments yields a *bound symbol* that carries ``fn`` in its call context, which is how
the generated computation reaches the kernel.  There is no tracing compiler behind it.
"""

from __future__ import annotations

import itertools
import os
from collections.abc import Callable, Hashable, Sequence
from dataclasses import dataclass, field
from typing import Any

import torch


# ------------------------------------------------------------------------------------------------
# proxies and symbols
# ------------------------------------------------------------------------------------------------


class TensorProxy:
    """Metadata stand-in for a tensor (cf. thunder/core/proxies.py:1442): what a ``meta`` function
    receives and returns.  ``TensorProxy(like=x, shape=...)`` copies everything else from ``x``."""

    __slots__ = ("name", "shape", "dtype", "device", "requires_grad", "tags")

    def __init__(self, name=None, *, like=None, shape=None, dtype=None, device=None, requires_grad=None, tags=None):
        if like is not None:
            shape = tuple(like.shape) if shape is None else shape
            dtype = like.dtype if dtype is None else dtype
            device = like.device if device is None else device
            requires_grad = bool(getattr(like, "requires_grad", False)) if requires_grad is None else requires_grad
        self.name = name
        self.shape = tuple(int(s) for s in shape)
        self.dtype = dtype
        self.device = torch.device(device) if device is not None else None
        self.requires_grad = bool(requires_grad)
        self.tags = set(tags or ())

    @property
    def ndim(self) -> int:
        return len(self.shape)

    def __repr__(self) -> str:
        return f"<TensorProxy(name={self.name!r}, dtype={self.dtype}, shape={self.shape}, device={self.device})>"


@dataclass(eq=False)
class BoundSymbol:
    """A symbol applied to arguments (cf. thunder/core/symbol.py:377)."""

    sym: "Symbol"
    args: tuple
    kwargs: dict = field(default_factory=dict)
    output: Any = None
    subsymbols: tuple = ()
    _call_ctx: dict | None = None

    def from_bsym(self, **changes) -> "BoundSymbol":
        new = BoundSymbol(self.sym, self.args, dict(self.kwargs), self.output, self.subsymbols, self._call_ctx)
        for k, v in changes.items():
            setattr(new, k, v)
        if "sym" in changes and changes["sym"]._bind_postprocess is not None:
            changes["sym"]._bind_postprocess(new)
        return new

    def __call__(self, *args, **kwargs):
        """Execute: the generated code of the reference calls ``fn`` by the symbol's name out of the
        call context (thunder/core/symbol.py:676-683)."""
        if not self._call_ctx or self.sym.name not in self._call_ctx:
            raise RuntimeError(f"symbol {self.sym.name} has no implementation in its call context")
        return self._call_ctx[self.sym.name](*args, **kwargs)

    def __repr__(self) -> str:
        def show(a):
            if isinstance(a, (TensorProxy, torch.Tensor)):
                return getattr(a, "name", None) or f"t{tuple(a.shape)}"
            return repr(a)

        return f"{self.sym.name}({', '.join(show(a) for a in self.args)})"


class Symbol:
    """A named operation (cf. thunder/core/symbol.py:120)."""

    def __init__(self, name, meta=None, *, id=None, is_prim=False, executor=None, tags=None, _bind_postprocess=None, _module=None):
        self.name = name
        self.id = name if id is None else id
        self.meta = meta
        self.is_prim = is_prim
        self.executor = executor
        self.tags = tags
        self._bind_postprocess = _bind_postprocess
        self._module = _module

    def bind(self, *args, output=None, subsymbols=(), **kwargs) -> BoundSymbol:
        b = BoundSymbol(self, tuple(args), dict(kwargs), output, tuple(subsymbols))
        if self._bind_postprocess is not None:
            self._bind_postprocess(b)
        return b

    def __call__(self, *args, **kwargs):
        """Calling a symbol on real tensors runs its implementation; on proxies its meta function."""
        leaves = list(args) + list(kwargs.values())
        if any(isinstance(a, TensorProxy) for a in leaves):
            return self.meta(*args, **kwargs)
        return self.bind(*args, **kwargs)(*args, **kwargs)

    def __repr__(self) -> str:
        return f"[Symbol name={self.name}]"


# The symbol the quantisation transform looks for (``thunder.torch.linear`` in the reference,
# thunder/torch/__init__.py:5801).
def _linear_meta(a, w, bias=None):
    return TensorProxy(like=a, shape=(*a.shape[:-1], w.shape[0]))


linear = Symbol("linear", _linear_meta, id="torch.nn.functional.linear")
linear._bind_postprocess = lambda b: setattr(b, "_call_ctx", {"linear": torch.nn.functional.linear})


# ------------------------------------------------------------------------------------------------
# executors
# ------------------------------------------------------------------------------------------------


class ImplInfo:
    """What an executor knows about a symbol it can run (thunder/extend/__init__.py:33-50)."""

    def __init__(self, symbol=None, checker=None, execution_transform=None, grad_transform=None):
        self.symbol = symbol
        self.checker = checker  # None: always executable
        self.execution_transform = execution_transform  # None: called as is
        self.grad_transform = grad_transform


class Executor:
    """thunder/extend/__init__.py:53-198.  Executors hash and compare by name."""

    def __init__(self, name: Hashable, *, version: Any = None):
        self._name = name
        self._version = version
        self._implmap: dict[Hashable, ImplInfo] = {}
        self._lookasides: dict[Callable, Symbol] = {}
        self._opmap: dict[str, Symbol] = {}

    name = property(lambda self: self._name)
    version = property(lambda self: self._version)
    implmap = property(lambda self: self._implmap)
    opmap = property(lambda self: self._opmap)

    def __repr__(self) -> str:
        return f"{self.__class__.__module__}.{self.__class__.__name__}('{self.name}')"

    def __hash__(self) -> int:
        return hash(self.name)

    def __eq__(self, other) -> bool:
        return isinstance(other, Executor) and other.name == self.name

    def can_execute(self, bsym: BoundSymbol) -> bool:
        impl = self.implmap.get(bsym.sym.id)
        if impl is None:
            return False
        return True if impl.checker is None else bool(impl.checker(*bsym.args, **bsym.kwargs))

    def can_fuse(self, bsym: BoundSymbol) -> bool:
        if self.can_execute(bsym):
            return True
        return len(bsym.subsymbols) > 0 and all(self.can_fuse(s) for s in bsym.subsymbols)

    def can_execute_or_fuse(self, bsym: BoundSymbol) -> bool:
        return self.can_execute(bsym) or self.can_fuse(bsym)

    def get_execution_transform(self, bsym: BoundSymbol):
        impl = self.implmap.get(bsym.sym.id)
        if impl is None or not (impl.checker is None or impl.checker(*bsym.args, **bsym.kwargs)):
            return None
        return impl.execution_transform

    def get_grad_transform(self, sym: Symbol):
        impl = self.implmap.get(sym.id)
        return None if impl is None else impl.grad_transform

    def register_operator(self, name: str, *, like: Symbol | None = None, meta: Callable | None = None, tags=None,
                          module=None, fn: Callable | None = None, bind_postprocess: Callable | None = None,
                          replaces=None) -> Symbol:
        """Create a symbol owned by this executor.  Exactly one of ``like`` / ``meta``; ``fn`` becomes
        the call context of every bound symbol; ``replaces`` registers look-asides
        (thunder/extend/__init__.py:146-198)."""
        ln, mn = like is None, meta is None
        assert ln ^ mn, (
            f"Expected one and only one of 'like' and 'meta' to be specified. {'Neither' if ln and mn else 'Both'} were specified."
        )
        is_prim = meta is not None
        if tags is None and like is not None:
            tags = getattr(like, "tags", None)
        meta = meta if meta is not None else like
        call_ctx = None if fn is None else {name: fn}

        def _bind_postprocess(bsym: BoundSymbol) -> None:
            bsym._call_ctx = call_ctx
            if bind_postprocess is not None:
                bind_postprocess(bsym)

        sym = Symbol(name, meta, id=name, is_prim=is_prim, executor=self, tags=tags,
                     _bind_postprocess=_bind_postprocess, _module=module)
        self.opmap[name] = sym
        if callable(replaces):
            replaces = (replaces,)
        self._lookasides.update({r: sym for r in replaces or ()})
        return sym


class OperatorExecutor(Executor):
    """thunder/extend/__init__.py:260-281."""

    def register_implementation(self, sym_or_id, op: Symbol | None = None, *, checker=None, execution_transform=None,
                                grad_transform=None) -> None:
        if execution_transform is None:
            assert op is not None
        _id = sym_or_id.id if isinstance(sym_or_id, Symbol) else sym_or_id
        self.implmap[_id] = ImplInfo(op, checker, execution_transform, grad_transform)


# ------------------------------------------------------------------------------------------------
# registries (thunder/extend/__init__.py:518-651)
# ------------------------------------------------------------------------------------------------

_executor_map: dict[Hashable, Executor] = {}
_default_executors: list[Executor] = []
_always_executors: list[Executor] = []


def register_executor(ex: Executor) -> Executor:
    _executor_map[ex.name] = ex
    return ex


def deregister_executor(ex) -> None:
    _id = ex.name if isinstance(ex, Executor) else ex
    _executor_map.pop(_id, None)
    remove_always_executor(_id)
    remove_default_executor(_id)


def get_all_executors() -> tuple[Executor, ...]:
    return tuple(_executor_map.values())


def get_executor(name) -> Executor | None:
    return _executor_map.get(name)


def get_default_executors() -> tuple[Executor, ...]:
    return tuple(_default_executors)


def get_always_executors() -> tuple[Executor, ...]:
    return tuple(_always_executors)


def add_default_executor(ex: Executor) -> list[Executor]:
    global _default_executors
    _default_executors = [ex] + _default_executors
    return _default_executors


def add_always_executor(ex: Executor) -> list[Executor]:
    global _always_executors
    _always_executors = [ex] + _always_executors
    return _always_executors


def remove_default_executor(ex) -> list[Executor]:
    global _default_executors
    _id = ex.name if isinstance(ex, Executor) else ex
    _default_executors = [x for x in _default_executors if x.name != _id]
    return _default_executors


def remove_always_executor(ex) -> list[Executor]:
    global _always_executors
    _id = ex.name if isinstance(ex, Executor) else ex
    _always_executors = [x for x in _always_executors if x.name != _id]
    return _always_executors


def resolve_executors(executors: Sequence[Executor | str] | None) -> tuple[Executor, ...]:
    """Instances pass through, names are looked up; ``None`` means the defaults.  Unknown names and
    foreign objects raise ``ValueError`` (thunder/extend/__init__.py:622-651)."""
    if executors is None:
        return get_default_executors()
    failed: list[str] = []
    resolved: list[Executor] = []
    for e in executors:
        if isinstance(e, str):
            ex = get_executor(e)
            if ex is None:
                failed.append(e)
            else:
                resolved.append(ex)
        elif not isinstance(e, Executor):
            raise ValueError(f"An object of type {type(e)} is not a valid Executor. Executor list: {executors}")
        else:
            resolved.append(e)
    if failed:
        raise ValueError(
            f"Expected an Executor or the name of a registered Executor, instead got: {failed[0] if len(failed) == 1 else failed}"
            + os.linesep + f"Registered executors: {get_all_executors()}"
        )
    return tuple(resolved)


def add_executor_lists(exc_list, other_exc_list) -> list[Executor]:
    out: list[Executor] = []
    for exc in itertools.chain(resolve_executors(exc_list), resolve_executors(other_exc_list)):
        if exc not in out:
            out.append(exc)
    return out


def single_op_executor(exc_name, op_name: str, fn: Callable, meta: Callable, *, version=None, replaces=None, tags=None,
                       checker=None, execution_transform=None, grad_transform=None) -> OperatorExecutor:
    """One executor with one operator implemented by ``fn`` (thunder/extend/__init__.py:459-514)."""
    exc = OperatorExecutor(exc_name, version=version)
    register_executor(exc)
    sym = exc.register_operator(op_name, fn=fn, replaces=fn if replaces is None else replaces, meta=meta, tags=tags)
    exc.register_implementation(sym, op=sym, checker=checker, execution_transform=execution_transform,
                                grad_transform=grad_transform)
    return exc
