"""Executor / operator registration, mirroring the part of ``thunder.extend`` that the 4-bit path
sits behind (thunder/extend/__init__.py:53-198, 260-281, 459-651).

Only what the NF4 path needs is modelled: an executor owns named operator *symbols*; a symbol has
a ``meta`` function (shape/dtype inference on proxies) and an implementation ``fn``; binding a
symbol to arguments yields a *bound symbol* that carries ``fn`` in its call context, which is how
the generated computation reaches the kernel.  There is no tracing compiler behind it.
"""

from __future__ import annotations

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
    """An executor owns operator symbols and knows which foreign symbols it can run
    (interface of thunder/extend/__init__.py:53-198).  Two executors are the same executor when their
    names are equal: they hash and compare by name."""

    def __init__(self, name: Hashable, *, version: Any = None):
        self._name, self._version = name, version
        self._implmap: dict[Hashable, ImplInfo] = {}
        self._lookasides: dict[Callable, Symbol] = {}
        self._opmap: dict[str, Symbol] = {}

    @property
    def name(self) -> Hashable:
        return self._name

    @property
    def version(self) -> Any:
        return self._version

    @property
    def implmap(self) -> dict:
        return self._implmap

    @property
    def opmap(self) -> dict:
        return self._opmap

    def __repr__(self) -> str:
        return f"{type(self).__module__}.{type(self).__name__}('{self._name}')"

    def __hash__(self) -> int:
        return hash(self._name)

    def __eq__(self, other) -> bool:
        return isinstance(other, Executor) and self._name == other._name

    # ---- which bound symbols this executor takes --------------------------------------------------
    def _accepting_impl(self, bsym: BoundSymbol) -> ImplInfo | None:
        """The registered implementation for the bound symbol's id whose checker accepts its arguments."""
        info = self._implmap.get(bsym.sym.id)
        if info is None:
            return None
        if info.checker is not None and not info.checker(*bsym.args, **bsym.kwargs):
            return None
        return info

    def can_execute(self, bsym: BoundSymbol) -> bool:
        return self._accepting_impl(bsym) is not None

    def can_fuse(self, bsym: BoundSymbol) -> bool:
        if self.can_execute(bsym):
            return True
        subs = bsym.subsymbols
        return bool(subs) and all(self.can_fuse(sub) for sub in subs)

    def can_execute_or_fuse(self, bsym: BoundSymbol) -> bool:
        return self.can_fuse(bsym)  # can_fuse already covers direct execution

    def get_execution_transform(self, bsym: BoundSymbol):
        info = self._accepting_impl(bsym)
        return info.execution_transform if info is not None else None

    def get_grad_transform(self, sym: Symbol):
        info = self._implmap.get(sym.id)
        return info.grad_transform if info is not None else None

    # ---- operators ---------------------------------------------------------------------------------
    def register_operator(self, name: str, *, like: Symbol | None = None, meta: Callable | None = None, tags=None,
                          module=None, fn: Callable | None = None, bind_postprocess: Callable | None = None,
                          replaces=None) -> Symbol:
        """Create the symbol ``name`` owned by this executor (thunder/extend/__init__.py:146-198).

        Give either ``meta`` (the symbol is a primitive with that shape/dtype inference) or ``like`` (it
        borrows the inference, and by default the tags, of an existing symbol).  ``fn`` is the
        implementation: every bound symbol carries ``{name: fn}`` as its call context.  ``replaces`` names
        callables this symbol stands in for (look-asides)."""
        given = [k for k, v in (("like", like), ("meta", meta)) if v is not None]
        assert len(given) == 1, (
            f"register_operator({name!r}): pass exactly one of `like` and `meta` -- "
            f"{'neither was' if not given else 'both were'} given"
        )
        infer = meta if meta is not None else like
        if like is not None and tags is None:
            tags = getattr(like, "tags", None)
        ctx = {name: fn} if fn is not None else None

        def on_bind(bsym: BoundSymbol) -> None:
            bsym._call_ctx = ctx
            if bind_postprocess is not None:
                bind_postprocess(bsym)

        sym = Symbol(name, infer, id=name, is_prim=meta is not None, executor=self, tags=tags, _bind_postprocess=on_bind,
                     _module=module)
        self._opmap[name] = sym
        if replaces is not None:
            for target in (replaces,) if callable(replaces) else tuple(replaces):
                self._lookasides[target] = sym
        return sym


class OperatorExecutor(Executor):
    """An executor that runs symbols one by one (thunder/extend/__init__.py:260-281)."""

    def register_implementation(self, sym_or_id, op: Symbol | None = None, *, checker=None, execution_transform=None,
                                grad_transform=None) -> None:
        """Claim a symbol (given as such or by id): run it with ``op``, or rewrite it with
        ``execution_transform``; ``checker(*args)`` may decline individual calls."""
        assert op is not None or execution_transform is not None, "register_implementation needs `op` or `execution_transform`"
        key = sym_or_id.id if isinstance(sym_or_id, Symbol) else sym_or_id
        self._implmap[key] = ImplInfo(op, checker, execution_transform, grad_transform)


# ------------------------------------------------------------------------------------------------
# registries (interface of thunder/extend/__init__.py:518-651)
# ------------------------------------------------------------------------------------------------


class _Registry:
    """All registered executors by name, plus the two ordered preference lists.  The most recently added
    default / always executor comes first."""

    def __init__(self):
        self.by_name: dict[Hashable, Executor] = {}
        self.defaults: list[Executor] = []
        self.always: list[Executor] = []

    @staticmethod
    def key(ex_or_name) -> Hashable:
        return ex_or_name.name if isinstance(ex_or_name, Executor) else ex_or_name

    def prepend(self, which: str, ex: Executor) -> list[Executor]:
        setattr(self, which, [ex, *getattr(self, which)])
        return getattr(self, which)

    def drop(self, which: str, ex_or_name) -> list[Executor]:
        k = self.key(ex_or_name)
        setattr(self, which, [e for e in getattr(self, which) if e.name != k])
        return getattr(self, which)


_registry = _Registry()


def register_executor(ex: Executor) -> Executor:
    _registry.by_name[ex.name] = ex
    return ex


def deregister_executor(ex) -> None:
    _registry.by_name.pop(_registry.key(ex), None)
    _registry.drop("always", ex)
    _registry.drop("defaults", ex)


def get_all_executors() -> tuple[Executor, ...]:
    return tuple(_registry.by_name.values())


def get_executor(name) -> Executor | None:
    return _registry.by_name.get(name)


def get_default_executors() -> tuple[Executor, ...]:
    return tuple(_registry.defaults)


def get_always_executors() -> tuple[Executor, ...]:
    return tuple(_registry.always)


def add_default_executor(ex: Executor) -> list[Executor]:
    return _registry.prepend("defaults", ex)


def add_always_executor(ex: Executor) -> list[Executor]:
    return _registry.prepend("always", ex)


def remove_default_executor(ex) -> list[Executor]:
    return _registry.drop("defaults", ex)


def remove_always_executor(ex) -> list[Executor]:
    return _registry.drop("always", ex)


def resolve_executors(executors: Sequence[Executor | str] | None) -> tuple[Executor, ...]:
    """``None`` -> the default executors; otherwise every entry is an :class:`Executor` (kept) or the name of a
    registered one (looked up).  Anything else, and any unknown name, is a ``ValueError``
    (thunder/extend/__init__.py:622-651)."""
    if executors is None:
        return get_default_executors()
    out: list[Executor] = []
    unknown: list[str] = []
    for entry in executors:
        if isinstance(entry, Executor):
            out.append(entry)
        elif isinstance(entry, str):
            found = get_executor(entry)
            (out if found is not None else unknown).append(found if found is not None else entry)
        else:
            raise ValueError(f"executors={executors!r}: {entry!r} ({type(entry).__name__}) is neither an Executor nor the name of one")
    if unknown:
        known = ", ".join(repr(e.name) for e in get_all_executors())
        raise ValueError(f"no executor registered under {', '.join(map(repr, unknown))}; registered: {known or 'none'}")
    return tuple(out)


def add_executor_lists(exc_list, other_exc_list) -> list[Executor]:
    """Concatenation of the two (resolved) lists without repeats, first occurrence wins."""
    merged: dict[Executor, None] = {}
    for ex in (*resolve_executors(exc_list), *resolve_executors(other_exc_list)):
        merged.setdefault(ex, None)
    return list(merged)


def single_op_executor(exc_name, op_name: str, fn: Callable, meta: Callable, *, version=None, replaces=None, tags=None,
                       checker=None, execution_transform=None, grad_transform=None) -> OperatorExecutor:
    """A registered executor holding one operator implemented by ``fn``, which it also claims for itself
    (thunder/extend/__init__.py:459-514)."""
    ex = register_executor(OperatorExecutor(exc_name, version=version))
    lookaside = fn if replaces is None else replaces
    sym = ex.register_operator(op_name, meta=meta, fn=fn, tags=tags, replaces=lookaside)
    ex.register_implementation(sym, op=sym, checker=checker, execution_transform=execution_transform, grad_transform=grad_transform)
    return ex
