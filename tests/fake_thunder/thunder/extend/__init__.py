"""Executor registry of the stand-in `thunder` package (see thunder/__init__.py next to this folder)."""

_executors = {}


class Symbol:
    def __init__(self, name, meta, fn, executor):
        self.name, self.meta, self.fn, self.executor = name, meta, fn, executor

    def __call__(self, *args):
        return self.fn(*args)


class OperatorExecutor:
    def __init__(self, name, version=None):
        self.name, self.version, self.opmap = name, version, {}

    def register_operator(self, name, *, meta, fn):
        sym = Symbol(name, meta, fn, self)
        self.opmap[name] = sym
        return sym


def get_executor(name):
    return _executors.get(name)


def register_executor(ex):
    _executors[ex.name] = ex
    return ex
