"""A minimal stand-in for the `thunder` package, for the CPU test of thunder_adapter.install() only.

It models just the surface the adapter touches -- thunder.extend's executor registry with
register_operator / opmap, thunder.TensorProxy(like=, shape=), and a BitsAndBytesLinearQuant4bit whose
transform_traces_pre_prologue binds whatever the module global ``bnb_matmul_nf4`` names at call time
(thunder/transforms/quantization.py:262-266 builds its bound symbol from that global) -- and none of
Thunder's behaviour beyond that.  Written for this test; nothing here comes from the reference's sources.
"""

from . import extend  # noqa: F401


class TensorProxy:
    def __init__(self, like=None, shape=None):
        self.shape = tuple(shape if shape is not None else like.shape)
        self.dtype = getattr(like, "dtype", None)
        self.device = getattr(like, "device", None)
