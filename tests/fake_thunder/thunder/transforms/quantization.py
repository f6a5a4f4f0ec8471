"""Stand-in for thunder.transforms.quantization: a transform class whose trace hook records which symbol the
module global ``bnb_matmul_nf4`` names while the hook runs (the real hook builds its bound symbol from that
global, thunder/transforms/quantization.py:262-266)."""


class BitsAndBytesLinearQuant4bit:
    def __init__(self):
        raise ImportError("bitsandbytes is not installed")  # the real __init__ imports it; the adapter must not get here

    def transform_traces_pre_prologue(self, prologue_trace, computation_trace, epilogue_trace, **kwargs):
        bound = globals().get("bnb_matmul_nf4")
        if kwargs.get("fail"):
            raise RuntimeError("trace rewrite failed")
        return prologue_trace, (computation_trace, bound), epilogue_trace
