"""MI355X-native NF4 weight-only quantized linear path (hand-written HIP for gfx950) behind the
interface of Thunder's ``BitsAndBytesLinearQuant4bit`` transform and its executor operator.

The directory name contains a hyphen, so import it with
``importlib.import_module("lightning-thunder_amd")``.
"""

from . import _lib, functional  # noqa: F401
from .functional import (  # noqa: F401
    NestedAbsmax,
    compress_absmax,
    dequantize_nf4,
    dynamic_map,
    matmul_nf4,
    nf4_code,
    quantize_nf4,
    reconstruct_absmax,
)
