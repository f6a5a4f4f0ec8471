"""MI355X-native NF4 weight-only quantized linear path (hand-written HIP for gfx950) behind the
interface of Thunder's ``BitsAndBytesLinearQuant4bit`` transform and its executor operator.

The directory name contains a hyphen, so import it with
``importlib.import_module("lightning-thunder_amd")``.
"""

from . import _lib, extend, functional, plugins, trace, transforms  # noqa: F401
from .api import (  # noqa: F401
    cache_hits,
    cache_misses,
    compile,
    compile_data,
    compile_stats,
    jit,
    last_prologue_traces,
    last_traces,
)
from .extend import TensorProxy  # noqa: F401
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
from .module import ThunderModule  # noqa: F401
from .plugins import Plugin, PluginPolicy, QuantizeInt4, get_plugin, get_plugin_names, register_plugin  # noqa: F401
from .transform_common import Transform  # noqa: F401
from .transforms import BitsAndBytesLinearQuant4bit, MaterializationTransform, get_bitsandbytes_executor, get_hip_nf4_executor  # noqa: F401
