from .materialization import MaterializationTransform  # noqa: F401
from .quantization import BitsAndBytesLinearQuant4bit, get_bitsandbytes_executor, get_hip_nf4_executor  # noqa: F401
