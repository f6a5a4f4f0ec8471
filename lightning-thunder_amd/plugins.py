"""Plugins (thunder/core/recipe.py:30-45, thunder/plugins/__init__.py:7-25,
thunder/plugins/quantization.py:4-37): named bundles of transforms + executors for ``compile``."""

from __future__ import annotations

from enum import Enum, auto


class PluginPolicy(Enum):
    PRE = auto()
    POST = auto()


class Plugin:
    policy: PluginPolicy = PluginPolicy.PRE

    def setup_lookasides(self):
        return None

    def setup_transforms(self):
        return None

    def setup_executors(self):
        return None


class QuantizeInt4(Plugin):
    """4-bit (NF4) weight-only quantisation of every ``nn.Linear``."""

    def setup_transforms(self):
        from .transforms.quantization import BitsAndBytesLinearQuant4bit

        return [BitsAndBytesLinearQuant4bit()]

    def setup_executors(self):
        from .transforms.quantization import get_hip_nf4_executor

        return [get_hip_nf4_executor()]


class ReduceOverhead(Plugin):
    """Replay the forward pass from a HIP graph (cf. thunder/plugins/reduce_overhead.py:5-19,
    thunder/transforms/cudagraph.py)."""

    policy = PluginPolicy.POST

    def setup_transforms(self):
        from .graphs import HIPGraphTransform

        return [HIPGraphTransform()]


names_to_plugins: dict[str, type[Plugin]] = {
    "quantize-int4": QuantizeInt4,
    "reduce-overhead": ReduceOverhead,
}


def get_plugin(name: str):
    return names_to_plugins.get(name)


def get_plugin_names() -> list[str]:
    return list(names_to_plugins.keys())


def register_plugin(name: str, cls) -> None:
    names_to_plugins[name] = cls
