"""The ``Transform`` hook interface (thunder/core/transform_common.py:397-445)."""

from __future__ import annotations

from abc import ABC
from typing import Any


class Transform(ABC):
    """Hooks are called at fixed points: ``transform_module`` once when the transform is applied
    (thunder/__init__.py:914-916), ``transform_traces_pre_prologue`` when a call has to be
    (re)planned (thunder/__init__.py:507-527), ``transform_state_dict_for_submodule`` while an
    original state dict is streamed in (thunder/core/module.py:149-150)."""

    def transform_traces_pre_prologue(self, prologue_trace, computation_trace, epilogue_trace, **kwargs):
        return prologue_trace, computation_trace, epilogue_trace

    def transform_module(self, model) -> None:
        pass

    def transform_state_dict_for_submodule(self, model, submodule_name: str, state_dict: dict[str, Any]) -> dict[str, Any]:
        return state_dict

    def transform_trace_post_optimization(self, computation_trace, **kwargs):
        return computation_trace

    def reverse_transform_state_dict_for_submodule(self, model, submodule_name: str, state_dict: dict[str, Any]) -> dict[str, Any]:
        return state_dict

    def __repr__(self) -> str:
        return f"{self.__class__.__module__}.{self.__class__.__name__}()"
