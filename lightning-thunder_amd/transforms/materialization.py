"""``MaterializationTransform``: give a meta-device model real storage AFTER the other transforms
have run, so that e.g. bf16 weights never exist on the device, only their NF4 form
(thunder/transforms/materialization.py:15-172)."""

from __future__ import annotations

import copy
from collections.abc import Callable
from itertools import chain

import torch

from ..transform_common import Transform


def module_init_from_original_module_init(transform: "MaterializationTransform", tm, *, non_persistent_only: bool = False):
    """Initialise materialised tensors with the wrapped module's own ``reset_parameters``, one
    submodule at a time, and push the result through the other transforms (so a freshly
    initialised Linear weight is quantised right away)."""
    if non_persistent_only:
        non_persistent = tm._non_persistent_buffers()

        def skip(n):
            return n not in non_persistent
    else:

        def skip(n):
            return False

    shared_names = tm._get_shared_names()
    processed: set[str] = set()
    for module_name, _ in tm._model.named_modules():
        submodule = tm.get_submodule(module_name)
        own = list(chain(submodule.named_parameters(recurse=False, prefix=module_name),
                         submodule.named_buffers(recurse=False, prefix=module_name)))
        if not any((n in transform.have_materialized) and not skip(n) for n, _ in own):
            continue
        module_copy = copy.copy(submodule)  # leave the user's module alone
        module_copy._parameters = module_copy._parameters.copy()
        module_copy._buffers = module_copy._buffers.copy()
        module_copy._modules = module_copy._modules.__class__()
        need_init = not all((shared_names[n] & processed) or skip(n) for n, _ in own)
        if need_init:
            module_copy.to_empty(device=transform.device, recurse=False)
            if not hasattr(module_copy, "reset_parameters"):
                raise TypeError(
                    f"Materialization requires that the `{type(submodule).__name__}.reset_parameters` method is implemented."
                    " This method is used to initialize any children parameters or buffers in this module."
                )
            module_copy.reset_parameters()
        sd = {n: p for n, p in chain(module_copy.named_parameters(recurse=False), module_copy.named_buffers(recurse=False))}
        tm._transform_and_load_for_submodule(module_name, sd, shared_names, processed)


class MaterializationTransform(Transform):
    """``MaterializationTransform(device, init=...)`` with ``init`` one of
    ``init_from_original_state_dict(sd)``, ``init_from_transformed_state_dict(sd)``,
    ``init_from_original_module_init()``."""

    def __init__(self, device, *, init: Callable) -> None:
        self.device = torch.device(device)
        self.init = init

    def transform_module(self, model) -> None:
        for p in chain(model._model.parameters(), model._model.buffers()):
            if p.device.type == "meta" and not hasattr(p, "_thunder_device"):
                p._thunder_device = self.device
        shared_names = model._get_shared_names()
        self.have_materialized: set[str] = set()
        for n, p in list(model.named_parameters()):
            if p.device.type == "meta":
                new = torch.empty_like(p, device=getattr(p, "_thunder_device", self.device))
                if isinstance(p, torch.nn.Parameter):
                    new = torch.nn.Parameter(new, requires_grad=p.requires_grad)
                for n2 in shared_names[n]:
                    model._overrides_parameters[n2] = new
                    self.have_materialized.add(n2)
        for n, b in list(model.named_buffers()):
            if b.device.type == "meta":
                new = torch.empty_like(b, device=getattr(b, "_thunder_device", self.device), requires_grad=b.requires_grad)
                for n2 in shared_names[n]:
                    model._overrides_buffers[n2] = new
                    self.have_materialized.add(n2)
        self.init(self, model)

    @staticmethod
    def init_from_original_state_dict(state_dict):
        def init(transform, model):
            module_init_from_original_module_init(transform, model, non_persistent_only=True)
            model.load_original_state_dict(state_dict)

        return init

    @staticmethod
    def init_from_transformed_state_dict(state_dict):
        def init(transform, model):
            module_init_from_original_module_init(transform, model, non_persistent_only=True)
            model.load_state_dict(state_dict)

        return init

    @staticmethod
    def init_from_original_module_init():
        return module_init_from_original_module_init
