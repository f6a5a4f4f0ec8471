"""``MaterializationTransform``: give a meta-device model real storage AFTER the other transforms have
run, so that e.g. bf16 weights never exist on the device -- only their NF4 form does
(interface of thunder/transforms/materialization.py:15-172).

Order of events in ``transform_module``:

1. every meta parameter / buffer of the wrapped module is tagged with the device it will live on
   (``_thunder_device``, which earlier transforms and the planner read instead of ``.device``);
2. every override that is still a meta tensor is replaced by uninitialised storage on that device -- tied
   names keep sharing one tensor -- and its names are remembered in ``have_materialized``;
3. the ``init`` strategy fills the storage: from a state dict of the original model, from a state dict of the
   transformed model, or by running each submodule's own ``reset_parameters``.
"""

from __future__ import annotations

import copy
from collections.abc import Callable

import torch

from ..transform_common import Transform


class MaterializationTransform(Transform):
    """``MaterializationTransform(device, init=...)`` with ``init`` one of
    ``init_from_original_state_dict(sd)``, ``init_from_transformed_state_dict(sd)``,
    ``init_from_original_module_init()``."""

    def __init__(self, device, *, init: Callable) -> None:
        self.device = torch.device(device)
        self.init = init
        self.have_materialized: set[str] = set()

    # ---- step 1 and 2 -------------------------------------------------------------------------------
    def _target_device(self, t: torch.Tensor) -> torch.device:
        return getattr(t, "_thunder_device", self.device)

    def _materialize_table(self, table, entries, groups) -> None:
        for name, meta_tensor in entries:
            if meta_tensor.device.type != "meta" or name in self.have_materialized:
                continue
            storage = torch.empty_like(meta_tensor, device=self._target_device(meta_tensor), requires_grad=meta_tensor.requires_grad)
            if isinstance(meta_tensor, torch.nn.Parameter):
                storage = torch.nn.Parameter(storage, requires_grad=meta_tensor.requires_grad)
            for tied in groups[name]:
                table[tied] = storage
            self.have_materialized |= groups[name]

    def transform_module(self, model) -> None:
        wrapped = model._model
        for t in (*wrapped.parameters(), *wrapped.buffers()):
            if t.device.type == "meta" and not hasattr(t, "_thunder_device"):
                t._thunder_device = self.device
        groups = model._get_shared_names()
        self.have_materialized = set()
        self._materialize_table(model._overrides_parameters, list(model.named_parameters()), groups)
        self._materialize_table(model._overrides_buffers, list(model.named_buffers()), groups)
        self.init(self, model)

    # ---- step 3 -------------------------------------------------------------------------------------
    def _run_module_inits(self, model, *, only_non_persistent: bool) -> None:
        """Fill materialised tensors with what the owning submodule's ``reset_parameters`` produces, and send
        the result through the other transforms (a freshly initialised Linear weight is quantised at once).
        With ``only_non_persistent`` just the buffers that no state dict carries are of interest."""
        transient = model._non_persistent_buffers() if only_non_persistent else None

        def wanted(name: str) -> bool:
            return name in self.have_materialized and (transient is None or name in transient)

        groups = model._get_shared_names()
        done: set[str] = set()
        for module_name in [n for n, _ in model._model.named_modules()]:
            submodule = model.get_submodule(module_name)
            own = [n for n, _ in (*submodule.named_parameters(recurse=False, prefix=module_name),
                                  *submodule.named_buffers(recurse=False, prefix=module_name))]
            pending = [n for n in own if wanted(n)]
            if not pending:
                continue
            # a private, childless stand-in for the submodule: the user's module keeps its meta tensors
            stand_in = copy.copy(submodule)
            stand_in._parameters = dict(submodule._parameters)
            stand_in._buffers = dict(submodule._buffers)
            stand_in._modules = type(submodule._modules)()
            # nothing to compute if every wanted tensor is tied to one that an earlier submodule initialised
            if any(not (groups[n] & done) for n in pending):
                init_fn = getattr(stand_in, "reset_parameters", None)
                if init_fn is None:
                    raise TypeError(f"cannot materialise {module_name or 'the root module'!r}: "
                                    f"{type(submodule).__name__} has no reset_parameters() to initialise its tensors with")
                stand_in.to_empty(device=self.device, recurse=False)
                init_fn()
            fresh = dict(stand_in.named_parameters(recurse=False))
            fresh.update(stand_in.named_buffers(recurse=False))
            model._transform_and_load_for_submodule(module_name, fresh, groups, done)

    @staticmethod
    def init_from_original_state_dict(state_dict) -> Callable:
        """Weights come from a state dict of the ORIGINAL model (streamed through the other transforms);
        non-persistent buffers, which no state dict holds, from the modules' own init."""

        def init(transform: "MaterializationTransform", model) -> None:
            transform._run_module_inits(model, only_non_persistent=True)
            model.load_original_state_dict(state_dict)

        return init

    @staticmethod
    def init_from_transformed_state_dict(state_dict) -> Callable:
        """Weights come from a state dict of the TRANSFORMED model (e.g. packed NF4 tensors), loaded as is."""

        def init(transform: "MaterializationTransform", model) -> None:
            transform._run_module_inits(model, only_non_persistent=True)
            model.load_state_dict(state_dict)

        return init

    @staticmethod
    def init_from_original_module_init() -> Callable:
        """Every materialised tensor is initialised by its submodule's ``reset_parameters``."""

        def init(transform: "MaterializationTransform", model) -> None:
            transform._run_module_inits(model, only_non_persistent=False)

        return init
