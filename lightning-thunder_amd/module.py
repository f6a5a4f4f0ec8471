"""``ThunderModule``: what ``jit`` returns for an ``nn.Module`` (interface of thunder/core/module.py:30-404).

The user's module is never modified.  The wrapper holds two *override tables* -- one for parameters, one
for buffers, keyed by dotted name -- and everything that reads the module's tensors (lookups, iteration,
state dicts, the forward pass) consults the tables before the wrapped module.  Transforms put their
results there: the packed NF4 weight under the Linear weight's own name, its statistics under
``<weight>.absmax`` / ``<weight>.code`` (names with no counterpart in the wrapped module).

The forward pass runs a structure-sharing *shadow* of the wrapped module: a shallow copy of every
submodule whose ``_parameters`` / ``_buffers`` point at the tables' tensors.
"""

from __future__ import annotations

import collections
import copy
from collections.abc import Iterable, Mapping
from typing import Any

import torch


def _split_by_submodule(state_dict: Mapping[str, Any], module_names: set[str]) -> dict[str, dict[str, Any]]:
    """Group the entries of a flat state dict by owning submodule.  The owner of ``"a.b.weight.absmax"`` is
    the longest dotted prefix that names a module (``"a.b"``, entry ``"weight.absmax"``); the root module is
    ``""``.  Groups keep the order in which their first key appears (thunder/core/module.py:19-27)."""
    groups: dict[str, dict[str, Any]] = {}
    for key, value in state_dict.items():
        parts = key.split(".")
        for cut in range(len(parts) - 1, -1, -1):
            owner = ".".join(parts[:cut])
            if owner in module_names:
                groups.setdefault(owner, {})[".".join(parts[cut:])] = value
                break
        else:
            raise KeyError(f"state dict entry {key!r} belongs to no submodule")
    return groups


class _Overrides(dict):
    """An override table that counts how often an entry was (re)bound, so the forward path can tell when
    its shadow module and prologue checks are stale.  Writing INTO an entry (``copy_``) does not count."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.version = 0

    def __setitem__(self, k, v):
        self.version += 1
        super().__setitem__(k, v)

    def __delitem__(self, k):
        self.version += 1
        super().__delitem__(k)

    def update(self, *args, **kwargs):
        self.version += 1
        super().update(*args, **kwargs)

    def pop(self, *args):
        self.version += 1
        return super().pop(*args)


class ThunderModule(torch.nn.Module):
    def __init__(self, model: torch.nn.Module, compiled_model_call):
        super().__init__()
        self._model = model
        del self.training  # answered by the wrapped module (see __getattr__)
        self._forward_fn = compiled_model_call
        self._overrides_parameters = _Overrides(model.named_parameters())
        self._overrides_buffers = _Overrides(model.named_buffers())
        self._submodules = dict(model.named_modules())
        self._lc_transforms: list = []

    def forward(self, *args, **kwargs):
        return self._forward_fn(*args, **kwargs)

    def __getattr__(self, name: str) -> Any:
        """Attributes this wrapper does not have are the wrapped module's."""
        try:
            return super().__getattr__(name)
        except AttributeError:
            wrapped = self.__dict__.get("_modules", {}).get("_model")
            if wrapped is None:
                raise
            return getattr(wrapped, name)

    # ---- lookups: the tables first, then the wrapped module ---------------------------------------
    def get_parameter(self, name: str):
        table = self._overrides_parameters
        return table[name] if name in table else self._model.get_parameter(name)

    def get_buffer(self, name: str):
        table = self._overrides_buffers
        return table[name] if name in table else self._model.get_buffer(name)

    def set_buffer(self, name: str, value) -> None:
        self._overrides_buffers[name] = value

    def get_submodule(self, name: str):
        known = self._submodules
        return known[name] if name in known else self._model.get_submodule(name)

    # ---- iteration --------------------------------------------------------------------------------
    @staticmethod
    def _merge(table: Mapping[str, Any], wrapped: Iterable[tuple[str, Any]], prefix: str, recurse: bool, remove_duplicate: bool):
        """Table entries in insertion order, then the wrapped module's entries under names the table
        does not have.  With ``remove_duplicate`` a tensor object is reported once, under its first name.
        ``recurse=False`` keeps the root module's own entries (names without a dot)."""
        named: dict[str, Any] = dict(table)
        for name, tensor in wrapped:
            named.setdefault(name, tensor)
        reported: set[int] = set()
        for name, tensor in named.items():
            if not recurse and "." in name:
                continue
            if remove_duplicate:
                if id(tensor) in reported:
                    continue
                reported.add(id(tensor))
            yield (f"{prefix}.{name}" if prefix else name), tensor

    def named_parameters(self, prefix: str = "", recurse: bool = True, remove_duplicate: bool = True):
        wrapped = self._model.named_parameters(remove_duplicate=remove_duplicate)
        yield from self._merge(self._overrides_parameters, wrapped, prefix, recurse, remove_duplicate)

    def named_buffers(self, prefix: str = "", recurse: bool = True, remove_duplicate: bool = True, *, persistent=None):
        wrapped = self._model.named_buffers(remove_duplicate=remove_duplicate)
        entries = self._merge(self._overrides_buffers, wrapped, prefix, recurse, remove_duplicate)
        if persistent is None:
            yield from entries
            return
        transient = self._non_persistent_buffers(prefix)
        for name, tensor in entries:
            if (name not in transient) == bool(persistent):
                yield name, tensor

    def _get_shared_names(self) -> dict[str, set[str]]:
        """For every parameter / buffer name the set of all names bound to the same tensor object (tied weights
        give sets of more than one), thunder/core/module.py:125-135."""
        group_of: dict[int, set[str]] = {}
        keep_alive = []  # ids are only unique among live objects
        for name, tensor in (*self.named_parameters(remove_duplicate=False), *self.named_buffers(remove_duplicate=False)):
            keep_alive.append(tensor)
            group_of.setdefault(id(tensor), set()).add(name)
        return {name: group for group in group_of.values() for name in group}

    def _non_persistent_buffers(self, prefix: str = "") -> set[str]:
        names: set[str] = set()
        for mod_name, sub in self._model.named_modules(prefix=prefix):
            head = f"{mod_name}." if mod_name else ""
            names |= {head + b for b in sub._non_persistent_buffers_set}
        return names

    # ---- loading ----------------------------------------------------------------------------------
    def _table_holding(self, full_name: str) -> _Overrides:
        for table in (self._overrides_parameters, self._overrides_buffers):
            if full_name in table:
                return table
        raise NotImplementedError(f"{full_name!r} is neither a parameter nor a buffer of the transformed module")

    def load_original_state_dict(self, state_dict: Mapping[str, Any]) -> None:
        """Load a state dict of the UNtransformed model: it is cut up by submodule, every part goes through
        each transform's ``transform_state_dict_for_submodule`` (bf16 weights are quantised as they arrive) and
        is then installed (thunder/core/module.py:137-145)."""
        groups = self._get_shared_names()
        done: set[str] = set()
        for submodule_name, part in _split_by_submodule(state_dict, set(self._submodules)).items():
            self._transform_and_load_for_submodule(submodule_name, part, groups, done)

    def _transform_and_load_for_submodule(self, submodule_name: str, sd_part: dict, shared_names: dict, processed_names: set) -> None:
        """One submodule's entries (keys without the submodule prefix): transform, then install.  A name tied to
        one that was installed earlier in the same load receives that tensor instead of a copy of its own."""
        for transform in self._lc_transforms:
            sd_part = transform.transform_state_dict_for_submodule(self, submodule_name, sd_part)
        head = f"{submodule_name}." if submodule_name else ""
        for key, incoming in sd_part.items():
            name = head + key
            table = self._table_holding(name)
            tied_and_loaded = (shared_names.get(name, set()) - {name}) & processed_names
            if tied_and_loaded:
                table[name] = self._table_holding(min(tied_and_loaded))[min(tied_and_loaded)]
            else:
                self._install(table, name, incoming)
            processed_names.add(name)

    @staticmethod
    def _install(table: _Overrides, name: str, incoming: torch.Tensor) -> None:
        """Copy into the current tensor where dtype and shape agree (its identity, and with it every plan
        made so far, survives); otherwise rebind the entry to the incoming tensor moved to the old device."""
        current = table[name]
        with torch.no_grad():
            if current.dtype == incoming.dtype and current.shape == incoming.shape:
                current.copy_(incoming)
                return
            moved = incoming.to(current.device)
            differentiable = moved.is_floating_point() or moved.is_complex()
            if isinstance(current, torch.nn.Parameter) and differentiable:
                moved = torch.nn.Parameter(moved, requires_grad=current.requires_grad)
            elif differentiable and not isinstance(current, torch.nn.Parameter):
                moved = moved.to(current.dtype).requires_grad_(current.requires_grad)
            table[name] = moved  # e.g. packed uint8 codes taking the place of a bf16 weight: a plain tensor

    def load_state_dict(self, state_dict: Mapping[str, Any], strict: bool = True, assign: bool = False):
        """Load a state dict of the TRANSFORMED module -- the keys :meth:`state_dict` writes
        (thunder/core/module.py:267-338).  ``assign`` rebinds the tables to the given tensors instead of copying."""
        transient = self._non_persistent_buffers()
        expected = {n: t for n, t in (*self.named_parameters(), *self.named_buffers()) if n not in transient}
        missing = [n for n in expected if n not in state_dict]
        unexpected = [k for k in state_dict if k not in expected]
        problems: list[str] = []
        accepted: list[tuple[str, torch.Tensor, torch.Tensor]] = []
        for name, current in expected.items():
            if name not in state_dict:
                continue
            incoming = state_dict[name]
            if not torch.overrides.is_tensor_like(incoming):
                problems.append(f'"{name}": the checkpoint holds a {type(incoming).__name__}, not a tensor')
            elif incoming.shape != current.shape:
                problems.append(f'size mismatch for "{name}": {tuple(incoming.shape)} in the checkpoint, {tuple(current.shape)} in the module')
            else:
                accepted.append((name, current, incoming))
        with torch.no_grad():
            for name, current, incoming in accepted:
                if not assign:
                    current.copy_(incoming)
                    continue
                if isinstance(current, torch.nn.Parameter):
                    if isinstance(incoming, torch.nn.Parameter):
                        incoming.requires_grad_(current.requires_grad)
                    else:
                        incoming = torch.nn.Parameter(incoming, requires_grad=current.requires_grad)
                    self._overrides_parameters[name] = incoming
                else:  # a plain tensor: an override a transform installed, or a buffer
                    table = self._overrides_parameters if name in self._overrides_parameters else self._overrides_buffers
                    table[name] = incoming
        if strict:
            if unexpected:
                problems.insert(0, "unexpected keys: " + ", ".join(f'"{k}"' for k in unexpected))
            if missing:
                problems.insert(0, "Missing keys: " + ", ".join(f'"{k}"' for k in missing))
        if problems:
            raise RuntimeError("load_state_dict failed:\n  " + "\n  ".join(problems))
        return torch.nn.modules.module._IncompatibleKeys(missing, unexpected)

    # ---- saving -----------------------------------------------------------------------------------
    @staticmethod
    def _new_destination():
        destination = collections.OrderedDict()
        destination._metadata = collections.OrderedDict()
        return destination

    def state_dict(self, *, destination=None, prefix: str = "", keep_vars: bool = False):
        """State dict of the TRANSFORMED module: parameters (original order, packed tensors in place of quantised
        weights, then the entries transforms added, in the order they added them), then persistent buffers."""
        destination = self._new_destination() if destination is None else destination
        transient = self._non_persistent_buffers(prefix)
        entries = [*self.named_parameters(prefix=prefix), *((n, b) for n, b in self.named_buffers(prefix=prefix) if n not in transient)]
        for name, tensor in entries:
            if tensor is not None:
                destination[name] = tensor if keep_vars else tensor.detach()
        return destination

    def original_state_dict(self, *, destination=None, prefix: str = "", keep_vars: bool = False):
        """State dict with the transforms undone, last transform first (thunder/core/module.py:230-265)."""
        destination = self._new_destination() if destination is None else destination
        for submodule_name, part in _split_by_submodule(self.state_dict(keep_vars=keep_vars), set(self._submodules)).items():
            for transform in reversed(self._lc_transforms):
                part = transform.reverse_transform_state_dict_for_submodule(self, submodule_name, part)
            head = prefix + (f"{submodule_name}." if submodule_name else "")
            for key, value in part.items():
                destination[head + key] = value
        return destination

    # ---- the shadow module the forward pass runs --------------------------------------------------
    def _build_shadow(self, weight_wrappers: dict[str, Any]) -> torch.nn.Module:
        """A copy of the module TREE (not of any tensor): every submodule is shallow-copied and given
        fresh ``_parameters`` / ``_buffers`` / ``_modules`` dicts that point at the overrides.
        ``weight_wrappers[name]`` replaces the override of ``name`` (used for packed NF4 weights)."""

        def clone(mod: torch.nn.Module, prefix: str) -> torch.nn.Module:
            new = copy.copy(mod)
            new._parameters = {k: self._shadow_value(f"{prefix}{k}", v, weight_wrappers, self._overrides_parameters)
                               for k, v in mod._parameters.items()}
            new._buffers = {k: self._shadow_value(f"{prefix}{k}", v, {}, self._overrides_buffers)
                            for k, v in mod._buffers.items()}
            new._modules = {k: (None if c is None else clone(c, f"{prefix}{k}.")) for k, c in mod._modules.items()}
            return new

        return clone(self._model, "")

    @staticmethod
    def _shadow_value(full_name, original, wrappers, overrides):
        if full_name in wrappers:
            return wrappers[full_name]
        return overrides[full_name] if full_name in overrides else original
