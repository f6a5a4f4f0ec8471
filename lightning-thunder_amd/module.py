"""``ThunderModule``: the wrapper ``jit`` returns for an ``nn.Module`` (thunder/core/module.py:30-404).

It keeps the user's module untouched and holds *overrides* for parameters and buffers, which is
where transforms put the packed NF4 weights, their absmax and code tensors.  The forward pass runs
a structure-sharing shadow of the wrapped module whose parameters and buffers are the overrides.
"""

from __future__ import annotations

import collections
import copy
import itertools
from collections.abc import Mapping
from typing import Any

import torch
from torch.utils.weak import WeakTensorKeyDictionary


def _convert_state_dict_to_per_module(state_dict: dict[str, Any], module_names: set[str]) -> dict[str, dict[str, Any]]:
    """``"a.b.weight.absmax"`` belongs to module ``"a.b"`` with key ``"weight.absmax"``: strip name
    components from the right until the prefix names a module (thunder/core/module.py:19-27)."""
    per_module: dict[str, dict[str, Any]] = collections.defaultdict(dict)
    for k, v in state_dict.items():
        prefix, sep, _ = k.rpartition(".")
        while prefix not in module_names:
            prefix, sep, _ = prefix.rpartition(".")
        per_module[prefix][k[len(prefix) + len(sep):]] = v
    return per_module


class _Overrides(dict):
    """Override table that counts rebinding of entries, so the forward path can tell when its
    shadow module (and the prologue checks) are stale.  In-place ``copy_`` keeps entries valid."""

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
        del self.training  # served by the wrapped module through __getattr__
        self._forward_fn = compiled_model_call
        self._overrides_parameters = _Overrides(self._model.named_parameters())
        self._overrides_buffers = _Overrides(self._model.named_buffers())
        self._module_cache = {k: v for k, v in self._model.named_modules()}
        self._null = object()
        self._lc_transforms: list = []

    # ---- lookups --------------------------------------------------------------------------------
    def get_buffer(self, name):
        p = self._overrides_buffers.get(name, self._null)
        return p if p is not self._null else self._model.get_buffer(name)

    def set_buffer(self, name, value):
        self._overrides_buffers[name] = value

    def get_parameter(self, name):
        p = self._overrides_parameters.get(name, self._null)
        return p if p is not self._null else self._model.get_parameter(name)

    def get_submodule(self, name):
        p = self._module_cache.get(name, self._null)
        return p if p is not self._null else self._model.get_submodule(name)

    def forward(self, *args, **kwargs):
        return self._forward_fn(*args, **kwargs)

    def _named_parameters_or_buffers(self, overrides, orig_iter, prefix="", recurse=True, remove_duplicate=True):
        seen_ids, seen_names = set(), set()
        for k, v in itertools.chain(overrides.items(), orig_iter):
            if remove_duplicate:
                if id(v) in seen_ids:
                    continue
                seen_ids.add(id(v))
            mod, _, _ = k.rpartition(".")
            if (recurse or not mod) and k not in seen_names:
                seen_names.add(k)
                yield (f"{prefix}.{k}" if prefix else k, v)

    def named_parameters(self, prefix="", recurse=True, remove_duplicate=True):
        yield from self._named_parameters_or_buffers(
            self._overrides_parameters, self._model.named_parameters(remove_duplicate=remove_duplicate),
            prefix=prefix, recurse=recurse, remove_duplicate=remove_duplicate)

    def named_buffers(self, prefix="", recurse=True, remove_duplicate=True, *, persistent=None):
        kw = {} if persistent is None else {"persistent": persistent}
        try:
            orig = self._model.named_buffers(remove_duplicate=remove_duplicate, **kw)
        except TypeError:  # older torch: no `persistent` keyword
            orig = self._model.named_buffers(remove_duplicate=remove_duplicate)
        yield from self._named_parameters_or_buffers(
            self._overrides_buffers, orig, prefix=prefix, recurse=recurse, remove_duplicate=remove_duplicate)

    def _get_shared_names(self) -> dict[str, set[str]]:
        """name -> all names bound to the same tensor (tied weights), thunder/core/module.py:125-135."""
        names_of = WeakTensorKeyDictionary()
        for name, v in itertools.chain(self.named_parameters(remove_duplicate=False), self.named_buffers(remove_duplicate=False)):
            names_of.setdefault(v, set()).add(name)
        shared: dict[str, set[str]] = {}
        for s in names_of.values():
            for n in s:
                shared[n] = s
        return shared

    # ---- state dicts ----------------------------------------------------------------------------
    def _non_persistent_buffers(self, prefix="") -> set[str]:
        out = set()
        for name, sub in self._model.named_modules(prefix=prefix):
            p = f"{name}." if name else name
            out.update(f"{p}{b}" for b in sub._non_persistent_buffers_set)
        return out

    def load_original_state_dict(self, state_dict):
        """Stream a state dict of the UNtransformed model through every transform, one submodule at
        a time, so that e.g. bf16 weights are quantised as they arrive (module.py:137-145)."""
        per_module = _convert_state_dict_to_per_module(state_dict, {n for n, _ in self._model.named_modules()})
        shared_names = self._get_shared_names()
        processed: set[str] = set()
        for submodule_name, sd_part in per_module.items():
            self._transform_and_load_for_submodule(submodule_name, sd_part, shared_names, processed)

    def _transform_and_load_for_submodule(self, submodule_name, sd_part, shared_names, processed_names):
        prefix = submodule_name + ("." if submodule_name else "")
        for transform in self._lc_transforms:
            sd_part = transform.transform_state_dict_for_submodule(self, submodule_name, sd_part)
        for k, v in sd_part.items():
            full_k = prefix + k
            done_copies = shared_names.get(full_k, {full_k}) & processed_names
            if done_copies:  # tied to something already loaded: share it
                copy_name = next(iter(done_copies))
                if full_k in self._overrides_parameters:
                    self._overrides_parameters[full_k] = self._overrides_parameters[copy_name]
                elif full_k in self._overrides_buffers:
                    self._overrides_buffers[full_k] = self._overrides_buffers[copy_name]
                else:
                    raise NotImplementedError(f"don't know how to handle {full_k}")
                processed_names.add(full_k)
                continue
            if full_k in self._overrides_parameters:
                p = self._overrides_parameters[full_k]
                with torch.no_grad():
                    if p.dtype == v.dtype and p.shape == v.shape:
                        p.copy_(v)
                    else:
                        self._overrides_parameters[full_k] = torch.nn.Parameter(v.to(p.device), requires_grad=p.requires_grad)
            elif full_k in self._overrides_buffers:
                b = self._overrides_buffers[full_k]
                with torch.no_grad():
                    if b.dtype == v.dtype and b.shape == v.shape:
                        b.copy_(v)
                    else:
                        self._overrides_buffers[full_k] = v.to(device=b.device, dtype=b.dtype).requires_grad_(b.requires_grad)
            else:
                raise NotImplementedError(f"don't know how to handle {full_k}")
            processed_names.add(full_k)

    def state_dict(self, *, destination=None, prefix="", keep_vars=False):
        """State dict of the TRANSFORMED module: for a quantised Linear ``<lin>.weight`` is the packed
        uint8 tensor, followed later by ``<lin>.weight.absmax`` and ``<lin>.weight.code``."""
        if destination is None:
            destination = collections.OrderedDict()
            destination._metadata = collections.OrderedDict()
        for name, param in self.named_parameters(prefix=prefix):
            if param is not None:
                destination[name] = param if keep_vars else param.detach()
        non_persistent = self._non_persistent_buffers(prefix=prefix)
        for name, buf in self.named_buffers(prefix=prefix):
            if buf is not None and name not in non_persistent:
                destination[name] = buf if keep_vars else buf.detach()
        return destination

    def original_state_dict(self, *, destination=None, prefix="", keep_vars=False):
        """State dict with every transform's reverse applied (module.py:230-265)."""
        module_names = {name for name, _ in self._model.named_modules()}
        per_module = _convert_state_dict_to_per_module(self.state_dict(), module_names)
        if destination is None:
            destination = collections.OrderedDict()
            destination._metadata = collections.OrderedDict()
        for submodule_name, sd in per_module.items():
            for transform in reversed(self._lc_transforms):
                sd = transform.reverse_transform_state_dict_for_submodule(self, submodule_name, sd)
            sub_prefix = f"{submodule_name}." if submodule_name else ""
            destination.update({f"{prefix}{sub_prefix}{k}": v for k, v in sd.items()})
        return destination

    def load_state_dict(self, state_dict: Mapping[str, Any], strict: bool = True, assign: bool = False):
        """Load a state dict of the TRANSFORMED module (module.py:267-338)."""
        non_persistent = self._non_persistent_buffers()
        keys_unused = dict.fromkeys(state_dict.keys())
        keys_missing: list[str] = []
        errors: list[str] = []
        for name, v in itertools.chain(self.named_parameters(), self.named_buffers()):
            if name in non_persistent:
                continue
            if name not in state_dict:
                keys_missing.append(name)
                continue
            keys_unused.pop(name, None)
            sd_v = state_dict[name]
            if not torch.overrides.is_tensor_like(sd_v):
                errors.append(f'While copying the parameter named "{name}", expected torch.Tensor or Tensor-like '
                              f"object from checkpoint but received {type(sd_v)}")
                continue
            if sd_v.shape != v.shape:
                errors.append(f"size mismatch for {name}: copying a param with shape {sd_v.shape} from checkpoint, "
                              f"the shape in current model is {v.shape}.")
                continue
            with torch.no_grad():
                if assign:
                    if isinstance(v, torch.nn.Parameter):
                        if not isinstance(sd_v, torch.nn.Parameter):
                            sd_v = torch.nn.Parameter(sd_v, requires_grad=v.requires_grad)
                        else:
                            sd_v.requires_grad_(v.requires_grad)
                        self._overrides_parameters[name] = sd_v
                    elif name in self._overrides_parameters:
                        self._overrides_parameters[name] = sd_v
                    else:
                        self._overrides_buffers[name] = sd_v
                else:
                    v.copy_(sd_v)
        if strict:
            if keys_unused:
                errors.insert(0, "Unexpected key(s) in state_dict: {}. ".format(", ".join(f'"{k}"' for k in keys_unused)))
            if keys_missing:
                errors.insert(0, "Missing key(s) in state_dict: {}. ".format(", ".join(f'"{k}"' for k in keys_missing)))
        if errors:
            raise RuntimeError("Error(s) in loading state_dict:\n\t{}".format("\n\t".join(errors)))
        return torch.nn.modules.module._IncompatibleKeys(keys_missing, list(keys_unused))

    # ---- the shadow module the forward pass runs ------------------------------------------------
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

    def _shadow_value(self, full_name, original, wrappers, overrides):
        if full_name in wrappers:
            return wrappers[full_name]
        v = overrides.get(full_name, self._null)
        return original if v is self._null else v

    def __getattr__(self, name: str) -> Any:
        try:
            return super().__getattr__(name)
        except AttributeError:
            model = self.__dict__.get("_modules", {}).get("_model")
            if model is None:
                raise
            return getattr(model, name)
