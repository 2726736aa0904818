"""Minimal LoRA containers with the attribute surface the patched forward reads.

The reference relies on PEFT for the *container* only: ``lora_A`` / ``lora_B``
``ModuleDict``s of bias-free ``nn.Linear``, ``lora_dropout``, ``active_adapters``,
``disable_adapters``, ``_check_forward_args`` and ``_cast_input_dtype`` are the
attributes its forward touches (src/twinkle/model/multi_lora.py:301-327).  PEFT's
own ``LoraLayer`` works unchanged with :class:`twinkle_amd.MultiLora`; the classes
here provide the same surface where PEFT is not installed.
"""
from __future__ import annotations

import math
import re
from dataclasses import dataclass, field
from typing import List, Optional, Union

import torch
from torch import nn


@dataclass
class LoraConfig:
    """The fields of ``peft.LoraConfig`` that the multi-LoRA path reads."""
    r: int = 8
    lora_alpha: float = 8
    target_modules: Optional[Union[List[str], str]] = None
    exclude_modules: Optional[Union[List[str], str]] = None
    lora_dropout: float = 0.0
    use_rslora: bool = False
    use_dora: bool = False
    fan_in_fan_out: bool = False
    lora_bias: bool = False
    target_parameters: Optional[List[str]] = None
    bias: str = 'none'
    extra: dict = field(default_factory=dict)


class LoraLinear(nn.Module):
    """A frozen ``base_layer`` plus named LoRA slots (PEFT ``lora.Linear`` surface)."""

    def __init__(self, base_layer: nn.Module):
        super().__init__()
        self.base_layer = base_layer
        self.in_features = base_layer.in_features
        self.out_features = base_layer.out_features
        self.lora_A = nn.ModuleDict()
        self.lora_B = nn.ModuleDict()
        self.lora_dropout = nn.ModuleDict()
        self.r = {}
        self.lora_alpha = {}
        self.scaling = {}
        self._active_adapter: List[str] = []
        self.disable_adapters = False
        for p in base_layer.parameters():
            p.requires_grad_(False)

    @property
    def active_adapters(self) -> List[str]:
        return list(self._active_adapter)

    @property
    def weight(self):
        return self.base_layer.weight

    def update_layer(self, adapter_name: str, r: int, lora_alpha: float, lora_dropout: float = 0.0) -> None:
        if r <= 0:
            raise ValueError(f'`r` should be a positive integer value but the value passed is {r}')
        w = self.base_layer.weight
        a = nn.Linear(self.in_features, r, bias=False, device=w.device, dtype=w.dtype)
        b = nn.Linear(r, self.out_features, bias=False, device=w.device, dtype=w.dtype)
        nn.init.kaiming_uniform_(a.weight, a=math.sqrt(5))
        nn.init.zeros_(b.weight)
        self.lora_A[adapter_name] = a
        self.lora_B[adapter_name] = b
        self.lora_dropout[adapter_name] = nn.Dropout(lora_dropout) if lora_dropout > 0 else nn.Identity()
        self.r[adapter_name] = r
        self.lora_alpha[adapter_name] = lora_alpha
        self.scaling[adapter_name] = lora_alpha / r
        if not self._active_adapter:
            self._active_adapter = [adapter_name]

    def set_adapter(self, adapter_names) -> None:
        if isinstance(adapter_names, str):
            adapter_names = [adapter_names]
        self._active_adapter = list(adapter_names)

    def enable_adapters(self, enabled: bool) -> None:
        self.disable_adapters = not enabled

    def _check_forward_args(self, x, *args, **kwargs) -> None:
        if kwargs.get('adapter_names') is not None:
            raise ValueError('mixed-batch `adapter_names` is not part of this path; use MultiLora.batch(...)')

    def _cast_input_dtype(self, x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
        return x if x.dtype == dtype else x.to(dtype)

    def forward(self, x: torch.Tensor, *args, **kwargs) -> torch.Tensor:
        # Plain single-adapter LoRA; MultiLora.patch() rebinds this per instance.
        result = self.base_layer(x, *args, **kwargs)
        if self.disable_adapters:
            return result
        for name in self._active_adapter:
            if name not in self.lora_A:
                continue
            xa = self._cast_input_dtype(x, self.lora_A[name].weight.dtype)
            result = result + self.lora_B[name](self.lora_A[name](self.lora_dropout[name](xa))) * self.scaling[name]
        return result


def _name_matches(name: str, target_modules) -> bool:
    if target_modules is None:
        return False
    if target_modules == 'all-linear' or (isinstance(target_modules, (list, set, tuple)) and
                                          'all-linear' in target_modules):
        return True
    if isinstance(target_modules, str):
        return re.fullmatch(target_modules, name) is not None
    return any(name == t or name.endswith('.' + t) for t in target_modules)


class LoraModel(nn.Module):
    """Holder returned by :func:`inject_adapter` (the part of ``PeftModel`` the multi-LoRA path uses)."""

    def __init__(self, model: nn.Module):
        super().__init__()
        self.model = model
        self.active_adapter: Optional[str] = None
        self.peft_config = {}

    @property
    def active_adapters(self) -> List[str]:
        return [self.active_adapter] if self.active_adapter else []

    def lora_layers(self):
        for name, m in self.named_modules():
            if isinstance(m, LoraLinear):
                yield name, m

    def add_adapter(self, adapter_name: str, config: LoraConfig, **_) -> None:
        inject_adapter(self, config, adapter_name)

    def set_adapter(self, adapter_name: str) -> None:
        self.active_adapter = adapter_name
        for _, layer in self.lora_layers():
            layer.set_adapter(adapter_name)

    def disable_adapter_layers(self) -> None:
        for _, layer in self.lora_layers():
            layer.enable_adapters(False)

    def enable_adapter_layers(self) -> None:
        for _, layer in self.lora_layers():
            layer.enable_adapters(True)

    def forward(self, *args, **kwargs):
        return self.model(*args, **kwargs)


def inject_adapter(model: nn.Module, config: LoraConfig, adapter_name: str) -> LoraModel:
    """Wrap every targeted ``nn.Linear`` in a :class:`LoraLinear` and add the named slot to it."""
    holder = model if isinstance(model, LoraModel) else LoraModel(model)
    root = holder.model
    exclude = config.exclude_modules or []
    if isinstance(exclude, str):
        exclude = [exclude]
    wrapped = 0
    inside = tuple(n + '.' for n, m in root.named_modules() if isinstance(m, LoraLinear))
    for name, module in list(root.named_modules()):
        if isinstance(module, LoraLinear):
            module.update_layer(adapter_name, config.r, config.lora_alpha, config.lora_dropout)
            wrapped += 1
            continue
        if not isinstance(module, nn.Linear) or name.startswith(inside):   # base layers and slot weights stay as they are
            continue
        if not _name_matches(name, config.target_modules) or any(name.endswith(e) for e in exclude):
            continue
        parent_name, _, child = name.rpartition('.')
        parent = root.get_submodule(parent_name) if parent_name else root
        layer = LoraLinear(module)
        layer.update_layer(adapter_name, config.r, config.lora_alpha, config.lora_dropout)
        setattr(parent, child, layer)
        wrapped += 1
    if wrapped == 0:
        raise ValueError(f'Target modules {config.target_modules} not found in the base model')
    holder.peft_config[adapter_name] = config
    if holder.active_adapter is None:
        holder.set_adapter(adapter_name)
    return holder
