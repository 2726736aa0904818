"""LoRA on packed expert weights (3-D parameters), per (expert, tenant) segment.

The reference keeps, per slot, ``lora_A [E, max_r, in]`` and ``lora_B [E, out, max_r]``
and merges ``W + einsum(B, A) * scaling`` into the expert weights through a
parametrization for the one active tenant
(src/twinkle/model/multi_lora_target_parameters.py:97-114, :158-209); the
per-expert loop then runs on the merged weights
(src/twinkle/model/transformers/moe/expert_parallel.py:347-371).  Here the same
slot tensors are read in place by the segmented kernels: rows are grouped by
``expert * num_tenants + tenant`` and each group adds
``scale * (x A_e^T) B_e^T`` to the expert's output rows, so the ``[E, out, in]``
delta is never materialised and many tenants share one pass.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch
from torch import nn

from .ops import AdapterGroups, multi_lora_delta
from .segments import SegmentTable


class ExpertLoraSlots(nn.Module):
    """Slot storage of one packed expert parameter (the reference's ``TargetParameterLoraWrapper`` state)."""

    def __init__(self, num_experts: int, in_features: int, out_features: int, max_loras: int, max_r: int,
                 dtype=torch.float32, device=None, key_prefix: str = ''):
        super().__init__()
        self.num_experts = num_experts
        self.in_features = in_features
        self.out_features = out_features
        self.max_loras = max_loras
        self.max_r = max_r
        self.peft_key_prefix = key_prefix
        self.lora_A = nn.ParameterDict()
        self.lora_B = nn.ParameterDict()
        self.scaling: Dict[str, float] = {}
        self.r: Dict[str, int] = {}
        self._initial_lora_A: Dict[str, torch.Tensor] = {}
        for index in range(max_loras):
            name = f'lora_{index}'
            self.lora_A[name] = nn.Parameter(torch.empty(num_experts, max_r, in_features, device=device, dtype=dtype))
            self.lora_B[name] = nn.Parameter(torch.empty(num_experts, out_features, max_r, device=device, dtype=dtype))
            self.r[name] = max_r
            self.scaling[name] = 1.0
            self.reset_slot(name)

    def reset_slot(self, slot_name: str) -> None:
        """A back to its first initialisation (kaiming-uniform, a = sqrt(5)), B to zero (reference :119-134)."""
        if slot_name not in self._initial_lora_A:
            nn.init.kaiming_uniform_(self.lora_A[slot_name], a=math.sqrt(5))
            self._initial_lora_A[slot_name] = self.lora_A[slot_name].detach().clone().cpu()
        else:
            init = self._initial_lora_A[slot_name]
            self.lora_A[slot_name].data.copy_(init.to(device=self.lora_A[slot_name].device,
                                                      dtype=self.lora_A[slot_name].dtype))
        nn.init.zeros_(self.lora_B[slot_name])

    def configure_slot(self, slot_name: str, config) -> None:
        """Rank and scaling of the tenant that takes the slot; same checks and messages as reference :136-156."""
        if slot_name not in self.lora_A:
            raise ValueError(f'Unknown target-parameter LoRA slot: {slot_name}')
        if config.r <= 0:
            raise ValueError(f'`r` should be a positive integer value but the value passed is {config.r}')
        if config.r > self.max_r:
            raise ValueError(f'LoRA rank {config.r} exceeds max_r={self.max_r}')
        if getattr(config, 'lora_dropout', 0):
            raise ValueError('target_parameters LoRA does not support lora_dropout != 0')
        if getattr(config, 'fan_in_fan_out', False):
            raise ValueError('target_parameters LoRA does not support fan_in_fan_out=True')
        if getattr(config, 'use_dora', False):
            raise ValueError('target_parameters LoRA does not support use_dora=True')
        if getattr(config, 'lora_bias', False):
            raise ValueError('target_parameters LoRA does not support lora_bias=True')
        self.r[slot_name] = config.r
        self.scaling[slot_name] = config.lora_alpha / (math.sqrt(config.r) if getattr(config, 'use_rslora', False)
                                                       else config.r)

    def get_delta_weight(self, slot_name: str, out_in_layout: bool = True) -> torch.Tensor:
        """The merged ``[E, out, in]`` (or ``[E, in, out]``) delta of the reference (:158-179); for export and checks."""
        if slot_name not in self.lora_A:
            raise ValueError(f'Unknown target-parameter LoRA slot: {slot_name}')
        r = self.r[slot_name]
        a, b = self.lora_A[slot_name][:, :r, :], self.lora_B[slot_name][:, :, :r]
        pattern = 'eor,eri->eoi' if out_in_layout else 'eor,eri->eio'
        return torch.einsum(pattern, b, a) * self.scaling[slot_name]

    def get_state_dict(self, slot_name: str) -> Dict[str, torch.Tensor]:
        r = self.r[slot_name]
        return {
            f'{self.peft_key_prefix}.lora_A.weight': self.lora_A[slot_name][:, :r, :].detach().clone(),
            f'{self.peft_key_prefix}.lora_B.weight': self.lora_B[slot_name][:, :, :r].detach().clone(),
        }

    def set_state_dict(self, slot_name: str, state_dict: Dict[str, torch.Tensor]) -> set:
        key_a, key_b = f'{self.peft_key_prefix}.lora_A.weight', f'{self.peft_key_prefix}.lora_B.weight'
        if key_a not in state_dict and key_b not in state_dict:
            return set()
        if key_a not in state_dict or key_b not in state_dict:
            raise KeyError(f'Missing target-parameter LoRA pair for {self.peft_key_prefix}')
        r = self.r[slot_name]
        a, b = state_dict[key_a], state_dict[key_b]
        if tuple(a.shape) != (self.num_experts, r, self.in_features):
            raise ValueError(f'Expected lora_A shape {(self.num_experts, r, self.in_features)}, got {tuple(a.shape)}')
        if tuple(b.shape) != (self.num_experts, self.out_features, r):
            raise ValueError(f'Expected lora_B shape {(self.num_experts, self.out_features, r)}, got {tuple(b.shape)}')
        with torch.no_grad():
            pa, pb = self.lora_A[slot_name], self.lora_B[slot_name]
            pa.zero_()
            pb.zero_()
            pa[:, :r, :].copy_(a.to(device=pa.device, dtype=pa.dtype))
            pb[:, :, :r].copy_(b.to(device=pb.device, dtype=pb.dtype))
        return {key_a, key_b}

    def groups(self, tenant_slots: Sequence[str]) -> AdapterGroups:
        """Group table for keys ``expert * len(tenant_slots) + tenant``: one block of a slot tensor per group."""
        nt = len(tenant_slots)
        a = [self.lora_A[s] for s in tenant_slots]
        b = [self.lora_B[s] for s in tenant_slots]
        n = self.num_experts * nt
        idx = [i % nt for i in range(n)]
        a_off = [(i // nt) * self.max_r * self.in_features for i in range(n)]
        b_off = [(i // nt) * self.out_features * self.max_r for i in range(n)]
        ranks = [self.r[tenant_slots[i % nt]] for i in range(n)]
        scales = [self.scaling[tenant_slots[i % nt]] for i in range(n)]
        return AdapterGroups(a, b, ranks, scales, a_index=idx, a_offset=a_off, b_index=idx, b_offset=b_off)


def expert_lora_delta(x_sorted: torch.Tensor, y_sorted: torch.Tensor, seg: SegmentTable, slots: ExpertLoraSlots,
                      tenant_slots: Sequence[str], groups: Optional[AdapterGroups] = None) -> torch.Tensor:
    """Adds every (expert, tenant) group's LoRA term onto the expert outputs, in place and differentiably.

    ``x_sorted`` / ``y_sorted`` are the expert inputs / outputs in segment order (what
    :func:`twinkle_amd.permute` and the per-expert base GEMMs produce); ``seg`` was built from keys
    ``expert * len(tenant_slots) + tenant``.
    """
    if groups is None:
        groups = slots.groups(tenant_slots)
    return multi_lora_delta(x_sorted, y_sorted, seg, groups, map_rows=False)
