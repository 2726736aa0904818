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
from contextlib import contextmanager
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
        # building the table costs a few host-to-device copies: kept until a slot's rank or scaling changes (moved
        # parameter storage is picked up by AdapterGroups.refresh at every call)
        key = (tuple(tenant_slots), tuple(self.r[s] for s in tenant_slots),
               tuple(self.scaling[s] for s in tenant_slots))
        cache = self.__dict__.setdefault('_groups_cache', {})
        hit = cache.get(key)
        if hit is not None and all(x is y for x, y in zip(hit.a_tensors + hit.b_tensors,
                                                           [self.lora_A[s] for s in tenant_slots] +
                                                           [self.lora_B[s] for s in tenant_slots])):
            return hit
        a = [self.lora_A[s] for s in tenant_slots]
        b = [self.lora_B[s] for s in tenant_slots]
        n = self.num_experts * nt
        idx = [i % nt for i in range(n)]
        a_off = [(i // nt) * self.max_r * self.in_features for i in range(n)]
        b_off = [(i // nt) * self.out_features * self.max_r for i in range(n)]
        ranks = [self.r[tenant_slots[i % nt]] for i in range(n)]
        scales = [self.scaling[tenant_slots[i % nt]] for i in range(n)]
        if len(cache) > 16:
            cache.clear()
        cache[key] = AdapterGroups(a, b, ranks, scales, a_index=idx, a_offset=a_off, b_index=idx, b_offset=b_off)
        return cache[key]


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


class ExpertLoraManager:
    """Finds packed expert parameters in a model, gives each its slot storage and keeps the tenant -> slot map.

    Host-side mirror of the reference's ``TargetParameterLoraManager``
    (src/twinkle/model/multi_lora_target_parameters.py:281-383): same method names, arguments and errors.  What
    differs is how a slot takes effect: the reference merges ``W + B A * scaling`` into the parameter through a
    parametrization while a tenant is active (:182-209); here the expert forward adds the low-rank term of every
    (expert, tenant) segment with :func:`expert_lora_delta`, and :meth:`adapter` only records which tenant is the
    active one for callers that run one tenant per pass.

    The slot tensors have the reference's shapes for both storage layouts (``lora_A [E, max_r, in_features]``,
    ``lora_B [E, out_features, max_r]`` with the reference's naming of the two trailing dimensions).  The segmented
    kernels apply ``scale * (x A^T) B^T``, which is the reference's merged form when the expert computes
    ``F.linear(x, W[e])`` on ``[E, out, in]`` storage (its expert forward, moe/expert_parallel.py:360-371);
    for modules that compute ``x @ W[e]`` the merged delta of :meth:`ExpertLoraSlots.get_delta_weight` applies.
    """

    def __init__(self, max_loras: int, max_r: int):
        self.max_loras = max_loras
        self.max_r = max_r
        self.wrappers: List[ExpertLoraSlots] = []
        self.tenant_to_slot: Dict[str, str] = {}
        self.tenant_configs: Dict[str, object] = {}
        self._target_parameters: Optional[tuple] = None

    def patch(self, model: nn.Module, target_parameters) -> None:
        """Attach slot storage to every parameter named (or suffixed ``.name``) in ``target_parameters``
        (reference :291-319).  3-D parameters are ``[E, out, in]`` unless the owning module says
        ``is_transposed`` (then ``[E, in, out]``), 2-D ones ``[out, in]`` with one expert (:47-52)."""
        target_parameters = tuple(target_parameters)
        if not target_parameters:
            return
        if self._target_parameters is not None:
            if self._target_parameters != target_parameters:
                raise ValueError(
                    f'target_parameters already patched as {self._target_parameters}, got {target_parameters}')
            return
        found = []
        for module_name, module in model.named_modules():
            for param_name, parameter in module.named_parameters(recurse=False):
                key = f'{module_name}.{param_name}' if module_name else param_name
                if key in target_parameters or any(key.endswith(f'.{t}') for t in target_parameters):
                    if parameter.ndim not in (2, 3):
                        raise ValueError(
                            f'target parameter {key} has {parameter.ndim} dimensions; only 2D and 3D are supported')
                    found.append((module_name, module, param_name, parameter))
        if not found:
            raise ValueError(f'target_parameters={target_parameters} were set but no parameter was matched')
        per_module: Dict[str, List[ExpertLoraSlots]] = {}
        for module_name, module, param_name, parameter in found:
            if parameter.ndim == 3:
                out_in = not getattr(module, 'is_transposed', False)
                experts = parameter.shape[0]
                fin, fout = (parameter.shape[-1], parameter.shape[-2]) if out_in else (parameter.shape[-2],
                                                                                      parameter.shape[-1])
            else:
                out_in, experts = True, 1
                fout, fin = parameter.shape
            device = 'cpu' if parameter.device.type == 'meta' else parameter.device
            slots = ExpertLoraSlots(experts, fin, fout, self.max_loras, self.max_r, dtype=parameter.dtype, device=device)
            slots.parameter_key = f'{module_name}.{param_name}' if module_name else param_name
            slots.out_in_layout = out_in
            slots.active_adapter, slots.disable_adapters = None, False
            module.add_module(f'_twinkle_lora_{param_name}', slots)
            self.wrappers.append(slots)
            per_module.setdefault(module_name, []).append(slots)
        # PEFT nests one wrapper per target parameter of a module: the first one found is the innermost (:321-330)
        for module_name, group in per_module.items():
            prefix = f'base_model.model.{module_name}' if module_name else 'base_model.model'
            for index, slots in enumerate(group):
                nested = '.'.join(['base_layer'] * (len(group) - index - 1))
                slots.peft_key_prefix = f'{prefix}.{nested}' if nested else prefix
        self._target_parameters = target_parameters

    def acquire(self, tenant_adapter_name: str, slot_name: str, config) -> None:
        if tenant_adapter_name in self.tenant_to_slot:
            raise ValueError(f'Lora {tenant_adapter_name} already exists')
        if getattr(config, 'target_parameters', None) and not self.wrappers:
            raise ValueError('target_parameters LoRA slots must be patched before acquire')
        self.tenant_to_slot[tenant_adapter_name] = slot_name
        self.tenant_configs[tenant_adapter_name] = config
        for slots in self.wrappers:
            slots.configure_slot(slot_name, config)

    def release(self, tenant_adapter_name: str) -> None:
        slot_name = self.tenant_to_slot.pop(tenant_adapter_name, None)
        self.tenant_configs.pop(tenant_adapter_name, None)
        if slot_name is None:
            return
        for slots in self.wrappers:
            slots.reset_slot(slot_name)

    @contextmanager
    def adapter(self, tenant_adapter_name: str, disable_lora: bool = False):
        """One tenant per pass: every slot storage learns which slot is active (``None`` for unknown tenants)."""
        slot_name = self.tenant_to_slot.get(tenant_adapter_name)
        previous = [(s.active_adapter, s.disable_adapters) for s in self.wrappers]
        for s in self.wrappers:
            s.active_adapter, s.disable_adapters = slot_name, disable_lora
        try:
            yield
        finally:
            for s, (a, d) in zip(self.wrappers, previous):
                s.active_adapter, s.disable_adapters = a, d

    def slots_of(self, tenant_adapter_names: Sequence[str]) -> List[str]:
        """Slot names of the tenants of a mixed batch, in the order their ids appear in the group keys."""
        return [self.tenant_to_slot[t] for t in tenant_adapter_names]

    def parameters_for_tenant(self, tenant_adapter_name: str) -> List[nn.Parameter]:
        return [p for _, p in self.named_slot_parameters(tenant_adapter_name)]

    def named_slot_parameters(self, tenant_adapter_name: str):
        slot_name = self.tenant_to_slot[tenant_adapter_name]
        for slots in self.wrappers:
            if slot_name in slots.lora_A:
                yield f'{slots.parameter_key}.lora_A.{slot_name}.weight', slots.lora_A[slot_name]
                yield f'{slots.parameter_key}.lora_B.{slot_name}.weight', slots.lora_B[slot_name]

    def get_state_dict(self, tenant_adapter_name: str) -> Dict[str, torch.Tensor]:
        slot_name = self.tenant_to_slot[tenant_adapter_name]
        state = {}
        for slots in self.wrappers:
            state.update(slots.get_state_dict(slot_name))
        return state

    def set_state_dict(self, tenant_adapter_name: str, state_dict: Dict[str, torch.Tensor]) -> set:
        slot_name = self.tenant_to_slot[tenant_adapter_name]
        consumed = set()
        for slots in self.wrappers:
            consumed.update(slots.set_state_dict(slot_name, state_dict))
        return consumed


def _is_silu(fn) -> bool:
    return fn is torch.nn.functional.silu or isinstance(fn, nn.SiLU)


def _gated_activation(experts_mod: nn.Module, gate_up_out: torch.Tensor, fused: bool = True) -> torch.Tensor:
    """``_apply_gate`` if the module has one, else ``act_fn(gate) * up`` (moe/expert_parallel.py:363-366); with
    SiLU on the GPU the one-pass kernel does the same arithmetic in fp32 with one rounding."""
    from .ops import swiglu, swiglu_applies
    if hasattr(experts_mod, '_apply_gate'):
        return experts_mod._apply_gate(gate_up_out)
    if fused and _is_silu(experts_mod.act_fn) and swiglu_applies(gate_up_out):
        return swiglu(gate_up_out)
    gate, up = gate_up_out.chunk(2, dim=-1)
    return experts_mod.act_fn(gate) * up


def grouped_gemm_applies(weight: torch.Tensor, rows: torch.Tensor) -> bool:
    """Frozen bf16 packed weights whose two widths are multiples of 128: what ``tk_grouped_linear`` takes in the
    forward direction (``in`` a multiple of 64, ``out`` of 128) and, with the roles swapped, in the backward one."""
    return (weight.dtype == torch.bfloat16 and rows.dtype == torch.bfloat16 and weight.is_contiguous() and
            not weight.requires_grad and weight.shape[1] % 128 == 0 and weight.shape[2] % 128 == 0)


def experts_forward(experts_mod: nn.Module, rows: torch.Tensor, seg: SegmentTable, tenant_slots: Sequence[str],
                    gate_up_slots: Optional[ExpertLoraSlots] = None,
                    down_slots: Optional[ExpertLoraSlots] = None, grouped: Optional[bool] = None,
                    fused_activation: bool = True) -> torch.Tensor:
    """Packed experts on rows in (expert, tenant) segment order, every tenant's LoRA terms included.

    The per-expert loop of the reference's expert forward (moe/expert_parallel.py:333-378: ``F.linear`` with
    ``gate_up_proj[e]``, gate activation, ``F.linear`` with ``down_proj[e]`` on contiguous chunks), with two
    differences: the chunk boundaries come from the segment table in one device-to-host copy (the reference
    synchronises once per expert, :347-349), and the LoRA terms are added per (expert, tenant) segment by the
    segmented kernels instead of being merged into the weights.  ``seg`` was built from keys
    ``expert * len(tenant_slots) + tenant`` with ``want_offsets=True``; ``experts_mod`` holds
    ``gate_up_proj [E, 2 I, H]`` and ``down_proj [E, H, I]`` and either ``_apply_gate`` or ``act_fn``.

    ``grouped`` (default: whenever the shapes allow, i.e. frozen bf16 weights with widths that are multiples of
    64 / 128 in both directions) replaces the loop by one grouped GEMM per projection with the LoRA terms in its
    epilogue: no host copy of the boundaries at all, one launch instead of one per expert, and the expert outputs
    are written once.  Its backward runs the same kernel in its transposing form on the same weights.
    ``fused_activation`` lets a SiLU gate run as one kernel forward and one backward instead of torch's five.
    """
    if rows.shape[0] == 0:
        return rows                                                   # keeps the autograd edge (reference :340-344)
    nt = len(tenant_slots)
    gate_up, down = experts_mod.gate_up_proj, experts_mod.down_proj
    experts = gate_up.shape[0]
    if seg.num_groups != experts * nt:
        raise ValueError('the segment table must be built from expert * num_tenants + tenant keys')
    input_dtype = rows.dtype
    x = rows if rows.dtype == gate_up.dtype else rows.to(gate_up.dtype)
    can_group = x.is_cuda and grouped_gemm_applies(gate_up, x) and grouped_gemm_applies(down, x)
    if grouped and not can_group:
        raise ValueError('grouped=True needs frozen bf16 expert weights with widths that are multiples of 128')
    if grouped or (grouped is None and can_group):
        from .ops import grouped_experts_linear
        x = x.contiguous()
        gate_up_out = grouped_experts_linear(x, gate_up, seg, nt,
                                             gate_up_slots.groups(tenant_slots) if gate_up_slots is not None else None)
        hidden = _gated_activation(experts_mod, gate_up_out, fused_activation)
        out = grouped_experts_linear(hidden.contiguous(), down, seg, nt,
                                     down_slots.groups(tenant_slots) if down_slots is not None else None)
        return out if out.dtype == input_dtype else out.to(input_dtype)
    if seg.offsets is None:
        raise ValueError('the per-expert loop needs a segment table built with want_offsets=True')
    bounds = seg.offsets[::nt].tolist()                               # first sorted position of every expert

    def per_expert(inp, weight):
        chunks = [torch.nn.functional.linear(inp[bounds[e]:bounds[e + 1]], weight[e]) for e in range(experts)
                  if bounds[e + 1] > bounds[e]]
        return torch.cat(chunks, dim=0)

    gate_up_out = per_expert(x, gate_up)
    if gate_up_slots is not None:
        gate_up_out = expert_lora_delta(x, gate_up_out, seg, gate_up_slots, tenant_slots)
    hidden = _gated_activation(experts_mod, gate_up_out, fused_activation).contiguous()
    out = per_expert(hidden, down)
    if down_slots is not None:
        out = expert_lora_delta(hidden, out, seg, down_slots, tenant_slots)
    return out if out.dtype == input_dtype else out.to(input_dtype)


def moe_experts_block(hidden_states: torch.Tensor, selected_experts: torch.Tensor, routing_weights: torch.Tensor,
                      tenant: Optional[torch.Tensor], experts_mod: nn.Module, tenant_slots: Sequence[str],
                      gate_up_slots: Optional[ExpertLoraSlots] = None,
                      down_slots: Optional[ExpertLoraSlots] = None) -> torch.Tensor:
    """Routed tokens through the packed experts and back: segment build, permute, :func:`experts_forward`,
    weighted unpermute (the single-rank part of the reference's patched block forward,
    moe/expert_parallel.py:253-255 and moe/ep_utils.py:99-149, :280-287).  ``tenant [T]`` gives every token's
    index into ``tenant_slots`` (``None``: one tenant)."""
    from .segments import build_segments, flat_keys_from_topk, permute, unpermute
    nt = len(tenant_slots)
    experts = experts_mod.gate_up_proj.shape[0]
    tokens = hidden_states.shape[0]
    keys = flat_keys_from_topk(selected_experts, tenant if nt > 1 else None, nt)
    seg = build_segments(keys, experts * nt, num_tokens=tokens)
    rows, _ = permute(hidden_states, seg)
    out_rows = experts_forward(experts_mod, rows, seg, tenant_slots, gate_up_slots, down_slots)
    return unpermute(out_rows, routing_weights.to(hidden_states.dtype), seg)
