"""Slot pool, tenant bookkeeping and the patched LoRA forward, on the HIP kernels.

Host-side mirror of ``twinkle.model.multi_lora.MultiLora``
(src/twinkle/model/multi_lora.py): same method names, argument meaning and
exceptions, so that code written against the reference's class runs unchanged.
Two things differ underneath:

* the LoRA arithmetic of the patched forward (reference :315-326) runs in the
  segmented HIP kernels instead of two ``F.linear`` calls, and
* :meth:`MultiLora.batch` widens :meth:`MultiLora.adapter` from one adapter per
  call to one adapter per row, so that many tenants share one forward/backward.
  ``adapter(name)`` is the one-segment special case and needs no change in callers.
"""
from __future__ import annotations

import re
from contextlib import contextmanager
from dataclasses import dataclass, field
from types import MethodType
from typing import Any, Dict, List, Optional, Sequence, Tuple, Union

import torch

from .expert_lora import ExpertLoraManager
from .lora_layer import LoraConfig, LoraLinear, LoraModel, inject_adapter
from .ops import AdapterGroups, multi_lora_delta, multi_lora_linear, multi_lora_linear_shared
from .segments import SegmentTable, build_segments


@dataclass
class LoraTenant:
    """One pre-allocated slot and the tenant that holds it (reference :20-28)."""
    index: int
    adapter_name: str
    config: Any
    tenant_adapter_name: Optional[str] = None
    tenant_config: Optional[Any] = None
    lora_A_weights: Dict[str, torch.Tensor] = field(default_factory=dict)


class _SharedInputGroup:
    """Layers that are called one after the other on the same tensor (q / k / v, gate / up)."""

    def __init__(self, layers):
        self.layers = list(layers)
        self.source = None       # the input the pending outputs were computed from
        self.version = -1
        self.pending = {}        # id(layer) -> output not handed out yet

    def take(self, layer, x):
        if self.source is x and self.version == x._version and id(layer) in self.pending:
            out = self.pending.pop(id(layer))
            if not self.pending:
                self.source = None
            return out
        return None

    def fill(self, x, outs, first):
        self.pending = {id(layer): out for layer, out in zip(self.layers, outs) if layer is not first}
        self.source, self.version = (x, x._version) if self.pending else (None, -1)


def _is_lora_layer(module) -> bool:
    return all(hasattr(module, a) for a in ('base_layer', 'lora_A', 'lora_B', 'lora_dropout'))


# ---------------------------------------------------------------------------------------------------------------
# What the patched forward needs beyond the reference's ``MultiLora`` surface (``loras``, ``find_lora``,
# ``find_lora_by_tenant``, ``match_target_modules``, ``max_loras``): the per-layer group tables, the segment table of
# the open batch and the one-segment tables of ``adapter()``.  It lives in one object that is attached to the
# ``MultiLora`` instance the first time it is needed, and every helper below takes that instance as an argument,
# so the functions work on the reference's own class as well as on the one in this file.
# ---------------------------------------------------------------------------------------------------------------
class _PathState:

    def __init__(self):
        self.layer_groups: Dict[tuple, tuple] = {}
        self.batch_table: Optional[SegmentTable] = None
        self.uniform_tables: Dict[tuple, SegmentTable] = {}


def _path_state(ml) -> _PathState:
    state = ml.__dict__.get('_tk_path_state')
    if state is None:
        state = ml.__dict__['_tk_path_state'] = _PathState()
    return state


def _hashable(v):
    return tuple(sorted(v)) if isinstance(v, (list, set, tuple)) else v


def _ownership(ml):
    """Changes whenever a slot changes hands or its tenant's settings do: the key the group tables are cached by.
    The class in this file counts its acquire / release calls; for any other object the tenants' settings are read."""
    version = ml.__dict__.get('_version')
    if version is not None:
        return version
    return tuple((t.tenant_adapter_name, getattr(t.tenant_config, 'r', None), getattr(t.tenant_config, 'lora_alpha', None),
                  bool(getattr(t.tenant_config, 'use_rslora', False)),
                  _hashable(getattr(t.tenant_config, 'target_modules', None))) for t in ml.loras)


def _table_for(ml, rows: int, slot_index: int, device) -> SegmentTable:
    """The one-segment table of ``adapter()``: every row belongs to slot ``slot_index``."""
    tables = _path_state(ml).uniform_tables
    key = (rows, slot_index, str(device))
    table = tables.get(key)
    if table is None:
        if len(tables) >= 64:
            tables.clear()
        keys = torch.full((rows,), slot_index, dtype=torch.int32, device=device)
        table = tables[key] = build_segments(keys, len(ml.loras), want_perm=False, want_offsets=False)
    return table


def _groups_for(ml, layer, only_slot: Union[None, str, Tuple[str, ...]],
                x_dtype: Optional[torch.dtype] = None) -> Optional[AdapterGroups]:
    """Rank/scale table of a layer: slots whose tenant targets this layer are live, the rest rank 0.
    ``only_slot`` narrows the live slots to one name or a tuple of names (``None``: every slot with a tenant).
    ``x_dtype`` is the dtype of the activations the layer is called with: fp32 adapters under bf16 activations
    (PEFT keeps adapters in fp32 under a bf16 base) run on the bf16 matrix-core kernels, which read the fp32
    parameters where they are and write fp32 gradients, unless ``lora_compute_dtype=torch.float32`` asks for the
    reference's arithmetic (activations cast to fp32, :320)."""
    cache = _path_state(ml).layer_groups
    mixed = (x_dtype == torch.bfloat16 and getattr(ml, 'lora_compute_dtype', None) != torch.float32)
    key = (id(layer), only_slot, mixed)
    owners = _ownership(ml)
    cached = cache.get(key)
    if cached is not None and cached[0] == owners:
        return cached[1]
    a, b, ranks, scales = [], [], [], []
    for slot in ml.loras:
        name = slot.adapter_name
        if name not in layer.lora_A.keys():
            raise ValueError(f'layer {layer.layer_name} has no slot {name}')
        a.append(layer.lora_A[name].weight)
        b.append(layer.lora_B[name].weight)
        cfg = slot.tenant_config
        wanted = only_slot is None or only_slot == name or (isinstance(only_slot, tuple) and name in only_slot)
        live = cfg is not None and wanted and ml.match_target_modules(layer.layer_name, cfg.target_modules)
        if live:
            ranks.append(cfg.r)
            scales.append(cfg.lora_alpha / (cfg.r**0.5 if getattr(cfg, 'use_rslora', False) else cfg.r))
        else:
            ranks.append(0)
            scales.append(0.0)
    if max(ranks) == 0:
        groups = None
    elif mixed and a[0].dtype == torch.float32:
        groups = AdapterGroups(a, b, ranks, scales, act_dtype=torch.bfloat16)
    else:
        groups = AdapterGroups(a, b, ranks, scales)
    if len(cache) > 8192:   # batches over ever-changing tenant sets: start over
        cache.clear()
    cache[key] = (owners, groups)
    return groups


def _slot_dropout(ml, layer, only_slot: Optional[str], table):
    """The dropout module the LoRA branch applies: the slot's own (reference :317).  In a mixed batch one module
    serves every row, which is what the reference computes only if the live slots' modules agree (identity, or
    one probability): anything else is refused rather than applied to the wrong rows."""
    if only_slot is not None:
        return layer.lora_dropout[only_slot]
    names = getattr(table, 'live_slots', None) or [t.adapter_name for t in ml.loras]
    mods = [layer.lora_dropout[n] for n in names if n in layer.lora_dropout.keys()]
    first = mods[0] if mods else torch.nn.Identity()
    for m in mods[1:]:
        if type(m) is not type(first) or getattr(m, 'p', 0.0) != getattr(first, 'p', 0.0):
            raise NotImplementedError(
                f'layer {layer.layer_name}: the slots of a mixed batch have different lora_dropout modules')
    return first


@contextmanager
def batch(ml, tenant_adapter_names: Sequence[str], row_tenant: torch.Tensor, check: bool = False):
    """Many tenants in one forward/backward: row ``i`` uses ``tenant_adapter_names[row_tenant[i]]``.

    ``ml`` is a ``MultiLora`` whose layers carry the forward of :meth:`MultiLora._patch_lora_forward` (the class in
    this file, or the reference's ``twinkle.model.multi_lora.MultiLora``).
    ``row_tenant`` is an integer GPU tensor with one entry per row of the
    flattened ``[rows, features]`` activations (so ``batch * seq`` entries for
    ``[batch, seq, features]`` inputs).  The segment table is built once here
    and shared by every patched layer called inside the context.  A row whose entry is negative (padding,
    ignored rows) or not below ``len(tenant_adapter_names)`` belongs to no tenant: it keeps the base output and
    adds to nobody's gradients.  ``check=True`` instead verifies that every entry of ``row_tenant`` indexes
    ``tenant_adapter_names`` (one device synchronisation) and raises ``ValueError`` otherwise.
    """
    slots = [ml.find_lora_by_tenant(n).index for n in tenant_adapter_names]
    if check and row_tenant.numel():
        lo, hi = int(row_tenant.min()), int(row_tenant.max())
        if lo < 0 or hi >= len(slots):
            raise ValueError(f'row_tenant holds {lo}..{hi} but the batch has {len(slots)} tenants')
    lut = torch.tensor(slots, dtype=torch.int32, device=row_tenant.device)
    rt = row_tenant.reshape(-1).long()
    known = (rt >= 0) & (rt < len(slots))
    keys = torch.where(known, lut[rt.clamp(0, len(slots) - 1)], torch.full_like(lut[:1], -1))
    table = build_segments(keys, len(ml.loras), want_perm=False, want_offsets=False)
    # only the tenants of this batch are live inside the context: the others get no gradient, like the
    # adapters the reference leaves inactive
    table.live_slots = tuple(sorted({ml.loras[i].adapter_name for i in slots}))
    state = _path_state(ml)
    previous, state.batch_table = state.batch_table, table
    experts = getattr(getattr(ml, 'target_parameter_manager', None), 'batch', None)   # this file's manager only
    try:
        if experts is not None:
            with experts(tenant_adapter_names, rt):
                yield table
        else:
            yield table
    finally:
        state.batch_table = previous


def _modules_of(ml):
    return ml.module if isinstance(ml.module, list) else [ml.module]


def share_inputs(ml, layer_groups: Sequence[Sequence]) -> None:
    """Declare groups of patched layers that the model calls one after the other on the same tensor
    (``[[q_proj, k_proj, v_proj], [gate_proj, up_proj]]`` per block; modules or their names inside the
    patched module).  Model code stays as it is: the first layer of a group that sees a new input computes
    the outputs of the whole group through :func:`forward_shared` and the siblings, called with the same
    tensor, pick theirs up.  A sibling called with another tensor (or twice) simply starts a new group
    computation, so results never depend on the call pattern; outputs nobody collects are dropped at the next
    call.  ``share_inputs([])`` clears nothing: call :func:`unshare_inputs` for that.
    """
    named = {n: sub for m in _modules_of(ml) for n, sub in m.named_modules()}
    for group in layer_groups:
        layers = [named[m] if isinstance(m, str) else m for m in group]
        if not 2 <= len(layers) <= 4:
            raise ValueError(f'a group of shared inputs has 2 to 4 layers, got {len(layers)}')
        for layer in layers:
            if not _is_lora_layer(layer) or not hasattr(layer, 'layer_name'):
                raise ValueError('share_inputs takes layers that patch() has patched')
        if len({layer.in_features for layer in layers}) != 1:
            raise ValueError('layers that share an input must agree in in_features')
        state = _SharedInputGroup(layers)
        for layer in layers:
            layer._tk_shared_inputs = state

def unshare_inputs(ml) -> None:
    for m in _modules_of(ml):
        for sub in m.modules():
            if hasattr(sub, '_tk_shared_inputs'):
                del sub._tk_shared_inputs

def forward_shared(ml, layers: Sequence, x: torch.Tensor) -> Tuple[torch.Tensor, ...]:
    """``tuple(layer(x) for layer in layers)`` for patched layers that read the same ``x`` (q / k / v,
    gate / up), with the LoRA terms of all of them computed by one shared call: ``x`` is read once in
    forward, and once in backward for every layer's dA, and the gradient of ``x`` is updated once.

    The reference has no per-input entry (every projection runs its own two ``F.linear`` calls, :322-326);
    a caller opts in by routing such a group of projections through this function.  Falls back to calling
    the layers one by one whenever one of them would not take the plain in-place path (adapters disabled,
    a layer without a live adapter, dtype casts, non-``nn.Linear`` base layers).
    """
    layers = list(layers)
    table = _path_state(ml).batch_table
    only_slot = None
    ok = 2 <= len(layers) <= 4 and x.is_cuda
    groups_list = []
    for layer in layers if ok else ():
        if table is None:
            active = [n for n in layer.active_adapters if n in layer.lora_A.keys()]
            slot = active[0] if active else None
            # several active adapters on one layer: the reference adds the term of every one of them
            # (multi_lora.py:306-326), which the layer's own forward does and one shared call does not
            if len(active) != 1 or (only_slot is not None and slot != only_slot):
                ok = False
                break
            only_slot = slot
        groups = None if layer.disable_adapters else _groups_for(
            ml, layer, only_slot if table is None else getattr(table, 'live_slots', None), x.dtype)
        base = layer.base_layer
        if (groups is None or groups.dtype != x.dtype or type(base) is not torch.nn.Linear
                or base.weight.dtype != x.dtype or base._forward_hooks or base._forward_pre_hooks
                or not isinstance(_slot_dropout(ml, layer, only_slot, table), torch.nn.Identity)):
            ok = False
            break
        groups_list.append(groups)
    if not ok:
        return tuple(getattr(layer, '_tk_forward_one', layer)(x) for layer in layers)
    x2 = x.reshape(-1, x.shape[-1])
    if x2.stride(-1) != 1 or (x2.shape[0] > 1 and x2.stride(0) < x2.shape[1]):
        x2 = x2.contiguous()
    if table is None:
        table = _table_for(ml, x2.shape[0], ml.find_lora(only_slot).index, x2.device)
    elif table.rows != x2.shape[0]:
        raise ValueError(f'batch() was given {table.rows} rows but the shared input has {x2.shape[0]}')
    outs = multi_lora_linear_shared(x2, [layer.base_layer.weight for layer in layers],
                                    [layer.base_layer.bias for layer in layers], table, groups_list)
    return tuple(y.view(*x.shape[:-1], y.shape[-1]) for y in outs)


class MultiLora:

    def __init__(self, max_loras=5, max_r=32, max_length: int = 8192, lora_compute_dtype: Optional[torch.dtype] = None):
        self.max_loras = max_loras
        self.max_r = max_r
        self.max_length = max_length
        # Adapter weights kept in fp32 under a bf16 base model (what PEFT's adapter autocast produces): the bf16
        # matrix-core kernels run, reading the fp32 parameters where they are (converted on the fly inside the
        # library, no copies kept on this side) and writing fp32 gradients: the bf16 kernels' speed at bf16
        # accuracy of the LoRA term.  lora_compute_dtype=torch.float32 instead casts the activations to fp32 like
        # the reference (:320) and runs the fp32 kernels.
        self.lora_compute_dtype = lora_compute_dtype
        self.loras: List[LoraTenant] = []
        self.module = None
        self._version = 0                 # bumped whenever slot ownership changes (see _ownership)
        # packed expert parameters (reference :40): slot storage per target parameter, same tenant -> slot map
        self.target_parameter_manager = ExpertLoraManager(max_loras=max_loras, max_r=max_r)

    def patch_target_parameters(self, module, target_parameters):
        """Slot storage for packed expert parameters such as ``gate_up_proj`` / ``down_proj`` (reference :151-152)."""
        self.target_parameter_manager.patch(module, target_parameters)

    def get_target_parameter_trainable_parameters(self, tenant_adapter_name):
        return dict(self.target_parameter_manager.named_slot_parameters(tenant_adapter_name))

    @staticmethod
    def _is_target_parameter_lora_name(name: str) -> bool:
        return '._twinkle_lora_' in name

    # ------------------------------------------------------------------ slots
    def _get_available_lora(self) -> Optional[LoraTenant]:
        return next((t for t in self.loras if t.tenant_adapter_name is None), None)

    def _count_available_loras(self) -> int:
        return sum(1 for t in self.loras if t.tenant_adapter_name is None)

    def has_lora(self, adapter_name: str) -> bool:
        return any(t.tenant_adapter_name == adapter_name for t in self.loras)

    def find_lora_by_tenant(self, tenant_adapter_name) -> LoraTenant:
        for t in self.loras:
            if t.tenant_adapter_name == tenant_adapter_name:
                return t
        raise ValueError(f'No lora found for tenant {tenant_adapter_name}')

    def find_lora(self, adapter_name) -> LoraTenant:
        for t in self.loras:
            if t.adapter_name == adapter_name:
                return t
        raise ValueError(f'No lora found for real adapter_name {adapter_name}')

    def acquire_lora(self, tenant_adapter_name: str, config) -> str:
        """Give the tenant the first free slot (reference :209-226; same exceptions)."""
        if self.has_lora(tenant_adapter_name):
            raise ValueError(f'Lora {tenant_adapter_name} already exists')
        slot = self._get_available_lora()
        if slot is None:
            raise RuntimeError(f'No lora available for tenant {tenant_adapter_name}. Max loras: {self.max_loras}')
        if config.r > self.max_r:
            raise RuntimeError(f'Too big rank for lora: {config.r}')
        slot.tenant_config = config
        slot.tenant_adapter_name = tenant_adapter_name
        if getattr(config, 'target_parameters', None):
            self.target_parameter_manager.acquire(tenant_adapter_name=tenant_adapter_name, slot_name=slot.adapter_name,
                                                  config=config)
        self._version += 1
        return slot.adapter_name

    def release_lora(self, tenant_adapter_name: str) -> Optional[str]:
        """Free the tenant's slot: A back to its saved initial values, B to zero (reference :228-237)."""
        try:
            slot = self.find_lora_by_tenant(tenant_adapter_name)
        except ValueError:
            return None
        slot.tenant_config = None
        slot.tenant_adapter_name = None
        self._load_initial_weights(slot.adapter_name)
        self.target_parameter_manager.release(tenant_adapter_name)
        self._version += 1
        return None

    def check_length(self, inputs) -> None:
        total_length = sum(len(i['input_ids']) for i in inputs)
        if total_length > self.max_length:
            raise ValueError(f'Max length exceeds {self.max_length}')

    # ------------------------------------------------------- target matching
    @staticmethod
    def match_target_modules(module_name: str, target_modules: Optional[Union[List[str], str]]) -> bool:
        """Does a tenant's ``target_modules`` select this layer?  Same rules as reference :256-287."""
        if target_modules is None:
            return False
        many = isinstance(target_modules, (list, set))
        if many and len(target_modules) == 0:
            return False
        if target_modules == 'all-linear' or (many and len(target_modules) == 1
                                              and next(iter(target_modules)) == 'all-linear'):
            return True
        name = module_name
        if '.lora_' in name:  # a parameter name such as "...proj.lora_A.default.weight"
            name = re.sub(r'\.lora_\w+(\.[\w-]+)*$', '', name)
        if isinstance(target_modules, str):
            return re.fullmatch(target_modules, name) is not None
        if many:
            return any(name.endswith(t) for t in target_modules)
        return False

    # --------------------------------------------------------- activation
    def _modules(self):
        return self.module if isinstance(self.module, list) else [self.module]

    def activate_adapter(self, tenant_adapter_name: str, call_enable=False):
        if not self.has_lora(tenant_adapter_name):
            raise ValueError(f'Adapter {tenant_adapter_name} does not exist')
        adapter_name = self.find_lora_by_tenant(tenant_adapter_name).adapter_name
        for m in self._modules():
            if call_enable:
                m.enable_adapter_layers()
            if getattr(m, 'active_adapter', None) != adapter_name:
                m.set_adapter(adapter_name)

    def deactivate_adapter(self):
        for m in self._modules():
            m.disable_adapter_layers()

    def reset_adapter_status(self):
        for m in self._modules():
            m.set_adapter('lora_0')

    @contextmanager
    def adapter(self, tenant_adapter_name: str, disable_lora: bool = False):
        """One tenant for every row of the calls inside (reference :154-163)."""
        self.activate_adapter(tenant_adapter_name)
        try:
            with self.target_parameter_manager.adapter(tenant_adapter_name, disable_lora=disable_lora):
                if disable_lora:
                    with self._disable_lora_context(tenant_adapter_name):
                        yield self.find_lora_by_tenant(tenant_adapter_name).adapter_name
                else:
                    yield self.find_lora_by_tenant(tenant_adapter_name).adapter_name
        finally:
            _path_state(self).uniform_tables.clear()

    @contextmanager
    def _disable_lora_context(self, tenant_adapter_name):
        self.deactivate_adapter()
        try:
            yield
        finally:
            self.activate_adapter(tenant_adapter_name, call_enable=True)

    def batch(self, tenant_adapter_names: Sequence[str], row_tenant: torch.Tensor, check: bool = False):
        """Many tenants in one forward/backward: row ``i`` uses ``tenant_adapter_names[row_tenant[i]]`` (see the
        module-level :func:`batch`, which this calls).  No counterpart in the reference, whose ``adapter()``
        activates one tenant per call."""
        return batch(self, tenant_adapter_names, row_tenant, check)

    @property
    def _batch_table(self) -> Optional[SegmentTable]:
        return _path_state(self).batch_table

    # ------------------------------------------------------------- patching
    def _groups_for(self, layer, only_slot=None, x_dtype=None) -> Optional[AdapterGroups]:
        return _groups_for(self, layer, only_slot, x_dtype)

    def _patch_lora_forward(_self, name, base_layer):
        """Rebind ``forward`` on one LoRA layer (reference :289-331, Linear branch)."""
        if not (_is_lora_layer(base_layer) and hasattr(base_layer, 'in_features')):
            return

        def _linear_forward(self, x: torch.Tensor, *args, **kwargs) -> torch.Tensor:
            shared = getattr(self, '_tk_shared_inputs', None)
            if shared is None or args or kwargs:
                return _forward_one(self, x, *args, **kwargs)
            # a sibling has computed this layer's output from the same tensor already, or this call computes
            # the outputs of all siblings (see MultiLora.share_inputs)
            self._check_forward_args(x)
            out = shared.take(self, x)
            if out is None:
                outs = forward_shared(_self, shared.layers, x)
                shared.fill(x, outs, self)
                out = outs[shared.layers.index(self)]
            return out

        def _forward_one(self, x: torch.Tensor, *args, **kwargs) -> torch.Tensor:
            self._check_forward_args(x, *args, **kwargs)
            if _path_state(_self).batch_table is None and not self.disable_adapters:
                # the reference adds the term of every active adapter the layer has, one after the other
                # (:306-326); one is the usual case, the others are added onto its result the same way
                active = [n for n in self.active_adapters if n in self.lora_A.keys()]
                if len(active) > 1:
                    out = _with_slot(self, x, active[0], None, args, kwargs)
                    for slot in active[1:]:
                        out = _with_slot(self, x, slot, out, (), {})
                    return out
            return _with_slot(self, x, None, None, args, kwargs)

        def _with_slot(self, x, forced_slot, onto, args, kwargs):
            """The layer's output with one adapter's term (``forced_slot``; ``None``: the open batch, or the first
            active adapter) added onto ``onto`` (``None``: onto the base layer's output)."""
            table = _path_state(_self).batch_table
            only_slot = None
            if table is None:
                # one adapter per call: the active slot, if this layer has it (reference :306-309)
                active = [n for n in self.active_adapters if n in self.lora_A.keys()]
                only_slot = forced_slot if forced_slot is not None else (active[0] if active else None)
            skip = self.disable_adapters or (table is None and only_slot is None)
            groups = None if skip else _groups_for(
                _self, self, only_slot if table is None else getattr(table, 'live_slots', None), x.dtype)
            if groups is None:
                return self.base_layer(x, *args, **kwargs) if onto is None else onto

            wdtype = groups.dtype    # what the kernels take as activations: the adapters' dtype, or bf16 (see _groups_for)
            xw = self._cast_input_dtype(x, wdtype)
            xw = _slot_dropout(_self, self, only_slot, table)(xw)
            x2 = xw.reshape(-1, xw.shape[-1])
            if x2.stride(-1) != 1 or (x2.shape[0] > 1 and x2.stride(0) < x2.shape[1]):
                x2 = x2.contiguous()
            if table is None:
                table = _table_for(_self, x2.shape[0], _self.find_lora(only_slot).index, x2.device)
            elif table.rows != x2.shape[0]:
                raise ValueError(f'batch() was given {table.rows} rows but layer {self.layer_name} sees {x2.shape[0]}')

            base = self.base_layer
            plain = (onto is None and type(base) is torch.nn.Linear and not args and not kwargs and xw is x
                     and x.dtype == wdtype and base.weight.dtype == wdtype and not base._forward_hooks
                     and not base._forward_pre_hooks)
            if plain:
                y2 = multi_lora_linear(x2, base.weight, base.bias, table, groups)
                return y2.reshape(*x.shape[:-1], y2.shape[-1])

            result = base(x, *args, **kwargs) if onto is None else onto
            result_dtype = result.dtype
            if result_dtype == wdtype and result.is_contiguous():
                y2 = multi_lora_delta(x2, result.view(-1, result.shape[-1]), table, groups)
                return y2.view(result.shape)
            delta = multi_lora_delta(x2, torch.zeros(x2.shape[0], groups.out_features, dtype=wdtype, device=x2.device),
                                     table, groups)
            return (result + delta.view(*result.shape[:-1], -1)).to(result_dtype)

        base_layer.forward = MethodType(_linear_forward, base_layer)
        base_layer._tk_forward_one = MethodType(_forward_one, base_layer)   # this layer alone, whatever it shares
        base_layer.layer_name = name

    def share_inputs(self, layer_groups: Sequence[Sequence]) -> None:
        """Declare groups of patched layers that read the same tensor (see the module-level :func:`share_inputs`)."""
        share_inputs(self, layer_groups)

    def unshare_inputs(self) -> None:
        unshare_inputs(self)

    def forward_shared(self, layers: Sequence, x: torch.Tensor) -> Tuple[torch.Tensor, ...]:
        """``tuple(layer(x) for layer in layers)`` with one shared LoRA call (see the module-level
        :func:`forward_shared`)."""
        return forward_shared(self, layers, x)

    def patch(self, module, target_modules='all-linear', *args, **kwargs):
        """Pre-allocate ``max_loras`` slots of rank ``max_r`` on ``module`` and patch every LoRA layer.

        Follows reference :477-556: slots are named ``lora_0 .. lora_{max_loras-1}``,
        built from ``lora_config`` (default ``r=max_r, lora_alpha=32``), every LoRA
        parameter is trainable.  With PEFT installed a ``PeftModel`` can be passed
        and is used as is; otherwise the in-tree container is injected.
        """
        for i in range(self.max_loras):
            config = kwargs.get('lora_config', None)
            if config is None:
                config = LoraConfig(r=self.max_r, target_modules=target_modules, lora_alpha=32,
                                    exclude_modules=['o_a_proj'])
            slot = LoraTenant(index=i, adapter_name=f'lora_{i}', config=config)
            self.loras.append(slot)
            if hasattr(module, 'add_adapter') and hasattr(module, 'peft_config'):
                module.add_adapter(slot.adapter_name, config)
            else:
                module = inject_adapter(module, config, slot.adapter_name)
            for name, sub in module.named_modules():
                if _is_lora_layer(sub):
                    self._patch_lora_forward(name, sub)
        for name, param in module.named_parameters():
            if 'lora_' in name and not param.requires_grad:
                param.requires_grad_(True)
        self.module = module
        return module

    # --------------------------------------------------- weights and state
    @staticmethod
    def _slice_rank_tensor(name: str, tensor, rank: int):
        if tensor is None:
            return None
        if 'embedding_A' in name:
            return tensor[:, :rank]
        if 'embedding_B' in name:
            return tensor[:rank, :]
        if '_A' in name:
            return tensor[:rank, :]
        if '_B' in name:
            return tensor[:, :rank]
        return tensor

    @staticmethod
    def _copy_rank_tensor(name: str, target, value):
        if target is None or value is None:
            return None
        if 'embedding_A' in name:
            target[:, :value.shape[1]].copy_(value)
        elif 'embedding_B' in name:
            target[:value.shape[0], :].copy_(value)
        elif '_A' in name:
            target[:value.shape[0], :].copy_(value)
        elif '_B' in name:
            target[:, :value.shape[1]].copy_(value)
        else:
            target.copy_(value)
        return target

    def _named_parameters(self):
        for m in self._modules():
            yield from m.named_parameters()

    def save_initial_weights(self):
        """Keep a CPU copy of every slot's initial A (reference :558-574)."""
        for slot in self.loras:
            pattern = re.compile(rf'\.lora_(?:A|embedding_A)\.{re.escape(slot.adapter_name)}\.')
            for name, p in self._named_parameters():
                if pattern.search(name):
                    slot.lora_A_weights[name] = p.detach().clone().to('cpu')

    def _load_initial_weights(self, origin_adapter_name):
        slot = self.find_lora(origin_adapter_name)
        pat_a = re.compile(rf'\.lora_(?:A|embedding_A)\.{re.escape(origin_adapter_name)}\.')
        pat_b = re.compile(rf'\.lora_(?:B|embedding_B)\.{re.escape(origin_adapter_name)}\.')
        if self.module is None:
            return
        with torch.no_grad():
            for name, p in self._named_parameters():
                if pat_a.search(name) and name in slot.lora_A_weights:
                    p.copy_(slot.lora_A_weights[name].to(device=p.device, dtype=p.dtype))
                if pat_b.search(name):
                    p.zero_()

    def set_state_dict(self, tenant_adapter_name, state_dict):
        """Load rank-sliced tensors into the prefix of the tenant's slot (reference :676-699)."""
        slot = self.find_lora_by_tenant(tenant_adapter_name)
        pattern = re.compile(rf'\.lora_\w+\.{re.escape(slot.adapter_name)}\.')
        with torch.no_grad():
            for name, p in self._named_parameters():
                if self._is_target_parameter_lora_name(name):
                    continue
                if pattern.search(name) and self.match_target_modules(name, slot.tenant_config.target_modules):
                    key = name.replace(f'.{slot.adapter_name}.', '.')
                    src = state_dict[key].to(dtype=p.dtype, device=p.device)
                    self._copy_rank_tensor(name, p.data, src)
        if tenant_adapter_name in self.target_parameter_manager.tenant_to_slot:
            self.target_parameter_manager.set_state_dict(tenant_adapter_name, state_dict)

    def get_state_dict(self, tenant_adapter_name):
        """Tenant's live ``[:r]`` blocks under slot-free names (reference :701-729)."""
        slot = self.find_lora_by_tenant(tenant_adapter_name)
        pattern = re.compile(rf'\.lora_\w+\.{re.escape(slot.adapter_name)}\.')
        out = {}
        for name, p in self._named_parameters():
            if self._is_target_parameter_lora_name(name):
                continue
            if pattern.search(name) and self.match_target_modules(name, slot.tenant_config.target_modules):
                out[name.replace(f'.{slot.adapter_name}.', '.')] = self._slice_rank_tensor(name, p.detach(),
                                                                                           slot.tenant_config.r)
        if tenant_adapter_name in self.target_parameter_manager.tenant_to_slot:
            expert_state = self.target_parameter_manager.get_state_dict(tenant_adapter_name)
            overlap = out.keys() & expert_state.keys()
            if overlap:
                raise ValueError(f'Duplicate LoRA state keys: {sorted(overlap)[:5]}')
            out.update(expert_state)
        return out

    # ---- adapter checkpoints in PEFT's on-disk format -----------------------------------------------------------
    _PEFT_PREFIX = 'base_model.'

    @classmethod
    def _peft_key(cls, key: str) -> str:
        """A state-dict key under PEFT's root: ``base_model.model.<path inside the wrapped model>...``.  The in-tree
        holder stands where ``PeftModel.base_model`` stands, so its parameter names lack only ``base_model.``; a real
        ``PeftModel``'s names and the keys of the packed expert parameters carry the root already."""
        return key if key.startswith(cls._PEFT_PREFIX) else cls._PEFT_PREFIX + key

    def save_adapter(self, tenant_adapter_name: str, checkpoint_dir: str) -> str:
        """Write the tenant's adapter as ``adapter_model.safetensors`` + ``adapter_config.json``.

        Same content as the reference's save for a tenant (transformers.py:1001-1033 with the state dict of
        multi_lora_transformers.py:265-267): the live ``[:r]`` blocks, slot name removed from the keys, on the
        CPU, contiguous.  Every key starts with ``base_model.model.`` like in PEFT's files (see :meth:`_peft_key`),
        linear layers and packed expert parameters alike, and loads with ``peft.utils.load_peft_weights``."""
        import json
        import os

        from safetensors.torch import save_file
        slot = self.find_lora_by_tenant(tenant_adapter_name)
        state = {self._peft_key(k): v.detach().to('cpu').contiguous()
                 for k, v in self.get_state_dict(tenant_adapter_name).items()}
        os.makedirs(checkpoint_dir, exist_ok=True)
        save_file(state, os.path.join(checkpoint_dir, 'adapter_model.safetensors'))
        cfg = slot.tenant_config
        target = cfg.target_modules
        config = {
            'peft_type': 'LORA', 'task_type': 'CAUSAL_LM', 'base_model_name_or_path': None, 'inference_mode': True,
            'r': cfg.r, 'lora_alpha': cfg.lora_alpha, 'lora_dropout': getattr(cfg, 'lora_dropout', 0.0),
            'target_modules': sorted(target) if isinstance(target, (set, list, tuple)) else target,
            'exclude_modules': getattr(cfg, 'exclude_modules', None), 'use_rslora': bool(getattr(cfg, 'use_rslora', False)),
            'use_dora': False, 'fan_in_fan_out': False, 'bias': 'none',
            'target_parameters': getattr(cfg, 'target_parameters', None),
        }
        with open(os.path.join(checkpoint_dir, 'adapter_config.json'), 'w') as f:
            json.dump(config, f, indent=2, sort_keys=True)
        return checkpoint_dir

    def load_adapter(self, tenant_adapter_name: str, checkpoint_dir: str) -> None:
        """Read ``adapter_model.safetensors`` into the prefix of the tenant's slot (the reference's load,
        multi_lora_transformers.py:280-300: weights to the CPU first, then ``set_state_dict``); tensors saved at a
        rank below the slot's are padded by leaving the rest of the slot untouched."""
        import os

        from safetensors.torch import load_file
        state = load_file(os.path.join(checkpoint_dir, 'adapter_model.safetensors'), device='cpu')
        # the linear layers are looked up under the names this model's parameters have (holder-relative when the
        # holder is the in-tree one), the packed expert parameters under PEFT's absolute names: offer both
        n = len(self._PEFT_PREFIX)
        relative = {k[n:]: v for k, v in state.items() if k.startswith(self._PEFT_PREFIX)}
        self.set_state_dict(tenant_adapter_name, {**relative, **state})

    def get_nb_trainable_parameters(self, tenant_adapter_name):
        """(trainable, all) parameter counts as the tenant sees them (reference :756-813)."""
        slot = self.find_lora_by_tenant(tenant_adapter_name)
        pattern = re.compile(rf'\.lora_\w+\.{re.escape(slot.adapter_name)}\.')
        trainable = total = 0
        for name, p in self._named_parameters():
            mine = pattern.search(name) is not None
            if not mine and 'lora_' in name:
                continue
            if mine and not self.match_target_modules(name, slot.tenant_config.target_modules):
                continue
            n = self._slice_rank_tensor(name, p, slot.tenant_config.r).numel() if mine else p.numel()
            total += n
            if p.requires_grad:
                trainable += n
        return trainable, total

    def get_trainable_parameters_example(self, tenant_adapter_name):
        """First and last five trainable parameter names of the tenant, slot name replaced by the tenant's
        (reference :815-837)."""
        slot = self.find_lora_by_tenant(tenant_adapter_name)
        pattern = re.compile(rf'\.lora_\w+\.{re.escape(slot.adapter_name)}\.')
        names = []
        for name, p in self._named_parameters():
            if p.requires_grad and pattern.search(name) and \
                    self.match_target_modules(name, slot.tenant_config.target_modules):
                for side in ('A', 'B'):
                    name = name.replace(f'{side}.{slot.adapter_name}', f'{side}.{tenant_adapter_name}')
                names.append(name)
        return '\n'.join(names[:5] + ['...'] + names[-5:])

    # ---- per-tensor converters of a checkpoint stream (one parameter at a time) ----------------------------------
    def save_lora_converter(self, name, parameter, adapter_name):
        """``(key, tensor)`` to write for one parameter of slot ``adapter_name``, or ``None`` to skip it: other
        slots' weights are dropped, the slot's own are cut to the tenant's rank and lose the slot name
        (reference :659-674)."""
        slot = self.find_lora(adapter_name)
        if re.search(r'\.lora_\w+\.\w+\.', name) and not re.search(rf'\.lora_\w+\.{re.escape(adapter_name)}\.', name):
            return None
        if not re.search(rf'\.lora_\w+\.({re.escape(adapter_name)}|weight)', name):
            return None
        tensor = self._slice_rank_tensor(name, parameter.detach() if hasattr(parameter, 'detach') else parameter,
                                         slot.tenant_config.r)
        return name.replace(f'.{slot.adapter_name}.', '.'), (tensor.clone() if tensor is not None else None)

    def load_lora_converter(self, name, parameter, **kwargs):
        """``(name, tensor)`` with a rank-``r`` LoRA tensor zero-padded to the slot's ``max_r`` (reference :576-608,
        the linear branches: A grows by rows, B by columns)."""
        if '_A' in name and parameter.shape[0] < self.max_r:
            pad = torch.zeros(self.max_r - parameter.shape[0], parameter.shape[1], dtype=parameter.dtype,
                              device=parameter.device)
            parameter = torch.cat((parameter, pad), dim=0)
        elif '_B' in name and parameter.shape[1] < self.max_r:
            pad = torch.zeros(parameter.shape[0], self.max_r - parameter.shape[1], dtype=parameter.dtype,
                              device=parameter.device)
            parameter = torch.cat((parameter, pad), dim=1)
        return name, parameter
