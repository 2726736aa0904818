"""Host-side mirror of the reference's MultiLora / target-parameter LoRA bookkeeping (no GPU needed)."""
import pytest
import torch
from torch import nn

import oracle
from twinkle_amd import LoraConfig, LoraLinear, MultiLora
from twinkle_amd.expert_lora import ExpertLoraSlots


class TinyBlock(nn.Module):

    def __init__(self, d=16, f=24):
        super().__init__()
        self.q_proj = nn.Linear(d, d, bias=False)
        self.up_proj = nn.Linear(d, f, bias=True)
        self.down_proj = nn.Linear(f, d, bias=False)

    def forward(self, x):
        return self.down_proj(torch.relu(self.up_proj(self.q_proj(x))))


def _patched(max_loras=3, max_r=8):
    torch.manual_seed(0)
    ml = MultiLora(max_loras=max_loras, max_r=max_r)
    model = ml.patch(TinyBlock(), target_modules='all-linear')
    ml.save_initial_weights()
    return ml, model


def test_patch_preallocates_slots_at_max_rank():
    ml, model = _patched()
    assert [t.adapter_name for t in ml.loras] == ['lora_0', 'lora_1', 'lora_2']
    layers = [m for m in model.modules() if isinstance(m, LoraLinear)]
    assert len(layers) == 3
    for layer in layers:
        assert set(layer.lora_A.keys()) == {'lora_0', 'lora_1', 'lora_2'}
        assert layer.lora_A['lora_1'].weight.shape == (8, layer.in_features)
        assert layer.lora_B['lora_1'].weight.shape == (layer.out_features, 8)
        assert torch.count_nonzero(layer.lora_B['lora_2'].weight) == 0       # B starts at zero
        assert hasattr(layer, 'layer_name')
    assert all(p.requires_grad for n, p in model.named_parameters() if 'lora_' in n)
    assert not any(p.requires_grad for n, p in model.named_parameters() if 'lora_' not in n)


def test_acquire_release_and_errors():
    """Same exceptions as the reference (multi_lora.py:128, :211-216, :247)."""
    ml, _ = _patched(max_loras=2, max_r=8)
    cfg = LoraConfig(r=4, lora_alpha=8, target_modules='all-linear')
    assert ml.acquire_lora('alice', cfg) == 'lora_0'
    assert ml.acquire_lora('bob', cfg) == 'lora_1'
    with pytest.raises(ValueError):
        ml.acquire_lora('alice', cfg)                      # duplicate tenant
    with pytest.raises(RuntimeError):
        ml.acquire_lora('carol', cfg)                      # no free slot
    ml.release_lora('alice')
    with pytest.raises(RuntimeError):
        ml.acquire_lora('carol', LoraConfig(r=16, lora_alpha=8, target_modules='all-linear'))   # r > max_r
    assert ml.acquire_lora('carol', cfg) == 'lora_0'       # first free slot is reused
    with pytest.raises(ValueError):
        ml.find_lora_by_tenant('alice')
    with pytest.raises(ValueError):
        ml.activate_adapter('nobody')
    assert ml.release_lora('nobody') is None               # unknown tenant: silently ignored, as in the reference
    with pytest.raises(ValueError):
        ml.check_length([{'input_ids': [0] * 5000}, {'input_ids': [0] * 5000}])


def test_release_restores_initial_a_and_zeroes_b():
    """Reference invariant (tests/model/test_multi_lora_target_parameters.py:103-134, and multi_lora.py:731-754)."""
    ml, model = _patched()
    ml.acquire_lora('alice', LoraConfig(r=4, lora_alpha=8, target_modules='all-linear'))
    before = {n: p.detach().clone() for n, p in model.named_parameters() if '.lora_0.' in n}
    with torch.no_grad():
        for n, p in model.named_parameters():
            if '.lora_0.' in n:
                p.add_(1.0)
    ml.release_lora('alice')
    for n, p in model.named_parameters():
        if '.lora_A.lora_0.' in n:
            assert torch.equal(p, before[n])
        if '.lora_B.lora_0.' in n:
            assert torch.count_nonzero(p) == 0


def test_state_dict_is_rank_sliced_renamed_and_round_trips():
    """Slicing / renaming of multi_lora.py:85-113, :676-729; round trip as in the reference test :188-213."""
    ml, model = _patched()
    ml.acquire_lora('alice', LoraConfig(r=4, lora_alpha=8, target_modules=['q_proj', 'down_proj']))
    with torch.no_grad():
        for n, p in model.named_parameters():
            if '.lora_0.' in n:
                p.uniform_(-0.1, 0.1)
    sd = ml.get_state_dict('alice')
    assert set(sd) == {'model.q_proj.lora_A.weight', 'model.q_proj.lora_B.weight', 'model.down_proj.lora_A.weight',
                       'model.down_proj.lora_B.weight'}
    assert sd['model.q_proj.lora_A.weight'].shape == (4, 16) and sd['model.q_proj.lora_B.weight'].shape == (16, 4)
    ml2, model2 = _patched()
    ml2.acquire_lora('zed', LoraConfig(r=4, lora_alpha=8, target_modules='all-linear'))
    ml2.acquire_lora('alice', LoraConfig(r=4, lora_alpha=8, target_modules=['q_proj', 'down_proj']))   # lands in lora_1
    ml2.set_state_dict('alice', sd)
    sd2 = ml2.get_state_dict('alice')
    for k in sd:
        assert torch.equal(sd[k], sd2[k])
    # only the live [:r] block of the slot was written
    a_full = dict(model2.named_parameters())['model.q_proj.lora_A.lora_1.weight']
    assert torch.equal(a_full[:4], sd['model.q_proj.lora_A.weight'])
    for name, t in [('m.lora_A.weight', torch.randn(8, 5)), ('m.lora_B.weight', torch.randn(5, 8))]:
        assert torch.equal(MultiLora._slice_rank_tensor(name, t, 3), oracle.slice_rank_tensor(name, t, 3))
    trainable, total = ml.get_nb_trainable_parameters('alice')
    assert trainable == 4 * 16 + 16 * 4 + 4 * 24 + 16 * 4


def test_match_target_modules_agrees_with_oracle():
    cases = [('model.layers.0.q_proj', None), ('x', []), ('a', 'all-linear'), ('a', ['all-linear']),
             ('model.layers.0.attn.proj', ['attn.proj']), ('model.layers.0.attn.proj', ['mlp.up']),
             ('model.layers.0.attn.proj.lora_A.default.weight', ['attn.proj']), ('model.layers.3.q_proj', r'.*\.q_proj'),
             ('model.layers.3.k_proj', r'.*\.q_proj'), ('m.q_proj', {'q_proj'})]
    for name, tm in cases:
        assert MultiLora.match_target_modules(name, tm) == oracle.match_target_modules(name, tm)


def test_adapter_context_selects_the_slot():
    ml, model = _patched()
    ml.acquire_lora('alice', LoraConfig(r=4, lora_alpha=8, target_modules='all-linear'))
    ml.acquire_lora('bob', LoraConfig(r=8, lora_alpha=8, target_modules='all-linear'))
    with ml.adapter('bob') as slot:
        assert slot == 'lora_1' and model.active_adapter == 'lora_1'
        assert all(m.active_adapters == ['lora_1'] for m in model.modules() if isinstance(m, LoraLinear))
    with ml.adapter('alice', disable_lora=True):
        assert all(m.disable_adapters for m in model.modules() if isinstance(m, LoraLinear))
        x = torch.randn(3, 16)
        assert torch.equal(model(x), model.model.down_proj.base_layer(
            torch.relu(model.model.up_proj.base_layer(model.model.q_proj.base_layer(x)))))   # base only, runs on CPU
    assert not any(m.disable_adapters for m in model.modules() if isinstance(m, LoraLinear))


def test_expert_slots_follow_the_reference_rules():
    """Checks of multi_lora_target_parameters.py:136-156 and the state-dict shape rules :232-278."""
    torch.manual_seed(0)
    slots = ExpertLoraSlots(num_experts=2, in_features=4, out_features=12, max_loras=2, max_r=4, key_prefix='m.experts')
    assert slots.lora_A['lora_0'].shape == (2, 4, 4) and slots.lora_B['lora_1'].shape == (2, 12, 4)
    assert torch.count_nonzero(slots.lora_B['lora_0']) == 0
    assert slots.lora_A['lora_0'].abs().max() <= 1.0
    with pytest.raises(ValueError):
        slots.configure_slot('lora_9', LoraConfig(r=2, lora_alpha=4))
    with pytest.raises(ValueError):
        slots.configure_slot('lora_0', LoraConfig(r=0, lora_alpha=4))
    with pytest.raises(ValueError):
        slots.configure_slot('lora_0', LoraConfig(r=8, lora_alpha=4))
    for bad in (dict(lora_dropout=0.1), dict(fan_in_fan_out=True), dict(use_dora=True), dict(lora_bias=True)):
        with pytest.raises(ValueError):
            slots.configure_slot('lora_0', LoraConfig(r=2, lora_alpha=4, **bad))
    slots.configure_slot('lora_0', LoraConfig(r=2, lora_alpha=4))
    slots.configure_slot('lora_1', LoraConfig(r=4, lora_alpha=4, use_rslora=True))
    assert slots.scaling['lora_0'] == 2.0 and slots.scaling['lora_1'] == 2.0 and slots.r['lora_0'] == 2
    with torch.no_grad():
        slots.lora_A['lora_0'].uniform_(-0.1, 0.1)
        slots.lora_B['lora_0'].uniform_(-0.1, 0.1)
    dw = slots.get_delta_weight('lora_0')
    want = oracle.expert_delta_weight(slots.lora_A['lora_0'].detach(), slots.lora_B['lora_0'].detach(), 2, 2.0)
    assert torch.allclose(dw, want) and dw.shape == (2, 12, 4)
    assert slots.get_delta_weight('lora_0', out_in_layout=False).shape == (2, 4, 12)
    sd = slots.get_state_dict('lora_0')
    assert sd['m.experts.lora_A.weight'].shape == (2, 2, 4) and sd['m.experts.lora_B.weight'].shape == (2, 12, 2)
    other = ExpertLoraSlots(2, 4, 12, 2, 4, key_prefix='m.experts')
    other.configure_slot('lora_1', LoraConfig(r=2, lora_alpha=4))
    assert other.set_state_dict('lora_1', sd) == set(sd)
    assert torch.allclose(other.get_delta_weight('lora_1'), dw, atol=1e-6)       # reference round-trip bar: atol 1e-6
    with pytest.raises(KeyError):
        other.set_state_dict('lora_1', {'m.experts.lora_A.weight': sd['m.experts.lora_A.weight']})
    with pytest.raises(ValueError):
        other.set_state_dict('lora_1', {k: v[:1] for k, v in sd.items()})
    a0 = slots._first_A['lora_0'].clone()
    slots.reset_slot('lora_0')
    assert torch.equal(slots.lora_A['lora_0'].detach(), a0) and torch.count_nonzero(slots.lora_B['lora_0']) == 0


def test_custom_ops_are_registered_and_traceable():
    """torch.ops.twinkle_amd.* exist, declare their mutations, and their fake kernels give exact shapes."""
    import twinkle_amd  # noqa: F401
    from torch._subclasses.fake_tensor import FakeTensorMode
    from twinkle_amd import _lib
    for name in ('segment_build', 'lora_fwd', 'lora_bwd', 'lora_fwd_shared', 'lora_bwd_shared'):
        assert hasattr(torch.ops.twinkle_amd, name)
    schema = str(torch.ops.twinkle_amd.lora_fwd_shared.default._schema)
    assert '!)[] ys' in schema and '!)[] hs' in schema
    schema = str(torch.ops.twinkle_amd.lora_bwd_shared.default._schema)
    assert '!) dx' in schema and '!)[] grad_a' in schema and '!)[] grad_b' in schema and '!)[] workspaces' in schema
    schema = str(torch.ops.twinkle_amd.lora_fwd.default._schema)
    assert 'Tensor(a1!) y' in schema and 'Tensor(a2!) h' in schema
    schema = str(torch.ops.twinkle_amd.lora_bwd.default._schema)
    for arg in ('dx', 'grad_a', 'grad_b', 'workspace'):
        assert f'!) {arg}' in schema
    with FakeTensorMode():
        keys = torch.empty(1000, dtype=torch.int32)
        ws = torch.ops.twinkle_amd.segment_build(keys, 7)
    assert ws.dtype == torch.uint8 and ws.numel() == _lib.load().tk_segment_workspace_bytes(1000, 7)
    with pytest.raises(RuntimeError, match='GPU'):
        torch.ops.twinkle_amd.segment_build(torch.zeros(4, dtype=torch.int32), 2)


def test_adapter_checkpoint_round_trip_in_peft_format(tmp_path):
    """adapter_model.safetensors holds the tenant's [:r] blocks under slot-free, PEFT-prefixed keys; loading into
    another slot (even of another MultiLora) reproduces them and leaves the rest of the slot alone."""
    import json

    from safetensors.torch import load_file

    class Tiny(nn.Module):

        def __init__(self):
            super().__init__()
            self.q_proj = nn.Linear(12, 12, bias=False)
            self.up_proj = nn.Linear(12, 20, bias=False)

        def forward(self, x):
            return self.up_proj(self.q_proj(x))

    torch.manual_seed(0)
    ml = MultiLora(max_loras=3, max_r=8)
    model = ml.patch(Tiny(), target_modules='all-linear')
    ml.save_initial_weights()
    ml.acquire_lora('alice', LoraConfig(r=4, lora_alpha=8, target_modules=['q_proj']))
    with torch.no_grad():
        for n, p in model.named_parameters():
            if 'lora_' in n:
                p.copy_(torch.randn(p.shape))
    out = ml.save_adapter('alice', str(tmp_path / 'ckpt'))
    saved = load_file(f'{out}/adapter_model.safetensors')
    # key and shape KAT: PEFT layout, rank-sliced, only the targeted module
    assert sorted(saved) == ['base_model.model.q_proj.lora_A.weight', 'base_model.model.q_proj.lora_B.weight']
    assert saved['base_model.model.q_proj.lora_A.weight'].shape == (4, 12)
    assert saved['base_model.model.q_proj.lora_B.weight'].shape == (12, 4)
    cfg = json.load(open(f'{out}/adapter_config.json'))
    assert cfg['peft_type'] == 'LORA' and cfg['r'] == 4 and cfg['lora_alpha'] == 8 and cfg['target_modules'] == ['q_proj']
    slot = ml.find_lora_by_tenant('alice').adapter_name
    a_src = dict(model.named_parameters())[f'model.q_proj.lora_A.{slot}.weight'].detach().clone()
    assert torch.equal(saved['base_model.model.q_proj.lora_A.weight'], a_src[:4])

    ml2 = MultiLora(max_loras=2, max_r=8)
    model2 = ml2.patch(Tiny(), target_modules='all-linear')
    ml2.save_initial_weights()
    ml2.acquire_lora('x', LoraConfig(r=2, lora_alpha=4, target_modules='all-linear'))     # takes the first slot
    ml2.acquire_lora('alice', LoraConfig(r=4, lora_alpha=8, target_modules=['q_proj']))
    slot2 = ml2.find_lora_by_tenant('alice').adapter_name
    before = dict(model2.named_parameters())[f'model.q_proj.lora_A.{slot2}.weight'].detach().clone()
    ml2.load_adapter('alice', out)
    after = dict(model2.named_parameters())[f'model.q_proj.lora_A.{slot2}.weight'].detach()
    assert torch.equal(after[:4], a_src[:4]) and torch.equal(after[4:], before[4:])
    for k, v in ml2.get_state_dict('alice').items():
        assert torch.equal(v, saved['base_model.' + k])


def test_share_inputs_bookkeeping_without_a_gpu(monkeypatch):
    """share_inputs: the first sibling that sees a tensor computes the group, the others collect; no stale results."""
    from torch import nn

    class QKV(nn.Module):
        def __init__(self):
            super().__init__()
            self.q_proj, self.k_proj, self.v_proj = nn.Linear(16, 16), nn.Linear(16, 8), nn.Linear(16, 8)

        def forward(self, x):
            return self.q_proj(x), self.k_proj(x), self.v_proj(x)

    torch.manual_seed(0)
    ml = MultiLora(max_loras=2, max_r=4)
    model = ml.patch(QKV(), target_modules='all-linear')
    ml.acquire_lora('alice', LoraConfig(r=4, lora_alpha=8, target_modules='all-linear'))
    x = torch.randn(5, 16)
    with ml.adapter('alice', disable_lora=True):                    # base path only: runs on the CPU
        want = model(x)
        calls = []
        import twinkle_amd.multi_lora as host
        original = host.forward_shared
        monkeypatch.setattr(host, 'forward_shared', lambda m, layers, t: calls.append(len(layers)) or original(m, layers, t))
        ml.share_inputs([['model.q_proj', 'model.k_proj', 'model.v_proj']])
        got = model(x)
        assert calls == [3]                                         # one group computation for three layer calls
        for a, b in zip(got, want):
            assert torch.equal(a, b)
        m = model.model
        state = m.q_proj._tk_shared_inputs
        assert state.source is None and not state.pending           # everything was collected
        # a sibling called with another tensor starts over instead of handing out a stale result
        k1 = m.k_proj(x)
        x2 = torch.randn(5, 16)
        v2 = m.v_proj(x2)
        assert torch.equal(k1, want[1]) and torch.equal(v2, torch.nn.functional.linear(x2, m.v_proj.base_layer.weight,
                                                                                      m.v_proj.base_layer.bias))
        x2.add_(1.0)                                                # same object, new version: recomputed
        assert torch.equal(m.q_proj(x2), torch.nn.functional.linear(x2, m.q_proj.base_layer.weight,
                                                                    m.q_proj.base_layer.bias))
        ml.unshare_inputs()
        assert not hasattr(m.q_proj, '_tk_shared_inputs')
    with pytest.raises(ValueError):
        ml.share_inputs([['model.q_proj']])


def test_checkpoint_stream_converters_slice_and_pad():
    """save_lora_converter cuts to the tenant's rank and renames; load_lora_converter pads back to max_r."""
    from torch import nn
    torch.manual_seed(0)
    ml = MultiLora(max_loras=2, max_r=8)
    model = ml.patch(nn.Sequential(nn.Linear(12, 6)), target_modules='all-linear')
    ml.acquire_lora('alice', LoraConfig(r=3, lora_alpha=6, target_modules='all-linear'))
    slot = ml.find_lora_by_tenant('alice').adapter_name
    other = 'lora_1' if slot == 'lora_0' else 'lora_0'
    params = dict(model.named_parameters())
    name_a = next(n for n in params if f'lora_A.{slot}.' in n)
    name_b = next(n for n in params if f'lora_B.{slot}.' in n)
    with torch.no_grad():
        params[name_b].normal_()
    key_a, a = ml.save_lora_converter(name_a, params[name_a], slot)
    key_b, b = ml.save_lora_converter(name_b, params[name_b], slot)
    assert slot not in key_a and a.shape == (3, 12) and b.shape == (6, 3)
    assert torch.equal(a, params[name_a][:3]) and torch.equal(b, params[name_b][:, :3])
    assert ml.save_lora_converter(name_a.replace(slot, other), params[name_a], slot) is None    # another slot's weight
    assert ml.save_lora_converter('model.0.base_layer.weight', params[name_a], slot) is None    # not a LoRA weight
    _, a8 = ml.load_lora_converter('x.lora_A.weight', a)
    _, b8 = ml.load_lora_converter('x.lora_B.weight', b)
    assert a8.shape == (8, 12) and b8.shape == (6, 8)
    assert torch.equal(a8[:3], a) and a8[3:].abs().sum() == 0 and torch.equal(b8[:, :3], b) and b8[:, 3:].abs().sum() == 0
    example = ml.get_trainable_parameters_example('alice')
    assert 'lora_A.alice' in example and slot not in example


# ---- packed expert parameters through MultiLora (the reference's tests/model/test_multi_lora_target_parameters.py) ----

class _PackedExperts(torch.nn.Module):
    """Two experts, hidden 4, intermediate 6; ``[E, out, in]`` storage, or ``[E, in, out]`` with is_transposed."""

    def __init__(self, is_transposed=False):
        super().__init__()
        self.is_transposed = is_transposed
        shape_gu, shape_d = ((2, 4, 12), (2, 6, 4)) if is_transposed else ((2, 12, 4), (2, 4, 6))
        self.gate_up_proj = torch.nn.Parameter(torch.randn(*shape_gu))
        self.down_proj = torch.nn.Parameter(torch.randn(*shape_d))


def _expert_model(is_transposed=False):
    from twinkle_amd import LoraTenant
    model = torch.nn.Module()
    model.mlp = torch.nn.Module()
    model.mlp.experts = _PackedExperts(is_transposed)
    model.active_adapter = 'lora_0'
    model.set_adapter = lambda name: setattr(model, 'active_adapter', name)
    model.disable_adapter_layers = lambda: None
    model.enable_adapter_layers = lambda: None
    targets = ['mlp.experts.gate_up_proj', 'mlp.experts.down_proj']
    cfg = lambda r: LoraConfig(r=r, lora_alpha=2 * r, target_modules=[], target_parameters=targets)  # noqa: E731
    ml = MultiLora(max_loras=2, max_r=4)
    ml.module = model
    ml.loras = [LoraTenant(index=i, adapter_name=f'lora_{i}', config=cfg(4)) for i in range(2)]
    ml.patch_target_parameters(model, targets)
    return ml, model, cfg


@pytest.mark.parametrize('is_transposed', [False, True])
def test_target_parameter_slots_keys_shapes_release_and_round_trip(is_transposed):
    torch.manual_seed(0)
    ml, model, cfg = _expert_model(is_transposed)
    manager = ml.target_parameter_manager
    gate_up, down = manager.wrappers
    assert (gate_up.in_features, gate_up.out_features, down.in_features, down.out_features) == (4, 12, 6, 4)
    ml.acquire_lora('adapter_a', cfg(2))
    named = dict(manager.named_slot_parameters('adapter_a'))
    assert {k: tuple(v.shape) for k, v in named.items()} == {
        'mlp.experts.gate_up_proj.lora_A.lora_0.weight': (2, 4, 4),
        'mlp.experts.gate_up_proj.lora_B.lora_0.weight': (2, 12, 4),
        'mlp.experts.down_proj.lora_A.lora_0.weight': (2, 4, 6),
        'mlp.experts.down_proj.lora_B.lora_0.weight': (2, 4, 4),
    }
    assert ml.get_target_parameter_trainable_parameters('adapter_a').keys() == named.keys()
    # the first target parameter of a module is the innermost wrapper in PEFT's nesting (reference :321-330)
    state = ml.get_state_dict('adapter_a')
    assert {k: tuple(v.shape) for k, v in state.items()} == {
        'base_model.model.mlp.experts.base_layer.lora_A.weight': (2, 2, 4),
        'base_model.model.mlp.experts.base_layer.lora_B.weight': (2, 12, 2),
        'base_model.model.mlp.experts.lora_A.weight': (2, 2, 6),
        'base_model.model.mlp.experts.lora_B.weight': (2, 4, 2),
    }
    # the merged delta has the parameter's own layout
    assert gate_up.get_delta_weight('lora_0', gate_up.out_in_layout).shape == model.mlp.experts.gate_up_proj.shape
    # state-dict round trip into a fresh model (reference test :188-213, atol 1e-6)
    with torch.no_grad():
        for p in named.values():
            p.uniform_(-0.1, 0.1)
    state = ml.get_state_dict('adapter_a')
    ml2, _, cfg2 = _expert_model(is_transposed)
    ml2.acquire_lora('adapter_a', cfg2(2))
    ml2.set_state_dict('adapter_a', state)
    for w1, w2 in zip(manager.wrappers, ml2.target_parameter_manager.wrappers):
        assert torch.allclose(w1.get_delta_weight('lora_0'), w2.get_delta_weight('lora_0'), atol=1e-6)
    # adapter() tells the manager which slot the expert modules apply, and restores what was there before
    with ml.adapter('adapter_a'):
        assert manager.active_pass.slots == ['lora_0'] and not manager.active_pass.disabled
        with ml.adapter('adapter_a', disable_lora=True):
            assert manager.active_pass.disabled
        assert not manager.active_pass.disabled
    assert manager.active_pass is None
    # release: A back to its first initialisation, B to zero (reference test :103-134)
    ml3, _, cfg3 = _expert_model(is_transposed)
    ml3.acquire_lora('adapter_a', cfg3(2))
    first = {k: v.detach().clone() for k, v in ml3.target_parameter_manager.named_slot_parameters('adapter_a')
             if '.lora_A.' in k}
    with torch.no_grad():
        for _, p in ml3.target_parameter_manager.named_slot_parameters('adapter_a'):
            p.add_(1.0)
    ml3.release_lora('adapter_a')
    for w in ml3.target_parameter_manager.wrappers:
        for k in ('lora_A', 'lora_B'):
            p = getattr(w, k)['lora_0'].detach()
            if k == 'lora_A':
                assert torch.equal(p, first[f'{w.parameter_key}.lora_A.lora_0.weight'])
            else:
                assert torch.count_nonzero(p) == 0
    with pytest.raises(ValueError):
        manager.patch(model, ['mlp.experts.down_proj'])              # another target list after patching
    with pytest.raises(ValueError):
        ml.acquire_lora('adapter_b', LoraConfig(r=2, lora_alpha=4, target_modules=[], lora_dropout=0.1,
                                                target_parameters=['mlp.experts.down_proj']))


def test_grouped_gemm_applicability():
    """experts_forward takes the grouped GEMMs only for frozen bf16 weights whose widths are multiples of 128."""
    from twinkle_amd.expert_lora import grouped_gemm_applies
    rows = torch.zeros(4, 256, dtype=torch.bfloat16)
    ok = torch.nn.Parameter(torch.zeros(3, 384, 256, dtype=torch.bfloat16), requires_grad=False)
    assert grouped_gemm_applies(ok, rows)
    assert not grouped_gemm_applies(torch.nn.Parameter(ok.detach().clone()), rows)                 # trainable
    assert not grouped_gemm_applies(ok.float(), rows.float())                                       # fp32
    assert not grouped_gemm_applies(torch.zeros(3, 384, 192, dtype=torch.bfloat16), rows)          # in = 192
    assert not grouped_gemm_applies(torch.zeros(3, 320, 256, dtype=torch.bfloat16), rows)          # out = 320
    assert not grouped_gemm_applies(ok.transpose(1, 2), rows)                                       # not contiguous


# ---- the documented way of installing the path into the reference's own MultiLora ------------------------------------

class ReferenceSurfaceMultiLora:
    """An object with the attributes and methods of the reference's ``MultiLora`` (src/twinkle/model/multi_lora.py:
    33-40 ``__init__``, :209-254 ``acquire_lora / release_lora / find_lora*``, :256-287 ``match_target_modules``,
    :126-163 ``activate_adapter / adapter``) and nothing of this package's own class."""

    def __init__(self, module, max_loras, max_r):
        from twinkle_amd import LoraTenant
        self.max_loras, self.max_r, self.max_length = max_loras, max_r, 8192
        self.module = module
        self.loras = [LoraTenant(index=i, adapter_name=f'lora_{i}', config=None) for i in range(max_loras)]

    def has_lora(self, name):
        return any(t.tenant_adapter_name == name for t in self.loras)

    def find_lora_by_tenant(self, name):
        found = [t for t in self.loras if t.tenant_adapter_name == name]
        if not found:
            raise ValueError(f'No lora found for tenant {name}')
        return found[0]

    def find_lora(self, adapter_name):
        found = [t for t in self.loras if t.adapter_name == adapter_name]
        if not found:
            raise ValueError(f'No lora found for real adapter_name {adapter_name}')
        return found[0]

    def acquire_lora(self, tenant, config):
        free = [t for t in self.loras if t.tenant_adapter_name is None]
        if self.has_lora(tenant):
            raise ValueError(f'Lora {tenant} already exists')
        if not free or config.r > self.max_r:
            raise RuntimeError('no slot / rank too big')
        free[0].tenant_adapter_name, free[0].tenant_config = tenant, config
        return free[0].adapter_name

    def release_lora(self, tenant):
        slot = self.find_lora_by_tenant(tenant)
        slot.tenant_adapter_name = slot.tenant_config = None

    match_target_modules = staticmethod(oracle.match_target_modules)

    def adapter(self, tenant, disable_lora=False):
        from contextlib import contextmanager

        @contextmanager
        def ctx():
            self.module.set_adapter(self.find_lora_by_tenant(tenant).adapter_name)
            if disable_lora:
                self.module.disable_adapter_layers()
            try:
                yield
            finally:
                if disable_lora:
                    self.module.enable_adapter_layers()
        return ctx()


def reference_surface_setup(device='cpu', dtype=torch.float32):
    """TinyBlock with three slots of rank 8 injected, held by an object that has only the reference's surface."""
    from twinkle_amd import inject_adapter
    torch.manual_seed(0)
    holder = TinyBlock().to(dtype).to(device)
    for i in range(3):
        holder = inject_adapter(holder, LoraConfig(r=8, lora_alpha=32, target_modules='all-linear'), f'lora_{i}')
    ref = ReferenceSurfaceMultiLora(holder, max_loras=3, max_r=8)
    with torch.no_grad():
        for n, p in holder.named_parameters():
            if '.lora_B.' in n:
                p.normal_(0, 0.05)
    return ref, holder


def test_use_mi355x_path_on_an_object_with_only_the_reference_surface():
    """The installer of twinkle_amd.integration needs nothing but the reference's MultiLora surface: after it, a
    forward under adapter() gets as far as the HIP op (which refuses CPU tensors), disable_lora gives the base
    model, and acquire / release through the object's own methods are seen without any notification."""
    import twinkle_amd
    ref, holder = reference_surface_setup()
    assert not hasattr(ref, '_groups_for') and not hasattr(ref, 'batch') and not hasattr(ref, '_version')
    twinkle_amd.use_mi355x_path(ref)
    x = torch.randn(6, 16)
    base_only = TinyBlock.forward(holder.model, x)         # no tenant holds the active slot: LoRA is skipped
    assert torch.isfinite(base_only).all()
    ref.acquire_lora('alice', LoraConfig(r=4, lora_alpha=8, target_modules='all-linear'))
    with ref.adapter('alice', disable_lora=True):
        assert torch.equal(holder(x), base_only)
    with ref.adapter('alice'):
        with pytest.raises(RuntimeError, match='GPU'):     # reached the op: the path has no CPU implementation
            holder(x)
    with pytest.raises(RuntimeError, match='GPU'):
        with twinkle_amd.batch(ref, ['alice'], torch.zeros(6, dtype=torch.long)):
            holder(x)
    ref.release_lora('alice')                              # the slot is free again: base output, no op call
    holder.set_adapter('lora_0')
    assert torch.equal(holder(x), base_only)
    with pytest.raises(ValueError):
        twinkle_amd.use_mi355x_path(ReferenceSurfaceMultiLora(TinyBlock(), 1, 8))   # nothing patched yet


def test_adapter_checkpoint_keys_with_linear_and_packed_expert_parameters(tmp_path):
    """One naming root in adapter_model.safetensors: base_model.model.<path inside the wrapped model> for linear
    layers and packed expert parameters alike (reference: PeftModel parameter names for the former,
    multi_lora_target_parameters.py:321-330 for the latter), and the file loads back into a fresh model."""
    from safetensors.torch import load_file

    class Moe(nn.Module):

        def __init__(self):
            super().__init__()
            self.q_proj = nn.Linear(4, 4, bias=False)
            self.mlp = nn.Module()
            self.mlp.experts = _PackedExperts()

        def forward(self, x):
            return self.q_proj(x)

    def build():
        torch.manual_seed(0)
        ml = MultiLora(max_loras=2, max_r=4)
        model = ml.patch(Moe(), target_modules=['q_proj'])
        ml.save_initial_weights()
        targets = ['mlp.experts.gate_up_proj', 'mlp.experts.down_proj']
        ml.patch_target_parameters(model, targets)
        ml.acquire_lora('alice', LoraConfig(r=2, lora_alpha=4, target_modules=['q_proj'], target_parameters=targets))
        return ml, model

    ml, model = build()
    with torch.no_grad():
        for n, p in model.named_parameters():
            if 'lora_' in n:
                p.uniform_(-0.1, 0.1)
    out = ml.save_adapter('alice', str(tmp_path / 'ckpt'))
    saved = load_file(f'{out}/adapter_model.safetensors')
    assert {k: tuple(v.shape) for k, v in saved.items()} == {
        'base_model.model.q_proj.lora_A.weight': (2, 4),
        'base_model.model.q_proj.lora_B.weight': (4, 2),
        'base_model.model.mlp.experts.base_layer.lora_A.weight': (2, 2, 4),
        'base_model.model.mlp.experts.base_layer.lora_B.weight': (2, 12, 2),
        'base_model.model.mlp.experts.lora_A.weight': (2, 2, 6),
        'base_model.model.mlp.experts.lora_B.weight': (2, 4, 2),
    }
    ml2, model2 = build()
    ml2.load_adapter('alice', out)
    want, got = ml.get_state_dict('alice'), ml2.get_state_dict('alice')
    assert want.keys() == got.keys()
    for k in want:
        assert torch.equal(want[k], got[k]), k
