"""Committed fixtures (tests/golden/*.json, written by tests/golden/make_golden.py from the oracle):
the oracle must still reproduce them (CPU), and the HIP path must match them (GPU)."""
import json
import os

import pytest
import torch

import oracle
from conftest import max_rel_err

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')


def _load(name):
    with open(os.path.join(GOLDEN, name)) as f:
        return json.load(f)


def test_oracle_reproduces_lora_fixture():
    c = _load('lora_small.json')
    t64 = lambda v: torch.tensor(v, dtype=torch.double)  # noqa: E731
    y, dx, da, db = oracle.multi_lora_linear_grads(t64(c['x']), t64(c['base']), torch.tensor(c['ids']),
                                                    [t64(v) for v in c['A']], [t64(v) for v in c['B']], c['ranks'],
                                                    c['scales'], t64(c['dy']))
    assert torch.allclose(y, t64(c['Y']), atol=1e-12) and torch.allclose(dx, t64(c['dX']), atol=1e-12)
    for g in range(len(c['A'])):
        assert torch.allclose(da[g], t64(c['dA'][g]), atol=1e-12) and torch.allclose(db[g], t64(c['dB'][g]), atol=1e-12)


def test_oracle_reproduces_segment_fixture():
    for c in _load('segments_small.json'):
        perm, _, offsets = oracle.segment_build_sort(torch.tensor(c['keys'], dtype=torch.long), c['groups'])
        assert perm.tolist() == c['perm'] and offsets.tolist() == c['offsets']
        assert perm.tolist() == oracle.segment_build_bruteforce(torch.tensor(c['keys'], dtype=torch.long), c['groups'])[0].tolist()
        if 'num_tokens' in c:
            assert (perm % c['num_tokens']).tolist() == c['row_token_of_reference_mask_order']


@pytest.mark.gpu
def test_hip_segment_builder_matches_fixture(dev):
    from twinkle_amd import build_segments
    for c in _load('segments_small.json'):
        keys = torch.tensor(c['keys'], dtype=torch.int32, device=dev)
        seg = build_segments(keys, c['groups'], num_tokens=c.get('num_tokens'), check=True)
        assert seg.perm.tolist() == c['perm'] and seg.offsets.tolist() == c['offsets']
        if 'num_tokens' in c:
            assert seg.row_token.tolist() == c['row_token_of_reference_mask_order']


@pytest.mark.gpu
@pytest.mark.parametrize('dtype,tol', [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
def test_hip_lora_matches_fixture(dev, dtype, tol):
    from twinkle_amd import AdapterGroups, build_segments, multi_lora_delta
    c = _load('lora_small.json')
    td = lambda v: torch.tensor(v, dtype=torch.double).to(dtype).to(dev)  # noqa: E731
    x = td(c['x']).requires_grad_(True)
    a = [td(v).requires_grad_(True) for v in c['A']]
    b = [td(v).requires_grad_(True) for v in c['B']]
    seg = build_segments(torch.tensor(c['ids'], dtype=torch.int32, device=dev), len(a))
    y = multi_lora_delta(x, td(c['base']), seg, AdapterGroups(a, b, c['ranks'], c['scales']))
    y.backward(td(c['dy']))
    t64 = lambda v: torch.tensor(v, dtype=torch.double)  # noqa: E731
    assert max_rel_err(y, t64(c['Y'])) < tol and max_rel_err(x.grad, t64(c['dX'])) < tol
    # the LoRA term alone (zero base) against fixture Y minus fixture base: the bar scales with the term itself
    from twinkle_amd import lora_fwd_
    delta = torch.zeros_like(y)
    lora_fwd_(x.detach(), delta, seg, AdapterGroups([v.detach() for v in a], [v.detach() for v in b], c['ranks'],
                                                    c['scales']))
    assert max_rel_err(delta, t64(c['Y']) - td(c['base']).double().cpu()) < tol
    for g in range(len(a)):
        assert max_rel_err(a[g].grad, t64(c['dA'][g])) < tol and max_rel_err(b[g].grad, t64(c['dB'][g])) < tol


def _experts_inputs():
    import importlib.util
    spec = importlib.util.spec_from_file_location('make_golden', os.path.join(GOLDEN, 'make_golden.py'))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod.experts_inputs()


def test_oracle_reproduces_experts_fixture():
    c, want = _experts_inputs(), _load('experts_small.json')
    assert want['expert'] == c['expert'].tolist() and want['shape']['out'] == c['out']
    order = torch.argsort(c['expert'], stable=True)
    offsets = torch.cat([torch.zeros(1, dtype=torch.long), torch.bincount(c['expert'], minlength=c['experts']).cumsum(0)])
    y = torch.empty(c['tokens'], c['out'], dtype=torch.double)
    y[order] = oracle.experts_linear(c['x'][order], offsets, c['w'])
    assert torch.allclose(y, torch.tensor(want['Y'], dtype=torch.double), atol=1e-12)
    assert torch.allclose(oracle.swiglu(y), torch.tensor(want['swiglu_of_Y'], dtype=torch.double), atol=1e-12)


@pytest.mark.gpu
def test_hip_grouped_linear_and_swiglu_match_fixture(dev):
    from twinkle_amd import build_segments, grouped_linear_, swiglu
    c, want = _experts_inputs(), _load('experts_small.json')
    keys = (c['expert'] * c['tenants'] + c['tenant']).to(torch.int32).to(dev)
    seg = build_segments(keys, c['experts'] * c['tenants'])
    y = grouped_linear_(c['x'].bfloat16().to(dev), c['w'].bfloat16().to(dev), seg, c['tenants'], map_rows=True)
    y64 = torch.tensor(want['Y'], dtype=torch.double)
    assert max_rel_err(y, y64) < 2e-2
    assert max_rel_err(swiglu(y64.float().to(dev)), torch.tensor(want['swiglu_of_Y'], dtype=torch.double)) < 1e-5
