"""Writes tests/golden/*.json from the CPU oracle (not from the reference, which cannot be imported here).

Small cases only: the fixtures hold the inputs and the oracle's float64 results as plain numbers, so a
later change of the oracle or of torch that moves any value shows up as a diff.  Run from the repo root:
    python tests/golden/make_golden.py
"""
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def lora_case():
    g = torch.Generator().manual_seed(20240607)
    t, k, m, n, max_r = 16, 16, 12, 3, 4
    ranks, alphas = [2, 4, 3], [4.0, 4.0, 9.0]
    scales = [oracle.lora_scaling(a, r) for a, r in zip(alphas, ranks)]
    # values on a coarse grid: exactly representable in bf16, so the same fixture serves both dtypes
    grid = lambda *s: torch.randint(-8, 9, s, generator=g).double() / 8  # noqa: E731
    x, base, dy = grid(t, k), grid(t, m), grid(t, m)
    a = [grid(max_r, k) / 4 for _ in range(n)]
    b = [grid(m, max_r) / 4 for _ in range(n)]
    ids = torch.tensor([2, 0, 1, 1, 0, 2, 2, 1, 0, 0, 1, 2, 1, 1, 0, 2])
    y, dx, da, db = oracle.multi_lora_linear_grads(x, base, ids, a, b, ranks, scales, dy)
    return {
        'shape': {'tokens': t, 'in': k, 'out': m, 'adapters': n, 'max_r': max_r},
        'ranks': ranks, 'scales': scales, 'ids': ids.tolist(),
        'x': x.tolist(), 'base': base.tolist(), 'dy': dy.tolist(),
        'A': [v.tolist() for v in a], 'B': [v.tolist() for v in b],
        'Y': y.tolist(), 'dX': dx.tolist(), 'dA': [v.tolist() for v in da], 'dB': [v.tolist() for v in db],
    }


def segment_cases():
    cases = []
    g = torch.Generator().manual_seed(7)
    for rows, groups in [(0, 3), (1, 1), (9, 9), (40, 5), (70, 3), (130, 17)]:
        keys = torch.randint(0, groups, (rows,), generator=g)
        perm, counts, offsets = oracle.segment_build_sort(keys, groups)
        cases.append({'groups': groups, 'keys': keys.tolist(), 'perm': perm.tolist(), 'offsets': offsets.tolist()})
    # top-k routing in the reference's mask order: flat row f = k * T + t
    sel = torch.tensor([[1, 0], [0, 2], [1, 2], [2, 1], [0, 1]])
    keys = oracle.flat_keys_from_topk(sel)
    perm, _, offsets = oracle.segment_build_sort(keys, 3)
    _, sorted_indices = oracle.permute_by_mask(torch.zeros(5, 1), oracle.expert_mask_from_topk(sel, 3))
    cases.append({'groups': 3, 'keys': keys.tolist(), 'perm': perm.tolist(), 'offsets': offsets.tolist(),
                  'num_tokens': 5, 'row_token_of_reference_mask_order': sorted_indices.tolist()})
    return cases


def experts_inputs():
    """Inputs of the packed-experts fixture, from integer formulas instead of stored numbers (the weights alone
    would be 16 k values): coarse-grid values, exactly representable in bf16."""
    e, nt, t, k, n, inter = 2, 2, 12, 64, 128, 64
    ar = torch.arange
    x = ((ar(t)[:, None] * 5 + ar(k)[None, :] * 3) % 17 - 8).double() / 8
    w = ((ar(e)[:, None, None] * 7 + ar(n)[None, :, None] * 3 + ar(k)[None, None, :] * 5) % 13 - 6).double() / 16
    expert = torch.tensor([1, 0, 0, 1, 1, 0, 1, 1, 0, 1, 0, 1])
    tenant = torch.tensor([0, 1, 1, 0, 1, 0, 0, 1, 1, 1, 0, 0])
    return {'experts': e, 'tenants': nt, 'tokens': t, 'in': k, 'out': n, 'inter': inter,
            'x': x, 'w': w, 'expert': expert, 'tenant': tenant}


def experts_case():
    c = experts_inputs()
    order = torch.argsort(c['expert'], stable=True)
    counts = torch.bincount(c['expert'], minlength=c['experts'])
    offsets = torch.cat([torch.zeros(1, dtype=torch.long), counts.cumsum(0)])
    y_sorted = oracle.experts_linear(c['x'][order], offsets, c['w'])
    y = torch.empty_like(y_sorted)
    y[order] = y_sorted
    return {'inputs': 'tests/golden/make_golden.py::experts_inputs (integer formulas)',
            'shape': {k: c[k] for k in ('experts', 'tenants', 'tokens', 'in', 'out', 'inter')},
            'expert': c['expert'].tolist(), 'tenant': c['tenant'].tolist(),
            'Y': y.tolist(),                                  # y[row] = x[row] W_e^T, rows in their original order
            'swiglu_of_Y': oracle.swiglu(y).tolist()}         # silu(Y[:, :64]) * Y[:, 64:]


if __name__ == '__main__':
    with open(os.path.join(HERE, 'experts_small.json'), 'w') as f:
        json.dump(experts_case(), f)
    with open(os.path.join(HERE, 'lora_small.json'), 'w') as f:
        json.dump(lora_case(), f)
    with open(os.path.join(HERE, 'segments_small.json'), 'w') as f:
        json.dump(segment_cases(), f)
    print('wrote', os.listdir(HERE))
