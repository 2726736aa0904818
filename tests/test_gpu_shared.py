"""Projections that share their input (q / k / v, gate / up) through tk_lora_fwd_shared / tk_lora_bwd_shared.

One call for all projections must give what one call per projection gives: y, dA and dB bit for bit (same
kernels' arithmetic in the same order), dx within the bf16 bar of the oracle (the shared kernel rounds the
sum over the projections once, separate calls round after every projection).
"""
import pytest
import torch

import oracle
from conftest import max_rel_err
from twinkle_amd import AdapterGroups, build_segments, multi_lora_delta, multi_lora_delta_shared

pytestmark = pytest.mark.gpu


def _projections(k, outs, n, max_r, ranks_per_proj, seed, dtype, dev):
    g = torch.Generator().manual_seed(seed)
    projs = []
    for m, ranks in zip(outs, ranks_per_proj):
        a = [((torch.rand(max_r, k, generator=g) * 2 - 1) / k**0.5).to(dtype) for _ in range(n)]
        b = [(torch.randn(m, max_r, generator=g) * 0.05).to(dtype) for _ in range(n)]
        scales = [2.0 if i % 2 == 0 else 0.5 for i in range(n)]
        projs.append((a, b, list(ranks), scales))
    return projs


def _groups(projs, dev):
    out = []
    for a, b, ranks, scales in projs:
        ad = [t.to(dev).requires_grad_(True) for t in a]
        bd = [t.to(dev).requires_grad_(True) for t in b]
        out.append((AdapterGroups(ad, bd, ranks, scales), ad, bd))
    return out


def _compare(dev, dtype, t, k, outs, n, max_r, ranks_per_proj, seed=0, exact=True):
    g = torch.Generator().manual_seed(seed + 100)
    x = torch.randn(t, k, generator=g).to(dtype)
    bases = [torch.randn(t, m, generator=g).to(dtype) for m in outs]
    dys = [torch.randn(t, m, generator=g).to(dtype) for m in outs]
    ids = torch.randint(0, n, (t,), generator=g)
    projs = _projections(k, outs, n, max_r, ranks_per_proj, seed, dtype, dev)
    seg = build_segments(ids.to(torch.int32).to(dev), n, check=True)

    # one call per projection
    xs = x.to(dev).requires_grad_(True)
    sep = _groups(projs, dev)
    ys = [multi_lora_delta(xs, b.to(dev) * 1.0, seg, grp) for b, (grp, _, _) in zip(bases, sep)]
    torch.autograd.backward(ys, [d.to(dev) for d in dys])

    # one call for all
    xj = x.to(dev).requires_grad_(True)
    joint = _groups(projs, dev)
    yj = multi_lora_delta_shared(xj, [b.to(dev) * 1.0 for b in bases], seg, [grp for grp, _, _ in joint])
    torch.autograd.backward(list(yj), [d.to(dev) for d in dys])

    tol = 2e-2 if dtype == torch.bfloat16 else 1e-5
    dx_ref = torch.zeros(t, k, dtype=torch.float64)
    for p, (a, b, ranks, scales) in enumerate(projs):
        yo, dxo, dao, dbo = oracle.multi_lora_linear_grads(x.double(), bases[p].double(), ids, [w.double() for w in a],
                                                           [w.double() for w in b], ranks, scales, dys[p].double())
        dx_ref += dxo
        assert max_rel_err(yj[p], yo) < tol, f'Y[{p}]'
        for gi in range(n):
            assert max_rel_err(joint[p][1][gi].grad, dao[gi]) < tol, f'dA[{p}][{gi}]'
            assert max_rel_err(joint[p][2][gi].grad, dbo[gi]) < tol, f'dB[{p}][{gi}]'
        if exact:
            assert torch.equal(yj[p], ys[p]), f'Y[{p}] differs from the single-projection call'
            for gi in range(n):
                assert torch.equal(joint[p][1][gi].grad, sep[p][1][gi].grad), f'dA[{p}][{gi}] bits'
                assert torch.equal(joint[p][2][gi].grad, sep[p][2][gi].grad), f'dB[{p}][{gi}] bits'
    assert max_rel_err(xj.grad, dx_ref) < tol, 'dX'
    assert max_rel_err(xs.grad, dx_ref) < tol, 'dX of separate calls'


@pytest.mark.parametrize('outs,ranks_per_proj', [
    ((1024, 512), ((16, 8, 4, 16, 1), (16, 16, 2, 8, 16))),                              # gate / up
    ((1024, 512, 512), ((16, 8, 4, 16, 1), (8, 8, 8, 8, 8), (16, 0, 3, 16, 5))),          # q / k / v, a dead adapter
    ((512, 512, 1024, 512), ((4, 4, 4, 4, 4), (16, 16, 16, 16, 16), (1, 2, 3, 4, 5), (0, 0, 16, 16, 0))),
])
def test_shared_matches_separate_calls_bf16(dev, outs, ranks_per_proj):
    _compare(dev, torch.bfloat16, 777, 2048, outs, 5, 16, ranks_per_proj)


def test_shared_llama_qkv_shape(dev):
    """q / k / v of a grouped-query attention block: 4096 -> 4096, 1024, 1024 on 4096 tokens of 16 adapters."""
    _compare(dev, torch.bfloat16, 4096, 4096, (4096, 1024, 1024), 16, 16, [(16,) * 16, (8,) * 16, (16,) * 16], seed=3)


@pytest.mark.parametrize('dtype,k,outs,max_r', [
    (torch.float32, 256, (128, 64), 8),         # fp32: one call per projection inside the library
    (torch.bfloat16, 2048, (1024, 512), 32),    # rank above 16
    (torch.bfloat16, 200, (96, 40), 8),         # shapes outside the MFMA kernels
    (torch.bfloat16, 2048, (1024,), 16),        # a single projection
])
def test_shared_falls_back_to_one_call_per_projection(dev, dtype, k, outs, max_r):
    ranks = [(max_r, max_r // 2, 1)] * len(outs)
    _compare(dev, dtype, 300, k, outs, 3, max_r, ranks, seed=5, exact=False)


def test_shared_argument_errors(dev):
    projs = _projections(2048, (512, 512), 2, 16, [(16, 16), (16, 16)], 0, torch.bfloat16, dev)
    grp = [g for g, _, _ in _groups(projs, dev)]
    other = AdapterGroups([torch.zeros(16, 1024, dtype=torch.bfloat16, device=dev)] * 2,
                          [torch.zeros(512, 16, dtype=torch.bfloat16, device=dev)] * 2, [16, 16], [1.0, 1.0])
    seg = build_segments(torch.zeros(64, dtype=torch.int32, device=dev), 2)
    x = torch.zeros(64, 2048, dtype=torch.bfloat16, device=dev)
    y = [torch.zeros(64, 512, dtype=torch.bfloat16, device=dev) for _ in range(2)]
    with pytest.raises(ValueError):
        multi_lora_delta_shared(x, y, seg, [grp[0], other])       # in_features differ
    with pytest.raises(ValueError):
        multi_lora_delta_shared(x, y * 3, seg, grp * 3)           # more than four projections
    with pytest.raises(ValueError):
        multi_lora_delta_shared(x, [y[0], y[1][:, :256]], seg, grp)  # an output of the wrong width
