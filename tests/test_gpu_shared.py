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


def _projections(k, outs, n, max_r, ranks_per_proj, seed, dtype, dev, weights_f32=False):
    g = torch.Generator().manual_seed(seed)
    projs = []
    max_rs = max_r if isinstance(max_r, tuple) else (max_r,) * len(outs)
    # weights_f32: fp32 adapters under bf16 activations (values that bf16 holds exactly, so the oracle sees what the
    # kernels' bf16 copies hold)
    wdt = (lambda v: v.to(dtype).float()) if weights_f32 else (lambda v: v.to(dtype))
    for m, ranks, mr in zip(outs, ranks_per_proj, max_rs):
        a = [wdt((torch.rand(mr, k, generator=g) * 2 - 1) / k**0.5) for _ in range(n)]
        b = [wdt(torch.randn(m, mr, generator=g) * 0.05) for _ in range(n)]
        scales = [2.0 if i % 2 == 0 else 0.5 for i in range(n)]
        projs.append((a, b, list(ranks), scales))
    return projs


def _groups(projs, dev, rank_classes=True, act_dtype=None):
    out = []
    for a, b, ranks, scales in projs:
        ad = [t.to(dev).requires_grad_(True) for t in a]
        bd = [t.to(dev).requires_grad_(True) for t in b]
        out.append((AdapterGroups(ad, bd, ranks, scales, rank_classes=rank_classes, act_dtype=act_dtype), ad, bd))
    return out


def _compare(dev, dtype, t, k, outs, n, max_r, ranks_per_proj, seed=0, exact=True, weights_f32=False):
    g = torch.Generator().manual_seed(seed + 100)
    x = torch.randn(t, k, generator=g).to(dtype)
    bases = [torch.randn(t, m, generator=g).to(dtype) for m in outs]
    dys = [torch.randn(t, m, generator=g).to(dtype) for m in outs]
    ids = torch.randint(0, n, (t,), generator=g)
    projs = _projections(k, outs, n, max_r, ranks_per_proj, seed, dtype, dev, weights_f32)
    act = dtype if weights_f32 else None
    seg = build_segments(ids.to(torch.int32).to(dev), n, check=True)

    # one call per projection (every group on the kernels of the projection's largest padded rank, like the shared
    # entry points: the bit-for-bit comparison below is between the same kernels)
    xs = x.to(dev).requires_grad_(True)
    sep = _groups(projs, dev, rank_classes=False, act_dtype=act)
    ys = [multi_lora_delta(xs, b.to(dev) * 1.0, seg, grp) for b, (grp, _, _) in zip(bases, sep)]
    torch.autograd.backward(ys, [d.to(dev) for d in dys])

    # one call for all
    xj = x.to(dev).requires_grad_(True)
    joint = _groups(projs, dev, act_dtype=act)
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
            if ranks[gi] == 0:        # not live: no gradient at all, from either entry point
                assert all(v[p][s][gi].grad is None for v in (joint, sep) for s in (1, 2)), f'adapter {gi} of {p}'
                assert torch.count_nonzero(dao[gi]) == 0 and torch.count_nonzero(dbo[gi]) == 0
                continue
            assert max_rel_err(joint[p][1][gi].grad, dao[gi]) < tol, f'dA[{p}][{gi}]'
            assert max_rel_err(joint[p][2][gi].grad, dbo[gi]) < tol, f'dB[{p}][{gi}]'
        if exact:
            assert torch.equal(yj[p], ys[p]), f'Y[{p}] differs from the single-projection call'
            for gi in range(n):
                if ranks[gi] == 0:
                    continue
                assert torch.equal(joint[p][1][gi].grad, sep[p][1][gi].grad), f'dA[{p}][{gi}] bits'
                assert torch.equal(joint[p][2][gi].grad, sep[p][2][gi].grad), f'dB[{p}][{gi}] bits'
    assert max_rel_err(xj.grad, dx_ref) < tol, 'dX'
    assert max_rel_err(xs.grad, dx_ref) < tol, 'dX of separate calls'


@pytest.mark.parametrize('outs,ranks_per_proj', [
    ((1024, 512), ((16, 8, 4, 16, 1), (16, 16, 2, 8, 16))),                              # gate / up
    ((1024, 512, 512), ((16, 8, 4, 16, 1), (8, 8, 8, 8, 8), (16, 0, 3, 16, 5))),          # q / k / v, a dead adapter
    ((512, 512, 1024, 512), ((4, 4, 4, 4, 4), (16, 16, 16, 16, 16), (1, 2, 3, 4, 5), (0, 0, 16, 16, 0))),
])
@pytest.mark.parametrize('weights_f32', [False, True])
def test_shared_matches_separate_calls_bf16(dev, outs, ranks_per_proj, weights_f32):
    _compare(dev, torch.bfloat16, 777, 2048, outs, 5, 16, ranks_per_proj, weights_f32=weights_f32)


@pytest.mark.parametrize('max_r,outs,ranks_per_proj', [
    (32, (1024, 512), ((32, 17, 4, 32, 1), (32, 32, 2, 24, 16))),                              # gate / up
    (32, (1024, 512, 512), ((32, 8, 4, 16, 1), (24, 24, 24, 24, 24), (32, 0, 3, 16, 5))),       # q / k / v, a dead adapter
    (32, (384, 640), ((32, 8, 4, 16, 1), (17, 32, 3, 16, 5))),                                  # widths off the fused dy pass
    (64, (1024, 512), ((64, 33, 4, 16, 1), (64, 64, 2, 48, 16))),
    (64, (512, 512, 1024, 512), ((64,) * 5, (33,) * 5, (1, 20, 33, 48, 64), (0, 0, 64, 40, 0))),
])
@pytest.mark.parametrize('weights_f32', [False, True])
def test_shared_matches_separate_calls_above_rank_16(dev, max_r, outs, ranks_per_proj, weights_f32):
    """Padded rank 32 and 64: one shrink launch for all projections, one dX read-modify-write, one dA launch.
    weights_f32: fp32 adapters and gradients under the bf16 activations (the state of a PEFT model on a bf16 base)."""
    _compare(dev, torch.bfloat16, 777, 2048, outs, 5, max_r, ranks_per_proj, weights_f32=weights_f32)


@pytest.mark.parametrize('max_r', [32, 64])
def test_shared_above_rank_16_input_width_off_four_column_groups(dev, max_r):
    """An input of 1152 columns is nine groups of 128: the last block of the dX kernel has one live wave out of four,
    and 131 rows end in a tile pair with one tile."""
    ranks = ((max_r, max_r // 2 + 1, 3), (max_r, max_r, max_r - 7))
    _compare(dev, torch.bfloat16, 131, 1152, (512, 256), 3, max_r, ranks, seed=5)


def test_shared_rank_64_attention_shape(dev):
    """q / k / v at rank 64: 4096 -> 4096, 1024, 1024 on 2048 tokens of 8 adapters, one of them without rows."""
    ranks = [(64, 64, 48, 64, 33, 64, 64, 64)] * 3
    _compare(dev, torch.bfloat16, 2048, 4096, (4096, 1024, 1024), 8, 64, ranks, seed=11)


def test_shared_llama_qkv_shape(dev):
    """q / k / v of a grouped-query attention block: 4096 -> 4096, 1024, 1024 on 4096 tokens of 16 adapters."""
    _compare(dev, torch.bfloat16, 4096, 4096, (4096, 1024, 1024), 16, 16, [(16,) * 16, (8,) * 16, (16,) * 16], seed=3)


@pytest.mark.parametrize('dtype,k,outs,max_r', [
    (torch.float32, 256, (128, 64), 8),         # fp32: one call per projection inside the library
    (torch.bfloat16, 200, (96, 40), 8),         # shapes outside the MFMA kernels
    (torch.bfloat16, 2048, (1024,), 16),        # a single projection
])
def test_shared_falls_back_to_one_call_per_projection(dev, dtype, k, outs, max_r):
    ranks = [(max_r, max_r // 2, 1)] * len(outs)
    _compare(dev, dtype, 300, k, outs, 3, max_r, ranks, seed=5, exact=False)


def test_shared_projections_of_different_padded_rank(dev):
    """One projection of rank 16, one of rank 64: no common kernel family, so one call per projection."""
    _compare(dev, torch.bfloat16, 300, 2048, (1024, 512), 3, (16, 64), [(16, 8, 1), (64, 32, 1)], seed=6, exact=True)


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


# ---- through the MultiLora mirror: q / k / v of one block routed through forward_shared --------------------

class _QKV(torch.nn.Module):

    def __init__(self, d, kv):
        super().__init__()
        self.q_proj = torch.nn.Linear(d, d, bias=True)
        self.k_proj = torch.nn.Linear(d, kv, bias=False)
        self.v_proj = torch.nn.Linear(d, kv, bias=False)

    def forward(self, x):
        return self.q_proj(x), self.k_proj(x), self.v_proj(x)


@pytest.mark.parametrize('dtype,d,kv', [(torch.bfloat16, 2048, 512), (torch.float32, 128, 64)])
def test_forward_shared_equals_layer_by_layer(dev, dtype, d, kv):
    from twinkle_amd import LoraConfig, MultiLora
    torch.manual_seed(0)
    ml = MultiLora(max_loras=4, max_r=16)
    model = ml.patch(_QKV(d, kv).to(dtype).to(dev), target_modules='all-linear')
    ml.acquire_lora('alice', LoraConfig(r=8, lora_alpha=16, target_modules='all-linear'))
    ml.acquire_lora('bob', LoraConfig(r=16, lora_alpha=32, target_modules=['q_proj', 'v_proj']))   # k_proj not targeted
    ml.acquire_lora('carol', LoraConfig(r=4, lora_alpha=16, target_modules='all-linear', use_rslora=True))
    g = torch.Generator().manual_seed(1)
    with torch.no_grad():
        for n, p in model.named_parameters():
            if '.lora_B.' in n:
                p.copy_((torch.randn(p.shape, generator=g) * 0.05).to(dtype))
    x = torch.randn(2, 150, d, generator=g).to(dtype).to(dev)
    row_tenant = torch.randint(0, 3, (300,), generator=g).to(dev)
    wq, wk, wv = (torch.randn(2, 150, n, generator=g).to(dtype).to(dev) for n in (d, kv, kv))
    m = model.model
    layers = [m.q_proj, m.k_proj, m.v_proj]

    def run(shared):
        for p in model.parameters():
            p.grad = None
        xi = x.clone().requires_grad_(True)
        with ml.batch(['alice', 'bob', 'carol'], row_tenant):
            q, k, v = ml.forward_shared(layers, xi) if shared else model(xi)
            ((q * wq).sum() + (k * wk).sum() + (v * wv).sum()).backward()
        grads = {n: p.grad.clone() for n, p in model.named_parameters() if p.grad is not None}
        return (q, k, v), xi.grad, grads

    (q0, k0, v0), dx0, g0 = run(False)
    (q1, k1, v1), dx1, g1 = run(True)
    bf16 = dtype == torch.bfloat16

    def same(outs, dx, grads):
        for a, b in zip((q0, k0, v0), outs):
            assert torch.equal(a, b) if bf16 else max_rel_err(b, a) < 1e-6
        assert g0.keys() == grads.keys()
        for n in g0:
            assert (torch.equal(g0[n], grads[n]) if bf16 and 'lora_' in n
                    else max_rel_err(grads[n], g0[n].double()) < 1e-5), n
        assert max_rel_err(dx, dx0.double()) < (2e-2 if bf16 else 1e-5)

    same((q1, k1, v1), dx1, g1)
    # the module's own forward (q_proj(x), k_proj(x), v_proj(x) one after the other) with the group declared
    ml.share_inputs([layers])
    calls = []
    import twinkle_amd.multi_lora as host
    original = host.forward_shared
    host.forward_shared = lambda m, ls, t: calls.append(len(ls)) or original(m, ls, t)
    try:
        outs2, dx2, g2 = run(False)
    finally:
        host.forward_shared = original
    ml.unshare_inputs()
    assert calls == [3]
    same(outs2, dx2, g2)
    # one adapter per call (the reference's adapter() context) takes the same route
    with ml.adapter('carol'):
        a = ml.forward_shared(layers, x)
        b = model(x)
    for u, w in zip(a, b):
        assert torch.equal(u, w) if bf16 else max_rel_err(u, w) < 1e-6
    with ml.adapter('carol', disable_lora=True):
        a = ml.forward_shared(layers, x)
    assert torch.equal(a[1], torch.nn.functional.linear(x, m.k_proj.base_layer.weight))


def test_shared_calls_replay_from_a_hip_graph(dev):
    """Segment build + shared forward + shared backward captured once and replayed: every replay equals eager."""
    from twinkle_amd import (lora_bwd_shared_, lora_bwd_workspace_bytes, lora_fwd_shared_, lora_h_bytes)
    t, k, outs, n = 1500, 1024, (1024, 512, 512), 4
    ranks = [(16, 7, 16, 3), (8, 8, 0, 8), (16, 16, 16, 16)]
    g = torch.Generator().manual_seed(31)
    dt = torch.bfloat16
    x = torch.randn(t, k, generator=g).to(dt).to(dev)
    bases = [torch.randn(t, m, generator=g).to(dt).to(dev) for m in outs]
    dys = [torch.randn(t, m, generator=g).to(dt).to(dev) for m in outs]
    keys = torch.randint(0, n, (t,), generator=g).to(torch.int32).to(dev)
    groups = [grp for grp, _, _ in _groups(_projections(k, outs, n, 16, ranks, 7, dt, dev), dev)]
    seg0 = build_segments(keys, n, want_perm=False, want_offsets=False)
    hs = [torch.empty(lora_h_bytes(seg0, grp), dtype=torch.uint8, device=dev) for grp in groups]
    wss = [torch.empty(lora_bwd_workspace_bytes(seg0, grp), dtype=torch.uint8, device=dev) for grp in groups]
    gas = [torch.zeros(grp.a_arena_elems, dtype=dt, device=dev) for grp in groups]
    gbs = [torch.zeros(grp.b_arena_elems, dtype=dt, device=dev) for grp in groups]
    pas = [grp._grad_a_rel + ga.data_ptr() for grp, ga in zip(groups, gas)]
    pbs = [grp._grad_b_rel + gb.data_ptr() for grp, gb in zip(groups, gbs)]
    ys = [torch.empty_like(b) for b in bases]
    dx = torch.empty_like(x)

    def step():
        for y, b in zip(ys, bases):
            y.copy_(b)
        dx.fill_(0)
        seg = build_segments(keys, n, want_perm=False, want_offsets=False)
        lora_fwd_shared_(x, ys, seg, groups, hs=hs)
        lora_bwd_shared_(dys, x, hs, dx, pas, pbs, seg, groups, workspaces=wss)

    step()
    torch.cuda.synchronize()
    want = [v.clone() for v in (*ys, dx, *gas, *gbs)]
    assert want[3].abs().max() > 0
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        step()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            step()
    torch.cuda.current_stream().wait_stream(side)
    for _ in range(3):
        for v in (*ys, dx):
            v.fill_(1)
        for v in (*gas, *gbs):
            v.zero_()                # regions beyond an adapter's rank are never written: keep them comparable
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, ref in zip((*ys, dx, *gas, *gbs), want):
            assert torch.equal(got, ref)


@pytest.mark.parametrize('seed', range(12))
def test_shared_random_projection_sets(dev, seed):
    """Seeded draws: 2..4 projections, widths on and off the single-pass backward's multiples, ranks 0..16, few rows."""
    g = torch.Generator().manual_seed(500 + seed)
    pick = lambda xs: xs[int(torch.randint(0, len(xs), (1,), generator=g))]  # noqa: E731
    p = pick([2, 3, 4])
    t, k, n = pick([1, 33, 500, 2100]), pick([1024, 2048]), pick([1, 3, 9])
    outs = tuple(pick([256, 512, 1024, 1536]) for _ in range(p))
    ranks = [tuple(int(torch.randint(0, 17, (1,), generator=g)) for _ in range(n)) for _ in range(p)]
    ranks = [tuple(16 if i == 0 else r for i, r in enumerate(rs)) for rs in ranks]    # keep every projection live
    print(f'case {seed}: t={t} k={k} outs={outs} n={n} ranks={ranks}', flush=True)
    # forward through the shared kernels always; backward too when every width is a multiple of 512
    _compare(dev, torch.bfloat16, t, k, outs, n, 16, ranks, seed=seed)


def test_shared_custom_ops_match_direct_calls(dev):
    """torch.ops.twinkle_amd.lora_fwd_shared / lora_bwd_shared give what the ctypes wrappers give, bit for bit."""
    from twinkle_amd import lora_bwd_shared_, lora_bwd_workspace_bytes, lora_fwd_shared_, lora_h_bytes
    t, k, outs, n = 900, 1024, (1024, 512), 3
    dt = torch.bfloat16
    g = torch.Generator().manual_seed(41)
    x = torch.randn(t, k, generator=g).to(dt).to(dev)
    bases = [torch.randn(t, m, generator=g).to(dt).to(dev) for m in outs]
    dys = [torch.randn(t, m, generator=g).to(dt).to(dev) for m in outs]
    keys = torch.randint(0, n, (t,), generator=g).to(torch.int32).to(dev)
    groups = [grp for grp, _, _ in _groups(_projections(k, outs, n, 16, [(16, 5, 9), (8, 16, 0)], 9, dt, dev), dev)]
    seg = build_segments(keys, n, want_perm=False, want_offsets=False)

    def buffers():
        return ([b.clone() for b in bases], torch.zeros_like(x),
                [torch.empty(lora_h_bytes(seg, grp), dtype=torch.uint8, device=dev) for grp in groups],
                [torch.empty(lora_bwd_workspace_bytes(seg, grp), dtype=torch.uint8, device=dev) for grp in groups],
                [torch.zeros(grp.a_arena_elems, dtype=dt, device=dev) for grp in groups],
                [torch.zeros(grp.b_arena_elems, dtype=dt, device=dev) for grp in groups])

    ys, dx, hs, wss, gas, gbs = buffers()
    pas = [grp._grad_a_rel + ga.data_ptr() for grp, ga in zip(groups, gas)]
    pbs = [grp._grad_b_rel + gb.data_ptr() for grp, gb in zip(groups, gbs)]
    lora_fwd_shared_(x, ys, seg, groups, hs=hs)
    lora_bwd_shared_(dys, x, hs, dx, pas, pbs, seg, groups, workspaces=wss)

    ys2, dx2, hs2, wss2, gas2, gbs2 = buffers()
    pas2 = [grp._grad_a_rel + ga.data_ptr() for grp, ga in zip(groups, gas2)]
    pbs2 = [grp._grad_b_rel + gb.data_ptr() for grp, gb in zip(groups, gbs2)]
    for grp in groups:
        grp.refresh()
    meta = [v for grp in groups for v in (grp.max_rank, grp.lda, grp.ldb)]
    common = (seg.workspace, [grp.a_ptrs for grp in groups], [grp.b_ptrs for grp in groups],
              [grp.rank_dev for grp in groups], [grp.scale_dev for grp in groups], meta, True)
    torch.ops.twinkle_amd.lora_fwd_shared(x, ys2, hs2, *common)
    torch.ops.twinkle_amd.lora_bwd_shared(dys, x, hs2, dx2, gas2, gbs2, pas2, pbs2, wss2, *common, False)
    for a, b in zip((*ys, dx, *gas, *gbs), (*ys2, dx2, *gas2, *gbs2)):
        assert torch.equal(a, b)
    assert dx.abs().max() > 0 and gas[0].abs().max() > 0
