"""The larger BASELINE configurations: full shapes on the GPU, checked by sampling against the oracle and
by properties that do not need a CPU pass over the whole problem."""
import pytest
import torch

import oracle
from conftest import max_rel_err
from twinkle_amd import AdapterGroups, build_segments, lora_bwd_, lora_bwd_workspace_bytes, lora_fwd_
from twinkle_amd import packed_cu_seqlens, token_groups_from_sequences, workloads

pytestmark = pytest.mark.gpu


def _device_problem(w, dev, weights_f32=False):
    dt = torch.bfloat16
    wdt = torch.float32 if weights_f32 else dt     # fp32 adapters under bf16 activations: tk_lora_desc::weights_f32
    a = [t.to(wdt).to(dev) for t in w.lora_A]
    b = [t.to(wdt).to(dev) for t in w.lora_B]
    seg = build_segments(w.ids.to(dev), w.num_adapters, check=True)
    return a, b, seg, AdapterGroups(a, b, w.ranks, w.scales, act_dtype=dt)


def _check_sampled(w, dev, sample_groups, sample_rows=64, weights_f32=False):
    """Forward/backward at full size; Y and dX on sampled rows, dA/dB of sampled adapters, against float64
    (with ``weights_f32`` on the unrounded fp32 weights, and the gradients must come back as fp32)."""
    dt = torch.bfloat16
    a, b, seg, groups = _device_problem(w, dev, weights_f32)
    x = w.x.to(dt).to(dev)
    y = w.base_out.to(dt).to(dev)
    dy = w.dy.to(dt).to(dev)
    h = lora_fwd_(x, y, seg, groups)
    delta = torch.zeros_like(y)                   # the LoRA term alone, on a zero base
    lora_fwd_(x, delta, seg, groups)
    ga = [torch.full_like(t, 7.0) for t in a]
    gb = [torch.full_like(t, 7.0) for t in b]
    pa = torch.tensor([t.data_ptr() for t in ga], dtype=torch.int64, device=dev)
    pb = torch.tensor([t.data_ptr() for t in gb], dtype=torch.int64, device=dev)
    dx = torch.zeros_like(x)
    lora_bwd_(dy, x, h, dx, pa, pb, seg, groups, accumulate=False)
    f64 = lambda t: t.to(dt).double()  # noqa: E731
    w64 = (lambda t: t.float().double()) if weights_f32 else f64  # noqa: E731
    assert all(t.dtype == (torch.float32 if weights_f32 else dt) for t in ga + gb)
    counts = torch.bincount(w.ids.long(), minlength=w.num_adapters)
    for g in sample_groups:
        r, s = w.ranks[g], w.scales[g]
        rows = (w.ids == g).nonzero().flatten()
        ag, bg = w64(w.lora_A[g])[:r], w64(w.lora_B[g])[:, :r]
        if rows.numel() == 0:
            assert torch.count_nonzero(ga[g][:r]) == 0 and torch.count_nonzero(gb[g][:, :r]) == 0
            continue
        xg, dyg = f64(w.x[rows]), f64(w.dy[rows])
        hg = s * xg @ ag.t()
        dh = s * dyg @ bg
        sub = rows[:sample_rows]
        assert max_rel_err(y[sub.to(dev)], f64(w.base_out[sub]) + (hg[:sample_rows] @ bg.t())) < 2e-2
        assert max_rel_err(delta[sub.to(dev)], hg[:sample_rows] @ bg.t()) < 2e-2, f'LoRA term of adapter {g}'
        assert max_rel_err(dx[sub.to(dev)], dh[:sample_rows] @ ag) < 2e-2
        assert max_rel_err(ga[g][:r], dh.t() @ xg) < 2e-2, f'dA[{g}] ({int(counts[g])} rows)'
        assert max_rel_err(gb[g][:, :r], dyg.t() @ (hg / 1.0)) < 2e-2, f'dB[{g}]'
        assert torch.all(ga[g][r:] == 7.0) and torch.all(gb[g][:, r:] == 7.0)       # outside the live block: untouched
    return y, dx, ga, gb


@pytest.mark.parametrize('direction', ['up', 'down'])
def test_config3_mixed_ranks_full_size(dev, direction):
    """BASELINE config 3: T=32768, 4096<->14336, 32 adapters with ranks {8,16,32,64}, adapters 5 and 17 empty."""
    w = workloads.config3_mlp(direction)
    assert int((w.ids == 5).sum()) == 0 and int((w.ids == 17).sum()) == 0
    _check_sampled(w, dev, sample_groups=[0, 3, 5, 9, 17, 22, 31])


def test_config2_fp32_adapters_full_size(dev):
    """BASELINE config 2 with PEFT-style fp32 adapters under the bf16 activations: every adapter, at full size."""
    w = workloads.config2_qproj()
    _check_sampled(w, dev, sample_groups=list(range(w.num_adapters)), weights_f32=True)


def test_config5_qkv_shared_inputs_rank64_full_size(dev):
    """q / k / v of one config-5 layer (4096 -> 4096, 1024, 1024; T = 32768, 8 tenants of rank 64, one per packed
    sequence) through the shared-input entry points: y, dA, dB equal to one call per projection bit for bit, dX
    (one rounding of the sum over the projections) against float64 on sampled rows."""
    from twinkle_amd import lora_bwd_shared_, lora_fwd_shared_
    dt, t, k, n, r = torch.bfloat16, 32768, 4096, 8, 64
    outs = (4096, 1024, 1024)
    g = torch.Generator().manual_seed(21)
    ids = torch.repeat_interleave(torch.arange(n, dtype=torch.int32), t // n)
    x = torch.randn(t, k, generator=g).to(dt)
    seg = build_segments(ids.to(dev), n, check=True)
    xd = x.to(dev)
    a_all, b_all, dys, groups = [], [], [], []
    for m in outs:
        a = [((torch.rand(r, k, generator=g) * 2 - 1) / 64).to(dt) for _ in range(n)]
        b = [(torch.randn(m, r, generator=g) * 0.02).to(dt) for _ in range(n)]
        a_all.append(a)
        b_all.append(b)
        dys.append(torch.randn(t, m, generator=g).to(dt))
        groups.append(AdapterGroups([w.to(dev) for w in a], [w.to(dev) for w in b], [r] * n, [2.0] * n))

    def grads():
        ga = [[torch.zeros(r, k, dtype=dt, device=dev) for _ in range(n)] for _ in outs]
        gb = [[torch.zeros(m, r, dtype=dt, device=dev) for _ in range(n)] for m in outs]
        pa = [torch.tensor([w.data_ptr() for w in ws], dtype=torch.int64, device=dev) for ws in ga]
        pb = [torch.tensor([w.data_ptr() for w in ws], dtype=torch.int64, device=dev) for ws in gb]
        return ga, gb, pa, pb

    # one call per projection
    ys = [torch.zeros(t, m, dtype=dt, device=dev) for m in outs]
    ga1, gb1, pa1, pb1 = grads()
    dx1 = torch.zeros(t, k, dtype=dt, device=dev)
    for p in range(3):
        h = lora_fwd_(xd, ys[p], seg, groups[p])
        lora_bwd_(dys[p].to(dev), xd, h, dx1, pa1[p], pb1[p], seg, groups[p])
    # all three at once
    yj = [torch.zeros(t, m, dtype=dt, device=dev) for m in outs]
    ga2, gb2, pa2, pb2 = grads()
    dx2 = torch.zeros(t, k, dtype=dt, device=dev)
    hs = lora_fwd_shared_(xd, yj, seg, groups)
    lora_bwd_shared_([d.to(dev) for d in dys], xd, hs, dx2, pa2, pb2, seg, groups)
    for p in range(3):
        assert torch.equal(yj[p], ys[p]), f'y[{p}]'
        for i in range(n):
            assert torch.equal(ga2[p][i], ga1[p][i]) and torch.equal(gb2[p][i], gb1[p][i]), f'gradients of {p}, {i}'
    for tenant in (0, 5):
        rows = (ids == tenant).nonzero().flatten()[:48]
        want = torch.zeros(rows.numel(), k, dtype=torch.float64)
        for p in range(3):
            dh = 2.0 * dys[p][rows].double() @ b_all[p][tenant].double()
            want += dh @ a_all[p][tenant].double()
            yo = (2.0 * x[rows].double() @ a_all[p][tenant].double().t()) @ b_all[p][tenant].double().t()
            assert max_rel_err(yj[p][rows.to(dev)], yo) < 2e-2
        assert max_rel_err(dx2[rows.to(dev)], want) < 2e-2, 'dX of the shared call'
        assert max_rel_err(dx1[rows.to(dev)], want) < 2e-2, 'dX of the separate calls'


def test_config3_linearity_and_repeatability(dev):
    """Size-independent properties at full size: the update is linear in B and bitwise repeatable."""
    w = workloads.config3_mlp('up', tokens=8192)
    dt = torch.bfloat16
    a, b, seg, groups = _device_problem(w, dev)
    x = w.x.to(dt).to(dev)
    zero = torch.zeros(w.tokens, w.out_features, dtype=dt, device=dev)
    y1 = zero.clone()
    lora_fwd_(x, y1, seg, groups)
    y1b = zero.clone()
    lora_fwd_(x, y1b, seg, groups)
    assert torch.equal(y1, y1b)
    b2 = [t * 2 for t in b]                      # exact in bf16
    y2 = zero.clone()
    lora_fwd_(x, y2, seg, AdapterGroups(a, b2, w.ranks, w.scales))
    assert torch.equal(y2, y1 * 2)
    bz = [torch.zeros_like(t) for t in b]        # B = 0: the base output comes back exactly
    base = w.base_out.to(dt).to(dev)
    y3 = base.clone()
    lora_fwd_(x, y3, seg, AdapterGroups(a, bz, w.ranks, w.scales))
    assert torch.equal(y3, base)


def test_config5_packed_sequences_one_tenant_each(dev):
    """BASELINE config 5, one projection: 8 sequences x 4096 packed, tenant j owns sequence j, rank 64, 4096 -> 1024."""
    g = torch.Generator().manual_seed(8)
    t, k, m, n, r = 32768, 4096, 1024, 8, 64
    pos = torch.cat([torch.arange(4096) for _ in range(n)])[None]
    cu = packed_cu_seqlens(pos.to(dev))
    assert cu.tolist() == oracle.packed_cu_seqlens(pos).tolist()
    ids = token_groups_from_sequences(cu, torch.arange(n, device=dev))
    x = torch.randn(t, k, generator=g)
    dy = torch.randn(t, m, generator=g)
    base = torch.randn(t, m, generator=g)
    a = [(torch.rand(r, k, generator=g) * 2 - 1) / 64 for _ in range(n)]
    b = [torch.randn(m, r, generator=g) * 0.02 for _ in range(n)]
    w = workloads.LoraWorkload('cfg5_k_proj', t, k, m, [r] * n, [2.0] * n, r, ids.cpu(), x, dy, base, a, b)
    _check_sampled(w, dev, sample_groups=[0, 4, 7])


def _config4_keys(dev, with_edge_groups):
    """(expert, tenant) keys of BASELINE config 4 in the reference's row order; optionally one group emptied and
    one cut down to a single row (their rows go to the neighbouring group)."""
    from twinkle_amd import flat_keys_from_topk
    sel, weights, tenant = workloads.moe_routing()
    keys = flat_keys_from_topk(sel.to(dev), tenant.to(dev), 4)
    if with_edge_groups:
        keys = keys.clone()
        keys[keys == 7] = 8                                   # group 7: empty
        rows300 = (keys == 300).nonzero().flatten()
        keys[rows300[1:]] = 301                               # group 300: one row
    return keys, sel.shape[0]


@pytest.mark.parametrize('k_in,m_out', [(2048, 1536), (768, 2048)])
def test_config4_backward_full_size(dev, k_in, m_out):
    """BASELINE config 4 at its own size, forward and backward: 65536 routed rows in (expert, tenant) order, 512
    groups of rank 8 reading blocks of packed [E, max_r, in] / [E, out, max_r] tensors, rows already in segment
    order (map_rows = 0); gate_up (2048 -> 1536) and down (768 -> 2048).  The LoRA term, dX on all rows of sampled
    groups, dA / dB of sampled groups (an empty one and a one-row one among them) against the closed forms in
    float64; gradients of groups that were not sampled are checked for finiteness and for zeros beyond the rank."""
    e, nt, r, max_r = 128, 4, 8, 8
    keys, tokens = _config4_keys(dev, with_edge_groups=True)
    rows = keys.numel()
    assert rows == 65536
    seg = build_segments(keys, e * nt, num_tokens=tokens, check=True)
    offsets = seg.offsets.cpu()
    assert int(offsets[8] - offsets[7]) == 0 and int(offsets[301] - offsets[300]) == 1
    g = torch.Generator().manual_seed(44)
    dt = torch.bfloat16
    x = torch.randn(rows, k_in, generator=g).to(dt)                      # rows in segment order
    dy = torch.randn(rows, m_out, generator=g).to(dt)
    a = [((torch.rand(e, max_r, k_in, generator=g) * 2 - 1) / k_in**0.5).to(dt) for _ in range(nt)]
    b = [(torch.randn(e, m_out, max_r, generator=g) * 0.02).to(dt) for _ in range(nt)]
    ad, bd = [v.to(dev) for v in a], [v.to(dev) for v in b]
    n = e * nt
    groups = AdapterGroups(ad, bd, [r] * n, [2.0] * n, a_index=[i % nt for i in range(n)],
                           a_offset=[(i // nt) * max_r * k_in for i in range(n)], b_index=[i % nt for i in range(n)],
                           b_offset=[(i // nt) * m_out * max_r for i in range(n)])
    xd, dyd = x.to(dev), dy.to(dev)
    y = torch.zeros(rows, m_out, dtype=dt, device=dev)                   # zero base: the LoRA term alone
    h = lora_fwd_(xd, y, seg, groups, map_rows=False)
    ga = torch.full((groups.a_arena_elems,), 7.0, dtype=dt, device=dev)
    gb = torch.full((groups.b_arena_elems,), 7.0, dtype=dt, device=dev)
    dx = torch.zeros_like(xd)
    lora_bwd_(dyd, xd, h, dx, groups._grad_a_rel + ga.data_ptr(), groups._grad_b_rel + gb.data_ptr(), seg, groups,
              map_rows=False, accumulate=False)
    grad_a, grad_b = groups.grad_views(ga, 'a'), groups.grad_views(gb, 'b')
    for i in (0, 7, 8, 77, 300, 301, 302, 511):
        s0, s1 = int(offsets[i]), int(offsets[i + 1])
        ex, tn = i // nt, i % nt
        got_a, got_b = grad_a[tn][ex].cpu(), grad_b[tn][ex].cpu()
        if s0 == s1:
            assert torch.count_nonzero(got_a[:r]) == 0 and torch.count_nonzero(got_b[:, :r]) == 0, i
            continue
        ag, bg = a[tn][ex, :r].double(), b[tn][ex, :, :r].double()
        xg, dyg = x[s0:s1].double(), dy[s0:s1].double()
        hg = 2.0 * xg @ ag.t()
        dh = 2.0 * dyg @ bg
        assert max_rel_err(y[s0:s1], hg @ bg.t()) < 2e-2, f'LoRA term, group {i} ({s1 - s0} rows)'
        assert max_rel_err(dx[s0:s1], dh @ ag) < 2e-2, f'dX, group {i}'
        assert max_rel_err(got_a[:r], dh.t() @ xg) < 2e-2, f'dA, group {i}'
        assert max_rel_err(got_b[:, :r], dyg.t() @ hg) < 2e-2, f'dB, group {i}'
    for tn in range(nt):
        assert torch.isfinite(grad_a[tn].float()).all() and torch.isfinite(grad_b[tn].float()).all()


def test_config4_grouped_linear_128_experts_both_directions(dev):
    """tk_grouped_linear at config 4's size (128 experts x 4 tenants, 65536 routed rows): y = x W_e^T for
    gate_up (2048 -> 1536) and the transposing form dx = dy W_e on the same weights, all rows of sampled experts
    against float64."""
    from twinkle_amd import grouped_linear_
    e, nt, hid, out = 128, 4, 2048, 1536
    keys, tokens = _config4_keys(dev, with_edge_groups=False)
    rows = keys.numel()
    seg = build_segments(keys, e * nt, num_tokens=tokens)
    offsets = seg.offsets.cpu()
    g = torch.Generator().manual_seed(45)
    dt = torch.bfloat16
    x = torch.randn(rows, hid, generator=g).to(dt)
    dy = torch.randn(rows, out, generator=g).to(dt)
    w = (torch.randn(e, out, hid, generator=g) * 0.02).to(dt)
    wd = w.to(dev)
    y = grouped_linear_(x.to(dev), wd, seg, nt, map_rows=False)
    dx = grouped_linear_(dy.to(dev), wd, seg, nt, map_rows=False, transposed=True)
    for ex in (0, 1, 63, 100, 127):
        s0, s1 = int(offsets[ex * nt]), int(offsets[(ex + 1) * nt])
        assert s1 > s0
        assert max_rel_err(y[s0:s1], x[s0:s1].double() @ w[ex].double().t()) < 2e-2, ex
        assert max_rel_err(dx[s0:s1], dy[s0:s1].double() @ w[ex].double()) < 2e-2, ex


def test_config5_one_full_layer_through_multilora_batch(dev):
    """BASELINE config 5, one decoder layer at full size: hidden 4096, 32 heads / 8 KV heads, intermediate 14336,
    rank 64 alpha 128 on all seven projections, 8 tenants, 8 packed sequences x 4096 with tenant j owning
    sequence j, through MultiLora.batch with q/k/v and gate/up declared as shared inputs.  Every projection's
    input, output, output gradient and input gradient is captured on the GPU and checked on the CPU in float64:
    outputs and input gradients on sampled rows of sampled tenants (base GEMM included: the same rows through the
    frozen weight), dA / dB of sampled tenants over all of their 4096 rows."""
    from test_gpu_multilora import _LlamaLayer
    from twinkle_amd import LoraConfig, MultiLora
    torch.manual_seed(7)
    d, heads, kv, inter, r, n, seq = 4096, 32, 8, 14336, 64, 8, 4096
    dt = torch.bfloat16
    layer = _LlamaLayer(d, heads, kv, inter).to(dt).to(dev)
    ml = MultiLora(max_loras=n, max_r=r)
    model = ml.patch(layer, target_modules='all-linear')
    names = [f'tenant_{j}' for j in range(n)]
    for name in names:
        ml.acquire_lora(name, LoraConfig(r=r, lora_alpha=2 * r, target_modules='all-linear'))
    gen = torch.Generator(device=dev).manual_seed(8)
    proj = ['q_proj', 'k_proj', 'v_proj', 'o_proj', 'gate_proj', 'up_proj', 'down_proj']
    mods = {p: getattr(model.model, p) for p in proj}
    with torch.no_grad():
        for p in proj:
            for s in mods[p].lora_B.keys():
                mods[p].lora_B[s].weight.copy_(torch.randn(mods[p].lora_B[s].weight.shape, generator=gen, device=dev) * 0.02)
    ml.share_inputs([['model.q_proj', 'model.k_proj', 'model.v_proj'], ['model.gate_proj', 'model.up_proj']])
    x = torch.randn(n, seq, d, generator=gen, device=dev, dtype=torch.float32).to(dt).requires_grad_(True)
    w = torch.randn(n, seq, d, generator=gen, device=dev, dtype=torch.float32).to(dt)
    cu = packed_cu_seqlens(torch.arange(seq, device=dev).repeat(n)[None])
    row_tenant = token_groups_from_sequences(cu, torch.arange(n, device=dev))
    seen = {}

    def capture(name):
        def hook(mod, args, out):
            inp = args[0]
            seen[name] = {'x': inp.detach(), 'y': out.detach()}
            out.register_hook(lambda gr: seen[name].__setitem__('dy', gr.detach()))
            if inp.requires_grad and name in ('q_proj', 'o_proj', 'gate_proj', 'down_proj'):
                inp.register_hook(lambda gr: seen[name].__setitem__('dx', gr.detach()))
        return hook

    handles = [mods[p].register_forward_hook(capture(p)) for p in proj]
    with ml.batch(names, row_tenant):
        y = model(x)
    (y * w).sum().backward()
    for hnd in handles:
        hnd.remove()
    assert torch.isfinite(y.float()).all() and torch.isfinite(x.grad.float()).all()

    f64 = lambda t: t.detach().double().cpu()  # noqa: E731
    sample = torch.arange(0, seq, 97)[:40]
    sharing = {'q_proj': ['q_proj', 'k_proj', 'v_proj'], 'o_proj': ['o_proj'], 'gate_proj': ['gate_proj', 'up_proj'],
               'down_proj': ['down_proj']}
    for j in (0, 5):                                                   # sampled tenants
        slot = ml.find_lora_by_tenant(names[j]).adapter_name
        rows = j * seq + sample
        allrows = slice(j * seq, (j + 1) * seq)
        dx_want = {}
        for p in proj:
            m = mods[p]
            wb = f64(m.base_layer.weight)
            a, b = f64(m.lora_A[slot].weight), f64(m.lora_B[slot].weight)
            xin = seen[p]['x'].reshape(-1, seen[p]['x'].shape[-1])
            yout = seen[p]['y'].reshape(-1, seen[p]['y'].shape[-1])
            dyo = seen[p]['dy'].reshape(-1, yout.shape[-1])
            xs, dys = f64(xin[rows.to(dev)]), f64(dyo[rows.to(dev)])
            want = xs @ wb.t() + 2.0 * (xs @ a.t()) @ b.t()
            assert max_rel_err(yout[rows.to(dev)], want) < 2e-2, (p, j, 'Y')
            dx_want[p] = dys @ wb + 2.0 * (dys @ b) @ a
            xa, dya = f64(xin[allrows]), f64(dyo[allrows])
            ha, dha = 2.0 * xa @ a.t(), 2.0 * dya @ b
            assert max_rel_err(m.lora_A[slot].weight.grad, dha.t() @ xa) < 2e-2, (p, j, 'dA')
            assert max_rel_err(m.lora_B[slot].weight.grad, dya.t() @ ha) < 2e-2, (p, j, 'dB')
        for first, group in sharing.items():
            got = seen[first]['dx'].reshape(-1, seen[first]['dx'].shape[-1])[rows.to(dev)]
            assert max_rel_err(got, sum(dx_want[p] for p in group)) < 2e-2, (first, j, 'dX')
    # The LoRA part of Y alone, at the same bar: every projection once more on the input it saw, with its frozen
    # weight set to zero, so that what comes out is the LoRA term itself and the bar scales with it (subtracting a
    # base output that was rounded to bf16 would leave that rounding in the difference).
    for p in proj:
        assert mods[p].base_layer.bias is None
    with torch.no_grad():
        for p in proj:
            mods[p].base_layer.weight.zero_()
        with ml.batch(names, row_tenant):
            for p in proj:
                xin = seen[p]['x']
                delta = mods[p](xin)
                delta = delta.reshape(-1, delta.shape[-1])
                for j in (0, 5):
                    slot = ml.find_lora_by_tenant(names[j]).adapter_name
                    rows = (j * seq + sample).to(dev)
                    xs = f64(xin.reshape(-1, xin.shape[-1])[rows])
                    a, b = f64(mods[p].lora_A[slot].weight), f64(mods[p].lora_B[slot].weight)
                    assert max_rel_err(delta[rows], 2.0 * (xs @ a.t()) @ b.t()) < 2e-2, (p, j, 'LoRA part of Y')
