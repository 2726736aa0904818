"""Grouped base GEMM of packed experts (tk_grouped_linear), alone and with the LoRA term in its epilogue,
against the CPU oracle's per-expert loop.  bf16 bar: max |got - ref| / max |ref| < 2e-2 against float64."""
import pytest
import torch

import oracle
from conftest import max_rel_err
from twinkle_amd import AdapterGroups, build_segments, grouped_linear_, lora_h_bytes, lora_shrink_

pytestmark = pytest.mark.gpu


def _case(e, nt, t, k, n, seed, empty=()):
    g = torch.Generator().manual_seed(seed)
    probs = torch.rand(e, generator=g) + 0.2
    for i in empty:
        probs[i] = 0
    expert = torch.multinomial(probs, t, replacement=True, generator=g)
    tenant = torch.randint(0, nt, (t,), generator=g)
    x = torch.randn(t, k, generator=g).bfloat16()
    w = (torch.randn(e, n, k, generator=g) / k**0.5).bfloat16()
    return expert, tenant, x, w


def _reference(x, w, expert):
    """Oracle's chunk loop on rows sorted by expert (stable), scattered back to the original row order."""
    order = torch.argsort(expert, stable=True)
    counts = torch.bincount(expert, minlength=w.shape[0])
    offsets = torch.cat([torch.zeros(1, dtype=torch.long), counts.cumsum(0)])
    out_sorted = oracle.experts_linear(x.double()[order], offsets, w.double())
    out = torch.empty_like(out_sorted)
    out[order] = out_sorted
    return out


@pytest.mark.parametrize('e,nt,t,k,n,empty', [
    (1, 1, 1, 64, 128, ()),            # one row, one expert, smallest legal widths
    (6, 1, 1000, 128, 256, (2,)),      # expert-only grouping (the reference's), one expert without rows
    (5, 3, 1500, 192, 384, (0, 4)),    # three tenants per expert: weights shared by consecutive groups
    (16, 4, 6000, 256, 128, ()),       # experts with more than one 128-row block
    (3, 2, 700, 64, 640, ()),
    (8, 2, 5000, 128, 512, (3,)),      # out_features a multiple of 256: 256-row blocks on 8 waves, experts of
    (2, 1, 300, 64, 256, ()),          # more and of less than one block, dead strips of rows
])
@pytest.mark.parametrize('map_rows', [True, False])
def test_base_term_matches_the_per_expert_loop(dev, e, nt, t, k, n, empty, map_rows):
    expert, tenant, x, w = _case(e, nt, t, k, n, seed=t + n, empty=empty)
    keys = (expert * nt + tenant).to(torch.int32).to(dev)
    seg = build_segments(keys, e * nt)
    want = _reference(x, w, expert)
    xd, wd = x.to(dev), w.to(dev)
    if map_rows:
        y = grouped_linear_(xd, wd, seg, nt, map_rows=True)
        got = y
    else:                                # rows already in segment order, as after permute()
        perm = seg.perm
        y = grouped_linear_(xd[perm].contiguous(), wd, seg, nt, map_rows=False)
        got = torch.empty_like(y)
        got[perm] = y
    assert max_rel_err(got, want) < 2e-2
    # bf16 rounding of an fp32 accumulation: far inside the bar
    assert max_rel_err(got, want) < 6e-3


@pytest.mark.parametrize('weights_f32', [False, True])
@pytest.mark.parametrize('max_r,ranks', [(8, [8, 4, 8]), (16, [16, 0, 9]), (32, [32, 17, 8]), (64, [64, 40, 16])])
@pytest.mark.parametrize('e,t,n', [(4, 1800, 384), (4, 1800, 512), (2, 2600, 512)])
def test_lora_term_in_the_epilogue(dev, max_r, ranks, e, t, n, weights_f32):
    """y = x W_e^T + s (x A_{e,t}^T) B_{e,t}^T per (expert, tenant) segment: oracle's low-rank form per tenant.
    The last shape (out_features a multiple of 256, more than 1024 rows per expert) takes the 256-row blocks on
    8 waves, the others the 128-row blocks on 4 waves."""
    nt, k = len(ranks), 256
    expert, tenant, x, w = _case(e, nt, t, k, n, seed=max_r)
    keys = (expert * nt + tenant).to(torch.int32).to(dev)
    seg = build_segments(keys, e * nt)
    g = torch.Generator().manual_seed(3)
    a = [(torch.randn(e, max_r, k, generator=g) / k**0.5).bfloat16().to(dev) for _ in range(nt)]
    b = [(torch.randn(e, n, max_r, generator=g) * 0.05).bfloat16().to(dev) for _ in range(nt)]
    if weights_f32:      # fp32 adapters under the bf16 activations: the epilogue reads the bf16 copy the call makes
        a, b = [v.float() for v in a], [v.float() for v in b]
    idx = [i % nt for i in range(e * nt)]
    # group i = expert i // nt, tenant i % nt: one block of the tenant's packed tensors (a rank-0 tenant is legal at
    # the kernel boundary: its term is skipped)
    groups = AdapterGroups(a, b, [ranks[i % nt] for i in range(e * nt)], [2.0] * (e * nt),
                           a_index=idx, a_offset=[(i // nt) * max_r * k for i in range(e * nt)],
                           b_index=idx, b_offset=[(i // nt) * n * max_r for i in range(e * nt)], rank_classes=False,
                           act_dtype=torch.bfloat16)
    xd, wd = x.to(dev), w.to(dev)
    h = torch.empty(lora_h_bytes(seg, groups), dtype=torch.uint8, device=dev)
    lora_shrink_(xd, seg, groups, h, map_rows=True)
    got = grouped_linear_(xd, wd, seg, nt, groups=groups, h=h, map_rows=True)
    want = _reference(x, w, expert)
    xs = x.double()
    for ei in range(e):
        for ti in range(nt):
            rows = ((expert == ei) & (tenant == ti)).nonzero().flatten()
            r = ranks[ti]
            if rows.numel() == 0 or r == 0:
                continue
            want[rows] += 2.0 * (xs[rows] @ a[ti][ei, :r].double().cpu().t()) @ b[ti][ei, :, :r].double().cpu().t()
    assert max_rel_err(got, want) < 2e-2


@pytest.mark.parametrize('k,n', [(128, 256), (512, 192), (384, 64), (256, 1024)])
def test_backward_of_the_base_term_on_the_same_weights(dev, k, n):
    """dx = dy W_e is the call with transposed=True on the forward's own weights (the kernel transposes the weight
    tiles on their way into LDS), and equally the plain call on a transposed copy.  in_features k of the forward is
    the output width here: 128 and 384 take the 4-wave kernel, 512 and 256 the 8-wave one."""
    e, nt, t = 5, 2, 1200
    expert, tenant, x, w = _case(e, nt, t, k, n, seed=9)
    dy = torch.randn(t, n, generator=torch.Generator().manual_seed(10)).bfloat16()
    keys = (expert * nt + tenant).to(torch.int32).to(dev)
    seg = build_segments(keys, e * nt)
    wt = w.transpose(1, 2).contiguous()                     # [E, in, out]
    want = _reference(dy, wt, expert)
    got = grouped_linear_(dy.to(dev), w.to(dev), seg, nt, map_rows=True, transposed=True)
    assert max_rel_err(got, want) < 6e-3
    if n % 64 == 0 and k % 128 == 0:
        copy = grouped_linear_(dy.to(dev), wt.to(dev), seg, nt, map_rows=True)
        assert torch.equal(copy, got), 'same products, same order of the sums'
    with pytest.raises(ValueError):
        grouped_linear_(dy.to(dev), w.to(dev), seg, nt, map_rows=True, transposed=True, groups=object(), h=None)


@pytest.mark.parametrize('depth', [64, 128, 192, 320, 384, 448, 832])
@pytest.mark.parametrize('transposed', [False, True])
def test_direct_kernel_depths_block_lengths_and_strides(dev, depth, transposed):
    """The 256-wide kernel that loads its tiles straight into LDS: contractions of 1, 2, 3, 5, 6, 7 and 13 steps of 64
    (its loop is unrolled six times, with a tail), experts of 1 to 8 tiles and of several row blocks (the step is
    compiled per number of live row blocks), x and the weights as views of wider buffers (row strides above the
    widths), in both weight layouts."""
    out_f, nt = 256, 1
    sizes = [20, 40, 70, 100, 130, 170, 200, 230, 600, 0, 257]
    expert = torch.cat([torch.full((c,), i) for i, c in enumerate(sizes)])
    expert = expert[torch.randperm(expert.numel(), generator=torch.Generator().manual_seed(depth))]
    e, t = len(sizes), expert.numel()
    g = torch.Generator().manual_seed(depth + 1)
    xbig = torch.randn(t, depth + 64, generator=g).bfloat16()
    rows, cols = (depth, out_f) if transposed else (out_f, depth)   # [E, in, out] when transposed, else [E, out, in]
    wbig = (torch.randn(e, rows, cols + 64, generator=g) / depth**0.5).bfloat16()
    x, w = xbig[:, :depth], wbig[:, :, :cols]
    seg = build_segments(expert.to(torch.int32).to(dev), e)
    want = _reference(x, w.transpose(1, 2) if transposed else w, expert)
    got = grouped_linear_(xbig.to(dev)[:, :depth], wbig.to(dev)[:, :, :cols], seg, nt, map_rows=True,
                          transposed=transposed)
    assert got.shape == (t, out_f)
    assert max_rel_err(got, want) < 6e-3


@pytest.mark.parametrize('transposed', [False, True])
def test_register_staged_kernels_behind_the_switch(dev, monkeypatch, transposed):
    """TK_GROUPED_DIRECT=0 keeps the 256-wide launches on the kernels that stage their operands through registers
    (what operands of 4 GB and more take): same bar against the oracle, with and without the LoRA term."""
    e, nt, t, k, n = 3, 2, 3400, 256, 512
    expert, tenant, x, w = _case(e, nt, t, k, n, seed=21)
    keys = (expert * nt + tenant).to(torch.int32).to(dev)
    seg = build_segments(keys, e * nt)
    monkeypatch.setenv('TK_GROUPED_DIRECT', '0')
    if transposed:
        dy = torch.randn(t, n, generator=torch.Generator().manual_seed(22)).bfloat16()
        want = _reference(dy, w.transpose(1, 2).contiguous(), expert)
        got = grouped_linear_(dy.to(dev), w.to(dev), seg, nt, map_rows=True, transposed=True)
        assert max_rel_err(got, want) < 6e-3
        monkeypatch.setenv('TK_GROUPED_DIRECT', '1')
        direct = grouped_linear_(dy.to(dev), w.to(dev), seg, nt, map_rows=True, transposed=True)
        assert max_rel_err(direct, want) < 6e-3
        return
    max_r = 16
    g = torch.Generator().manual_seed(23)
    a = [(torch.randn(e, max_r, k, generator=g) / k**0.5).bfloat16().to(dev) for _ in range(nt)]
    b = [(torch.randn(e, n, max_r, generator=g) * 0.05).bfloat16().to(dev) for _ in range(nt)]
    idx = [i % nt for i in range(e * nt)]
    ranks = [16, 9]
    groups = AdapterGroups(a, b, [ranks[i % nt] for i in range(e * nt)], [2.0] * (e * nt),
                           a_index=idx, a_offset=[(i // nt) * max_r * k for i in range(e * nt)],
                           b_index=idx, b_offset=[(i // nt) * n * max_r for i in range(e * nt)], rank_classes=False)
    xd, wd = x.to(dev), w.to(dev)
    h = torch.empty(lora_h_bytes(seg, groups), dtype=torch.uint8, device=dev)
    lora_shrink_(xd, seg, groups, h, map_rows=True)
    want = _reference(x, w, expert)
    assert max_rel_err(grouped_linear_(xd, wd, seg, nt, map_rows=True), want) < 6e-3
    xs = x.double()
    for ei in range(e):
        for ti in range(nt):
            rows = ((expert == ei) & (tenant == ti)).nonzero().flatten()
            if rows.numel():
                r = ranks[ti]
                want[rows] += 2.0 * (xs[rows] @ a[ti][ei, :r].double().cpu().t()) @ b[ti][ei, :, :r].double().cpu().t()
    assert max_rel_err(grouped_linear_(xd, wd, seg, nt, groups=groups, h=h, map_rows=True), want) < 2e-2


def test_unsupported_shapes_are_refused(dev):
    e, nt, t = 2, 1, 64
    keys = torch.zeros(t, dtype=torch.int32, device=dev)
    seg = build_segments(keys, e * nt)
    for k, n in [(96, 128), (64, 192), (32, 128)]:
        x = torch.zeros(t, k, dtype=torch.bfloat16, device=dev)
        w = torch.zeros(e, n, k, dtype=torch.bfloat16, device=dev)
        with pytest.raises(ValueError):
            grouped_linear_(x, w, seg, nt)
    x = torch.zeros(t, 64, dtype=torch.float32, device=dev)
    w = torch.zeros(e, 128, 64, dtype=torch.float32, device=dev)
    with pytest.raises(ValueError):
        grouped_linear_(x, w, seg, nt)                      # fp32: run the experts one by one
    with pytest.raises(ValueError):
        grouped_linear_(x.bfloat16(), w.bfloat16(), seg, 3)  # 2 experts x 3 tenants != 2 groups


def test_experts_forward_grouped_equals_the_per_expert_loop(dev):
    """experts_forward with the grouped GEMMs (the default for frozen bf16 weights of these widths) against its
    per-expert loop (the reference's form, checked against the float64 restatement elsewhere): outputs, dx and
    every tenant's adapter gradients."""
    from twinkle_amd import LoraConfig
    from twinkle_amd.expert_lora import ExpertLoraSlots, experts_forward
    torch.manual_seed(0)
    e, nt, hid, inter, t = 6, 2, 128, 256, 1400

    class Experts(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.gate_up_proj = torch.nn.Parameter((torch.randn(e, 2 * inter, hid) * 0.08).bfloat16(),
                                                   requires_grad=False)
            self.down_proj = torch.nn.Parameter((torch.randn(e, hid, inter) * 0.08).bfloat16(), requires_grad=False)
            self.act_fn = torch.nn.functional.silu

    experts = Experts().to(dev)
    names = ['lora_0', 'lora_1']
    gu = ExpertLoraSlots(e, hid, 2 * inter, max_loras=2, max_r=16, dtype=torch.bfloat16, device=dev)
    dn = ExpertLoraSlots(e, inter, hid, max_loras=2, max_r=16, dtype=torch.bfloat16, device=dev)
    for slots in (gu, dn):
        for name, r in zip(names, (16, 6)):
            slots.configure_slot(name, LoraConfig(r=r, lora_alpha=2 * r))
            with torch.no_grad():
                slots.lora_B[name].normal_(0, 0.05)
    g = torch.Generator().manual_seed(2)
    expert = torch.multinomial(torch.tensor([1.0, 0.2, 0.0, 2.0, 1.0, 0.5]), t, replacement=True, generator=g)
    tenant = torch.randint(0, nt, (t,), generator=g)
    keys = torch.sort(expert * nt + tenant).values.to(torch.int32).to(dev)      # rows already in segment order
    seg = build_segments(keys, e * nt)
    x0 = torch.randn(t, hid, generator=g).bfloat16().to(dev)
    dy = torch.randn(t, hid, generator=g).bfloat16().to(dev)

    def run(grouped):
        for slots in (gu, dn):
            for p in slots.parameters():
                p.grad = None
        x = x0.clone().requires_grad_(True)
        y = experts_forward(experts, x, seg, names, gu, dn, grouped=grouped)
        y.backward(dy)
        grads = [slots.lora_A[n].grad.clone() for slots in (gu, dn) for n in names] + \
                [slots.lora_B[n].grad.clone() for slots in (gu, dn) for n in names]
        return [y.detach(), x.grad] + grads

    loop, fused = run(False), run(True)
    default = run(None)
    for a, b in zip(fused, default):
        assert torch.equal(a, b), 'grouped is the default for these shapes'
    for i, (a, b) in enumerate(zip(fused, loop)):
        assert max_rel_err(a, b.double().cpu()) < 2e-2, i
    assert experts.gate_up_proj.grad is None and experts.down_proj.grad is None


def test_custom_op_matches_the_direct_call(dev):
    """torch.ops.twinkle_amd.grouped_linear gives bit-identical results to the direct binding, with and without
    the LoRA term."""
    import twinkle_amd.custom_ops  # noqa: F401  (registers the ops)
    e, nt, t, k, n, max_r = 4, 2, 900, 128, 256, 16
    expert, tenant, x, w = _case(e, nt, t, k, n, seed=5)
    keys = (expert * nt + tenant).to(torch.int32).to(dev)
    seg = build_segments(keys, e * nt)
    g = torch.Generator().manual_seed(6)
    a = [(torch.randn(e, max_r, k, generator=g) / k**0.5).bfloat16().to(dev) for _ in range(nt)]
    b = [(torch.randn(e, n, max_r, generator=g) * 0.05).bfloat16().to(dev) for _ in range(nt)]
    idx = [i % nt for i in range(e * nt)]
    groups = AdapterGroups(a, b, [16, 7] * e, [2.0] * (e * nt),
                           a_index=idx, a_offset=[(i // nt) * max_r * k for i in range(e * nt)],
                           b_index=idx, b_offset=[(i // nt) * n * max_r for i in range(e * nt)], rank_classes=False)
    xd, wd = x.to(dev), w.to(dev)
    h = torch.empty(lora_h_bytes(seg, groups), dtype=torch.uint8, device=dev)
    lora_shrink_(xd, seg, groups, h, map_rows=True)
    want_base = grouped_linear_(xd, wd, seg, nt, map_rows=True)
    want_lora = grouped_linear_(xd, wd, seg, nt, groups=groups, h=h, map_rows=True)
    empty_i64 = torch.empty(0, dtype=torch.int64, device=dev)
    y = torch.empty_like(want_base)
    torch.ops.twinkle_amd.grouped_linear(xd, wd, y, seg.workspace, nt, e * nt, True, h[:0], empty_i64, empty_i64,
                                         groups.rank_dev[:0], groups.scale_dev[:0], 0, 0, 0)
    assert torch.equal(y, want_base)
    y2 = torch.empty_like(want_base)
    torch.ops.twinkle_amd.grouped_linear(xd, wd, y2, seg.workspace, nt, e * nt, True, h, groups.a_ptrs, groups.b_ptrs,
                                         groups.rank_dev, groups.scale_dev, groups.max_rank, groups.lda, groups.ldb)
    assert torch.equal(y2, want_lora)
    assert not torch.equal(want_base, want_lora)


def test_hip_graph_replay_of_the_grouped_calls(dev):
    """Segment build, shrink, grouped GEMM with the LoRA term and the transposing backward call captured in one HIP
    graph (no host synchronisation anywhere in them) and replayed with fresh inputs: every replay equals eager."""
    e, nt, k, n, max_r = 4, 2, 256, 512, 16
    t = 3000
    g = torch.Generator().manual_seed(12)
    a = [(torch.randn(e, max_r, k, generator=g) / k**0.5).bfloat16().to(dev) for _ in range(nt)]
    b = [(torch.randn(e, n, max_r, generator=g) * 0.05).bfloat16().to(dev) for _ in range(nt)]
    idx = [i % nt for i in range(e * nt)]
    groups = AdapterGroups(a, b, [16, 5] * e, [2.0] * (e * nt),
                           a_index=idx, a_offset=[(i // nt) * max_r * k for i in range(e * nt)],
                           b_index=idx, b_offset=[(i // nt) * n * max_r for i in range(e * nt)], rank_classes=False)
    w = (torch.randn(e, n, k, generator=g) / k**0.5).bfloat16().to(dev)
    keys = torch.empty(t, dtype=torch.int32, device=dev)
    x = torch.empty(t, k, dtype=torch.bfloat16, device=dev)
    dy = torch.empty(t, n, dtype=torch.bfloat16, device=dev)

    def fill(seed):
        gg = torch.Generator().manual_seed(seed)
        keys.copy_(torch.randint(0, e * nt, (t,), generator=gg).to(torch.int32))
        x.copy_(torch.randn(t, k, generator=gg).bfloat16())
        dy.copy_(torch.randn(t, n, generator=gg).bfloat16())

    fill(0)
    seg0 = build_segments(keys, e * nt, want_perm=False, want_offsets=False)
    h = torch.empty(lora_h_bytes(seg0, groups), dtype=torch.uint8, device=dev)
    y = torch.empty(t, n, dtype=torch.bfloat16, device=dev)
    dx = torch.empty(t, k, dtype=torch.bfloat16, device=dev)

    def step():
        seg = build_segments(keys, e * nt, want_perm=False, want_offsets=False)
        lora_shrink_(x, seg, groups, h, map_rows=True)
        grouped_linear_(x, w, seg, nt, y=y, groups=groups, h=h, map_rows=True)
        grouped_linear_(dy, w, seg, nt, y=dx, map_rows=True, transposed=True)

    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                       # warm-up on the capture stream
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            step()
    torch.cuda.current_stream().wait_stream(side)
    for seed in (1, 2, 3):
        fill(seed)
        step()
        torch.cuda.synchronize()
        want_y, want_dx = y.clone(), dx.clone()
        y.zero_()
        dx.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want_y) and torch.equal(dx, want_dx), seed


def _random_grouped_case(seed):
    g = torch.Generator().manual_seed(5000 + seed)
    pick = lambda xs: xs[int(torch.randint(0, len(xs), (1,), generator=g))]  # noqa: E731
    e = pick([1, 2, 3, 7, 16, 40])
    nt = pick([1, 1, 2, 4])
    t = pick([1, 31, 200, 1000, 2500, 6000])
    k = pick([64, 128, 192, 256, 512, 1024])
    n = pick([128, 256, 384, 512, 768, 1024])
    max_r = pick([0, 8, 16, 32, 64])
    return g, e, nt, t, k, n, max_r


@pytest.mark.parametrize('seed', range(24))
def test_random_shapes_of_the_grouped_gemm(dev, seed):
    """Random expert counts, tenant counts, row counts (experts of no, few and thousands of rows), widths (both
    block sizes) and ranks; the forward with the LoRA term where there is one, and the transposing backward
    whenever in_features allows it as an output width."""
    g, e, nt, t, k, n, max_r = _random_grouped_case(seed)
    probs = torch.rand(e, generator=g) ** 3 + 1e-3
    probs[torch.rand(e, generator=g) < 0.2] = 0
    if probs.sum() == 0:
        probs[0] = 1
    expert = torch.multinomial(probs, t, replacement=True, generator=g)
    tenant = torch.randint(0, nt, (t,), generator=g)
    x = torch.randn(t, k, generator=g).bfloat16()
    w = (torch.randn(e, n, k, generator=g) / k**0.5).bfloat16()
    seg = build_segments((expert * nt + tenant).to(torch.int32).to(dev), e * nt)
    xd, wd = x.to(dev), w.to(dev)
    want = _reference(x, w, expert)
    if max_r == 0:
        got = grouped_linear_(xd, wd, seg, nt, map_rows=True)
    else:
        ranks = [int(torch.randint(0, max_r + 1, (1,), generator=g)) for _ in range(nt)]
        ranks[0] = max_r
        a = [(torch.randn(e, max_r, k, generator=g) / k**0.5).bfloat16().to(dev) for _ in range(nt)]
        b = [(torch.randn(e, n, max_r, generator=g) * 0.05).bfloat16().to(dev) for _ in range(nt)]
        idx = [i % nt for i in range(e * nt)]
        groups = AdapterGroups(a, b, [ranks[i % nt] for i in range(e * nt)], [0.5] * (e * nt),
                               a_index=idx, a_offset=[(i // nt) * max_r * k for i in range(e * nt)],
                               b_index=idx, b_offset=[(i // nt) * n * max_r for i in range(e * nt)], rank_classes=False)
        h = torch.empty(lora_h_bytes(seg, groups), dtype=torch.uint8, device=dev)
        lora_shrink_(xd, seg, groups, h, map_rows=True)
        got = grouped_linear_(xd, wd, seg, nt, groups=groups, h=h, map_rows=True)
        for ei in range(e):
            for ti in range(nt):
                rows = ((expert == ei) & (tenant == ti)).nonzero().flatten()
                r = ranks[ti]
                if rows.numel() and r:
                    want[rows] += 0.5 * (x.double()[rows] @ a[ti][ei, :r].double().cpu().t()) @ \
                        b[ti][ei, :, :r].double().cpu().t()
    assert max_rel_err(got, want) < 2e-2
    if k % 128 == 0:                     # the backward of the base term: output width k, contraction over n
        dy = torch.randn(t, n, generator=g).bfloat16()
        dx = grouped_linear_(dy.to(dev), wd, seg, nt, map_rows=True, transposed=True)
        assert max_rel_err(dx, _reference(dy, w.transpose(1, 2).contiguous(), expert)) < 6e-3


@pytest.mark.parametrize('dtype,tol', [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize('rows,inter', [(1, 8), (37, 24), (1000, 768), (5000, 1408)])
def test_swiglu_forward_and_backward(dev, dtype, tol, rows, inter):
    """silu(gate) * up in one pass and its backward against the oracle in float64 on the same rounded inputs."""
    from twinkle_amd import swiglu
    g = torch.Generator().manual_seed(rows + inter)
    gu = (torch.randn(rows, 2 * inter, generator=g) * 2).to(dtype)
    dout = torch.randn(rows, inter, generator=g).to(dtype)
    gud = gu.to(dev).requires_grad_(True)
    out = swiglu(gud)
    out.backward(dout.to(dev))
    gu64 = gu.double().requires_grad_(True)
    want = oracle.swiglu(gu64)
    want.backward(dout.double())
    assert out.dtype == dtype and max_rel_err(out, want) < tol
    assert max_rel_err(gud.grad, gu64.grad) < tol


def test_swiglu_refuses_what_it_cannot_vectorise(dev):
    from twinkle_amd import swiglu
    from twinkle_amd.ops import swiglu_applies
    bad = torch.zeros(4, 20, dtype=torch.bfloat16, device=dev)           # inter = 10
    assert not swiglu_applies(bad)
    with pytest.raises(ValueError):
        swiglu(bad)
    assert swiglu_applies(torch.zeros(4, 32, dtype=torch.bfloat16, device=dev))
    assert not swiglu_applies(torch.zeros(4, 32, dtype=torch.float16, device=dev))


def test_experts_forward_per_expert_loop_keeps_rows_without_an_expert(dev):
    """Keys outside [0, groups) sort behind every expert and belong to none: the per-expert loop (the reference's
    form) returns one row for every input row all the same, zeros for those, and nothing at all still works."""
    from twinkle_amd.expert_lora import experts_forward
    e, hid, inter, t = 3, 64, 96, 50

    class Experts(torch.nn.Module):
        def __init__(self):
            super().__init__()
            g = torch.Generator().manual_seed(1)
            self.gate_up_proj = torch.nn.Parameter(torch.randn(e, 2 * inter, hid, generator=g) * 0.1, requires_grad=False)
            self.down_proj = torch.nn.Parameter(torch.randn(e, hid, inter, generator=g) * 0.1, requires_grad=False)
            self.act_fn = torch.nn.functional.silu

    experts = Experts().to(dev)
    keys = torch.sort(torch.randint(0, e, (t,), generator=torch.Generator().manual_seed(2))).values.to(torch.int32)
    keys[-7:] = e + 1                                                     # rows without an expert, last in order
    seg = build_segments(keys.to(dev), e)
    x = torch.randn(t, hid, generator=torch.Generator().manual_seed(3)).to(dev)
    y = experts_forward(experts, x, seg, ['only'], grouped=False)
    assert y.shape == (t, hid) and torch.count_nonzero(y[-7:]) == 0
    for ex in range(e):
        rows = (keys == ex).nonzero().flatten().to(dev)
        gu = x[rows] @ experts.gate_up_proj[ex].t()
        want = (torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]) @ experts.down_proj[ex].t()
        assert max_rel_err(y[rows], want.double().cpu()) < 1e-5
    none = build_segments(torch.full((t,), -1, dtype=torch.int32, device=dev), e)
    assert torch.count_nonzero(experts_forward(experts, x, none, ['only'], grouped=False)) == 0
