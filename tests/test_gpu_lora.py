"""Segmented LoRA forward/backward through the C ABI against the CPU oracle.

Bars (BASELINE.json): fp32 within 1e-5 relative, bf16 within 2e-2 max relative error against a
float32-or-better reference; here the reference is the oracle in float64 on the same (rounded) inputs,
and "relative" is max|got - ref| / max|ref|.
"""
import pytest
import torch

import oracle
from conftest import max_rel_err
from twinkle_amd import AdapterGroups, build_segments, lora_bwd_, lora_fwd_, multi_lora_delta, multi_lora_linear
from twinkle_amd import workloads

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


def _problem(t, k, m, n, max_r, ranks, seed, ids=None):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(t, k, generator=g)
    base = torch.randn(t, m, generator=g)
    dy = torch.randn(t, m, generator=g)
    a = [(torch.rand(max_r, k, generator=g) * 2 - 1) / k**0.5 for _ in range(n)]
    b = [torch.randn(m, max_r, generator=g) * 0.05 for _ in range(n)]
    if ids is None:
        ids = torch.randint(0, n, (t,), generator=g)
    scales = [2.0 if i % 2 == 0 else 0.5 for i in range(n)]
    return x, base, dy, a, b, ids, list(ranks), scales


def lora_fwd_zero_base(x, seg, groups, map_rows=True):
    """The LoRA term of every row on its own: the forward applied to a base output of zeros."""
    y0 = torch.zeros(x.shape[0], groups.out_features, dtype=x.dtype, device=x.device)
    lora_fwd_(x, y0, seg, groups, map_rows)
    return y0


def _run(dev, dtype, x, base, dy, a, b, ids, ranks, scales, check_zero_beyond_rank=True, weights_f32=False):
    """GPU through autograd vs oracle in float64 on the same rounded inputs.  ``weights_f32``: the adapters stay
    fp32 tensors under activations of ``dtype`` (bf16); the oracle then works from the fp32 values, so the bar also
    covers the rounding of the weights inside the library."""
    cast = lambda t: t.to(dtype)  # noqa: E731
    wcast = (lambda t: t.float()) if weights_f32 else cast  # noqa: E731
    xd = cast(x).to(dev).requires_grad_(True)
    yd = cast(base).to(dev).requires_grad_(True)
    ad = [wcast(t).to(dev).requires_grad_(True) for t in a]
    bd = [wcast(t).to(dev).requires_grad_(True) for t in b]
    seg = build_segments(ids.to(torch.int32).to(dev), len(a), check=True)
    groups = AdapterGroups(ad, bd, ranks, scales, act_dtype=dtype if weights_f32 else None)
    y = multi_lora_delta(xd, yd * 1.0, seg, groups)
    y.backward(cast(dy).to(dev))
    f64 = lambda t: cast(t).double()  # noqa: E731
    w64 = lambda t: wcast(t).double()  # noqa: E731
    yo, dxo, dao, dbo = oracle.multi_lora_linear_grads(f64(x), f64(base), ids, [w64(t) for t in a],
                                                        [w64(t) for t in b], ranks, scales, f64(dy))
    tol = TOL[dtype]
    if weights_f32:
        assert all(t.grad is None or t.grad.dtype == torch.float32 for t in ad + bd), 'fp32 gradients'
    assert max_rel_err(y, yo) < tol, 'Y'
    # the LoRA term alone, on a zero base: the bar then scales with the term itself, not with the base output
    # (which at these shapes is an order of magnitude larger and would hide an error in the term)
    delta = lora_fwd_zero_base(xd.detach(), seg, groups)
    assert max_rel_err(delta, yo - f64(base)) < tol, 'LoRA term'
    assert max_rel_err(xd.grad, dxo) < tol, 'dX'
    assert torch.equal(yd.grad.cpu(), cast(dy)), 'dY passes through to the base output unchanged'
    for g in range(len(a)):
        if ranks[g] == 0:      # an adapter that is not live gets no gradient at all (the reference's inactive ones)
            assert ad[g].grad is None and bd[g].grad is None, f'adapter {g} has rank 0'
            assert torch.count_nonzero(dao[g]) == 0 and torch.count_nonzero(dbo[g]) == 0
            continue
        assert max_rel_err(ad[g].grad, dao[g]) < tol, f'dA[{g}]'
        assert max_rel_err(bd[g].grad, dbo[g]) < tol, f'dB[{g}]'
        if check_zero_beyond_rank:
            assert torch.count_nonzero(ad[g].grad[ranks[g]:]) == 0
            assert torch.count_nonzero(bd[g].grad[:, ranks[g]:]) == 0
    zeros = lambda ts: [t.grad if t.grad is not None else torch.zeros_like(t) for t in ts]  # noqa: E731
    return y, xd.grad, zeros(ad), zeros(bd)


def test_config1_fp32_plumbing(dev):
    """BASELINE config 1: T=512, 1024->1024, 4 adapters rank 8 alpha 16, contiguous segments; Y, dX, dA, dB."""
    w = workloads.config1_plumbing()
    _run(dev, torch.float32, w.x, w.base_out, w.dy, w.lora_A, w.lora_B, w.ids, w.ranks, w.scales)


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('t,k,m,n,max_r,ranks', [
    (1, 8, 8, 1, 4, [4]),
    (33, 40, 24, 3, 8, [2, 8, 5]),                 # odd widths: generic kernels
    (257, 128, 256, 4, 16, [16, 8, 16, 1]),
    (700, 256, 128, 5, 32, [32, 0, 16, 8, 24]),   # a rank-0 (skipped) adapter
    (1500, 384, 640, 6, 64, [64, 8, 16, 32, 64, 4]),
    (900, 256, 1024, 5, 16, [16, 3, 0, 9, 16]),    # rank <= 16, out width a multiple of 512: one pass over dy
    (2100, 128, 1536, 4, 8, [8, 8, 1, 5]),         # ... with groups that span several chunks
    (1300, 256, 1024, 5, 32, [32, 17, 0, 24, 5]),  # the same at rank 17..32 (two rank blocks per wave)
    (2600, 128, 2048, 3, 24, [24, 24, 20]),
])
def test_small_shapes(dev, dtype, t, k, m, n, max_r, ranks):
    _run(dev, dtype, *_problem(t, k, m, n, max_r, ranks, seed=t))


@pytest.mark.parametrize('t,k,m,n,max_r,ranks', [
    (33, 40, 24, 3, 8, [2, 8, 5]),                 # odd widths: generic kernels
    (257, 128, 256, 4, 16, [16, 8, 16, 1]),
    (900, 256, 1024, 5, 16, [16, 3, 0, 9, 16]),    # one pass over dy, a dead adapter
    (2100, 128, 1536, 4, 8, [8, 8, 1, 5]),         # groups that span several chunks: partial sums, fp32 reduction
    (1300, 256, 1024, 5, 32, [32, 17, 0, 24, 5]),
    (1500, 384, 640, 6, 64, [64, 8, 16, 32, 64, 4]),
    (2304, 2048, 512, 2, 64, [64, 48]),            # rank 64, long groups: the shrink with weights shared in LDS
])
def test_fp32_adapters_under_bf16_activations(dev, t, k, m, n, max_r, ranks):
    """tk_lora_desc::weights_f32: A and B are read as fp32 (converted to bf16 on the fly inside the library), the
    products run on the bf16 kernels, dA and dB come back as fp32 (PEFT's adapters under a bf16 base,
    multi_lora.py:320).  Bar: the bf16 bar against the fp64 oracle on the unrounded weights."""
    _run(dev, torch.bfloat16, *_problem(t, k, m, n, max_r, ranks, seed=t + 1), weights_f32=True)


def test_fp32_adapters_gradient_accumulation(dev):
    """accumulate=1 with fp32 gradients: a second backward adds onto the first in fp32."""
    from twinkle_amd import lora_bwd_, lora_fwd_
    x, base, dy, a, b, ids, ranks, scales = _problem(1100, 256, 1024, 3, 16, [16, 8, 16], seed=9)
    xd, yd, dyd = (t.bfloat16().to(dev) for t in (x, base, dy))
    ad, bd = [t.float().to(dev) for t in a], [t.float().to(dev) for t in b]
    seg = build_segments(ids.to(torch.int32).to(dev), 3)
    groups = AdapterGroups(ad, bd, ranks, scales, act_dtype=torch.bfloat16)
    h = lora_fwd_(xd, yd.clone(), seg, groups)
    ga, gb = [torch.zeros_like(t) for t in ad], [torch.zeros_like(t) for t in bd]
    pa = torch.tensor([t.data_ptr() for t in ga], dtype=torch.int64, device=dev)
    pb = torch.tensor([t.data_ptr() for t in gb], dtype=torch.int64, device=dev)
    lora_bwd_(dyd, xd, h, None, pa, pb, seg, groups, accumulate=False)
    once_a, once_b = [t.clone() for t in ga], [t.clone() for t in gb]
    lora_bwd_(dyd, xd, h, None, pa, pb, seg, groups, accumulate=True)
    for one, two in zip(once_a + once_b, ga + gb):
        assert torch.equal(two, one + one)     # fp32 adds of equal numbers are exact


@pytest.mark.parametrize('mask', [None, 0, 0b101, 0b110, 0b111])
def test_rank_class_masks_give_the_same_backward(dev, mask):
    """Per-group ranks (src/twinkle/model/multi_lora.py:318-325) with every way of telling the backward about them:
    the mask made from the live ranks (None), no mask (one class, everything padded to rank 64), and masks that
    leave a class out although groups of it exist (0b101: ranks 24 and 32 go to the 33..64 kernels; 0b110: ranks 5
    to 16 go to the 17..32 kernels).  Every variant against the oracle at the bf16 bar, and dX / dA / dB of every
    variant close to the single-class result (the classes use kernels with other summation orders, so not bitwise)."""
    ranks = [8, 16, 24, 32, 48, 64, 0, 5]
    t, k, m, max_r = 3000, 256, 512, 64
    x, base, dy, a, b, ids, ranks, scales = _problem(t, k, m, len(ranks), max_r, ranks, seed=77)
    cast = lambda v: v.bfloat16()  # noqa: E731
    seg = build_segments(ids.to(torch.int32).to(dev), len(a), check=True)
    f64 = lambda v: cast(v).double()  # noqa: E731
    _, dxo, dao, dbo = oracle.multi_lora_linear_grads(f64(x), f64(base), ids, [f64(v) for v in a], [f64(v) for v in b],
                                                      ranks, scales, f64(dy))

    def backward(rank_classes):
        xd = cast(x).to(dev).requires_grad_(True)
        ad = [cast(v).to(dev).requires_grad_(True) for v in a]
        bd = [cast(v).to(dev).requires_grad_(True) for v in b]
        groups = AdapterGroups(ad, bd, ranks, scales)
        assert groups.rank_classes == 0b111, 'ranks 5..64 span three classes'
        if rank_classes is not None:
            groups.rank_classes = rank_classes
        multi_lora_delta(xd, cast(base).to(dev), seg, groups).backward(cast(dy).to(dev))
        return xd.grad, [v.grad for v in ad], [v.grad for v in bd]

    dx, da, db = backward(mask)
    dx1, da1, db1 = backward(0)
    assert max_rel_err(dx, dxo) < 2e-2 and max_rel_err(dx, dx1.double().cpu()) < 1e-2
    for g, r in enumerate(ranks):
        if r == 0:
            assert da[g] is None and db[g] is None
            continue
        assert max_rel_err(da[g], dao[g]) < 2e-2 and max_rel_err(db[g], dbo[g]) < 2e-2, f'group {g} (rank {r})'
        assert max_rel_err(da[g], da1[g].double().cpu()) < 1e-2 and max_rel_err(db[g], db1[g].double().cpu()) < 1e-2
        assert torch.count_nonzero(da[g][r:]) == 0 and torch.count_nonzero(db[g][:, r:]) == 0


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_empty_and_huge_segments(dev, dtype):
    t, n = 2100, 6
    ids = torch.zeros(t, dtype=torch.long)
    ids[:40] = 3          # one tiny segment, adapters 1, 2, 4, 5 empty, adapter 0 spans several chunks
    ids = ids[torch.randperm(t, generator=torch.Generator().manual_seed(0))]
    x, base, dy, a, b, _, ranks, scales = _problem(t, 256, 128, n, 16, [16] * n, seed=3)
    _, _, da, db = _run(dev, dtype, x, base, dy, a, b, ids, ranks, scales)
    for g in (1, 2, 4, 5):
        assert torch.count_nonzero(da[g]) == 0 and torch.count_nonzero(db[g]) == 0


@pytest.mark.parametrize('dtype,t,k,m,max_r,ranks', [
    (torch.bfloat16, 3000, 256, 1024, 16, [16, 8, 16]),     # single pass over dy, several chunks per group
    (torch.bfloat16, 1500, 256, 384, 64, [64, 20, 33]),     # separate kernels, two streams
    (torch.float32, 700, 40, 24, 8, [8, 3, 5]),             # generic kernels
])
def test_rows_without_an_adapter_keep_the_base_output(dev, dtype, t, k, m, max_r, ranks):
    """Ids outside [0, adapters) (-1 for padding or ignored rows, or too large) belong to no adapter: such rows
    keep the base output, get no input gradient from the LoRA branch and add to nobody's dA / dB; the
    permutation places them after the last group.  The oracle skips them the same way."""
    n = len(ranks)
    x, base, dy, a, b, ids, _, scales = _problem(t, k, m, n, max_r, ranks, seed=t + 1)
    g = torch.Generator().manual_seed(t)
    ids = ids.clone()
    ids[torch.rand(t, generator=g) < 0.2] = -1
    ids[torch.rand(t, generator=g) < 0.05] = n + 3
    ids[:40] = -1                                  # more than a tile of them in a row
    none = (ids < 0) | (ids >= n)
    cast = lambda v: v.to(dtype)  # noqa: E731
    xd = cast(x).to(dev).requires_grad_(True)
    ad = [cast(v).to(dev).requires_grad_(True) for v in a]
    bd = [cast(v).to(dev).requires_grad_(True) for v in b]
    seg = build_segments(ids.to(torch.int32).to(dev), n)
    assert seg.bad_keys() == int(none.sum())
    perm, _, offsets = oracle.segment_build_sort(ids, n)
    assert torch.equal(seg.perm.cpu(), perm) and torch.equal(seg.offsets.cpu(), offsets)
    assert int(offsets[n]) == t - int(none.sum())
    groups = AdapterGroups(ad, bd, ranks, scales)
    based = cast(base).to(dev)
    y = multi_lora_delta(xd, based * 1.0, seg, groups)
    y.backward(cast(dy).to(dev))
    f64 = lambda v: cast(v).double()  # noqa: E731
    yo, dxo, dao, dbo = oracle.multi_lora_linear_grads(f64(x), f64(base), ids, [f64(v) for v in a],
                                                        [f64(v) for v in b], ranks, scales, f64(dy))
    tol = TOL[dtype]
    assert torch.equal(y[none.to(dev)], based[none.to(dev)]), 'rows without an adapter: base output, bit for bit'
    assert torch.count_nonzero(xd.grad[none.to(dev)]) == 0
    assert max_rel_err(y, yo) < tol and max_rel_err(xd.grad, dxo) < tol
    assert max_rel_err(lora_fwd_zero_base(xd.detach(), seg, groups), yo - f64(base)) < tol
    for i in range(n):
        assert max_rel_err(ad[i].grad, dao[i]) < tol and max_rel_err(bd[i].grad, dbo[i]) < tol


def test_results_are_bitwise_repeatable(dev):
    p = _problem(3000, 512, 256, 4, 16, [16, 8, 16, 16], seed=5)
    r1 = _run(dev, torch.bfloat16, *p)
    r2 = _run(dev, torch.bfloat16, *p)
    assert torch.equal(r1[0], r2[0]) and torch.equal(r1[1], r2[1])
    for u, v in zip(r1[2] + r1[3], r2[2] + r2[3]):
        assert torch.equal(u, v)


def test_my_gradients_ignore_other_tenants_rows(dev):
    """Reference invariant: only the active adapter is updated (tests/model/test_multi_lora_target_parameters.py:78-100)."""
    x, base, dy, a, b, ids, ranks, scales = _problem(900, 256, 256, 3, 16, [16, 16, 8], seed=6)
    _, _, da, db = _run(dev, torch.bfloat16, x, base, dy, a, b, ids, ranks, scales)
    x2 = x.clone()
    x2[ids != 0] = 7.0
    _, _, da2, db2 = _run(dev, torch.bfloat16, x2, base, dy, a, b, ids, ranks, scales)
    assert torch.equal(da[0], da2[0]) and torch.equal(db[0], db2[0])


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_fused_base_linear_node(dev, dtype):
    """F.linear + LoRA as one autograd node: dX of the base GEMM updated in place."""
    t, k, m, n = 600, 256, 384, 3
    x, _, dy, a, b, ids, ranks, scales = _problem(t, k, m, n, 16, [16, 4, 8], seed=7)
    w = torch.randn(m, k, generator=torch.Generator().manual_seed(8)) * 0.05
    bias = torch.randn(m, generator=torch.Generator().manual_seed(9))
    cast = lambda v: v.to(dtype)  # noqa: E731
    xd = cast(x).to(dev).requires_grad_(True)
    ad = [cast(v).to(dev).requires_grad_(True) for v in a]
    bd = [cast(v).to(dev).requires_grad_(True) for v in b]
    seg = build_segments(ids.to(torch.int32).to(dev), n)
    y = multi_lora_linear(xd, cast(w).to(dev), cast(bias).to(dev), seg, AdapterGroups(ad, bd, ranks, scales))
    y.backward(cast(dy).to(dev))
    f64 = lambda v: cast(v).double()  # noqa: E731
    x64 = f64(x).requires_grad_(True)
    a64 = [f64(v).requires_grad_(True) for v in a]
    b64 = [f64(v).requires_grad_(True) for v in b]
    base64 = torch.nn.functional.linear(x64, f64(w), f64(bias))
    if dtype == torch.bfloat16:
        base64 = base64.detach().bfloat16().double() + (base64 - base64.detach())  # base GEMM output is stored in bf16
    yo = oracle.multi_lora_linear(x64, base64, ids, a64, b64, ranks, scales)
    yo.backward(f64(dy))
    tol = TOL[dtype] * (2 if dtype == torch.bfloat16 else 20)   # the base GEMM runs in the library's own order
    assert max_rel_err(y, yo) < tol
    assert max_rel_err(xd.grad, x64.grad) < tol
    for g in range(n):
        assert max_rel_err(ad[g].grad, a64[g].grad) < TOL[dtype]
        assert max_rel_err(bd[g].grad, b64[g].grad) < TOL[dtype]


def test_rows_already_in_segment_order_and_packed_expert_weights(dev):
    """map_rows=0 with (expert, tenant) groups reading blocks of packed [E, max_r, in] tensors (config 4 shape, small)."""
    e, nt, t, k_in, m_out, max_r, r = 6, 2, 500, 128, 256, 8, 4
    g = torch.Generator().manual_seed(10)
    keys = torch.randint(0, e * nt, (t,), generator=g)
    a = [torch.randn(e, max_r, k_in, generator=g) * 0.1 for _ in range(nt)]
    b = [torch.randn(e, m_out, max_r, generator=g) * 0.1 for _ in range(nt)]
    x = torch.randn(t, k_in, generator=g)
    base = torch.randn(t, m_out, generator=g)
    dy = torch.randn(t, m_out, generator=g)
    dtype = torch.bfloat16
    cast = lambda v: v.to(dtype)  # noqa: E731
    seg = build_segments(keys.to(torch.int32).to(dev), e * nt)
    perm = seg.perm
    xs = cast(x).to(dev)[perm].requires_grad_(True)           # rows physically in segment order
    ys = cast(base).to(dev)[perm]
    ad = [cast(v).to(dev).requires_grad_(True) for v in a]
    bd = [cast(v).to(dev).requires_grad_(True) for v in b]
    groups = AdapterGroups(ad, bd, [r] * (e * nt), [2.0] * (e * nt),
                           a_index=[i % nt for i in range(e * nt)], a_offset=[(i // nt) * max_r * k_in for i in range(e * nt)],
                           b_index=[i % nt for i in range(e * nt)], b_offset=[(i // nt) * m_out * max_r for i in range(e * nt)])
    y = multi_lora_delta(xs, ys * 1.0, seg, groups, map_rows=False)
    y.backward(cast(dy).to(dev)[perm])
    # oracle: group i = (expert i // nt, tenant i % nt)
    f64 = lambda v: cast(v).double()  # noqa: E731
    a_list = [f64(a[i % nt][i // nt]) for i in range(e * nt)]
    b_list = [f64(b[i % nt][i // nt]) for i in range(e * nt)]
    yo, dxo, dao, dbo = oracle.multi_lora_linear_grads(f64(x), f64(base), keys, a_list, b_list, [r] * (e * nt),
                                                        [2.0] * (e * nt), f64(dy))
    pc = perm.cpu()
    assert max_rel_err(y, yo[pc]) < 2e-2
    assert max_rel_err(xs.grad, dxo[pc]) < 2e-2
    for i in range(e * nt):
        assert max_rel_err(ad[i % nt].grad[i // nt], dao[i]) < 2e-2
        assert max_rel_err(bd[i % nt].grad[i // nt], dbo[i]) < 2e-2
    # the same thing as the reference's merged-weight expert loop (W + dW)
    offsets = seg.offsets.cpu()
    for i in (0, 5, e * nt - 1):
        s, t_ = int(offsets[i]), int(offsets[i + 1])
        if s == t_:
            continue
        dw = oracle.expert_delta_weight(f64(a[i % nt]), f64(b[i % nt]), r, 2.0)[i // nt]
        want = f64(base)[pc][s:t_] + f64(x)[pc][s:t_] @ dw.t()
        assert max_rel_err(y[s:t_], want) < 2e-2


def test_accumulate_and_strided_inputs(dev):
    """C ABI directly: row strides larger than the width, accumulate=1 adds onto existing gradients."""
    t, k, m, n, max_r = 400, 256, 128, 2, 16
    x, base, dy, a, b, ids, ranks, scales = _problem(t, k, m, n, max_r, [16, 8], seed=11)
    dt = torch.bfloat16
    xbuf = torch.zeros(t, k + 64, dtype=dt, device=dev)
    ybuf = torch.zeros(t, m + 128, dtype=dt, device=dev)
    dybuf = torch.zeros(t, m + 8, dtype=dt, device=dev)
    xbuf[:, :k] = x.to(dt).to(dev)
    ybuf[:, :m] = base.to(dt).to(dev)
    dybuf[:, :m] = dy.to(dt).to(dev)
    xv, yv, dyv = xbuf[:, :k], ybuf[:, :m], dybuf[:, :m]
    ad = [v.to(dt).to(dev) for v in a]
    bd = [v.to(dt).to(dev) for v in b]
    seg = build_segments(ids.to(torch.int32).to(dev), n)
    groups = AdapterGroups(ad, bd, ranks, scales)
    h = lora_fwd_(xv, yv, seg, groups)
    ga = [torch.ones_like(v) for v in ad]
    gb = [torch.ones_like(v) for v in bd]
    pa = torch.tensor([v.data_ptr() for v in ga], dtype=torch.int64, device=dev)
    pb = torch.tensor([v.data_ptr() for v in gb], dtype=torch.int64, device=dev)
    dx = torch.ones(t, k, dtype=dt, device=dev)
    lora_bwd_(dyv, xv, h, dx, pa, pb, seg, groups, accumulate=True)
    f64 = lambda v: v.to(dt).double()  # noqa: E731
    yo, dxo, dao, dbo = oracle.multi_lora_linear_grads(f64(x), f64(base), ids, [f64(v) for v in a],
                                                        [f64(v) for v in b], ranks, scales, f64(dy))
    assert max_rel_err(yv, yo) < 2e-2
    assert torch.count_nonzero(ybuf[:, m:]) == 0, 'padding columns untouched'
    assert max_rel_err(dx, dxo + 1.0) < 2e-2
    for g in range(n):
        r = ranks[g]
        assert max_rel_err(ga[g][:r], dao[g][:r] + 1.0) < 2e-2
        assert max_rel_err(gb[g][:, :r], dbo[g][:, :r] + 1.0) < 2e-2
        assert torch.all(ga[g][r:] == 1) and torch.all(gb[g][:, r:] == 1), 'outside the live block: untouched'


def test_argument_errors(dev):
    x, base, dy, a, b, ids, ranks, scales = _problem(64, 32, 32, 2, 8, [8, 8], seed=12)
    ad = [v.to(dev) for v in a]
    bd = [v.to(dev) for v in b]
    seg = build_segments(ids.to(torch.int32).to(dev), 2)
    groups = AdapterGroups(ad, bd, ranks, scales)
    with pytest.raises(ValueError):
        lora_fwd_(x.to(dev)[:, :16], base.to(dev), seg, groups)            # wrong width
    with pytest.raises(ValueError):
        lora_fwd_(x.bfloat16().to(dev), base.to(dev), seg, groups)          # dtype mismatch
    with pytest.raises(RuntimeError):
        lora_fwd_(x, base, seg, groups)                                     # CPU tensors
    with pytest.raises(RuntimeError):
        AdapterGroups(ad, bd, [9, 8], scales)                               # rank above the slot size
    seg3 = build_segments(ids.to(torch.int32).to(dev), 3)
    with pytest.raises(ValueError):
        lora_fwd_(x.to(dev), base.to(dev), seg3, groups)                    # group count mismatch


def test_config2_full_size_bf16(dev):
    """BASELINE config 2 at full size: 4096->4096, T=16384, 16 adapters rank 16, Zipf ids, shuffled."""
    w = workloads.config2_qproj()
    _run(dev, torch.bfloat16, w.x, w.base_out, w.dy, w.lora_A, w.lora_B, w.ids, w.ranks, w.scales)


def test_custom_ops_match_direct_calls(dev):
    """torch.ops.twinkle_amd.{segment_build, lora_fwd, lora_bwd} give bit-identical results to the direct bindings."""
    from twinkle_amd import lora_bwd_, lora_bwd_workspace_bytes, lora_fwd_, lora_h_bytes
    t, k, m, n = 700, 256, 1024, 4
    x, base, dy, a, b, ids, ranks, scales = _problem(t, k, m, n, 16, [16, 8, 16, 3], seed=11)
    bf = lambda v: v.bfloat16().to(dev)  # noqa: E731
    xd, dyd = bf(x), bf(dy)
    ad, bd = [bf(v) for v in a], [bf(v) for v in b]
    groups = AdapterGroups(ad, bd, ranks, scales)
    keys = ids.to(torch.int32).to(dev)
    seg = build_segments(keys, n)

    def grads():
        ga = torch.zeros(groups.a_arena_elems, dtype=torch.bfloat16, device=dev)
        gb = torch.zeros(groups.b_arena_elems, dtype=torch.bfloat16, device=dev)
        return ga, gb, groups._grad_a_rel + ga.data_ptr(), groups._grad_b_rel + gb.data_ptr()

    # direct
    y1 = bf(base)
    h1 = lora_fwd_(xd, y1, seg, groups)
    dx1 = torch.zeros_like(xd)
    ga1, gb1, pa, pb = grads()
    lora_bwd_(dyd, xd, h1, dx1, pa, pb, seg, groups)
    # through the dispatcher
    ws = torch.ops.twinkle_amd.segment_build(keys, n)
    assert ws.numel() == seg.workspace.numel()
    y2 = bf(base)
    h2 = torch.empty(lora_h_bytes(seg, groups), dtype=torch.uint8, device=dev)
    args = (ws, groups.a_ptrs, groups.b_ptrs, groups.rank_dev, groups.scale_dev, groups.max_rank, groups.lda,
            groups.ldb, True)
    torch.ops.twinkle_amd.lora_fwd(xd, y2, h2, *args)
    dx2 = torch.zeros_like(xd)
    ga2, gb2, pa, pb = grads()
    wsb = torch.empty(lora_bwd_workspace_bytes(seg, groups), dtype=torch.uint8, device=dev)
    torch.ops.twinkle_amd.lora_bwd(dyd, xd, h2, dx2, ga2, gb2, pa, pb, wsb, *args, False)
    assert torch.equal(y1, y2) and torch.equal(dx1, dx2) and torch.equal(ga1, ga2) and torch.equal(gb1, gb2)
    assert y1.float().sub(bf(base).float()).abs().max() > 0


@pytest.mark.parametrize('max_r,ranks', [(16, [16, 7, 16]), (32, [32, 16, 24]), (64, [64, 16, 40])])
def test_hip_graph_replay_matches_eager(dev, max_r, ranks):
    """Segment build + forward + backward captured in a HIP graph and replayed: every replay equals the eager result.

    Ranks 16 and 32 take the single-pass dy kernel; rank 64 takes the separate kernels, whose backward forks onto
    the library's side stream and joins back (both must be capturable).  Eager work and synchronisations run
    between the replays.
    """
    from twinkle_amd import lora_bwd_, lora_bwd_workspace_bytes, lora_fwd_, lora_h_bytes
    t, k, m, n = 1200, 256, 1024, 3
    x, base, dy, a, b, ids, _, scales = _problem(t, k, m, n, max_r, ranks, seed=21)
    bf = lambda v: v.bfloat16().to(dev)  # noqa: E731
    xd, dyd, based = bf(x), bf(dy), bf(base)
    groups = AdapterGroups([bf(v) for v in a], [bf(v) for v in b], ranks, scales)
    keys = ids.to(torch.int32).to(dev)
    seg0 = build_segments(keys, n, want_perm=False, want_offsets=False)
    h = torch.empty(lora_h_bytes(seg0, groups), dtype=torch.uint8, device=dev)
    ws = torch.empty(lora_bwd_workspace_bytes(seg0, groups), dtype=torch.uint8, device=dev)
    ga = torch.zeros(groups.a_arena_elems, dtype=torch.bfloat16, device=dev)
    gb = torch.zeros(groups.b_arena_elems, dtype=torch.bfloat16, device=dev)
    pa, pb = groups._grad_a_rel + ga.data_ptr(), groups._grad_b_rel + gb.data_ptr()
    y, dx = torch.empty_like(based), torch.empty_like(xd)

    def step():
        y.copy_(based)
        dx.fill_(0)      # a fill kernel, not a memset node
        seg = build_segments(keys, n, want_perm=False, want_offsets=False)
        lora_fwd_(xd, y, seg, groups, h=h)
        lora_bwd_(dyd, xd, h, dx, pa, pb, seg, groups, accumulate=False, workspace=ws)

    step()
    torch.cuda.synchronize()
    want = [v.clone() for v in (y, dx, ga, gb)]
    assert want[1].abs().max() > 0 and want[3].abs().max() > 0
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        step()                       # warm-up on the capture stream
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            step()
    torch.cuda.current_stream().wait_stream(side)
    for _ in range(3):
        for v in (y, dx, ga, gb):
            v.fill_(1)               # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want[0]) and torch.equal(dx, want[1])
        # weight gradients are written up to each adapter's rank only: compare the live blocks
        for g, r in enumerate(ranks):
            got_a, ref_a = groups.grad_views(ga, 'a')[g], groups.grad_views(want[2], 'a')[g]
            got_b, ref_b = groups.grad_views(gb, 'b')[g], groups.grad_views(want[3], 'b')[g]
            assert torch.equal(got_a[:r], ref_a[:r]) and torch.equal(got_b[:, :r], ref_b[:, :r])


@pytest.mark.parametrize('dtype,t,k,m,max_r,ranks', [
    (torch.bfloat16, 20000, 128, 1024, 16, [16, 5, 16]),    # 32-tile chunks, single pass over dy
    (torch.bfloat16, 40000, 128, 256, 64, [64, 17, 40]),    # 64-tile chunks, rank indices split over two waves
    (torch.float32, 17000, 24, 40, 8, [8, 3]),              # generic kernels walk a chunk in passes of 512 slots
    (torch.bfloat16, 140000, 128, 1024, 16, [16, 5, 16]),   # 128-tile chunks (the largest), single pass over dy
    (torch.bfloat16, 140000, 256, 128, 64, [64, 30]),       # 128-tile chunks on the two-wave kernels
    (torch.float32, 140000, 24, 40, 8, [8, 3]),             # and on the generic ones
])
def test_chunks_larger_than_512_rows(dev, dtype, t, k, m, max_r, ranks):
    """Above 16384 rows a chunk of the row contractions holds 32 or more tiles; groups span several such chunks."""
    n = len(ranks)
    x, base, dy, a, b, _, _, scales = _problem(t, k, m, n, max_r, ranks, seed=t)
    ids = torch.zeros(t, dtype=torch.long)
    ids[: t // 7] = 1 % n
    ids[t // 7: t // 7 + 50] = n - 1          # one group far smaller than a chunk
    ids = ids[torch.randperm(t, generator=torch.Generator().manual_seed(1))]
    _run(dev, dtype, x, base, dy, a, b, ids, ranks, scales)


@pytest.mark.parametrize('weights_f32', [False, True])
def test_rank_64_chunk_pairs_with_odd_and_even_first_slots(dev, weights_f32):
    """At padded rank 64 a weight-gradient work item is two consecutive chunks of a group and the reduction reads
    every other partial slot.  Group sizes chosen so that groups start at even and at odd slots and have 1, 2, 3, 4,
    6 and 8 chunks of 128 rows (3000 rows: four tiles per chunk), one of them ending in a six-row chunk."""
    sizes = [390, 300, 1000, 130, 128, 700, 352]
    ranks = [64, 40, 64, 33, 64, 50, 64]
    t, k, m = sum(sizes), 256, 384
    ids = torch.cat([torch.full((n,), g) for g, n in enumerate(sizes)])
    ids = ids[torch.randperm(t, generator=torch.Generator().manual_seed(3))]
    x, base, dy, a, b, _, _, scales = _problem(t, k, m, len(sizes), 64, ranks, seed=11)
    _run(dev, torch.bfloat16, x, base, dy, a, b, ids, ranks, scales, weights_f32=weights_f32)


def _random_case(seed):
    g = torch.Generator().manual_seed(1000 + seed)
    pick = lambda xs: xs[int(torch.randint(0, len(xs), (1,), generator=g))]  # noqa: E731
    t = pick([1, 7, 32, 33, 100, 257, 1000, 2500])
    k = pick([64, 128, 192, 256, 512, 1024, 1088])
    m = pick([128, 256, 384, 512, 640, 1024, 1536])
    max_r = pick([4, 8, 16, 24, 32, 48, 64])
    n = pick([1, 2, 5, 17, 40])
    ranks = [int(torch.randint(0, max_r + 1, (1,), generator=g)) for _ in range(n)]
    ranks[int(torch.randint(0, n, (1,), generator=g))] = max_r            # at least one adapter at the slot's rank
    # ids over a random subset of the adapters, so that some stay empty
    live = torch.randperm(n, generator=g)[:max(1, int(torch.randint(1, n + 1, (1,), generator=g)))]
    ids = live[torch.randint(0, live.numel(), (t,), generator=g)]
    return t, k, m, n, max_r, ranks, ids


@pytest.mark.parametrize('seed', range(36))
def test_random_shapes_ranks_and_id_distributions(dev, seed):
    """Seeded draws over the kernels' boundary sizes (one row, one tile plus one, widths at and off the MFMA
    kernels' multiples, ranks 0 .. 64, many empty adapters), bf16 and fp32 alternating."""
    t, k, m, n, max_r, ranks, ids = _random_case(seed)
    print(f'case {seed}: t={t} k={k} m={m} n={n} max_r={max_r} ranks={ranks}', flush=True)
    dtype = torch.bfloat16 if seed % 3 else torch.float32
    x, base, dy, a, b, _, _, scales = _problem(t, k, m, n, max_r, ranks, seed=seed)
    _run(dev, dtype, x, base, dy, a, b, ids, ranks, scales)


_ENV_CHILD = r'''
import sys, torch
sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[1] + "/tests")
import oracle
from twinkle_amd import AdapterGroups, build_segments, multi_lora_delta
torch.manual_seed(0)
t, k, m, n, max_r, ranks = 700, 256, 512, 4, 32, [32, 9, 0, 17]
g = torch.Generator().manual_seed(5)
bf = lambda v: v.bfloat16()
x, base, dy = bf(torch.randn(t, k, generator=g)), bf(torch.randn(t, m, generator=g)), bf(torch.randn(t, m, generator=g))
a = [bf((torch.rand(max_r, k, generator=g) * 2 - 1) / k ** 0.5) for _ in range(n)]
b = [bf(torch.randn(m, max_r, generator=g) * 0.05) for _ in range(n)]
ids = torch.randint(0, n, (t,), generator=g)
scales = [2.0, 0.5, 1.0, 2.0]
dev = torch.device("cuda:0")
xd = x.to(dev).requires_grad_(True)
ad = [v.to(dev).requires_grad_(True) for v in a]; bd = [v.to(dev).requires_grad_(True) for v in b]
seg = build_segments(ids.to(torch.int32).to(dev), n)
y = multi_lora_delta(xd, base.to(dev) * 1.0, seg, AdapterGroups(ad, bd, ranks, scales))
y.backward(dy.to(dev))
yo, dxo, dao, dbo = oracle.multi_lora_linear_grads(x.double(), base.double(), ids, [v.double() for v in a],
                                                    [v.double() for v in b], ranks, scales, dy.double())
err = lambda got, ref: float((got.double().cpu() - ref).abs().max() / ref.abs().max().clamp_min(1e-30))
worst = max([err(y, yo), err(xd.grad, dxo)] + [err(ad[i].grad, dao[i]) for i in (0, 1, 3)] +
            [err(bd[i].grad, dbo[i]) for i in (0, 1, 3)])
print("worst", worst)
sys.exit(0 if worst < 2e-2 else 1)
'''


@pytest.mark.parametrize('env', [{'TK_FORCE_GENERIC': '1'}, {'TK_BWD_STREAMS': '0'}])
def test_environment_switches_in_a_child_process(dev, env):
    """TK_FORCE_GENERIC=1 (every launch on the shape-agnostic kernels) and TK_BWD_STREAMS=0 (backward on the
    caller's stream only) are read once per process, so each runs in a child: same bar against the oracle."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, '-c', _ENV_CHILD, root], env={**os.environ, **env}, capture_output=True,
                         text=True, timeout=300)
    assert out.returncode == 0, out.stdout[-2000:] + out.stderr[-2000:]


def test_two_host_threads_call_the_two_stream_backward(dev):
    """Rank 32 at an output width of 384 takes the backward that forks onto the library's per-device side stream;
    two host threads, each on its own stream with its own buffers, must get what they get alone (the kernels are
    deterministic: bit-equal)."""
    import threading
    dt = torch.bfloat16

    def make(seed):
        t, k, m, n, max_r = 3000, 512, 384, 3, 32
        x, base, dy, a, b, ids, ranks, scales = _problem(t, k, m, n, max_r, [32, 20, 32], seed=seed)
        p = {'x': x.to(dt).to(dev), 'dy': dy.to(dt).to(dev), 'y0': base.to(dt).to(dev)}
        ad, bd = [v.to(dt).to(dev) for v in a], [v.to(dt).to(dev) for v in b]
        p['seg'] = build_segments(ids.to(torch.int32).to(dev), n)
        p['groups'] = AdapterGroups(ad, bd, ranks, scales)
        p['keep'] = (ad, bd)
        return p

    def run(p, iters, out, stream=None):
        try:
            with torch.cuda.stream(stream if stream is not None else torch.cuda.current_stream()):
                for _ in range(iters):
                    ad, bd = p['keep']
                    y = p['y0'].clone()
                    h = lora_fwd_(p['x'], y, p['seg'], p['groups'])
                    ga, gb = [torch.zeros_like(v) for v in ad], [torch.zeros_like(v) for v in bd]
                    pa = torch.tensor([v.data_ptr() for v in ga], dtype=torch.int64, device=dev)
                    pb = torch.tensor([v.data_ptr() for v in gb], dtype=torch.int64, device=dev)
                    dx = torch.zeros_like(p['x'])
                    lora_bwd_(p['dy'], p['x'], h, dx, pa, pb, p['seg'], p['groups'])
                    res = [y, dx] + ga + gb
                (stream or torch.cuda.current_stream()).synchronize()
                out.append([v.clone() for v in res])
        except Exception as e:  # surfaced by the assertion on the main thread
            out.append(e)

    probs = [make(21), make(22)]
    alone = []
    for p in probs:
        o = []
        run(p, 1, o)
        alone.append(o[0])
    torch.cuda.synchronize()
    outs = [[], []]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for s in streams:
        s.wait_stream(torch.cuda.current_stream())
    threads = [threading.Thread(target=run, args=(probs[i], 8, outs[i], streams[i])) for i in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    torch.cuda.synchronize()
    for i in range(2):
        assert len(outs[i]) == 1 and not isinstance(outs[i][0], Exception), outs[i]
        for got, want in zip(outs[i][0], alone[i]):
            assert torch.equal(got, want)


@pytest.mark.parametrize('max_r,ranks', [(16, [16, 7, 0]), (32, [32, 20, 9]), (64, [64, 33, 16])])
def test_backward_with_a_subset_of_the_outputs(dev, max_r, ranks):
    """A caller may want only dX (frozen adapters), only the weight gradients (input without gradient) or one side
    of them: every subset goes through a different sequence of kernels and must agree with the full call."""
    dt = torch.bfloat16
    t, k, m, n = 1500, 256, 1024, 3
    x, base, dy, a, b, ids, _, scales = _problem(t, k, m, n, max_r, ranks, seed=77)
    xd, dyd = x.to(dt).to(dev), dy.to(dt).to(dev)
    ad, bd = [v.to(dt).to(dev) for v in a], [v.to(dt).to(dev) for v in b]
    seg = build_segments(ids.to(torch.int32).to(dev), n)
    groups = AdapterGroups(ad, bd, ranks, scales)
    h = lora_fwd_(xd, base.to(dt).to(dev), seg, groups)

    def call(want_dx, want_a, want_b):
        ga, gb = [torch.zeros_like(v) for v in ad], [torch.zeros_like(v) for v in bd]
        pa = torch.tensor([v.data_ptr() for v in ga], dtype=torch.int64, device=dev) if want_a else None
        pb = torch.tensor([v.data_ptr() for v in gb], dtype=torch.int64, device=dev) if want_b else None
        dx = torch.zeros_like(xd) if want_dx else None
        lora_bwd_(dyd, xd if want_a else None, h if want_b else None, dx, pa, pb, seg, groups)
        torch.cuda.synchronize()
        return dx, ga, gb

    full = call(True, True, True)
    for want in [(True, False, False), (False, True, True), (False, False, True), (False, True, False),
                 (True, True, False), (True, False, True)]:
        dx, ga, gb = call(*want)
        if want[0]:
            assert max_rel_err(dx, full[0].double().cpu()) < 1e-2, want
        for g in range(n):
            if want[1]:
                assert max_rel_err(ga[g], full[1][g].double().cpu()) < 1e-2, want
            else:
                assert torch.count_nonzero(ga[g]) == 0
            if want[2]:
                assert max_rel_err(gb[g], full[2][g].double().cpu()) < 1e-2, want
            else:
                assert torch.count_nonzero(gb[g]) == 0
