"""Pins for the floating-point part of the oracle: closed forms in fp64, gradcheck, special cases."""
import pytest
import torch
import torch.nn.functional as F

import oracle


def _problem(t=24, k=12, m=10, n=3, max_r=6, ranks=(2, 6, 4), seed=0, dtype=torch.double):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(t, k, generator=g, dtype=dtype)
    base = torch.randn(t, m, generator=g, dtype=dtype)
    dy = torch.randn(t, m, generator=g, dtype=dtype)
    a = [torch.randn(max_r, k, generator=g, dtype=dtype) for _ in range(n)]
    b = [torch.randn(m, max_r, generator=g, dtype=dtype) for _ in range(n)]
    ids = torch.randint(0, n, (t,), generator=g)
    scales = [oracle.lora_scaling(2.0 * r, r) for r in ranks]
    return x, base, dy, a, b, ids, list(ranks), scales


def test_forward_closed_form():
    x, base, _, a, b, ids, ranks, scales = _problem()
    y = oracle.multi_lora_linear(x, base, ids, a, b, ranks, scales)
    for t in range(x.shape[0]):
        g = int(ids[t])
        want = base[t] + scales[g] * (b[g][:, :ranks[g]] @ (a[g][:ranks[g]] @ x[t]))
        assert torch.allclose(y[t], want, atol=1e-12)


def test_backward_closed_form():
    """dB = s dY^T h, dh = s dY B, dA = dh^T x, dX = dh A, per adapter over its rows; zero beyond r."""
    x, base, dy, a, b, ids, ranks, scales = _problem(seed=1)
    _, dx, da, db = oracle.multi_lora_linear_grads(x, base, ids, a, b, ranks, scales, dy)
    for g in range(len(a)):
        rows = (ids == g).nonzero().flatten()
        r, s = ranks[g], scales[g]
        xg, dyg = x[rows], dy[rows]
        h = xg @ a[g][:r].t()
        dh = s * dyg @ b[g][:, :r]
        assert torch.allclose(db[g][:, :r], s * dyg.t() @ h, atol=1e-10)
        assert torch.allclose(da[g][:r], dh.t() @ xg, atol=1e-10)
        assert torch.allclose(dx[rows], dh @ a[g][:r], atol=1e-10)
        assert torch.count_nonzero(da[g][r:]) == 0 and torch.count_nonzero(db[g][:, r:]) == 0


def test_gradcheck_single_adapter():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(5, 4, generator=g, dtype=torch.double, requires_grad=True)
    base = torch.randn(5, 3, generator=g, dtype=torch.double, requires_grad=True)
    a = torch.randn(3, 4, generator=g, dtype=torch.double, requires_grad=True)
    b = torch.randn(3, 3, generator=g, dtype=torch.double, requires_grad=True)
    assert torch.autograd.gradcheck(lambda *t: oracle.lora_linear_forward(t[0], t[1], t[2], t[3], 2, 1.5),
                                    (x, base, a, b))


def test_b_zero_gives_base_exactly():
    x, base, _, a, b, ids, ranks, scales = _problem(seed=3, dtype=torch.float32)
    b = [torch.zeros_like(t) for t in b]
    assert torch.equal(oracle.multi_lora_linear(x, base, ids, a, b, ranks, scales), base)


def test_rank_slice_equals_zero_padded_full_rank():
    x, base, _, a, b, ids, ranks, scales = _problem(seed=4)
    a0 = [t.clone() for t in a]
    b0 = [t.clone() for t in b]
    for g, r in enumerate(ranks):
        a0[g][r:] = 0
        b0[g][:, r:] = 0
    full = [a[0].shape[0]] * len(ranks)
    assert torch.allclose(oracle.multi_lora_linear(x, base, ids, a, b, ranks, scales),
                          oracle.multi_lora_linear(x, base, ids, a0, b0, full, scales), atol=1e-12)


def test_single_segment_is_plain_linear_chain():
    x, base, _, a, b, _, ranks, scales = _problem(seed=5)
    ids = torch.zeros(x.shape[0], dtype=torch.long)
    want = base + F.linear(F.linear(x, a[0][:ranks[0]]), b[0][:, :ranks[0]]) * scales[0]
    assert torch.allclose(oracle.multi_lora_linear(x, base, ids, a, b, ranks, scales), want, atol=1e-12)


def test_rank_zero_or_negative_id_keeps_base():
    x, base, _, a, b, ids, ranks, scales = _problem(seed=6)
    ranks[1] = 0
    ids[0] = -1
    y = oracle.multi_lora_linear(x, base, ids, a, b, ranks, scales)
    keep = (ids == 1) | (ids < 0)
    assert torch.equal(y[keep], base[keep])


def test_other_adapters_do_not_change_my_gradients():
    """Reference invariant (tests/model/test_multi_lora_target_parameters.py:78-100): only the active adapter moves."""
    x, base, dy, a, b, ids, ranks, scales = _problem(seed=7)
    _, _, da, db = oracle.multi_lora_linear_grads(x, base, ids, a, b, ranks, scales, dy)
    x2 = x.clone()
    x2[ids != 0] = torch.randn_like(x2[ids != 0])
    _, _, da2, db2 = oracle.multi_lora_linear_grads(x2, base, ids, a, b, ranks, scales, dy)
    assert torch.allclose(da[0], da2[0]) and torch.allclose(db[0], db2[0])
    empty = torch.full_like(ids, 1)
    _, _, da3, db3 = oracle.multi_lora_linear_grads(x, base, empty, a, b, ranks, scales, dy)
    assert torch.count_nonzero(da3[0]) == 0 and torch.count_nonzero(db3[2]) == 0


def test_rslora_scaling():
    assert oracle.lora_scaling(32, 16) == 2.0
    assert oracle.lora_scaling(32, 16, use_rslora=True) == 8.0


@pytest.mark.parametrize('out_in', [True, False])
def test_expert_merged_weight_equals_low_rank(out_in):
    """x (W + dW)^T == x W^T + s (x A^T) B^T per expert (reference merged form vs segmented form)."""
    torch.manual_seed(0)  # the reference's test seed
    e, hid, inter, max_r, r, s = 2, 4, 6, 4, 2, 2.0  # FakePackedExperts sizes of the reference test
    a = torch.randn(e, max_r, hid, dtype=torch.double)
    b = torch.randn(e, 2 * inter, max_r, dtype=torch.double)
    w = torch.randn(e, 2 * inter, hid, dtype=torch.double)
    dw = oracle.expert_delta_weight(a, b, r, s, out_in_layout=out_in)
    assert dw.shape == ((e, 2 * inter, hid) if out_in else (e, hid, 2 * inter))
    dw_oi = dw if out_in else dw.transpose(1, 2)
    x = torch.randn(7, hid, dtype=torch.double)
    offsets = torch.tensor([0, 3, 7])
    base = torch.cat([F.linear(x[:3], w[0]), F.linear(x[3:], w[1])])
    merged = torch.cat([F.linear(x[:3], w[0] + dw_oi[0]), F.linear(x[3:], w[1] + dw_oi[1])])
    low = oracle.expert_lora_low_rank(x, offsets, base, a, b, r, s)
    assert torch.allclose(merged, low, atol=1e-12)


def test_experts_linear_is_each_rows_own_expert():
    """The chunk loop against a row-by-row product with each row's own expert (empty experts included), and
    against one F.linear when there is a single expert."""
    g = torch.Generator().manual_seed(5)
    e, hid, out = 5, 6, 4
    counts = [3, 0, 4, 1, 0]
    offsets = torch.tensor([0, 3, 3, 7, 8, 8])
    x = torch.randn(8, hid, generator=g, dtype=torch.double)
    w = torch.randn(e, out, hid, generator=g, dtype=torch.double)
    got = oracle.experts_linear(x, offsets, w)
    expert_of_row = [i for i, c in enumerate(counts) for _ in range(c)]
    want = torch.stack([sum(w[expert_of_row[i]][:, k] * x[i, k] for k in range(hid)) for i in range(8)])
    assert got.shape == (8, out) and torch.allclose(got, want, atol=1e-12)
    one = oracle.experts_linear(x, torch.tensor([0, 8]), w[:1])
    assert torch.equal(one, F.linear(x, w[0]))


def test_swiglu_closed_form_and_gradient():
    g = torch.Generator().manual_seed(6)
    gu = torch.randn(5, 8, generator=g, dtype=torch.double, requires_grad=True)
    gate, up = gu[:, :4], gu[:, 4:]
    want = gate / (1 + torch.exp(-gate)) * up
    assert torch.allclose(oracle.swiglu(gu), want, atol=1e-14)
    assert torch.autograd.gradcheck(oracle.swiglu, (gu,))


def test_slice_copy_round_trip():
    g = torch.Generator().manual_seed(8)
    for name, shape, r in [('m.lora_A.weight', (8, 5), 3), ('m.lora_B.weight', (5, 8), 3),
                           ('m.lora_embedding_A.weight', (8, 5), 2), ('m.lora_embedding_B.weight', (5, 8), 2)]:
        full = torch.randn(*shape, generator=g)
        live = oracle.slice_rank_tensor(name, full, r)
        target = torch.zeros(*shape)
        oracle.copy_rank_tensor(name, target, live)
        assert torch.equal(oracle.slice_rank_tensor(name, target, r), live)
        assert torch.count_nonzero(target) == torch.count_nonzero(live)


def test_match_target_modules_cases():
    m = oracle.match_target_modules
    assert not m('model.layers.0.q_proj', None) and not m('x', [])
    assert m('anything', 'all-linear') and m('anything', ['all-linear'])
    assert m('model.layers.0.attn.proj', ['attn.proj']) and not m('model.layers.0.attn.proj', ['mlp.up'])
    # the example in the reference's comment: parameter names are stripped of their LoRA suffix
    assert m('model.layers.0.attn.proj.lora_A.default.weight', ['attn.proj'])
    assert m('model.layers.3.q_proj', r'.*\.q_proj') and not m('model.layers.3.k_proj', r'.*\.q_proj')
