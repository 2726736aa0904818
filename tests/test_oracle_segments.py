"""Pins for the integer part of the oracle: two independent constructions, brute force, invariants."""
import pytest
import torch

import oracle


def _routing(t, e, k, seed):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(t, e, generator=g)
    return torch.topk(logits, k, dim=-1).indices


@pytest.mark.parametrize('t,e,k', [(1, 1, 1), (7, 3, 1), (16, 4, 2), (33, 8, 3), (64, 5, 5), (257, 16, 4)])
def test_sort_construction_equals_mask_construction(t, e, k):
    """Stable sort of flat keys f=k*T+t == the reference's one_hot/permute/masked_select order."""
    sel = _routing(t, e, k, seed=t * 31 + e)
    mask = oracle.expert_mask_from_topk(sel, e)
    assert mask.shape == (e, k, t)
    tokens = torch.arange(t, dtype=torch.float32)[:, None].repeat(1, 3)
    rows, sorted_indices = oracle.permute_by_mask(tokens, mask)
    perm, counts, offsets = oracle.segment_build_sort(oracle.flat_keys_from_topk(sel), e)
    assert torch.equal(perm % t, sorted_indices)
    assert torch.equal(counts, mask.sum(dim=(1, 2)))
    assert torch.equal(rows[:, 0].long(), sorted_indices)


@pytest.mark.parametrize('n,g,seed', [(0, 3, 0), (1, 1, 1), (5, 2, 2), (40, 7, 3), (64, 64, 4), (63, 9, 5)])
def test_sort_equals_bruteforce(n, g, seed):
    keys = torch.randint(0, g, (n,), generator=torch.Generator().manual_seed(seed))
    a = oracle.segment_build_sort(keys, g)
    b = oracle.segment_build_bruteforce(keys, g)
    for x, y in zip(a, b):
        assert torch.equal(x, y)


@pytest.mark.parametrize('n,g,seed', [(1, 1, 0), (9, 2, 1), (40, 7, 2), (200, 5, 3)])
def test_keys_outside_the_groups_sort_last_and_are_counted_nowhere(n, g, seed):
    """Rows whose key is negative or >= groups have no group: they follow every group in ascending row order."""
    keys = torch.randint(-2, g + 2, (n,), generator=torch.Generator().manual_seed(seed))
    a = oracle.segment_build_sort(keys, g)
    b = oracle.segment_build_bruteforce(keys, g)
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    perm, counts, offsets = a
    good = (keys >= 0) & (keys < g)
    assert sorted(perm.tolist()) == list(range(n))
    assert int(offsets[g]) == int(good.sum()) == int(counts.sum())
    tail = perm[int(offsets[g]):]
    assert torch.equal(tail, torch.nonzero(~good).flatten())
    # hand-computed: keys [1, -1, 0, 5, 0] over 2 groups -> rows 2, 4 | 0 | 1, 3
    p2, c2, o2 = oracle.segment_build_sort(torch.tensor([1, -1, 0, 5, 0]), 2)
    assert p2.tolist() == [2, 4, 0, 1, 3] and c2.tolist() == [2, 1] and o2.tolist() == [0, 2, 3]


def test_invariants_with_empty_groups():
    keys = torch.tensor([3, 3, 0, 7, 0, 3, 7, 7, 7])
    perm, counts, offsets = oracle.segment_build_sort(keys, 9)
    assert sorted(perm.tolist()) == list(range(9))                # a permutation
    assert torch.all(keys[perm][1:] >= keys[perm][:-1])           # non-decreasing keys
    for g in range(9):                                            # ascending rows inside a group
        seg = perm[offsets[g]:offsets[g + 1]]
        assert torch.all(seg[1:] > seg[:-1])
    assert offsets[0] == 0 and offsets[-1] == 9
    assert counts.tolist() == [2, 0, 0, 3, 0, 0, 0, 4, 0]
    assert perm.tolist() == [2, 4, 0, 1, 5, 3, 6, 7, 8]


def test_topk_order_is_group_then_k_then_token():
    sel = torch.tensor([[1, 0], [0, 1], [1, 0]])  # T=3, K=2
    perm, _, offsets = oracle.segment_build_sort(oracle.flat_keys_from_topk(sel), 2)
    # group 0: (k=0,t=1), (k=1,t=0), (k=1,t=2); group 1: (k=0,t=0), (k=0,t=2), (k=1,t=1)
    assert perm.tolist() == [1, 3, 5, 0, 2, 4]
    assert offsets.tolist() == [0, 3, 6]


def test_tenant_keys_refine_expert_groups():
    sel = _routing(50, 6, 2, seed=9)
    tenant = torch.randint(0, 3, (50,), generator=torch.Generator().manual_seed(10))
    keys = oracle.flat_keys_from_topk(sel, tenant, 3)
    perm, counts, _ = oracle.segment_build_sort(keys, 18)
    assert torch.equal(counts.view(6, 3).sum(1), oracle.expert_mask_from_topk(sel, 6).sum(dim=(1, 2)))
    assert torch.equal(keys[perm] % 3, tenant[perm % 50].long())


def test_unpermute_closed_form_and_identity():
    t, e, k, h = 19, 5, 2, 4
    sel = _routing(t, e, k, seed=3)
    w_tk = torch.rand(t, k, generator=torch.Generator().manual_seed(4)).double()
    x = torch.randn(t, h, generator=torch.Generator().manual_seed(5)).double()
    mask = oracle.expert_mask_from_topk(sel, e)
    # the reference's 2-D `unpermute` takes weights [T, E] and a folded routing map [E, T]; its row
    # order is (expert, token), i.e. `permute` on the folded map
    folded = mask.sum(1)
    rows2, mapping2 = oracle.permute_by_mask(x, folded[:, None, :])
    w_te = torch.zeros(t, e, dtype=torch.double).scatter_add_(1, sel, w_tk)
    got = oracle.unpermute(rows2, w_te, (t, h), mapping2, folded)
    want = x * w_tk.sum(1, keepdim=True)            # every copy of a token is the token itself
    assert torch.allclose(got, want, atol=1e-12)
    # the per-row form on the 3-D (expert, k, token) order, weight w[t, k] for row (k, t)
    # (ep_utils.py:238 and :280-287), gives the same sums
    rows, mapping = oracle.permute_by_mask(x, mask)
    perm = oracle.segment_build_sort(oracle.flat_keys_from_topk(sel), e)[0]
    assert torch.equal(perm % t, mapping)
    row_w = w_tk.t().reshape(-1)[perm]
    assert torch.equal(row_w, w_tk.t().contiguous().masked_select(mask.bool()))
    assert torch.allclose(oracle.unpermute_rows(rows, row_w, perm % t, t), got, atol=1e-12)
    # K=1, unit weights: permute then unpermute is the identity
    sel1 = sel[:, :1]
    m1 = oracle.expert_mask_from_topk(sel1, e)
    r1, map1 = oracle.permute_by_mask(x, m1)
    assert torch.equal(oracle.unpermute_rows(r1, None, map1, t), x)


@pytest.mark.parametrize('lens', [[5], [1, 1, 1], [4, 9, 2], [16, 16]])
def test_packed_cu_seqlens_bruteforce(lens):
    pos = torch.cat([torch.arange(n) for n in lens])[None]
    cu = oracle.packed_cu_seqlens(pos)
    want = [0]
    for n in lens:
        want.append(want[-1] + n)
    assert cu.dtype == torch.int32 and cu.tolist() == want
    ids = oracle.token_ids_from_cu_seqlens(cu, torch.arange(len(lens)))
    assert ids.tolist() == [j for j, n in enumerate(lens) for _ in range(n)]
