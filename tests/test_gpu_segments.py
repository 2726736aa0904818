"""Segment builder and row permute/unpermute against the oracle: integer results bit-exact."""
import pytest
import torch

import oracle
from conftest import max_rel_err
from twinkle_amd import build_segments, flat_keys_from_topk, packed_cu_seqlens, permute, unpermute
from twinkle_amd import workloads

pytestmark = pytest.mark.gpu


def _check(keys_cpu, groups, dev, dtype=torch.int32, num_tokens=None):
    seg = build_segments(keys_cpu.to(dtype).to(dev), groups, num_tokens=num_tokens, check=True)
    perm, counts, offsets = oracle.segment_build_sort(keys_cpu, groups)
    assert seg.perm.dtype == torch.int64 and seg.offsets.dtype == torch.int64
    assert torch.equal(seg.perm.cpu(), perm)
    assert torch.equal(seg.offsets.cpu(), offsets)
    assert torch.equal(seg.counts.cpu(), counts)
    seg.validate()      # every array of the device-side table, rebuilt on the host from the sizes and the order
    return seg


@pytest.mark.parametrize('rows,groups,seed', [(1, 1, 0), (5, 2, 1), (63, 3, 2), (64, 64, 3), (65, 7, 4), (511, 16, 5),
                                              (512, 16, 6), (513, 5, 7), (4097, 33, 8), (16384, 16, 9),
                                              (20000, 1000, 10), (70001, 4096, 11), (32768, 64, 12), (32769, 64, 13),
                                              (32768, 65, 14), (40000, 16, 15), (50000, 16384, 16)])
@pytest.mark.parametrize('dtype', [torch.int32, torch.int64])
def test_random_keys(dev, rows, groups, seed, dtype):
    keys = torch.randint(0, groups, (rows,), generator=torch.Generator().manual_seed(seed))
    _check(keys, groups, dev, dtype)


def test_empty_input_and_empty_groups(dev):
    _check(torch.zeros(0, dtype=torch.long), 4, dev)
    keys = torch.tensor([3, 3, 0, 7, 0, 3, 7, 7, 7])
    seg = _check(keys, 9, dev)
    assert seg.perm.tolist() == [2, 4, 0, 1, 5, 3, 6, 7, 8]


def test_all_rows_one_group_and_sorted_input(dev):
    _check(torch.full((3000,), 2), 5, dev)
    _check(torch.arange(4096) // 128, 32, dev)            # config 1 style: contiguous segments
    _check(torch.arange(4095, -1, -1) // 128, 32, dev)    # reversed


def test_bad_keys_are_reported(dev):
    keys = torch.tensor([0, 1, 9, -1, 1], dtype=torch.int32, device=dev)
    with pytest.raises(ValueError):
        build_segments(keys, 2, check=True)
    seg = build_segments(keys, 2)
    assert seg.bad_keys() == 2
    assert sorted(seg.perm.tolist()) == [0, 1, 2, 3, 4]   # still a permutation: clamped, not dropped


def test_limits(dev):
    with pytest.raises(ValueError):
        build_segments(torch.zeros(4, dtype=torch.int32, device=dev), 16385)
    with pytest.raises(ValueError):
        build_segments(torch.zeros(4, dtype=torch.float32, device=dev), 4)


def test_config2_and_config3_ids(dev):
    _check(workloads.zipf_ids(16384, 16).long(), 16, dev)
    ids = workloads.uneven_ids(32768, 32).long()
    seg = _check(ids, 32, dev)
    assert seg.counts[5] == 0 and seg.counts[17] == 0


def test_config4_expert_tenant_grouping_matches_reference_mask_order(dev):
    """65 536 routed rows, 512 (expert, tenant) groups; with one tenant the order is the reference's permute()."""
    sel, w, tenant = workloads.moe_routing()
    t, k = sel.shape
    keys = oracle.flat_keys_from_topk(sel, tenant, 4)
    seg = _check(keys, 512, dev, num_tokens=t)
    assert torch.equal(flat_keys_from_topk(sel.to(dev), tenant.to(dev), 4).cpu().long(), keys)
    # one tenant: identical to the masked_select order of the reference
    keys1 = oracle.flat_keys_from_topk(sel)
    seg1 = _check(keys1, 128, dev, num_tokens=t)
    mask = oracle.expert_mask_from_topk(sel.long(), 128)
    _, sorted_indices = oracle.permute_by_mask(torch.zeros(t, 1), mask)
    assert torch.equal(seg1.row_token.cpu(), sorted_indices)
    assert torch.equal(seg1.counts.cpu(), mask.sum(dim=(1, 2)))
    # tenant grouping refines the expert grouping
    assert torch.equal(seg.counts.view(128, 4).sum(1).cpu(), seg1.counts.cpu())


@pytest.mark.parametrize('dtype,tol', [(torch.float32, 1e-6), (torch.bfloat16, 2e-2)])
def test_permute_unpermute_round_trip_and_grads(dev, dtype, tol):
    t, e, k, h = 300, 12, 3, 40
    g = torch.Generator().manual_seed(0)
    sel = torch.topk(torch.randn(t, e, generator=g), k).indices
    w = torch.rand(t, k, generator=g)
    x = torch.randn(t, h, generator=g)
    keys = oracle.flat_keys_from_topk(sel)
    seg = build_segments(keys.to(torch.int32).to(dev), e, num_tokens=t)
    xd = x.to(dtype).to(dev).requires_grad_(True)
    wd = w.to(dtype).to(dev).requires_grad_(True)
    rows, row_token = permute(xd, seg)
    perm = oracle.segment_build_sort(keys, e)[0]
    assert torch.equal(row_token.cpu(), perm % t)
    assert torch.equal(rows.detach().cpu(), x.to(dtype)[perm % t])          # a gather: exact
    out = unpermute(rows * 1.0, wd, seg)
    # oracle in fp64 on the same rounded inputs
    x64 = x.to(dtype).double().requires_grad_(True)
    w64 = w.to(dtype).double().requires_grad_(True)
    rows64 = x64[perm % t]
    out64 = oracle.unpermute_rows(rows64, w64.t().reshape(-1)[perm], perm % t, t)
    assert max_rel_err(out, out64) < tol
    dy = torch.randn(t, h, generator=g)
    out.backward(dy.to(dtype).to(dev))
    out64.backward(dy.to(dtype).double())
    assert max_rel_err(xd.grad, x64.grad) < tol
    assert max_rel_err(wd.grad, w64.grad) < tol
    # unit weights, K = 1: permute then unpermute is the identity, bit for bit
    seg1 = build_segments(sel[:, 0].to(torch.int32).to(dev), e)
    r1, _ = permute(xd.detach(), seg1)
    assert torch.equal(unpermute(r1, None, seg1), xd.detach())


def test_unpermute_is_deterministic(dev):
    t, e, k, h = 2000, 16, 4, 64
    g = torch.Generator().manual_seed(1)
    sel = torch.topk(torch.randn(t, e, generator=g), k).indices
    seg = build_segments(oracle.flat_keys_from_topk(sel).to(torch.int32).to(dev), e, num_tokens=t)
    rows = torch.randn(t * k, h, generator=g).bfloat16().to(dev)
    w = torch.rand(t, k, generator=g).bfloat16().to(dev)
    a = unpermute(rows, w, seg)
    b = unpermute(rows, w, seg)
    assert torch.equal(a, b)


def test_packed_sequences(dev):
    lens = [4096] * 8
    pos = torch.cat([torch.arange(n) for n in lens])[None].to(dev)
    cu = packed_cu_seqlens(pos)
    assert torch.equal(cu.cpu(), oracle.packed_cu_seqlens(pos.cpu()))
    from twinkle_amd import token_groups_from_sequences
    ids = token_groups_from_sequences(cu, torch.arange(8, device=dev))
    seg = build_segments(ids, 8)
    assert seg.offsets.tolist() == [4096 * i for i in range(9)]
    assert torch.equal(seg.perm.cpu(), torch.arange(32768))


def test_tables_of_the_baseline_configs_validate(dev):
    """The device-side table of every BASELINE configuration's keys passes the host-side check entry by entry
    (config 1: contiguous segments; 2: Zipf ids shuffled; 3: uneven sizes with two empty adapters; 4: (expert, tenant)
    keys of top-8 routing; 5: one tenant per packed sequence), and so do keys with rows that have no group."""
    from twinkle_amd import validate_segment_table
    cases = [(workloads.config1_plumbing().ids, 4), (workloads.zipf_ids(16384, 16), 16), (workloads.uneven_ids(32768, 32), 32),
             (torch.repeat_interleave(torch.arange(8), 4096), 8)]
    selected, _, tenant = workloads.moe_routing()
    cases.append((flat_keys_from_topk(selected, tenant, 4), 512))
    keys = workloads.zipf_ids(5000, 16).clone()
    keys[::7] = -1
    keys[3::11] = 16
    cases.append((keys, 16))
    for keys, groups in cases:
        seg = build_segments(keys.to(torch.int32).to(dev), groups)
        validate_segment_table(seg)


def test_the_host_side_check_sees_a_changed_entry(dev):
    """The check itself: a copy of a good table with one entry changed (on the copy only: no kernel ever reads it) is
    reported, with the check that failed."""
    import ctypes
    from twinkle_amd import _lib
    keys = workloads.zipf_ids(3000, 8).to(dev)
    seg = build_segments(keys, 8)
    seg.validate()
    lib = _lib.load()
    words = seg.workspace.view(torch.int32)
    failed = set()
    for at in (2, 64 + 5):                    # header.groups; inv[5] (the header takes 64 words)
        copy = words.clone()
        copy[at] += 1
        check, index = ctypes.c_int32(0), ctypes.c_int64(-1)
        code = lib.tk_segment_validate(copy.data_ptr(), seg.rows, seg.num_groups, _lib.stream_ptr(), ctypes.byref(check),
                                       ctypes.byref(index))
        assert code == _lib.TK_ERR_INVALID and check.value > 0
        failed.add(check.value)
    assert failed == {1, 6}
