"""The larger BASELINE configurations: full shapes on the GPU, checked by sampling against the oracle and
by properties that do not need a CPU pass over the whole problem."""
import pytest
import torch

import oracle
from conftest import max_rel_err
from twinkle_amd import AdapterGroups, build_segments, lora_bwd_, lora_bwd_workspace_bytes, lora_fwd_
from twinkle_amd import packed_cu_seqlens, token_groups_from_sequences, workloads

pytestmark = pytest.mark.gpu


def _device_problem(w, dev):
    dt = torch.bfloat16
    a = [t.to(dt).to(dev) for t in w.lora_A]
    b = [t.to(dt).to(dev) for t in w.lora_B]
    seg = build_segments(w.ids.to(dev), w.num_adapters, check=True)
    return a, b, seg, AdapterGroups(a, b, w.ranks, w.scales)


def _check_sampled(w, dev, sample_groups, sample_rows=64):
    """Forward/backward at full size; Y and dX on sampled rows, dA/dB of sampled adapters, against float64."""
    dt = torch.bfloat16
    a, b, seg, groups = _device_problem(w, dev)
    x = w.x.to(dt).to(dev)
    y = w.base_out.to(dt).to(dev)
    dy = w.dy.to(dt).to(dev)
    h = lora_fwd_(x, y, seg, groups)
    ga = [torch.full_like(t, 7.0) for t in a]
    gb = [torch.full_like(t, 7.0) for t in b]
    pa = torch.tensor([t.data_ptr() for t in ga], dtype=torch.int64, device=dev)
    pb = torch.tensor([t.data_ptr() for t in gb], dtype=torch.int64, device=dev)
    dx = torch.zeros_like(x)
    lora_bwd_(dy, x, h, dx, pa, pb, seg, groups, accumulate=False)
    f64 = lambda t: t.to(dt).double()  # noqa: E731
    counts = torch.bincount(w.ids.long(), minlength=w.num_adapters)
    for g in sample_groups:
        r, s = w.ranks[g], w.scales[g]
        rows = (w.ids == g).nonzero().flatten()
        ag, bg = f64(w.lora_A[g])[:r], f64(w.lora_B[g])[:, :r]
        if rows.numel() == 0:
            assert torch.count_nonzero(ga[g][:r]) == 0 and torch.count_nonzero(gb[g][:, :r]) == 0
            continue
        xg, dyg = f64(w.x[rows]), f64(w.dy[rows])
        hg = s * xg @ ag.t()
        dh = s * dyg @ bg
        sub = rows[:sample_rows]
        assert max_rel_err(y[sub.to(dev)], f64(w.base_out[sub]) + (hg[:sample_rows] @ bg.t())) < 2e-2
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
