"""Expert (3-D parameter) LoRA per (expert, tenant) segment, and the MoE row pipeline around it (config 4)."""
import pytest
import torch

import oracle
from conftest import max_rel_err
from twinkle_amd import LoraConfig, build_segments, flat_keys_from_topk, permute, unpermute
from twinkle_amd import workloads
from twinkle_amd.expert_lora import ExpertLoraSlots, expert_lora_delta

pytestmark = pytest.mark.gpu


def test_low_rank_segments_equal_the_reference_merged_weights(dev):
    """y_e = x (W_e + dW_e)^T with dW from the reference's einsum == base + segmented low-rank update."""
    torch.manual_seed(0)
    e, nt, hid, out, max_r = 8, 3, 128, 256, 8
    t, k = 400, 2
    slots = ExpertLoraSlots(e, hid, out, max_loras=4, max_r=max_r, dtype=torch.float32, device=dev)
    tenants = ['lora_0', 'lora_2', 'lora_3']
    for s, r in zip(tenants, (4, 8, 2)):
        slots.configure_slot(s, LoraConfig(r=r, lora_alpha=2 * r))
        with torch.no_grad():
            slots.lora_B[s].normal_(0, 0.05)
    g = torch.Generator().manual_seed(1)
    sel = torch.topk(torch.randn(t, e, generator=g), k).indices
    tenant = torch.randint(0, nt, (t,), generator=g)
    w = torch.randn(e, out, hid, generator=g) * 0.05
    x = torch.randn(t, hid, generator=g)
    keys = flat_keys_from_topk(sel.to(dev), tenant.to(dev), nt)
    seg = build_segments(keys, e * nt, num_tokens=t)
    xd = x.to(dev).requires_grad_(True)
    rows, _ = permute(xd, seg)                                  # expert inputs in segment order
    offsets = seg.offsets.cpu()
    # frozen per-expert base GEMMs over contiguous chunks (expert_parallel.py:347-371); a group's expert is g // nt
    base = torch.cat([rows[offsets[i]:offsets[i + 1]] @ w[i // nt].to(dev).t() for i in range(e * nt)])
    y = expert_lora_delta(rows, base, seg, slots, tenants)
    y.pow(2).sum().backward()
    # reference: merged weights, per (expert, tenant)
    perm = seg.perm.cpu()
    x64 = x.double().requires_grad_(True)
    rows64 = x64[perm % t]
    a64 = {s: slots.lora_A[s].detach().double().cpu().requires_grad_(True) for s in tenants}
    b64 = {s: slots.lora_B[s].detach().double().cpu().requires_grad_(True) for s in tenants}
    outs = []
    for i in range(e * nt):
        s = tenants[i % nt]
        dw = oracle.expert_delta_weight(a64[s], b64[s], slots.r[s], slots.scaling[s])[i // nt]
        outs.append(rows64[offsets[i]:offsets[i + 1]] @ (w[i // nt].double() + dw).t())
    y64 = torch.cat(outs)
    y64.pow(2).sum().backward()
    assert max_rel_err(y, y64) < 1e-5
    assert max_rel_err(xd.grad, x64.grad) < 1e-4
    for s in tenants:
        assert max_rel_err(slots.lora_A[s].grad, a64[s].grad) < 1e-4
        assert max_rel_err(slots.lora_B[s].grad, b64[s].grad) < 1e-4
        assert torch.count_nonzero(slots.lora_A[s].grad[:, slots.r[s]:]) == 0
    assert slots.lora_A['lora_1'].grad is None                  # a slot no tenant of the batch holds


def test_config4_shapes_bf16(dev):
    """BASELINE config 4 at full size: 8192 tokens, top-8 of 128 experts, 4 tenants, rank 8, 2048 -> 1536 (gate_up)
    and 768 -> 2048 (down); LoRA deltas only, plus bit-exact permutation and the unpermute round trip."""
    sel, weights, tenant = workloads.moe_routing()
    t, k = sel.shape
    e, nt, hid, inter, r = 128, 4, 2048, 768, 8
    keys = flat_keys_from_topk(sel.to(dev), tenant.to(dev), nt)
    seg = build_segments(keys, e * nt, num_tokens=t, check=True)
    perm, counts, offsets = oracle.segment_build_sort(oracle.flat_keys_from_topk(sel, tenant, nt), e * nt)
    assert torch.equal(seg.perm.cpu(), perm) and torch.equal(seg.offsets.cpu(), offsets)     # bit-exact ordering
    g = torch.Generator().manual_seed(2)
    x = torch.randn(t, hid, generator=g).bfloat16()
    rows, row_token = permute(x.to(dev), seg)
    assert torch.equal(rows.cpu(), x[perm % t])
    gate_up = ExpertLoraSlots(e, hid, 2 * inter, max_loras=nt, max_r=r, dtype=torch.bfloat16, device=dev)
    down = ExpertLoraSlots(e, inter, hid, max_loras=nt, max_r=r, dtype=torch.bfloat16, device=dev)
    tenants = [f'lora_{i}' for i in range(nt)]
    for sl in (gate_up, down):
        for s in tenants:
            sl.configure_slot(s, LoraConfig(r=r, lora_alpha=2 * r))
            with torch.no_grad():
                sl.lora_B[s].normal_(0, 0.02)
    # gate_up delta on zero base, checked on a sample of groups against the oracle's per-expert loop
    y = expert_lora_delta(rows, torch.zeros(t * k, 2 * inter, dtype=torch.bfloat16, device=dev), seg, gate_up, tenants)
    for i in (0, 1, 77, 300, 511):
        s0, s1 = int(offsets[i]), int(offsets[i + 1])
        if s0 == s1:
            continue
        sname = tenants[i % nt]
        a = gate_up.lora_A[sname][i // nt, :r].detach().double().cpu()
        b = gate_up.lora_B[sname][i // nt, :, :r].detach().double().cpu()
        want = 2.0 * (x[perm[s0:s1] % t].double() @ a.t()) @ b.t()
        assert max_rel_err(y[s0:s1], want) < 2e-2
    # down projection input: rows of width 768 already in segment order
    act = torch.randn(t * k, inter, generator=g).bfloat16().to(dev)
    out = expert_lora_delta(act, torch.zeros(t * k, hid, dtype=torch.bfloat16, device=dev), seg, down, tenants)
    i = 123
    s0, s1 = int(offsets[i]), int(offsets[i + 1])
    a = down.lora_A[tenants[i % nt]][i // nt, :r].detach().double().cpu()
    b = down.lora_B[tenants[i % nt]][i // nt, :, :r].detach().double().cpu()
    assert max_rel_err(out[s0:s1], 2.0 * (act[s0:s1].double().cpu() @ a.t()) @ b.t()) < 2e-2
    # weighted scatter-back (ep_utils.py:280-287) against the oracle
    final = unpermute(out, weights.bfloat16().to(dev), seg)
    row_w = weights.bfloat16().t().reshape(-1)[perm]
    want = oracle.unpermute_rows((out.cpu().double() * row_w.double()[:, None]).bfloat16().double(), None, perm % t, t)
    assert max_rel_err(final, want) < 2e-2


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_moe_block_with_expert_lora_equals_merged_weights_per_tenant(dev, dtype):
    """Router outputs -> permute -> packed experts (gate_up, SiLU gate, down) with per-(expert, tenant) LoRA ->
    weighted unpermute, against the reference's form in float64: merged weights W + B A * scaling of every token's
    own tenant (multi_lora_target_parameters.py:158-209), the per-expert loop, zero-init + index_add.
    float32 takes the per-expert loop for the frozen weights, bfloat16 the grouped GEMMs (widths are multiples
    of 128); the float64 restatement starts from the same rounded values."""
    from twinkle_amd import LoraTenant, MultiLora
    from twinkle_amd.expert_lora import moe_experts_block
    torch.manual_seed(0)
    e, hid, inter, t, k = 6, 128, 256, 300, 2

    class Experts(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.gate_up_proj = torch.nn.Parameter((torch.randn(e, 2 * inter, hid) * 0.05).to(dtype),
                                                   requires_grad=False)
            self.down_proj = torch.nn.Parameter((torch.randn(e, hid, inter) * 0.05).to(dtype), requires_grad=False)
            self.act_fn = torch.nn.functional.silu

    model = torch.nn.Module()
    model.experts = Experts().to(dev)
    model.set_adapter = lambda name: None
    model.disable_adapter_layers = model.enable_adapter_layers = lambda: None
    targets = ['experts.gate_up_proj', 'experts.down_proj']
    ml = MultiLora(max_loras=3, max_r=8)
    ml.module = model
    ml.loras = [LoraTenant(index=i, adapter_name=f'lora_{i}', config=None) for i in range(3)]
    ml.patch_target_parameters(model, targets)
    tenants = ['alice', 'bob']
    for name, r in zip(tenants, (8, 4)):
        ml.acquire_lora(name, LoraConfig(r=r, lora_alpha=2 * r, target_modules=[], target_parameters=targets))
    manager = ml.target_parameter_manager
    gu_slots, down_slots = manager.wrappers
    with torch.no_grad():
        for name in tenants:
            for key, p in manager.named_slot_parameters(name):
                if '.lora_B.' in key:
                    p.normal_(0, 0.05)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(t, hid, generator=g).to(dtype)
    logits = torch.randn(t, e, generator=g)
    weights, sel = torch.topk(torch.softmax(logits, -1), k)
    weights = weights.to(dtype)
    tenant = torch.randint(0, 2, (t,), generator=g)
    xd = x.to(dev).requires_grad_(True)
    assert gu_slots.lora_A['lora_0'].dtype == dtype
    slots = manager.slots_of(tenants)
    y = moe_experts_block(xd, sel.to(dev), weights.to(dev), tenant.to(dev), model.experts, slots, gu_slots, down_slots)
    y.pow(2).sum().backward()

    # float64 restatement with merged weights, token by token group
    x64 = x.double().requires_grad_(True)
    leaf = {}
    for s in slots:
        for w in (gu_slots, down_slots):
            leaf[(id(w), s, 'a')] = w.lora_A[s].detach().double().cpu().requires_grad_(True)
            leaf[(id(w), s, 'b')] = w.lora_B[s].detach().double().cpu().requires_grad_(True)
    out = torch.zeros(t, hid, dtype=torch.float64)
    for kk in range(k):
        for ex in range(e):
            for ti, s in enumerate(slots):
                idx = ((sel[:, kk] == ex) & (tenant == ti)).nonzero().flatten()
                if idx.numel() == 0:
                    continue
                merged = []
                for w, base in ((gu_slots, model.experts.gate_up_proj), (down_slots, model.experts.down_proj)):
                    dw = oracle.expert_delta_weight(leaf[(id(w), s, 'a')], leaf[(id(w), s, 'b')], w.r[s], w.scaling[s])
                    merged.append(base.detach().double().cpu()[ex] + dw[ex])
                h = x64[idx] @ merged[0].t()
                gate, up = h.chunk(2, dim=-1)
                o = (torch.nn.functional.silu(gate) * up) @ merged[1].t()
                out = out.index_add(0, idx, o * weights[idx, kk].double()[:, None])
    out.pow(2).sum().backward()
    tight = dtype == torch.float32
    assert max_rel_err(y, out) < (2e-5 if tight else 2e-2)
    assert max_rel_err(xd.grad, x64.grad) < (1e-4 if tight else 2e-2)
    for s in slots:
        for w in (gu_slots, down_slots):
            assert max_rel_err(w.lora_A[s].grad, leaf[(id(w), s, 'a')].grad) < (2e-4 if tight else 2e-2)
            assert max_rel_err(w.lora_B[s].grad, leaf[(id(w), s, 'b')].grad) < (2e-4 if tight else 2e-2)
    assert gu_slots.lora_A['lora_2'].grad is None                      # the free slot
