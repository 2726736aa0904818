"""The MultiLora mirror on the GPU: mixed-tenant batches equal each tenant run alone, and both equal the oracle."""
import pytest
import torch
from torch import nn

import oracle
from conftest import max_rel_err
from twinkle_amd import LoraConfig, LoraLinear, MultiLora

pytestmark = pytest.mark.gpu


class Block(nn.Module):

    def __init__(self, d=128, f=256):
        super().__init__()
        self.q_proj = nn.Linear(d, d, bias=False)
        self.up_proj = nn.Linear(d, f, bias=True)
        self.down_proj = nn.Linear(f, d, bias=False)

    def forward(self, x):
        return self.down_proj(torch.nn.functional.silu(self.up_proj(self.q_proj(x))))


def _setup(dev, dtype, max_loras=4, max_r=16):
    torch.manual_seed(0)
    ml = MultiLora(max_loras=max_loras, max_r=max_r)
    model = ml.patch(Block().to(dtype).to(dev), target_modules='all-linear')
    ml.save_initial_weights()
    cfgs = {
        'alice': LoraConfig(r=8, lora_alpha=16, target_modules='all-linear'),
        'bob': LoraConfig(r=16, lora_alpha=32, target_modules=['q_proj', 'down_proj']),       # up_proj not targeted
        'carol': LoraConfig(r=4, lora_alpha=16, target_modules='all-linear', use_rslora=True),
    }
    for name, cfg in cfgs.items():
        ml.acquire_lora(name, cfg)
    g = torch.Generator().manual_seed(1)
    with torch.no_grad():
        for n, p in model.named_parameters():
            if '.lora_B.' in n:                   # B starts at zero: give it values so the LoRA term is visible
                p.copy_((torch.randn(p.shape, generator=g) * 0.05).to(dtype))
    return ml, model, cfgs


def _oracle_block(model, x64, tenant_of_row, cfgs, ml, dtype):
    """The block evaluated per layer with the oracle's per-adapter loop, in float64 on the rounded weights."""
    names = list(cfgs)
    slot = {n: ml.find_lora_by_tenant(n).adapter_name for n in names}

    def lora_layer(layer, name, h):
        w = layer.base_layer.weight.detach().double().cpu()
        b = layer.base_layer.bias.detach().double().cpu() if layer.base_layer.bias is not None else None
        base = torch.nn.functional.linear(h, w, b)
        a_list, b_list, ranks, scales = [], [], [], []
        for n in names:
            cfg = cfgs[n]
            live = oracle.match_target_modules(name, cfg.target_modules)
            a_list.append(layer.lora_A[slot[n]].weight.detach().double().cpu())
            b_list.append(layer.lora_B[slot[n]].weight.detach().double().cpu())
            ranks.append(cfg.r if live else 0)
            scales.append(oracle.lora_scaling(cfg.lora_alpha, cfg.r, cfg.use_rslora))
        return oracle.multi_lora_linear(h, base, tenant_of_row, a_list, b_list, ranks, scales)

    m = model.model
    h = lora_layer(m.q_proj, 'model.q_proj', x64)
    h = torch.nn.functional.silu(lora_layer(m.up_proj, 'model.up_proj', h))
    return lora_layer(m.down_proj, 'model.down_proj', h)


@pytest.mark.parametrize('dtype,tol', [(torch.float32, 2e-5), (torch.bfloat16, 3e-2)])
def test_mixed_batch_equals_each_tenant_alone_and_the_oracle(dev, dtype, tol):
    ml, model, cfgs = _setup(dev, dtype)
    names = list(cfgs)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(3, 70, 128, generator=g).to(dtype)                      # [batch, seq, features]
    row_tenant = torch.randint(0, 3, (3 * 70,), generator=g)
    xd = x.to(dev)
    with ml.batch(names, row_tenant.to(dev)):
        y_mixed = model(xd)
    # every tenant alone through the reference-style one-adapter context
    y_single = torch.empty_like(y_mixed)
    for i, n in enumerate(names):
        with ml.adapter(n):
            yi = model(xd)
        mask = (row_tenant == i).view(3, 70).to(dev)
        y_single[mask] = yi[mask]
    assert max_rel_err(y_mixed, y_single) < (1e-6 if dtype == torch.float32 else 1e-2)
    want = _oracle_block(model, x.double().view(-1, 128), row_tenant, cfgs, ml, dtype).view(3, 70, 128)
    assert max_rel_err(y_mixed, want) < tol


def test_batch_check_rejects_rows_without_a_tenant(dev):
    ml, model, cfgs = _setup(dev, torch.float32)
    rows = torch.tensor([0, 1, 3], device=dev)
    with pytest.raises(ValueError):
        with ml.batch(['alice', 'bob', 'carol'], rows, check=True):
            pass
    with pytest.raises(ValueError):
        with ml.batch(['alice', 'nobody'], rows[:2]):
            pass


def test_only_the_tenants_in_the_batch_get_gradients(dev):
    """Reference invariant: updates only the active adapter (tests/model/test_multi_lora_target_parameters.py:78-100)."""
    ml, model, cfgs = _setup(dev, torch.float32)
    x = torch.randn(50, 128, generator=torch.Generator().manual_seed(3)).to(dev)
    row_tenant = (torch.arange(50) % 2).to(dev)                             # alice and bob only
    with ml.batch(['alice', 'bob'], row_tenant):
        model(x).pow(2).mean().backward()
    params = dict(model.named_parameters())
    for n, p in params.items():
        if 'lora_' not in n:
            assert p.grad is None                                            # base stays frozen
            continue
        slot = n.split('.')[-2]
        if slot in ('lora_2', 'lora_3'):                                     # carol's slot and the free slot
            assert p.grad is None or torch.count_nonzero(p.grad) == 0, n
    ga = params['model.q_proj.lora_A.lora_0.weight'].grad
    assert torch.count_nonzero(ga[:8]) > 0 and torch.count_nonzero(ga[8:]) == 0   # alice: rank 8 of a 16-row slot
    assert params['model.up_proj.lora_A.lora_1.weight'].grad is None or \
        torch.count_nonzero(params['model.up_proj.lora_A.lora_1.weight'].grad) == 0  # bob does not target up_proj


def test_gradients_match_the_oracle_through_the_whole_block(dev):
    ml, model, cfgs = _setup(dev, torch.float32)
    names = list(cfgs)
    g = torch.Generator().manual_seed(4)
    x = torch.randn(90, 128, generator=g)
    row_tenant = torch.randint(0, 3, (90,), generator=g)
    xd = x.to(dev).requires_grad_(True)
    with ml.batch(names, row_tenant.to(dev)):
        model(xd).pow(2).sum().backward()
    # oracle: same block in float64 with autograd
    x64 = x.double().requires_grad_(True)
    m = model.model
    slot = {n: ml.find_lora_by_tenant(n).adapter_name for n in names}
    leaves = {}

    def layer64(layer, name, h):
        base = torch.nn.functional.linear(h, layer.base_layer.weight.detach().double().cpu(),
                                          None if layer.base_layer.bias is None else layer.base_layer.bias.detach().double().cpu())
        a_list, b_list, ranks, scales = [], [], [], []
        for n in names:
            cfg = cfgs[n]
            a = layer.lora_A[slot[n]].weight.detach().double().cpu().requires_grad_(True)
            b = layer.lora_B[slot[n]].weight.detach().double().cpu().requires_grad_(True)
            leaves[(name, n, 'A')], leaves[(name, n, 'B')] = a, b
            a_list.append(a)
            b_list.append(b)
            ranks.append(cfg.r if oracle.match_target_modules(name, cfg.target_modules) else 0)
            scales.append(oracle.lora_scaling(cfg.lora_alpha, cfg.r, cfg.use_rslora))
        return oracle.multi_lora_linear(h, base, row_tenant, a_list, b_list, ranks, scales)

    h = layer64(m.q_proj, 'model.q_proj', x64)
    h = torch.nn.functional.silu(layer64(m.up_proj, 'model.up_proj', h))
    layer64(m.down_proj, 'model.down_proj', h).pow(2).sum().backward()
    assert max_rel_err(xd.grad, x64.grad) < 1e-4
    params = dict(model.named_parameters())
    for (lname, tenant, side), leaf in leaves.items():
        got = params[f'{lname}.lora_{side}.{slot[tenant]}.weight'].grad
        want = leaf.grad if leaf.grad is not None else torch.zeros_like(leaf)
        if got is None:
            assert torch.count_nonzero(want) == 0
        else:
            assert max_rel_err(got, want) < 1e-4, (lname, tenant, side)


def test_disable_lora_and_unmatched_layers_return_the_base_output(dev):
    ml, model, _ = _setup(dev, torch.float32)
    x = torch.randn(10, 128, generator=torch.Generator().manual_seed(5)).to(dev)
    m = model.model
    base = m.down_proj.base_layer(torch.nn.functional.silu(m.up_proj.base_layer(m.q_proj.base_layer(x))))
    with ml.adapter('alice', disable_lora=True):
        assert torch.equal(model(x), base)
    with ml.adapter('bob'):                        # bob does not target up_proj: that layer must be the base layer
        q = m.q_proj(x)
        assert torch.equal(m.up_proj(q), m.up_proj.base_layer(q))
    # after release B is zero again: the tenant's rows are the base output exactly (reference :745-748)
    ml.release_lora('alice')
    ml.acquire_lora('dave', LoraConfig(r=8, lora_alpha=16, target_modules='all-linear'))
    with ml.adapter('dave'):
        assert torch.equal(model(x), base)


def test_activation_checkpointing_recompute_is_bitwise_identical(dev):
    """The reference runs with gradient checkpointing on (multi_lora_transformers.py:85): forward runs twice."""
    from torch.utils.checkpoint import checkpoint
    ml, model, cfgs = _setup(dev, torch.bfloat16)
    g = torch.Generator().manual_seed(6)
    x = torch.randn(200, 128, generator=g).bfloat16().to(dev).requires_grad_(True)
    row_tenant = torch.randint(0, 3, (200,), generator=g).to(dev)
    with ml.batch(list(cfgs), row_tenant):
        y1 = model(x)
        y1.float().pow(2).sum().backward()
        g1 = {n: p.grad.clone() for n, p in model.named_parameters() if p.grad is not None}
        gx1 = x.grad.clone()
        model.zero_grad()
        x.grad = None
        y2 = checkpoint(model, x, use_reentrant=False)
        y2.float().pow(2).sum().backward()
    assert torch.equal(y1, y2) and torch.equal(gx1, x.grad)
    for n, p in model.named_parameters():
        if p.grad is not None:
            assert torch.equal(p.grad, g1[n]), n


def test_mixed_dtype_base_bf16_adapters_fp32(dev):
    """x is cast to the adapter dtype and the sum back to the base output dtype (multi_lora.py:320, :327)."""
    torch.manual_seed(0)
    ml = MultiLora(max_loras=2, max_r=8)
    base = nn.Sequential(nn.Linear(64, 128, bias=False)).bfloat16().to(dev)
    model = ml.patch(base, target_modules='all-linear')
    for n, p in model.named_parameters():
        if 'lora_' in n:
            p.data = p.data.float()
    ml.acquire_lora('alice', LoraConfig(r=8, lora_alpha=16, target_modules='all-linear'))
    layer = [m for m in model.modules() if isinstance(m, LoraLinear)][0]
    with torch.no_grad():
        layer.lora_B['lora_0'].weight.normal_(0, 0.05)
    x = torch.randn(33, 64, generator=torch.Generator().manual_seed(7)).bfloat16().to(dev)
    with ml.adapter('alice'):
        y = model(x)
    assert y.dtype == torch.bfloat16
    want = oracle.lora_linear_forward(x.cpu(), layer.base_layer(x).cpu(), layer.lora_A['lora_0'].weight.detach().cpu(),
                                      layer.lora_B['lora_0'].weight.detach().cpu(), 8, 2.0)
    assert want.dtype == torch.bfloat16
    assert max_rel_err(y, want) < 1e-2
    # the adapters were read where they are (fp32) by the bf16 kernels, and their gradients arrive in fp32
    groups = ml._groups_for(layer, 'lora_0', torch.bfloat16)
    assert groups.dtype == torch.bfloat16 and groups.weights_f32
    y.float().pow(2).sum().backward()
    ga, gb = layer.lora_A['lora_0'].weight.grad, layer.lora_B['lora_0'].weight.grad
    assert ga.dtype == torch.float32 and gb.dtype == torch.float32 and ga.abs().max() > 0 and gb.abs().max() > 0
    # lora_compute_dtype=float32 asks for the reference's arithmetic instead: activations cast to fp32
    ml.lora_compute_dtype = torch.float32
    groups32 = ml._groups_for(layer, 'lora_0', torch.bfloat16)
    assert groups32.dtype == torch.float32 and not groups32.weights_f32
    with ml.adapter('alice'):
        y32 = model(x)
    assert y32.dtype == torch.bfloat16 and max_rel_err(y32, want) < 1e-2


def test_batched_training_step_equals_tenants_one_after_the_other(dev):
    """One mixed-tenant forward/backward and one multi-tenant optimizer launch set against the reference's
    schedule: every tenant alone (adapter context, its own rows), grads divided by its token count, clipped,
    torch.optim.AdamW per tenant."""
    from twinkle_amd import MultiTenantAdamW, trainable_parameters
    dtype = torch.float32
    names = ['alice', 'bob', 'carol']
    hyper = {'alice': dict(lr=1e-2, weight_decay=0.01), 'bob': dict(lr=5e-3, weight_decay=0.0),
             'carol': dict(lr=2e-2, weight_decay=0.1)}
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 90, 128, generator=g)
    target = torch.randn(2, 90, 128, generator=g)
    row_tenant = torch.randint(0, 3, (180,), generator=g)
    tokens = {n: int((row_tenant == i).sum()) for i, n in enumerate(names)}

    # (a) batched: one forward/backward, sum-of-squares loss per token, then one optimizer step for all tenants
    ml, model, cfgs = _setup(dev, dtype)
    opt = MultiTenantAdamW()
    slot = {n: ml.find_lora_by_tenant(n).adapter_name for n in names}
    for n in names:
        opt.add_tenant(n, trainable_parameters(model, slot[n]).values(), **hyper[n])
    with ml.batch(names, row_tenant.to(dev)):
        y = model(x.to(dev))
    ((y - target.to(dev))**2).sum().backward()
    norms = opt.clip_grad_and_step(tokens, max_grad_norm=1.0)
    got = {n: {k: p.detach().clone() for k, p in trainable_parameters(model, slot[n]).items()} for n in names}

    # (b) the reference's schedule on a fresh copy: tenants one after the other, each on its own rows
    ml2, model2, _ = _setup(dev, dtype)
    for i, n in enumerate(names):
        params = trainable_parameters(model2, slot[n])
        rows = (row_tenant == i).nonzero().flatten().to(dev)
        xs = x.to(dev).reshape(180, 128).index_select(0, rows)
        ts = target.to(dev).reshape(180, 128).index_select(0, rows)
        with ml2.adapter(n):
            ys = model2(xs)
        ((ys - ts)**2).sum().backward()
        tenant_params = [p for p in params.values() if p.grad is not None]
        for p in tenant_params:
            p.grad.div_(tokens[n])                                   # grad_clip.py:81-96
        want_norm = torch.nn.utils.clip_grad_norm_(tenant_params, 1.0)
        torch.optim.AdamW(tenant_params, **hyper[n]).step()
        assert abs(float(norms[n]) - float(want_norm)) < 1e-4 * float(want_norm)
        for k, p in params.items():
            assert max_rel_err(got[n][k], p.detach()) < 2e-5, (n, k)
        for p in model2.parameters():
            p.grad = None


# ---- a Llama-shaped block stack (BASELINE config 5 in miniature): seven projections per layer, packed sequences ----

class _RMSNorm(nn.Module):

    def __init__(self, d):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(d))

    def forward(self, x):
        v = x.float()
        return (v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + 1e-5)).to(x.dtype) * self.weight


class _LlamaLayer(nn.Module):

    def __init__(self, d, heads, kv_heads, inter):
        super().__init__()
        self.heads, self.kv_heads, self.hd = heads, kv_heads, d // heads
        self.input_layernorm, self.post_attention_layernorm = _RMSNorm(d), _RMSNorm(d)
        self.q_proj = nn.Linear(d, d, bias=False)
        self.k_proj = nn.Linear(d, kv_heads * self.hd, bias=False)
        self.v_proj = nn.Linear(d, kv_heads * self.hd, bias=False)
        self.o_proj = nn.Linear(d, d, bias=False)
        self.gate_proj = nn.Linear(d, inter, bias=False)
        self.up_proj = nn.Linear(d, inter, bias=False)
        self.down_proj = nn.Linear(inter, d, bias=False)

    def forward(self, x):                                            # x: [sequences, tokens, d], causal per sequence
        b, s, _ = x.shape
        h = self.input_layernorm(x)
        q = self.q_proj(h).view(b, s, self.heads, self.hd).transpose(1, 2)
        k = self.k_proj(h).view(b, s, self.kv_heads, self.hd).transpose(1, 2)
        v = self.v_proj(h).view(b, s, self.kv_heads, self.hd).transpose(1, 2)
        rep = self.heads // self.kv_heads
        a = torch.nn.functional.scaled_dot_product_attention(q, k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1),
                                                             is_causal=True)
        x = x + self.o_proj(a.transpose(1, 2).reshape(b, s, -1))
        h = self.post_attention_layernorm(x)
        return x + self.down_proj(torch.nn.functional.silu(self.gate_proj(h)) * self.up_proj(h))


class _LlamaStack(nn.Module):

    def __init__(self, layers=2, d=1024, heads=8, kv_heads=2, inter=2048):
        super().__init__()
        self.layers = nn.ModuleList(_LlamaLayer(d, heads, kv_heads, inter) for _ in range(layers))

    def forward(self, x):
        for layer in self.layers:
            x = layer(x)
        return x


def test_llama_shaped_stack_packed_sequences_one_tenant_each(dev):
    """Seven LoRA projections per layer (q/k/v and gate/up through the shared-input path), one tenant per packed
    sequence: the mixed batch equals every tenant run alone through the reference-style adapter context, outputs
    and every adapter gradient."""
    dtype = torch.bfloat16
    torch.manual_seed(0)
    ml = MultiLora(max_loras=4, max_r=16)
    model = ml.patch(_LlamaStack().to(dtype).to(dev), target_modules='all-linear')
    cfgs = {'alice': LoraConfig(r=16, lora_alpha=32, target_modules='all-linear'),
            'bob': LoraConfig(r=8, lora_alpha=16, target_modules=['q_proj', 'v_proj', 'down_proj']),
            'carol': LoraConfig(r=4, lora_alpha=16, target_modules='all-linear', use_rslora=True)}
    for n, c in cfgs.items():
        ml.acquire_lora(n, c)
    g = torch.Generator().manual_seed(1)
    with torch.no_grad():
        for n, p in model.named_parameters():
            if '.lora_B.' in n:
                p.copy_((torch.randn(p.shape, generator=g) * 0.02).to(dtype))
    names = list(cfgs)
    seqs, toks, d = 5, 96, 1024
    seq_tenant = torch.tensor([0, 1, 2, 1, 0])
    x = torch.randn(seqs, toks, d, generator=g).to(dtype).to(dev)
    w = torch.randn(seqs, toks, d, generator=g).to(dtype).to(dev)
    row_tenant = seq_tenant.repeat_interleave(toks).to(dev)
    lora = {n: p for n, p in model.named_parameters() if 'lora_' in n}

    def run(mixed, shared):
        for p in model.parameters():
            p.grad = None
        if shared:
            ml.share_inputs([[f'model.layers.{i}.{a}' for a in grp] for i in range(2)
                             for grp in (('q_proj', 'k_proj', 'v_proj'), ('gate_proj', 'up_proj'))])
        try:
            if mixed:
                with ml.batch(names, row_tenant):
                    y = model(x)
                (y * w).sum().backward()
            else:
                y = torch.empty_like(x)
                for i, n in enumerate(names):                        # the reference's schedule: one tenant per pass
                    mine = (seq_tenant == i).nonzero().flatten().to(dev)
                    with ml.adapter(n):
                        yi = model(x.index_select(0, mine))
                    (yi * w.index_select(0, mine)).sum().backward()
                    y[mine] = yi.detach()
        finally:
            ml.unshare_inputs()
        return y.detach().clone(), {n: (p.grad.clone() if p.grad is not None else None) for n, p in lora.items()}

    y_ref, g_ref = run(mixed=False, shared=False)
    for shared in (False, True):
        y, grads = run(mixed=True, shared=shared)
        assert max_rel_err(y, y_ref) < 2e-2, shared
        for n in lora:
            if g_ref[n] is None or g_ref[n].abs().max() == 0:
                assert grads[n] is None or grads[n].abs().max() == 0, n        # free slot, untargeted layer
            else:
                assert max_rel_err(grads[n], g_ref[n].double()) < 3e-2, (shared, n)


def test_fp32_adapters_computed_in_bf16_on_request(dev):
    """lora_compute_dtype=bfloat16: fp32 adapter parameters under a bf16 base run through the bf16 kernels (copies
    refreshed at every forward), gradients arrive in fp32 on the fp32 parameters, and an in-place update of the
    masters - by torch or by the multi-tenant optimizer kernel, which bumps no version counter - shows up in the
    next forward."""
    from twinkle_amd import MultiTenantAdamW, trainable_parameters
    torch.manual_seed(0)
    ml = MultiLora(max_loras=3, max_r=16, lora_compute_dtype=torch.bfloat16)
    model = ml.patch(Block(d=256, f=512).bfloat16().to(dev), target_modules='all-linear')
    g = torch.Generator().manual_seed(1)
    for n, p in model.named_parameters():
        if 'lora_' in n:
            p.data = p.data.float()
            if '.lora_B.' in n:
                with torch.no_grad():
                    p.copy_(torch.randn(p.shape, generator=g) * 0.05)
    cfgs = {'alice': LoraConfig(r=16, lora_alpha=32, target_modules='all-linear'),
            'bob': LoraConfig(r=8, lora_alpha=16, target_modules='all-linear')}
    for n, c in cfgs.items():
        ml.acquire_lora(n, c)
    names = list(cfgs)
    x = torch.randn(300, 256, generator=g).bfloat16()
    row_tenant = torch.randint(0, 2, (300,), generator=g)

    def forward():
        with ml.batch(names, row_tenant.to(dev)):
            return model(x.to(dev))

    def reference():
        # the reference's arithmetic on the fp32 masters, float64, per layer through the oracle's per-adapter loop
        m = model.model
        h = x.double()
        for layer, act in ((m.q_proj, None), (m.up_proj, torch.nn.functional.silu), (m.down_proj, None)):
            w = layer.base_layer.weight.detach().double().cpu()
            b = layer.base_layer.bias.detach().double().cpu() if layer.base_layer.bias is not None else None
            base = torch.nn.functional.linear(h, w, b)
            a_list = [layer.lora_A[ml.find_lora_by_tenant(n).adapter_name].weight.detach().double().cpu() for n in names]
            b_list = [layer.lora_B[ml.find_lora_by_tenant(n).adapter_name].weight.detach().double().cpu() for n in names]
            h = oracle.multi_lora_linear(h, base, row_tenant, a_list, b_list, [cfgs[n].r for n in names], [2.0, 2.0])
            if act is not None:
                h = act(h)
        return h

    y = forward()
    assert y.dtype == torch.bfloat16 and max_rel_err(y, reference()) < 3e-2
    y.float().pow(2).mean().backward()
    slot = ml.find_lora_by_tenant('alice').adapter_name
    pa = model.model.q_proj.lora_A[slot].weight
    assert pa.dtype == torch.float32 and pa.grad is not None and pa.grad.dtype == torch.float32
    assert pa.grad.abs().max() > 0
    for n, p in model.named_parameters():
        assert 'lora_' in n or p.grad is None
    # masters updated by the optimizer kernel: the next forward must see them
    opt = MultiTenantAdamW()
    for n in names:
        opt.add_tenant(n, trainable_parameters(model, ml.find_lora_by_tenant(n).adapter_name).values(), lr=0.05)
    before = pa.detach().clone()
    opt.clip_grad_and_step({'alice': 150, 'bob': 150}, max_grad_norm=1.0)
    assert (pa.detach() - before).abs().max() > 0
    y2 = forward()
    assert max_rel_err(y2, reference()) < 3e-2 and (y2.float() - y.float()).abs().max() > 0
