"""The boundary on the GPU: the installer on an object with only the reference's MultiLora surface, rows without a
tenant, idle slots, the patched packed-experts forward, and the accumulation schedule of batched steps."""
import pytest
import torch
from torch import nn

import oracle
import twinkle_amd
from conftest import max_rel_err
from test_gpu_multilora import Block, _setup
from test_host_logic import TinyBlock, reference_surface_setup
from twinkle_amd import BatchedStep, LoraConfig, LoraTenant, MultiLora, MultiTenantAdamW, trainable_parameters

pytestmark = pytest.mark.gpu


def _oracle_tiny_block(holder, x64, row_tenant, tenants):
    """TinyBlock layer by layer through the oracle's per-adapter loop; ``tenants``: [(slot name, config)]."""
    def layer(mod, name, h):
        w = mod.base_layer.weight.detach().double().cpu()
        b = None if mod.base_layer.bias is None else mod.base_layer.bias.detach().double().cpu()
        base = torch.nn.functional.linear(h, w, b)
        a_list = [mod.lora_A[s].weight.detach().double().cpu() for s, _ in tenants]
        b_list = [mod.lora_B[s].weight.detach().double().cpu() for s, _ in tenants]
        ranks = [c.r if oracle.match_target_modules(name, c.target_modules) else 0 for _, c in tenants]
        scales = [oracle.lora_scaling(c.lora_alpha, c.r, getattr(c, 'use_rslora', False)) for _, c in tenants]
        return oracle.multi_lora_linear(h, base, row_tenant, a_list, b_list, ranks, scales)
    m = holder.model
    h = layer(m.q_proj, 'model.q_proj', x64)
    h = torch.relu(layer(m.up_proj, 'model.up_proj', h))
    return layer(m.down_proj, 'model.down_proj', h)


def test_installer_on_the_reference_surface_mixed_batch_equals_the_oracle(dev):
    """use_mi355x_path on an object that has only what the reference's MultiLora has; then adapter() (the
    reference's own context) and twinkle_amd.batch() with padding rows, both against the oracle in float64."""
    ref, holder = reference_surface_setup(device=dev)
    twinkle_amd.use_mi355x_path(ref)
    cfgs = {'alice': LoraConfig(r=4, lora_alpha=8, target_modules='all-linear'),
            'bob': LoraConfig(r=8, lora_alpha=8, target_modules=['q_proj', 'down_proj'])}
    slots = {n: ref.acquire_lora(n, c) for n, c in cfgs.items()}
    g = torch.Generator().manual_seed(3)
    x = torch.randn(75, 16, generator=g)
    row_tenant = torch.randint(-1, 2, (75,), generator=g)              # -1: a row without a tenant
    tenants = [(slots[n], cfgs[n]) for n in cfgs]
    with twinkle_amd.batch(ref, list(cfgs), row_tenant.to(dev)):
        y = holder(x.to(dev))
    want = _oracle_tiny_block(holder, x.double(), row_tenant, tenants)
    assert max_rel_err(y, want) < 2e-5
    base = TinyBlock()
    base.load_state_dict({k.replace('.base_layer', ''): v for k, v in holder.model.state_dict().items()
                          if 'lora_' not in k})
    none = (row_tenant < 0)
    assert max_rel_err(y[none.to(dev)], base.double()(x.double())[none]) < 2e-5
    with ref.adapter('bob'):
        yb = holder(x.to(dev))
    assert max_rel_err(yb, _oracle_tiny_block(holder, x.double(), torch.ones(75, dtype=torch.long), tenants)) < 2e-5
    # ownership changes made through the object's own methods are seen by the next forward
    ref.release_lora('bob')
    with twinkle_amd.batch(ref, ['alice'], torch.zeros(75, dtype=torch.long, device=dev)):
        ya = holder(x.to(dev))
    assert max_rel_err(ya, _oracle_tiny_block(holder, x.double(), torch.zeros(75, dtype=torch.long), tenants[:1])) < 2e-5


def test_idle_slots_keep_no_gradient_and_their_optimizer_state(dev):
    """A batch over two of three tenants: the third tenant's slot and the free slot get no gradient at all (the
    reference updates only the active adapter), so a default optimizer call leaves their parameters, moments and
    step count alone; rows marked -1 add to nobody's gradients."""
    ml, model, cfgs = _setup(dev, torch.float32)
    names = list(cfgs)
    slot = {n: ml.find_lora_by_tenant(n).adapter_name for n in names}
    opt = MultiTenantAdamW()
    for n in names:
        opt.add_tenant(n, trainable_parameters(model, slot[n]).values(), lr=1e-2, weight_decay=0.1)
    g = torch.Generator().manual_seed(11)
    x = torch.randn(120, 128, generator=g).to(dev)
    rt = torch.randint(0, 2, (120,), generator=g)
    rt[::7] = -1
    carol_before = {k: p.detach().clone() for k, p in trainable_parameters(model, slot['carol']).items()}
    with ml.batch(['alice', 'bob'], rt.to(dev)):
        model(x).pow(2).sum().backward()
    for n, p in model.named_parameters():
        if 'lora_' not in n:
            continue
        s = n.split('.')[-2]
        if s in (slot['carol'], 'lora_3') or (s == slot['bob'] and '.up_proj.' in n):
            assert p.grad is None, n                                  # idle slot / untargeted layer
        else:
            assert p.grad is not None and torch.count_nonzero(p.grad) > 0, n
    # the same batch without the -1 rows of each tenant gives the same gradients: those rows add to nobody
    got = {n: p.grad.clone() for n, p in model.named_parameters() if p.grad is not None}
    model.zero_grad(set_to_none=True)
    keep = (rt >= 0).nonzero().flatten()
    with ml.batch(['alice', 'bob'], rt[keep].to(dev)):
        model(x[keep.to(dev)]).pow(2).sum().backward()
    for n, p in model.named_parameters():
        if p.grad is not None:
            assert max_rel_err(got[n], p.grad) < 1e-5, n
    norms = opt.clip_grad_and_step({'alice': 50, 'bob': 50, 'carol': 1}, max_grad_norm=1.0)   # names: all tenants
    assert opt.state('carol')['step'] == 0 and opt.state('alice')['step'] == 1
    assert all(v is None for v in opt.state('carol')['exp_avg'])
    for k, p in trainable_parameters(model, slot['carol']).items():
        assert torch.equal(p.detach(), carol_before[k]), k
    assert float(norms['alice']) > 0


class PackedExperts(nn.Module):
    """The packed-experts module of transformers' MoE models as the reference patches it: ``gate_up_proj
    [E, 2 I, H]``, ``down_proj [E, H, I]``, ``forward(hidden_states, top_k_index, top_k_weights)`` looping over the
    experts that were hit."""

    def __init__(self, experts, hidden, inter, dtype):
        super().__init__()
        self.num_experts = experts
        self.gate_up_proj = nn.Parameter((torch.randn(experts, 2 * inter, hidden) * 0.05).to(dtype), requires_grad=False)
        self.down_proj = nn.Parameter((torch.randn(experts, hidden, inter) * 0.05).to(dtype), requires_grad=False)
        self.act_fn = torch.nn.functional.silu

    def forward(self, hidden_states, top_k_index, top_k_weights, gate_up=None, down=None):
        gate_up = self.gate_up_proj if gate_up is None else gate_up
        down = self.down_proj if down is None else down
        out = torch.zeros_like(hidden_states)
        for e in range(self.num_experts):
            token, k = torch.where(top_k_index == e)
            if token.numel() == 0:
                continue
            g, u = torch.nn.functional.linear(hidden_states[token], gate_up[e]).chunk(2, dim=-1)
            o = torch.nn.functional.linear(self.act_fn(g) * u, down[e]) * top_k_weights[token, k, None]
            out = out.index_add(0, token, o.to(out.dtype))
        return out


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_patched_experts_forward_under_adapter_disable_and_batch(dev, dtype):
    """patch_target_parameters makes the model's own expert module apply the active tenant's expert LoRA
    (the reference does it by merging W + B A * scaling into the parameter, multi_lora_target_parameters.py:182-209):
    ``with adapter(t): model(...)`` equals the module's loop on merged weights in float64, ``disable_lora=True`` and
    no tenant give the frozen experts, and ``batch()`` gives every token its own tenant's merged weights."""
    torch.manual_seed(0)
    e, hid, inter, t, k = 4, 128, 256, 90, 2
    model = nn.Module()
    model.experts = PackedExperts(e, hid, inter, dtype).to(dev)
    model.set_adapter = lambda name: None
    model.disable_adapter_layers = model.enable_adapter_layers = lambda: None
    targets = ['experts.gate_up_proj', 'experts.down_proj']
    ml = MultiLora(max_loras=3, max_r=8)
    ml.module = model
    ml.loras = [LoraTenant(index=i, adapter_name=f'lora_{i}', config=None) for i in range(3)]
    ml.patch_target_parameters(model, targets)
    cfg = lambda r: LoraConfig(r=r, lora_alpha=2 * r, target_modules=[], target_parameters=targets)  # noqa: E731
    ml.acquire_lora('alice', cfg(8))
    ml.acquire_lora('bob', cfg(4))
    manager = ml.target_parameter_manager
    gu, dn = manager.wrappers
    with torch.no_grad():
        for name in ('alice', 'bob'):
            for key, p in manager.named_slot_parameters(name):
                if '.lora_B.' in key:
                    p.normal_(0, 0.05)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(t, hid, generator=g).to(dtype)
    weights, sel = torch.topk(torch.softmax(torch.randn(t, e, generator=g), -1), k)
    weights = weights.to(dtype)
    tenant = torch.randint(-1, 2, (t,), generator=g)                  # -1: a token without a tenant
    xd, seld, wd = x.to(dev), sel.to(dev), weights.to(dev)

    cpu = PackedExperts(e, hid, inter, torch.float64)
    w_gu, w_dn = model.experts.gate_up_proj.detach().double().cpu(), model.experts.down_proj.detach().double().cpu()

    def merged_forward(token_tenant):
        """float64: every token through the experts with the merged weights of its own tenant."""
        out = torch.zeros(t, hid, dtype=torch.float64)
        for ti, name in list(enumerate(('alice', 'bob'))) + [(-1, None)]:
            rows = (token_tenant == ti).nonzero().flatten()
            if rows.numel() == 0:
                continue
            a, b = w_gu, w_dn
            if name is not None:
                s = manager.tenant_to_slot[name]
                a = a + gu.get_delta_weight(s).detach().double().cpu()
                b = b + dn.get_delta_weight(s).detach().double().cpu()
            out[rows] = cpu(x.double()[rows], sel[rows], weights.double()[rows], a, b)
        return out

    tol = 2e-5 if dtype == torch.float32 else 2e-2
    frozen = merged_forward(torch.full((t,), -1))
    assert max_rel_err(model.experts(xd, seld, wd), frozen) < tol                       # no context: frozen experts
    with ml.adapter('alice', disable_lora=True):
        assert max_rel_err(model.experts(xd, seld, wd), frozen) < tol
    for ti, name in enumerate(('alice', 'bob')):
        with ml.adapter(name):
            y = model.experts(xd, seld, wd)
        want = merged_forward(torch.full((t,), ti))
        assert max_rel_err(y, want) < tol, name
        assert max_rel_err(y.double().cpu() - frozen, want - frozen) < 5 * tol, name   # the LoRA part on its own
    # a mixed batch: gradients of both tenants' expert adapters from one pass, against float64 autograd
    leaves = {}
    for w in (gu, dn):
        for name in ('alice', 'bob'):
            s = manager.tenant_to_slot[name]
            leaves[(id(w), name, 'a')] = w.lora_A[s].detach().double().cpu().requires_grad_(True)
            leaves[(id(w), name, 'b')] = w.lora_B[s].detach().double().cpu().requires_grad_(True)
    want = torch.zeros(t, hid, dtype=torch.float64)
    for ti, name in list(enumerate(('alice', 'bob'))) + [(-1, None)]:
        rows = (tenant == ti).nonzero().flatten()
        a, b = w_gu, w_dn
        if name is not None:
            s = manager.tenant_to_slot[name]
            a = a + oracle.expert_delta_weight(leaves[(id(gu), name, 'a')], leaves[(id(gu), name, 'b')], gu.r[s], gu.scaling[s])
            b = b + oracle.expert_delta_weight(leaves[(id(dn), name, 'a')], leaves[(id(dn), name, 'b')], dn.r[s], dn.scaling[s])
        want = want.index_add(0, rows, cpu(x.double()[rows], sel[rows], weights.double()[rows], a, b))
    with ml.batch(['alice', 'bob'], tenant.to(dev)):
        y = model.experts(xd, seld, wd)
    assert max_rel_err(y, want) < tol
    y.float().pow(2).sum().backward()
    want.pow(2).sum().backward()
    gtol = 2e-4 if dtype == torch.float32 else 3e-2
    for w in (gu, dn):
        for name in ('alice', 'bob'):
            s = manager.tenant_to_slot[name]
            assert max_rel_err(w.lora_A[s].grad, leaves[(id(w), name, 'a')].grad) < gtol, (name, 'A')
            assert max_rel_err(w.lora_B[s].grad, leaves[(id(w), name, 'b')].grad) < gtol, (name, 'B')
        assert w.lora_A['lora_2'].grad is None


def test_batched_steps_with_gradient_accumulation_equal_each_tenant_alone(dev):
    """Three tenants with gradient accumulation 1 / 2 / 3 share six mixed batches; BatchedStep reduces the token
    losses per tenant (sum reduction, ignore_index rows do not count) and steps the tenants that are due
    (optimizer_group.py:56-62).  Against the reference's schedule on a fresh copy: every tenant alone, its own rows
    under adapter(), loss_value / num_tokens accumulated, clip_grad_and_step's parts guarded by do_grad_sync."""
    names = ['alice', 'bob', 'carol']
    gas = {'alice': 1, 'bob': 2, 'carol': 3}
    hyper = {'alice': dict(lr=1e-2, weight_decay=0.01), 'bob': dict(lr=5e-3, weight_decay=0.0),
             'carol': dict(lr=2e-2, weight_decay=0.1)}
    vocab, steps, rows = 128, 6, 150
    g = torch.Generator().manual_seed(7)
    xs = [torch.randn(rows, 128, generator=g) for _ in range(steps)]
    labels = [torch.randint(0, vocab, (rows,), generator=g) for _ in range(steps)]
    for lab in labels:
        lab[torch.rand(rows, generator=g) < 0.15] = -100
    rts = [torch.randint(0, 3, (rows,), generator=g) for _ in range(steps)]
    rts[3][rts[3] == 2] = 0                                            # carol has no row in the fourth batch

    # (a) batched
    ml, model, _ = _setup(dev, torch.float32)
    slot = {n: ml.find_lora_by_tenant(n).adapter_name for n in names}
    opt = MultiTenantAdamW()
    for n in names:
        opt.add_tenant(n, trainable_parameters(model, slot[n]).values(), **hyper[n])
    sched = BatchedStep(opt, gradient_accumulation_steps=gas, reduction='sum')
    stepped = []
    for i in range(steps):
        present = [n for j, n in enumerate(names) if int((rts[i] == j).sum()) > 0]
        lut = torch.tensor([present.index(n) if n in present else -1 for n in names])
        rt = lut[rts[i]].to(dev)
        with ml.batch(present, rt):
            logits = model(xs[i].to(dev))
        loss = sched.loss(present, rt, labels[i].to(dev), logits=logits)
        sched.backward(loss)
        stepped.append(sorted(sched.due()))
        sched.clip_grad_and_step(max_grad_norm=1.0)
    got = {n: {k: p.detach().clone() for k, p in trainable_parameters(model, slot[n]).items()} for n in names}
    assert stepped[0] == ['alice'] and 'bob' in stepped[2] and 'bob' not in stepped[1]

    # (b) the reference's schedule, one tenant at a time on a fresh copy
    ml2, model2, _ = _setup(dev, torch.float32)
    for j, n in enumerate(names):
        params = trainable_parameters(model2, slot[n])
        plist = list(params.values())
        optim = torch.optim.AdamW(plist, **hyper[n])
        cur_step, num_tokens, did = 0, 0.0, []
        for i in range(steps):
            mine = (rts[i] == j).nonzero().flatten()
            if mine.numel() == 0:
                continue                                               # the tenant sent no batch this round
            with ml2.adapter(n):
                logits = model2(xs[i][mine].to(dev))
            lab = labels[i][mine].to(dev)
            logps = torch.log_softmax(logits, -1).gather(-1, lab.clamp(min=0)[:, None])[:, 0]
            mask = (lab != -100).float()
            (-(logps) * mask).sum().backward()                        # loss/cross_entropy.py:16-33, reduction='sum'
            num_tokens += float(mask.sum().clamp(min=1))
            cur_step += 1
            if twinkle_amd.do_grad_sync(cur_step, gas[n]):
                for p in plist:
                    if p.grad is not None:
                        p.grad.div_(num_tokens)
                torch.nn.utils.clip_grad_norm_([p for p in plist if p.grad is not None], 1.0)
                optim.step()
                optim.zero_grad(set_to_none=True)
                num_tokens = 0.0
                did.append(i)
        assert did == [i for i in range(steps) if n in stepped[i]], (n, did, stepped)
        for k, p in params.items():
            assert max_rel_err(got[n][k], p.detach()) < 5e-5, (n, k)

    # (c) one tenant's whole trajectory through the oracle on the CPU in float64: its rows of every batch through the
    # per-adapter forward (oracle.lora_linear_forward, autograd of it), the token-normalised clipped AdamW step of
    # oracle.TenantAdamW whenever the accumulation rule says so.  bob targets q_proj and down_proj (rank 16).
    n, j = 'bob', names.index('bob')
    _, fresh, cfgs3 = _setup(dev, torch.float32)
    cfg = cfgs3[n]
    blk = fresh.model
    scaling = oracle.lora_scaling(cfg.lora_alpha, cfg.r, cfg.use_rslora)
    cpu = lambda t: t.detach().double().cpu()  # noqa: E731
    w_q, w_up, b_up, w_down = cpu(blk.q_proj.base_layer.weight), cpu(blk.up_proj.base_layer.weight), \
        cpu(blk.up_proj.base_layer.bias), cpu(blk.down_proj.base_layer.weight)
    keys = [k for k in trainable_parameters(fresh, slot[n]) if '.q_proj.' in k or '.down_proj.' in k]
    start = trainable_parameters(fresh, slot[n])
    tenant_opt = oracle.TenantAdamW([cpu(start[k]) for k in keys], **hyper[n])
    by_key = dict(zip(keys, tenant_opt.params))
    pick = lambda layer, side: next(p for k, p in by_key.items() if f'.{layer}.' in k and f'.{side}.' in k)  # noqa: E731
    acc = [torch.zeros_like(p) for p in tenant_opt.params]
    cur_step, num_tokens = 0, 0.0
    for i in range(steps):
        mine = (rts[i] == j).nonzero().flatten()
        if mine.numel() == 0:
            continue
        x64 = xs[i][mine].double()
        h = oracle.lora_linear_forward(x64, torch.nn.functional.linear(x64, w_q), pick('q_proj', 'lora_A'),
                                       pick('q_proj', 'lora_B'), cfg.r, scaling)
        h = torch.nn.functional.silu(torch.nn.functional.linear(h, w_up, b_up))        # up_proj is not targeted
        logits = oracle.lora_linear_forward(h, torch.nn.functional.linear(h, w_down), pick('down_proj', 'lora_A'),
                                            pick('down_proj', 'lora_B'), cfg.r, scaling)
        lab = labels[i][mine]
        logps = torch.log_softmax(logits, -1).gather(-1, lab.clamp(min=0)[:, None])[:, 0]
        mask = (lab != -100).double()
        grads = torch.autograd.grad(-(logps * mask).sum(), tenant_opt.params)
        for a_, g_ in zip(acc, grads):
            a_ += g_
        num_tokens += float(mask.sum().clamp(min=1))
        cur_step += 1
        if twinkle_amd.do_grad_sync(cur_step, gas[n]):
            tenant_opt.clip_grad_and_step(acc, int(num_tokens), max_grad_norm=1.0)
            acc = [torch.zeros_like(p) for p in tenant_opt.params]
            num_tokens = 0.0
    for k, p in by_key.items():
        assert max_rel_err(got[n][k], p.detach()) < 2e-4, (n, k, 'oracle trajectory')
        assert (p.detach() - cpu(start[k])).abs().max() > 0, (k, 'the tenant was stepped')
    for k, p in start.items():                       # the layer bob does not target stays as it was
        if k not in by_key:
            assert torch.equal(got[n][k], p.detach()), k


@pytest.mark.parametrize('dtype,tol', [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
def test_several_active_adapters_on_one_layer_add_up(dev, dtype, tol):
    """The reference's patched forward loops over ``active_adapters`` and adds every adapter's term
    (multi_lora.py:306-326); with two active slots the layer gives base + term(alice) + term(bob)."""
    ml, model, cfgs = _setup(dev, dtype)
    slot = {n: ml.find_lora_by_tenant(n).adapter_name for n in cfgs}
    layer = model.model.q_proj
    g = torch.Generator().manual_seed(9)
    x = torch.randn(70, 128, generator=g).to(dtype)
    layer.set_adapter([slot['alice'], slot['bob']])
    y = layer(x.to(dev))
    want = layer.base_layer(x.to(dev)).double().cpu()
    for n in ('alice', 'bob'):
        cfg = cfgs[n]
        want = oracle.lora_linear_forward(x.double(), want, layer.lora_A[slot[n]].weight.detach().double().cpu(),
                                          layer.lora_B[slot[n]].weight.detach().double().cpu(), cfg.r,
                                          oracle.lora_scaling(cfg.lora_alpha, cfg.r, cfg.use_rslora))
    assert max_rel_err(y, want) < tol
    layer.set_adapter([slot['alice']])
    one = layer(x.to(dev))
    assert (y.float() - one.float()).abs().max() > 0


@pytest.mark.parametrize('dtype,tol', [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
def test_several_active_adapters_with_shared_inputs_add_up(dev, dtype, tol):
    """Layers declared with ``share_inputs`` route their calls through the shared entry; with two active slots every
    layer must still add every adapter's term (multi_lora.py:306-326), whether or not the group call is used."""
    ml, model, cfgs = _setup(dev, dtype)
    slot = {n: ml.find_lora_by_tenant(n).adapter_name for n in cfgs}
    layers = {'model.q_proj': model.model.q_proj, 'model.up_proj': model.model.up_proj}
    ml.share_inputs([list(layers)])
    try:
        g = torch.Generator().manual_seed(10)
        x = torch.randn(70, 128, generator=g).to(dtype)
        xd = x.to(dev)
        for layer in layers.values():
            layer.set_adapter([slot['alice'], slot['bob']])
        got = {name: layer(xd) for name, layer in layers.items()}       # same tensor: one group computation
        for name, layer in layers.items():
            want = layer.base_layer(xd).double().cpu()
            for n in ('alice', 'bob'):
                cfg = cfgs[n]
                if not oracle.match_target_modules(name, cfg.target_modules):
                    continue                                            # bob does not target up_proj
                want = oracle.lora_linear_forward(x.double(), want, layer.lora_A[slot[n]].weight.detach().double().cpu(),
                                                  layer.lora_B[slot[n]].weight.detach().double().cpu(), cfg.r,
                                                  oracle.lora_scaling(cfg.lora_alpha, cfg.r, cfg.use_rslora))
            assert max_rel_err(got[name], want) < tol, name
        # one active adapter: the group call proper gives the same as the layer alone
        for layer in layers.values():
            layer.set_adapter([slot['alice']])
        shared = {name: layer(xd) for name, layer in layers.items()}
        ml.unshare_inputs()
        for name, layer in layers.items():
            assert max_rel_err(shared[name], layer(xd).double().cpu()) < tol, name
            assert (got[name].float() - shared[name].float()).abs().max() > 0 or name == 'model.up_proj'
    finally:
        ml.unshare_inputs()
