"""Pins for oracle/optim.py: the reference's per-tenant clip + AdamW step, against closed forms."""
import math

import torch

import oracle


def test_parameter_selection_follows_the_reference_regex():
    names = ['model.layers.0.q_proj.lora_A.lora_1.weight', 'model.layers.0.q_proj.lora_B.lora_1.weight',
             'model.layers.0.q_proj.lora_A.lora_10.weight', 'model.layers.0.q_proj.base_layer.weight',
             'model.layers.0.mlp.experts.lora_A.lora_1']
    got = oracle.trainable_parameter_names(names, 'lora_1')
    # the pattern is a search, so lora_10 also matches lora_1 (reference behaviour, transformers.py:966)
    assert got == [names[0], names[1], names[2], names[4]]


def test_normalize_then_clip_matches_definition():
    g = torch.Generator().manual_seed(0)
    grads = [torch.randn(5, 7, generator=g, dtype=torch.float64), torch.randn(3, generator=g, dtype=torch.float64)]
    ref = [t.clone() for t in grads]
    norm = oracle.normalize_and_clip_grad_norm(grads, num_tokens=4, max_grad_norm=0.05, norm_type=2.0)
    total = math.sqrt(sum(float((t / 4).pow(2).sum()) for t in ref))
    assert abs(norm - total) < 1e-12
    coef = min(1.0, 0.05 / (total + 1e-6))
    for a, b in zip(grads, ref):
        assert torch.allclose(a, b / 4 * coef, rtol=1e-12, atol=0)
    # num_tokens <= 0 counts as 1; a large threshold leaves the gradients alone
    grads = [t.clone() for t in ref]
    norm = oracle.normalize_and_clip_grad_norm(grads, num_tokens=0, max_grad_norm=1e9, norm_type=float('inf'))
    assert abs(norm - max(float(t.abs().max()) for t in ref)) < 1e-12
    assert all(torch.equal(a, b) for a, b in zip(grads, ref))


def test_adamw_steps_match_the_closed_form():
    g = torch.Generator().manual_seed(1)
    p0 = torch.randn(4, 6, generator=g, dtype=torch.float64)
    opt = oracle.TenantAdamW([p0], lr=1e-2, betas=(0.8, 0.95), eps=1e-6, weight_decay=0.1)
    p, m, v = p0.clone(), torch.zeros_like(p0), torch.zeros_like(p0)
    for step in range(1, 4):
        grad = torch.randn(4, 6, generator=g, dtype=torch.float64)
        lr = 1e-2 / step                       # per-call override, as the server passes it
        opt.clip_grad_and_step([grad], num_tokens=3, max_grad_norm=1e9, optim_params={'lr': lr})
        gg = grad / 3
        p = p * (1 - lr * 0.1)
        m = 0.8 * m + 0.2 * gg
        v = 0.95 * v + 0.05 * gg * gg
        p = p - lr / (1 - 0.8**step) * m / (v.sqrt() / math.sqrt(1 - 0.95**step) + 1e-6)
        assert torch.allclose(opt.params[0].detach(), p, rtol=1e-12, atol=1e-14)
    # weight_decay is only overridden where it was positive (transformers.py:862-863)
    opt0 = oracle.TenantAdamW([p0], lr=1e-2, weight_decay=0.0)
    opt0.clip_grad_and_step([torch.ones_like(p0)], 1, 1e9, optim_params={'lr': 1e-2, 'weight_decay': 0.5})
    assert opt0.optimizer.param_groups[0]['weight_decay'] == 0.0
