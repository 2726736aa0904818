"""Multi-tenant gradient norm + AdamW on the GPU against the reference's per-tenant torch path (oracle/optim.py)."""
import math

import pytest
import torch

import oracle
from conftest import max_rel_err
from twinkle_amd import MultiTenantAdamW

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def dev():
    if not torch.cuda.is_available():
        pytest.skip('needs a GPU')
    return torch.device('cuda:0')


def _tenants(dtype, seed):
    g = torch.Generator().manual_seed(seed)
    shapes = {'a': [(16, 256), (512, 16), (1, 5)], 'b': [(8, 1000), (333, 8)], 'c': [(64, 4096), (4096, 64)]}
    hyper = {'a': dict(lr=1e-2, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2),
             'b': dict(lr=3e-3, betas=(0.8, 0.95), eps=1e-6, weight_decay=0.0),
             'c': dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-8, weight_decay=0.1)}
    params = {k: [torch.randn(s, generator=g).to(dtype) for s in v] for k, v in shapes.items()}
    return params, hyper, g


@pytest.mark.parametrize('norm_type', [2.0, float('inf')])
def test_fp32_three_tenants_three_steps(dev, norm_type):
    params, hyper, g = _tenants(torch.float32, 0)
    opt = MultiTenantAdamW()
    dev_params, refs = {}, {}
    for name, ps in params.items():
        dev_params[name] = [torch.nn.Parameter(p.to(dev)) for p in ps]
        opt.add_tenant(name, dev_params[name], **hyper[name])
        refs[name] = oracle.TenantAdamW([p.double() for p in ps], **hyper[name])
    tokens = {'a': 37, 'b': 1, 'c': 4096}
    for step in range(3):
        grads = {k: [torch.randn(p.shape, generator=g) * (10.0 if k == 'a' else 1.0) for p in ps]
                 for k, ps in params.items()}
        over = {'a': {'lr': 1e-2 / (step + 1), 'weight_decay': 0.05}, 'b': {'lr': 3e-3, 'weight_decay': 0.5},
                'c': {'lr': 2e-3, 'eps': 1e-7, 'betas': (0.85, 0.98)}}
        for k in params:
            for p, gr in zip(dev_params[k], grads[k]):
                p.grad = gr.to(dev)
        norms = opt.clip_grad_and_step(tokens, max_grad_norm=0.5, norm_type=norm_type, optim_params=over)
        for k in params:
            want = refs[k].clip_grad_and_step([t.double() for t in grads[k]], tokens[k], 0.5, norm_type, over[k])
            assert abs(float(norms[k]) - want) <= 1e-5 * max(want, 1e-12), (k, step)
            for p, q in zip(dev_params[k], refs[k].params):
                assert max_rel_err(p.detach(), q.detach()) < 1e-5, (k, step)
                assert torch.count_nonzero(p.grad) == 0      # zero_grad is part of clip_grad_and_step
    # moments against torch's own state
    for k in params:
        st = opt.state(k)
        assert st['step'] == 3
        for i, q in enumerate(refs[k].params):
            ref_state = refs[k].optimizer.state[q]
            assert max_rel_err(st['exp_avg'][i], ref_state['exp_avg']) < 1e-5
            assert max_rel_err(st['exp_avg_sq'][i], ref_state['exp_avg_sq']) < 1e-5


def test_bf16_parameters_one_step(dev):
    """bf16 parameters and gradients, fp32 arithmetic and moments: one step against the fp64 oracle on the same
    rounded inputs, to bf16 resolution."""
    params, hyper, g = _tenants(torch.bfloat16, 1)
    opt = MultiTenantAdamW()
    dev_params, refs, grads = {}, {}, {}
    for name, ps in params.items():
        dev_params[name] = [torch.nn.Parameter(p.to(dev)) for p in ps]
        opt.add_tenant(name, dev_params[name], **hyper[name])
        refs[name] = oracle.TenantAdamW([p.double() for p in ps], **hyper[name])
        grads[name] = [torch.randn(p.shape, generator=g).bfloat16() for p in ps]
        for p, gr in zip(dev_params[name], grads[name]):
            p.grad = gr.to(dev)
    tokens = {'a': 5, 'b': 7, 'c': 11}
    norms = opt.clip_grad_norm(tokens, max_grad_norm=1.0)
    opt.step(tokens, write_grads=True)
    for k in params:
        want = refs[k].clip_grad_and_step([t.double() for t in grads[k]], tokens[k], 1.0, 2.0)
        assert abs(float(norms[k]) - want) <= 1e-5 * want
        for p, q in zip(dev_params[k], refs[k].params):
            assert max_rel_err(p.detach(), q.detach()) < 2e-2
        # write_grads: .grad now holds the normalised, clipped gradient, as in the reference after clip_grad_norm
        coef = min(1.0, 1.0 / (want + 1e-6))
        for p, gr in zip(dev_params[k], grads[k]):
            assert max_rel_err(p.grad, gr.double() / tokens[k] * coef) < 2e-2


def test_skipped_tenants_missing_grads_and_repeatability(dev):
    params, hyper, g = _tenants(torch.float32, 2)
    runs = []
    for _ in range(2):
        opt = MultiTenantAdamW()
        dp = {}
        for name, ps in params.items():
            dp[name] = [torch.nn.Parameter(p.to(dev)) for p in ps]
            opt.add_tenant(name, dp[name], **hyper[name])
        gg = torch.Generator().manual_seed(9)
        for k in ('a', 'c'):
            for i, p in enumerate(dp[k]):
                if not (k == 'a' and i == 1):          # one parameter of tenant a has no gradient
                    p.grad = torch.randn(p.shape, generator=gg).to(dev)
        before_b = [p.detach().clone() for p in dp['b']]
        before_a1 = dp['a'][1].detach().clone()
        norms = opt.clip_grad_and_step({'a': 3, 'c': 9}, max_grad_norm=0.1, names=['a', 'c'])
        assert set(norms) == {'a', 'c'}
        assert all(torch.equal(p.detach(), q) for p, q in zip(dp['b'], before_b))      # tenant b did not step
        assert torch.equal(dp['a'][1].detach(), before_a1)                              # no gradient, no update
        assert opt.state('b')['step'] == 0 and opt.state('a')['step'] == 1
        runs.append([p.detach().clone() for k in ('a', 'c') for p in dp[k]] + [norms['a'].clone(), norms['c'].clone()])
    assert all(torch.equal(x, y) for x, y in zip(*runs))                                # bitwise repeatable


def test_argument_errors(dev):
    opt = MultiTenantAdamW()
    with pytest.raises(RuntimeError, match='GPU'):
        opt.add_tenant('cpu', [torch.nn.Parameter(torch.zeros(3))])
    with pytest.raises(ValueError):
        opt.add_tenant('half', [torch.nn.Parameter(torch.zeros(3, dtype=torch.float16, device=dev))])
    opt.add_tenant('x', [torch.nn.Parameter(torch.zeros(3, device=dev))])
    with pytest.raises(ValueError):
        opt.add_tenant('x', [])
    assert opt.clip_grad_and_step(1) == {}                # no gradients anywhere: nothing to do
