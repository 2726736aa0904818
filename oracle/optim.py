"""CPU restatement of the reference's per-tenant optimizer step (test infrastructure only).

The reference steps one tenant at a time (src/twinkle/model/transformers/transformers.py):
``clip_grad_norm`` (:732-778) calls ``normalize_and_clip_grad_norm``
(src/twinkle/utils/grad_clip.py:31-96), which divides every gradient by the tenant's token
count in place (``_normalize_grads`` :81-96, ``num_tokens <= 0`` counts as 1) and, on one GPU,
clips with ``torch.nn.utils.clip_grad_norm_`` (:118-123), returning the norm *before* clipping;
``step`` (:835-876) overrides lr / weight_decay (only where it was positive) / eps / betas from
``optim_params`` and runs the tenant's ``torch.optim.AdamW`` (or ``Adam``); ``clip_grad_and_step``
(:781-785) is clip, step, zero_grad, lr_step.  The tenant's parameters are those whose name
matches ``\\.lora_\\w+\\.<adapter name>`` (:962-972).

Pin status: pinned.  The arithmetic is ``torch.nn.utils.clip_grad_norm_`` and
``torch.optim.AdamW`` themselves (the library routines the reference calls), driven here on CPU
tensors; ``tests/test_oracle_optim.py`` additionally checks one AdamW step against the textbook
closed form and the clip coefficient against its definition.
"""
from __future__ import annotations

import re
from typing import Dict, Iterable, List, Optional, Sequence

import torch


def trainable_parameter_names(names: Iterable[str], adapter_name: str) -> List[str]:
    """Names that belong to one tenant's slot (transformers.py:962-972, non-default adapter)."""
    pattern = re.compile(rf'\.lora_\w+\.{re.escape(adapter_name)}')
    return [n for n in names if pattern.search(n)]


def normalize_and_clip_grad_norm(grads: Sequence[torch.Tensor], num_tokens: int, max_grad_norm: float,
                                 norm_type: float) -> float:
    """In place on ``grads``; returns the total norm after normalisation, before clipping (grad_clip.py:31-96)."""
    if num_tokens <= 0:
        num_tokens = 1
    holders = []
    for g in grads:
        g.div_(num_tokens)
        p = torch.nn.Parameter(torch.empty_like(g), requires_grad=True)
        p.grad = g
        holders.append(p)
    if not holders:
        return 0.0
    return float(torch.nn.utils.clip_grad_norm_(holders, max_grad_norm, norm_type=norm_type))


class TenantAdamW:
    """One tenant's ``torch.optim.AdamW`` on CPU copies, stepped with the reference's per-call overrides."""

    def __init__(self, params: Sequence[torch.Tensor], lr: float = 1e-3, betas=(0.9, 0.999), eps: float = 1e-8,
                 weight_decay: float = 1e-2):
        self.params = [torch.nn.Parameter(p.detach().clone()) for p in params]
        self.optimizer = torch.optim.AdamW(self.params, lr=lr, betas=betas, eps=eps, weight_decay=weight_decay)

    def clip_grad_and_step(self, grads: Sequence[torch.Tensor], num_tokens: int, max_grad_norm: float = 1.0,
                           norm_type: float = 2.0, optim_params: Optional[Dict] = None) -> float:
        grads = [g.detach().clone().to(p.dtype) for g, p in zip(grads, self.params)]
        norm = normalize_and_clip_grad_norm(grads, num_tokens, max_grad_norm, norm_type)
        for p, g in zip(self.params, grads):
            p.grad = g
        if optim_params:  # transformers.py:857-868
            for group in self.optimizer.param_groups:
                group['lr'] = optim_params['lr']
                if group['weight_decay'] > 0.0 and optim_params.get('weight_decay') is not None:
                    group['weight_decay'] = optim_params['weight_decay']
                if optim_params.get('eps') is not None:
                    group['eps'] = optim_params['eps']
                if optim_params.get('betas') is not None:
                    group['betas'] = optim_params['betas']
        self.optimizer.step()
        self.optimizer.zero_grad()
        return norm
