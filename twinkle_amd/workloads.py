"""Seeded synthetic inputs for the benchmark and parity configurations.

Everything is generated on the CPU in float32 with fixed seeds (and cast
afterwards), so the GPU kernels and the CPU checker see identical values.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List

import torch


@dataclass
class LoraWorkload:
    name: str
    tokens: int
    in_features: int
    out_features: int
    ranks: List[int]
    scales: List[float]
    max_rank: int
    ids: torch.Tensor            # [tokens] int32, adapter of each token
    x: torch.Tensor              # [tokens, in]  float32
    dy: torch.Tensor             # [tokens, out] float32
    base_out: torch.Tensor       # [tokens, out] float32 (output of the frozen base layer)
    lora_A: List[torch.Tensor] = field(default_factory=list)  # each [max_rank, in]
    lora_B: List[torch.Tensor] = field(default_factory=list)  # each [out, max_rank]

    @property
    def num_adapters(self) -> int:
        return len(self.ranks)

    def flops(self) -> float:
        counts = torch.bincount(self.ids.long(), minlength=self.num_adapters).tolist()
        return float(sum(6.0 * c * r * (self.in_features + self.out_features) for c, r in zip(counts, self.ranks)))

    def algorithmic_bytes(self, elt: int) -> float:
        """fwd+bwd bytes: x, y (r+w), dy, x, dx (r+w); weights read twice; fp32-sized grads written once."""
        w = sum(r * (self.in_features + self.out_features) for r in self.ranks)
        return float(elt * self.tokens * (4 * self.in_features + 3 * self.out_features) + (2 * elt + 4) * w)


def _weights(gen, n, max_rank, in_features, out_features):
    bound = 1.0 / math.sqrt(in_features)
    a = [(torch.rand(max_rank, in_features, generator=gen) * 2 - 1) * bound for _ in range(n)]
    b = [torch.randn(out_features, max_rank, generator=gen) * 0.02 for _ in range(n)]
    return a, b


def _acts(gen, tokens, in_features, out_features):
    x = torch.randn(tokens, in_features, generator=gen)
    dy = torch.randn(tokens, out_features, generator=gen)
    base = torch.randn(tokens, out_features, generator=gen) * 0.5
    return x, dy, base


def config1_plumbing() -> LoraWorkload:
    """T=512, 1024->1024, 4 adapters rank 8 alpha 16, contiguous 128-token segments, fp32."""
    gen = torch.Generator().manual_seed(0)
    t, k, m, n, r = 512, 1024, 1024, 4, 8
    x, dy, _ = _acts(gen, t, k, m)
    w = torch.randn(m, k, generator=gen) * 0.02
    a, b = _weights(gen, n, r, k, m)
    ids = torch.arange(t, dtype=torch.int32) // (t // n)
    return LoraWorkload('cfg1_plumbing_fp32', t, k, m, [r] * n, [2.0] * n, r, ids, x, dy, x @ w.t(), a, b)


def zipf_ids(tokens: int, n: int, s: float = 1.1, seed_draw: int = 1, seed_shuffle: int = 2) -> torch.Tensor:
    pmf = torch.tensor([1.0 / (i + 1)**s for i in range(n)])
    pmf = pmf / pmf.sum()
    ids = torch.multinomial(pmf, tokens, replacement=True, generator=torch.Generator().manual_seed(seed_draw))
    order = torch.randperm(tokens, generator=torch.Generator().manual_seed(seed_shuffle))
    return ids[order].to(torch.int32)


def config2_qproj(tokens: int = 16384, features: int = 4096, n: int = 16, r: int = 16) -> LoraWorkload:
    """Llama-3-8B q_proj: 4096->4096, T=16384, 16 adapters rank 16 alpha 32, Zipf(1.1) ids, shuffled."""
    gen = torch.Generator().manual_seed(11)
    x, dy, base = _acts(gen, tokens, features, features)
    a, b = _weights(gen, n, r, features, features)
    return LoraWorkload('cfg2_llama8b_qproj', tokens, features, features, [r] * n, [2.0] * n, r,
                        zipf_ids(tokens, n), x, dy, base, a, b)


def uneven_ids(tokens: int, n: int, empty=(5, 17), seed_sizes: int = 3, seed_shuffle: int = 4) -> torch.Tensor:
    u = torch.rand(n, generator=torch.Generator().manual_seed(seed_sizes)) * 2048
    for e in empty:
        if e < n:
            u[e] = 0
    exact = u / u.sum() * tokens
    sizes = exact.floor().long()
    rem = tokens - int(sizes.sum())
    frac = exact - sizes
    for e in empty:
        if e < n:
            frac[e] = -1
    sizes[torch.argsort(frac, descending=True)[:rem]] += 1
    ids = torch.repeat_interleave(torch.arange(n), sizes)
    order = torch.randperm(tokens, generator=torch.Generator().manual_seed(seed_shuffle))
    return ids[order].to(torch.int32)


def config3_mlp(direction: str = 'up', tokens: int = 32768, hidden: int = 4096, inter: int = 14336,
                n: int = 32) -> LoraWorkload:
    """Llama-3-8B MLP projection, 32 adapters with ranks cycled over {8,16,32,64}, two of them empty."""
    k, m = (hidden, inter) if direction == 'up' else (inter, hidden)
    gen = torch.Generator().manual_seed(33)
    ranks = [[8, 16, 32, 64][i % 4] for i in range(n)]
    x, dy, base = _acts(gen, tokens, k, m)
    a, b = _weights(gen, n, 64, k, m)
    return LoraWorkload(f'cfg3_llama8b_mlp_{direction}', tokens, k, m, ranks, [2.0] * n, 64, uneven_ids(tokens, n), x,
                        dy, base, a, b)


def moe_routing(tokens: int = 8192, experts: int = 128, top_k: int = 8, tenants: int = 4):
    """Top-k routing from softmax(N(0,1) logits) and a uniform tenant id per token (CPU, seeded)."""
    logits = torch.randn(tokens, experts, generator=torch.Generator().manual_seed(5))
    weights, selected = torch.topk(torch.softmax(logits, -1), top_k, dim=-1)
    tenant = torch.randint(0, tenants, (tokens,), generator=torch.Generator().manual_seed(6))
    return selected.to(torch.int32), weights, tenant.to(torch.int32)
