"""Oracle: token→group ordering, permute/unpermute, packed-sequence bounds.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  Integer results here
are the bit-exact target for the HIP segment builder.
"""
from __future__ import annotations

import torch


def expert_mask_from_topk(selected: torch.Tensor, num_groups: int) -> torch.Tensor:
    """Mask ``[G, K, T]`` from per-token group choices ``[T, K]``.

    Follows src/twinkle/model/transformers/moe/expert_parallel.py:254-255
    (``one_hot(selected_experts, num_classes).permute(2, 1, 0)``).
    """
    if selected.dim() == 1:
        selected = selected[:, None]
    return torch.nn.functional.one_hot(selected.long(), num_classes=num_groups).permute(2, 1, 0)


def permute_by_mask(tokens: torch.Tensor, mask: torch.Tensor):
    """Rows gathered in (group, k, token) order, plus the token index of each row.

    Follows src/twinkle/model/transformers/moe/ep_utils.py:99-118: a token-index
    tensor is expanded to the mask's shape ``[G, K, T]`` and ``masked_select``
    walks it row-major, so the order is group ascending, then top-k slot
    ascending, then token ascending.
    """
    num_tokens = tokens.shape[0]
    mask = mask.bool()
    token_indices = torch.arange(num_tokens).view(1, 1, num_tokens).expand_as(mask)
    sorted_indices = token_indices.masked_select(mask)
    return tokens.index_select(0, sorted_indices), sorted_indices


def segment_build_sort(keys: torch.Tensor, num_groups: int):
    """(perm, counts, offsets) for flat row keys, by a stable sort.

    ``keys[f]`` is the group of flat row ``f``; for top-k routing the flat row
    index is ``f = k*T + t`` (row-major over the last two axes of the
    reference's mask, expert_parallel.py:254-255 / ep_utils.py:112-113).
    ``perm[j]`` is the flat row placed at sorted position ``j``; ties keep
    ascending ``f``.  ``counts`` follows ep_utils.py:191
    (``expert_mask.sum((1, 2))``) and kernel/npu_impls/moe.py:117 (``bincount``
    with ``minlength``); ``offsets`` is the running sum the reference builds on
    the host at expert_parallel.py:347-349.  All int64, as in the reference.
    """
    keys = keys.reshape(-1).long()
    # a key outside [0, num_groups) is a row without a group (nothing in the reference, whose mask has no such
    # row): it sorts after every group and is counted nowhere, so offsets[num_groups] = rows that have a group
    keys = torch.where((keys < 0) | (keys >= num_groups), torch.full_like(keys, num_groups), keys)
    perm = torch.sort(keys, stable=True).indices
    counts = torch.bincount(keys, minlength=num_groups + 1)[:num_groups]
    offsets = torch.zeros(num_groups + 1, dtype=torch.long)
    offsets[1:] = torch.cumsum(counts, 0)
    return perm, counts, offsets


def segment_build_bruteforce(keys, num_groups: int):
    """Same contract as :func:`segment_build_sort`, by explicit loops (tiny inputs)."""
    keys = [int(k) for k in torch.as_tensor(keys).reshape(-1).tolist()]
    perm, counts = [], []
    for g in range(num_groups):
        rows = [f for f, k in enumerate(keys) if k == g]
        counts.append(len(rows))
        perm.extend(rows)
    perm.extend(f for f, k in enumerate(keys) if k < 0 or k >= num_groups)  # rows without a group come last
    offsets = [0]
    for c in counts:
        offsets.append(offsets[-1] + c)
    return (torch.tensor(perm, dtype=torch.long), torch.tensor(counts, dtype=torch.long),
            torch.tensor(offsets, dtype=torch.long))


def flat_keys_from_topk(selected: torch.Tensor, tenant: torch.Tensor | None = None, num_tenants: int = 1):
    """Flat keys in the reference's row order ``f = k*T + t``.

    ``key = expert * num_tenants + tenant[t]``; ``num_tenants == 1`` reproduces
    the reference's plain expert grouping exactly.
    """
    if selected.dim() == 1:
        selected = selected[:, None]
    keys = selected.long() * num_tenants
    if tenant is not None:
        keys = keys + tenant.long()[:, None]
    return keys.t().contiguous().reshape(-1)


def unpermute(rows: torch.Tensor, routing_weights: torch.Tensor, out_shape, mapping: torch.Tensor,
              routing_map: torch.Tensor) -> torch.Tensor:
    """Weighted scatter-add of permuted rows back to token positions.

    Follows src/twinkle/model/transformers/moe/ep_utils.py:121-149 (and the
    identical tail at :280-287): the per-row weight is
    ``routing_weights.T.masked_select(routing_map)``, ``out`` starts at zero and
    duplicate token indices add.  ``routing_map`` is ``[G, T]`` (top-k slots
    already folded) and ``routing_weights`` is ``[T, G]``.
    """
    w = routing_weights.T.contiguous().masked_select(routing_map.bool())
    rows = rows * w.unsqueeze(-1)
    out = torch.zeros(out_shape, dtype=rows.dtype)
    out.scatter_add_(0, mapping.unsqueeze(1).expand(-1, out_shape[-1]), rows)
    return out


def unpermute_rows(rows: torch.Tensor, row_weight: torch.Tensor | None, row_token: torch.Tensor,
                   num_tokens: int) -> torch.Tensor:
    """``out[row_token[j]] += rows[j] * row_weight[j]`` with ``out`` zero-initialised.

    The per-row form of ep_utils.py:280-287 (``local_assignment_weights`` is
    already one weight per permuted row there).
    """
    out = torch.zeros(num_tokens, rows.shape[1], dtype=rows.dtype)
    src = rows if row_weight is None else rows * row_weight.unsqueeze(-1).to(rows.dtype)
    out.index_add_(0, row_token.long(), src)
    return out


def packed_cu_seqlens(position_ids: torch.Tensor) -> torch.Tensor:
    """Sequence starts of a packed batch followed by the total length, int32.

    Follows src/twinkle/processor/base.py:502-513.
    """
    if position_ids.dim() > 1 and position_ids.shape[0] > 1:
        position_ids = position_ids[:1]
    flat = position_ids.flatten()
    idx = torch.arange(flat.shape[0], dtype=torch.int32)
    return torch.cat([idx[flat == 0], torch.tensor(flat.shape, dtype=torch.int32)])


def token_ids_from_cu_seqlens(cu_seqlens: torch.Tensor, seq_group: torch.Tensor) -> torch.Tensor:
    """Per-token group id when sequence ``j`` (``cu[j]..cu[j+1]``) belongs to ``seq_group[j]``."""
    lens = cu_seqlens[1:].long() - cu_seqlens[:-1].long()
    return torch.repeat_interleave(seq_group.long(), lens)
