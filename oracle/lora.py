"""Oracle: per-tenant LoRA linear forward/backward and expert (3-D) LoRA.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).
"""
from __future__ import annotations

import re
from typing import List, Optional, Sequence, Union

import torch
import torch.nn.functional as F


def lora_scaling(lora_alpha: float, r: int, use_rslora: bool = False) -> float:
    """``alpha / r`` or ``alpha / sqrt(r)``.

    Follows src/twinkle/model/multi_lora.py:318-319 and
    src/twinkle/model/multi_lora_target_parameters.py:152-156.
    """
    return lora_alpha / (r**0.5 if use_rslora else r)


def lora_linear_forward(x: torch.Tensor, base_out: torch.Tensor, lora_A: torch.Tensor, lora_B: torch.Tensor, r: int,
                        scaling: float) -> torch.Tensor:
    """One adapter on one call, exactly as the reference's patched forward runs it.

    Follows src/twinkle/model/multi_lora.py:303-327 with the slot's dropout
    being the identity (the slot config built at :490-495 has none):
    ``x`` is cast to the adapter weight dtype (:320), ``h = linear(x, A[:r])``
    (:322-323), ``u = linear(h, B[:, :r])`` (:324-325),
    ``result = base_out + u * scaling`` (:326) and the result is cast back to
    the base output dtype (:327).  ``lora_A`` is the full slot ``[max_r, K]``
    and ``lora_B`` the full slot ``[M, max_r]``.
    """
    result_dtype = base_out.dtype
    xa = x.to(lora_A.dtype)
    h = F.linear(xa, lora_A[:r, :], bias=None)
    u = F.linear(h, lora_B[:, :r], bias=None)
    result = base_out + u * scaling
    return result.to(result_dtype)


def multi_lora_linear(x: torch.Tensor, base_out: torch.Tensor, ids: torch.Tensor, lora_A: Sequence[torch.Tensor],
                      lora_B: Sequence[torch.Tensor], ranks: Sequence[int], scalings: Sequence[float]) -> torch.Tensor:
    """Batched multi-tenant result = each tenant's rows run alone with its adapter.

    The reference activates one adapter per call
    (src/twinkle/model/multi_lora.py:126-163); the batched path must give, for
    the rows of adapter ``g``, what :func:`lora_linear_forward` gives on those
    rows.  Rows whose id is negative or whose adapter has rank 0 keep the base
    output (the reference's skip rules at :308-313).
    Autograd through this function is the gradient oracle.
    """
    x2 = x.reshape(-1, x.shape[-1])
    y2 = base_out.reshape(-1, base_out.shape[-1])
    ids = ids.reshape(-1)
    out = y2.clone() if not y2.requires_grad else y2 + 0
    pieces = []
    index = []
    for g in range(len(lora_A)):
        rows = torch.nonzero(ids == g, as_tuple=False).flatten()
        if rows.numel() == 0 or ranks[g] == 0:
            continue
        yg = lora_linear_forward(x2.index_select(0, rows), y2.index_select(0, rows), lora_A[g], lora_B[g], ranks[g],
                                 scalings[g])
        pieces.append(yg)
        index.append(rows)
    if pieces:
        out = out.index_copy(0, torch.cat(index), torch.cat(pieces))
    return out.reshape(base_out.shape)


def multi_lora_linear_grads(x, base_out, ids, lora_A, lora_B, ranks, scalings, dy):
    """(Y, dX_lora, dA list, dB list) by autograd on :func:`multi_lora_linear`.

    ``dX_lora`` is the LoRA branch's contribution only (``base_out`` is treated
    as a constant), which is what the segmented backward adds onto the base
    GEMM's input gradient.  Gradients have full slot shape, zero beyond the
    tenant rank and for adapters with no rows.
    """
    xg = x.detach().clone().requires_grad_(True)
    A = [a.detach().clone().requires_grad_(True) for a in lora_A]
    B = [b.detach().clone().requires_grad_(True) for b in lora_B]
    y = multi_lora_linear(xg, base_out.detach(), ids, A, B, ranks, scalings)
    y.backward(dy.reshape(y.shape).to(y.dtype))
    zero = lambda t: torch.zeros_like(t)  # noqa: E731
    return (y.detach(), xg.grad if xg.grad is not None else zero(xg), [a.grad if a.grad is not None else zero(a) for a in A],
            [b.grad if b.grad is not None else zero(b) for b in B])


def expert_delta_weight(lora_A: torch.Tensor, lora_B: torch.Tensor, r: int, scaling: float,
                        out_in_layout: bool = True) -> torch.Tensor:
    """Merged ΔW for packed experts.

    Follows src/twinkle/model/multi_lora_target_parameters.py:158-179:
    ``einsum('e o r, e r i -> e o i', B[:, :, :r], A[:, :r, :]) * scaling`` when
    the module stores ``[E, out, in]`` (``out_in_layout``), ``-> e i o``
    otherwise.  ``lora_A`` is ``[E, max_r, in]``, ``lora_B`` is ``[E, out, max_r]``.
    """
    wa = lora_A[:, :r, :]
    wb = lora_B[:, :, :r]
    if out_in_layout:
        return torch.einsum('eor,eri->eoi', wb, wa) * scaling
    return torch.einsum('eor,eri->eio', wb, wa) * scaling


def experts_linear(x_sorted: torch.Tensor, offsets: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``y_e = F.linear(x_e, weight[e])`` over the contiguous per-expert chunks of rows in expert order.

    Follows src/twinkle/model/transformers/moe/expert_parallel.py:347-371 (one ``F.linear`` per projection per
    expert, empty experts skipped, chunks concatenated); ``offsets`` is the ``cumsum`` of :347-349,
    ``weight`` the packed ``[E, out, in]`` parameter (``gate_up_proj`` or ``down_proj``).
    """
    chunks = []
    for e in range(weight.shape[0]):
        s, t = int(offsets[e]), int(offsets[e + 1])
        chunks.append(F.linear(x_sorted[s:t], weight[e]))
    return torch.cat(chunks, dim=0) if chunks else x_sorted.new_empty(0, weight.shape[1])


def swiglu(gate_up: torch.Tensor) -> torch.Tensor:
    """``act_fn(gate) * up`` with ``gate, up = gate_up.chunk(2, dim=-1)`` and ``act_fn = SiLU``.

    Follows src/twinkle/model/transformers/moe/expert_parallel.py:363-366 (the branch without ``_apply_gate``).
    """
    gate, up = gate_up.chunk(2, dim=-1)
    return F.silu(gate) * up


def expert_lora_low_rank(x_sorted: torch.Tensor, offsets: torch.Tensor, base_out: torch.Tensor, lora_A: torch.Tensor,
                         lora_B: torch.Tensor, r: int, scaling: float) -> torch.Tensor:
    """``y_e = base_e + s (x_e A_e^T) B_e^T`` over contiguous per-expert chunks.

    The chunked per-expert loop follows
    src/twinkle/model/transformers/moe/expert_parallel.py:347-371; the low-rank
    form is the algebraic expansion of running that loop on ``W + ΔW`` with ΔW
    from :func:`expert_delta_weight`.
    """
    out = base_out.clone()
    for e in range(lora_A.shape[0]):
        s, t = int(offsets[e]), int(offsets[e + 1])
        if s == t:
            continue
        h = F.linear(x_sorted[s:t], lora_A[e, :r, :])
        out[s:t] = out[s:t] + F.linear(h, lora_B[e, :, :r]) * scaling
    return out


def slice_rank_tensor(name: str, tensor: Optional[torch.Tensor], rank: int):
    """Live sub-block of a slot tensor.  Follows src/twinkle/model/multi_lora.py:85-97."""
    if tensor is None:
        return None
    if 'embedding_A' in name:
        return tensor[:, :rank]
    if 'embedding_B' in name:
        return tensor[:rank, :]
    if '_A' in name:
        return tensor[:rank, :]
    if '_B' in name:
        return tensor[:, :rank]
    return tensor


def copy_rank_tensor(name: str, target: Optional[torch.Tensor], value: Optional[torch.Tensor]):
    """Copy a rank-sliced tensor into the prefix of a slot.  Follows multi_lora.py:99-113."""
    if target is None or value is None:
        return None
    if 'embedding_A' in name:
        target[:, :value.shape[1]].copy_(value)
    elif 'embedding_B' in name:
        target[:value.shape[0], :].copy_(value)
    elif '_A' in name:
        target[:value.shape[0], :].copy_(value)
    elif '_B' in name:
        target[:, :value.shape[1]].copy_(value)
    else:
        target.copy_(value)
    return target


def match_target_modules(module_name: str, target_modules: Optional[Union[List[str], str]]) -> bool:
    """Whether a tenant's ``target_modules`` selects a layer.  Follows multi_lora.py:256-287."""
    if target_modules is None:
        return False
    if isinstance(target_modules, (list, set)) and len(target_modules) == 0:
        return False
    if isinstance(target_modules, (list, set)) and len(target_modules) == 1 and next(iter(target_modules)) == 'all-linear':
        return True
    if target_modules == 'all-linear':
        return True
    cleaned = module_name
    if '.lora_' in module_name:
        cleaned = re.sub(r'\.lora_\w+(\.[\w-]+)*$', '', module_name)
    if isinstance(target_modules, str):
        return re.fullmatch(target_modules, cleaned) is not None
    if isinstance(target_modules, (list, set)):
        return any(cleaned.endswith(t) for t in target_modules)
    return False
