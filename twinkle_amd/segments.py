"""Segment table: rows grouped by adapter (or by (expert, tenant)), built on the GPU.

The table takes over what the reference does with a one-hot mask,
``masked_select`` and a host-side cumulative sum
(src/twinkle/model/transformers/moe/expert_parallel.py:254-255, :347-349;
src/twinkle/model/transformers/moe/ep_utils.py:99-118, :191), and is the
per-row form of ``MultiLora.adapter()``'s one-adapter-per-call selection
(src/twinkle/model/multi_lora.py:154-163).
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _lib


class SegmentTable:
    """Rows in stable group order.

    ``perm[j]`` is the flat row at sorted position ``j`` (for top-k routing the
    flat row of token ``t`` and slot ``k`` is ``k * num_tokens + t``, the
    reference's mask order) and ``offsets[g]:offsets[g+1]`` are the sorted
    positions of group ``g``; both int64 like the reference's tensors.
    ``workspace`` is the device-side table the kernels read.
    """

    def __init__(self, rows: int, num_groups: int, num_tokens: int, workspace: torch.Tensor,
                 perm: Optional[torch.Tensor], offsets: Optional[torch.Tensor]):
        self.rows = rows
        self.num_groups = num_groups
        self.num_tokens = num_tokens
        self.top_k = rows // num_tokens if num_tokens else 1
        self.workspace = workspace
        self.perm = perm
        self.offsets = offsets

    @property
    def device(self):
        return self.workspace.device

    @property
    def row_token(self) -> torch.Tensor:
        """Token index of each sorted row (``sorted_indices`` of ep_utils.py:113)."""
        return self.perm % self.num_tokens

    @property
    def counts(self) -> torch.Tensor:
        return self.offsets[1:] - self.offsets[:-1]

    def bad_keys(self) -> int:
        """Number of keys that were outside ``[0, num_groups)`` (synchronises)."""
        out = ctypes.c_int64(0)
        _lib.check(_lib.load().tk_segment_bad_keys(self.workspace.data_ptr(), _lib.stream_ptr(), ctypes.byref(out)),
                   'tk_segment_bad_keys')
        return out.value

    def validate(self) -> None:
        """Checks every array of the table on the host (``tk_segment_validate``: copies the table back, synchronises).
        ``ValueError`` naming the first failing check and index if the table is not one ``tk_segment_build`` writes."""
        check, index = ctypes.c_int32(0), ctypes.c_int64(-1)
        code = _lib.load().tk_segment_validate(self.workspace.data_ptr(), self.rows, self.num_groups, _lib.stream_ptr(),
                                               ctypes.byref(check), ctypes.byref(index))
        if code == _lib.TK_ERR_INVALID and check.value:
            names = {1: 'header', 2: 'offsets', 3: 'first tiles', 4: 'group of a tile', 5: 'slot rows / positions',
                     6: 'permutation and its inverse', 7: 'stable order', 8: 'walk orders', 9: 'chunks',
                     10: 'first chunks / partial slots'}
            raise ValueError(f'segment table fails check {check.value} ({names.get(check.value)}) at index {index.value}')
        _lib.check(code, 'tk_segment_validate')


def validate_segment_table(seg: SegmentTable) -> None:
    """See :meth:`SegmentTable.validate`."""
    seg.validate()


def build_segments(keys: torch.Tensor, num_groups: int, num_tokens: Optional[int] = None, want_perm: bool = True,
                   want_offsets: bool = True, check: bool = False) -> SegmentTable:
    """Group flat rows by ``keys`` (int32 or int64, on the GPU), stably.

    ``check=True`` raises ``ValueError`` for keys outside ``[0, num_groups)``
    (costs a device synchronisation; an index error in the reference).
    """
    if not keys.is_cuda:
        raise RuntimeError('build_segments needs keys on the GPU: this path has no CPU implementation')
    if keys.dtype not in (torch.int32, torch.int64):
        raise ValueError(f'keys must be int32 or int64, got {keys.dtype}')
    if num_groups <= 0:
        raise ValueError('num_groups must be positive')
    keys = keys.reshape(-1).contiguous()
    rows = keys.numel()
    num_tokens = rows if num_tokens is None else num_tokens
    if num_tokens and rows % num_tokens:
        raise ValueError(f'rows ({rows}) must be a multiple of num_tokens ({num_tokens})')
    lib = _lib.load()
    nbytes = lib.tk_segment_workspace_bytes(rows, num_groups)
    _lib.check(nbytes, 'tk_segment_workspace_bytes')
    ws = torch.empty(nbytes, dtype=torch.uint8, device=keys.device)
    perm = torch.empty(rows, dtype=torch.int64, device=keys.device) if want_perm else None
    offsets = torch.empty(num_groups + 1, dtype=torch.int64, device=keys.device) if want_offsets else None
    code = lib.tk_segment_build(keys.data_ptr() if rows else None, _lib.TK_KEY_I32 if keys.dtype == torch.int32 else
                                _lib.TK_KEY_I64, rows, num_groups, perm.data_ptr() if want_perm else None,
                                offsets.data_ptr() if want_offsets else None, ws.data_ptr(), nbytes, _lib.stream_ptr())
    _lib.check(code, 'tk_segment_build')
    table = SegmentTable(rows, num_groups, num_tokens, ws, perm, offsets)
    if check:
        bad = table.bad_keys()
        if bad:
            raise ValueError(f'{bad} keys outside [0, {num_groups})')
    return table


def flat_keys_from_topk(selected: torch.Tensor, tenant: Optional[torch.Tensor] = None,
                        num_tenants: int = 1) -> torch.Tensor:
    """Keys ``expert * num_tenants + tenant[t]`` in the reference's row order ``f = k * T + t``."""
    if selected.dim() == 1:
        selected = selected[:, None]
    keys = selected.to(torch.int32) * num_tenants
    if tenant is not None:
        keys = keys + tenant.to(torch.int32)[:, None]
    return keys.t().contiguous().reshape(-1)


def packed_cu_seqlens(position_ids: torch.Tensor) -> torch.Tensor:
    """Starts of the packed sequences plus the total length (int32).

    Same result as src/twinkle/processor/base.py:502-513.
    """
    if position_ids.dim() > 1 and position_ids.shape[0] > 1:
        position_ids = position_ids[:1]
    flat = position_ids.flatten()
    starts = torch.nonzero(flat == 0, as_tuple=False).flatten().to(torch.int32)
    total = torch.tensor([flat.shape[0]], dtype=torch.int32, device=flat.device)
    return torch.cat([starts, total])


def token_groups_from_sequences(cu_seqlens: torch.Tensor, seq_group: torch.Tensor) -> torch.Tensor:
    """Per-token group id when packed sequence ``j`` belongs to group ``seq_group[j]``."""
    lens = (cu_seqlens[1:] - cu_seqlens[:-1]).long()
    return torch.repeat_interleave(seq_group.to(torch.int32), lens)


# ---------------------------------------------------------------------------
# permute / unpermute with autograd (reference: ep_utils.py:99-149, :280-287)
# ---------------------------------------------------------------------------
def _rows_call(fn_name, a, ld_a, b, ld_b, w, seg: SegmentTable, width, dtype):
    lib = _lib.load()
    code = getattr(lib, fn_name)(a.data_ptr(), ld_a, b.data_ptr(), ld_b, w.data_ptr() if w is not None else None,
                                 seg.workspace.data_ptr(), seg.rows, seg.num_tokens, width, seg.num_groups,
                                 _lib.dtype_code(dtype), _lib.stream_ptr())
    _lib.check(code, fn_name)


def _check_2d(t: torch.Tensor, name: str):
    if t.dim() != 2 or t.stride(1) != 1 or not t.is_cuda:
        raise ValueError(f'{name} must be a 2-D GPU tensor with unit inner stride')


def _gather_rows(src, weights, seg):
    _check_2d(src, 'tokens')
    out = torch.empty(seg.rows, src.shape[1], dtype=src.dtype, device=src.device)
    if weights is not None:
        weights = weights.to(src.dtype).contiguous()
    _rows_call('tk_permute_rows', src, src.stride(0), out, out.stride(0), weights, seg, src.shape[1], src.dtype)
    return out


def _scatter_rows(rows, weights, seg):
    _check_2d(rows, 'rows')
    out = torch.empty(seg.num_tokens, rows.shape[1], dtype=rows.dtype, device=rows.device)
    if weights is not None:
        weights = weights.to(rows.dtype).contiguous()
    _rows_call('tk_unpermute_rows', rows, rows.stride(0), out, out.stride(0), weights, seg, rows.shape[1], rows.dtype)
    return out


class _Permute(torch.autograd.Function):

    @staticmethod
    def forward(ctx, tokens, seg):
        ctx.seg = seg
        return _gather_rows(tokens, None, seg)

    @staticmethod
    def backward(ctx, grad_rows):
        return _scatter_rows(grad_rows.contiguous(), None, ctx.seg), None


class _Unpermute(torch.autograd.Function):

    @staticmethod
    def forward(ctx, rows, weights, seg):
        ctx.seg = seg
        ctx.save_for_backward(rows, weights)
        return _scatter_rows(rows, weights, seg)

    @staticmethod
    def backward(ctx, grad_out):
        rows, weights = ctx.saved_tensors
        seg = ctx.seg
        grad_out = grad_out.contiguous()
        grad_rows = _gather_rows(grad_out, weights, seg) if ctx.needs_input_grad[0] else None
        grad_w = None
        if weights is not None and ctx.needs_input_grad[1]:
            dw = torch.empty(seg.num_tokens, seg.top_k, dtype=torch.float32, device=rows.device)
            lib = _lib.load()
            code = lib.tk_unpermute_weight_grad(grad_out.data_ptr(), grad_out.stride(0), rows.data_ptr(),
                                                rows.stride(0), dw.data_ptr(), seg.workspace.data_ptr(), seg.rows,
                                                seg.num_tokens, rows.shape[1], seg.num_groups,
                                                _lib.dtype_code(rows.dtype), _lib.stream_ptr())
            _lib.check(code, 'tk_unpermute_weight_grad')
            grad_w = dw.to(weights.dtype)
        return grad_rows, grad_w, None


def permute(tokens: torch.Tensor, seg: SegmentTable):
    """Rows of ``tokens [T, H]`` gathered into segment order; returns ``(rows, row_token)``.

    Same result as ``permute`` of ep_utils.py:99-118 when the table was built
    from the same routing (``num_tenants == 1``).
    """
    return _Permute.apply(tokens, seg), (seg.row_token if seg.perm is not None else None)


def unpermute(rows: torch.Tensor, routing_weights: Optional[torch.Tensor], seg: SegmentTable) -> torch.Tensor:
    """``out[t] = sum_k rows[pos(k, t)] * routing_weights[t, k]``.

    Same result as the zero-init + ``scatter_add_`` of ep_utils.py:121-149 /
    :280-287, with ``routing_weights`` given per selected slot ``[T, top_k]``
    and a fixed summation order (k ascending).
    """
    return _Unpermute.apply(rows, routing_weights, seg)
