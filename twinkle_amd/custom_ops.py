"""``torch.ops.twinkle_amd.*``: the C-ABI entry points registered as torch custom ops.

The functions in :mod:`twinkle_amd.ops` and :mod:`twinkle_amd.segments` call the
shared library directly (lowest launch overhead, used by the autograd nodes and
the benchmark).  The same entry points are registered here with
``torch.library.custom_op`` so that graph-capturing front ends
(``torch.compile``, ``torch.export``) see opaque ops with declared mutation and
shape behaviour instead of ``ctypes`` calls.  Every op takes plain tensors and
integers; the pointer tables of an :class:`~twinkle_amd.ops.AdapterGroups` are
passed as the int64 / int32 / float32 device tensors it already holds.

    segment_build(keys, num_groups)                  -> segment workspace (uint8)
    lora_fwd(x, y, h, seg_ws, a_ptrs, b_ptrs, rank, scale, ...)         y, h written
    lora_bwd(dy, x, h, dx, grad_a, grad_b, grad_a_ptrs, grad_b_ptrs, ws, seg_ws, ...)
                                                     dx, grad_a, grad_b, ws written
    lora_fwd_shared(x, ys, hs, seg_ws, ...) / lora_bwd_shared(dys, x, hs, dx, ...)
                                                     the same for projections that share x (tensor lists)
    grouped_linear(x, weight, y, seg_ws, ...)        y written: packed experts' base GEMM (+ LoRA term from h)
"""
from __future__ import annotations

import ctypes
from typing import List

import torch

from . import _lib


def _desc(rows, in_features, out_features, max_rank, dtype, map_rows, seg_ws, a_ptrs, b_ptrs, lda, ldb, rank, scale):
    d = _lib.LoraDesc()
    d.rows = rows
    d.in_features = in_features
    d.out_features = out_features
    d.num_groups = rank.numel()
    d.max_rank = max_rank
    d.dtype = _lib.dtype_code(dtype)
    d.map_rows = 1 if map_rows else 0
    d.seg_ws = seg_ws.data_ptr()
    d.lora_A = a_ptrs.data_ptr()
    d.lora_B = b_ptrs.data_ptr()
    d.lda = lda
    d.ldb = ldb
    d.rank = rank.data_ptr()
    d.scale = scale.data_ptr()
    return d


def _need_gpu(t: torch.Tensor, name: str):
    if not t.is_cuda:
        raise RuntimeError(f'{name} must live on the GPU: this path has no CPU implementation')


@torch.library.custom_op('twinkle_amd::segment_build', mutates_args=())
def segment_build(keys: torch.Tensor, num_groups: int) -> torch.Tensor:
    """The device-side segment table of ``keys`` (flat int32 / int64 group ids), as raw bytes."""
    _need_gpu(keys, 'keys')
    keys = keys.reshape(-1).contiguous()
    lib = _lib.load()
    nbytes = lib.tk_segment_workspace_bytes(keys.numel(), num_groups)
    _lib.check(nbytes, 'tk_segment_workspace_bytes')
    ws = torch.empty(nbytes, dtype=torch.uint8, device=keys.device)
    code = lib.tk_segment_build(keys.data_ptr(), 0 if keys.dtype == torch.int32 else 1, keys.numel(), num_groups, None,
                                None, ws.data_ptr(), ws.numel(), _lib.stream_ptr())
    _lib.check(code, 'tk_segment_build')
    return ws


@segment_build.register_fake
def _(keys, num_groups):
    # the size is a pure host-side function of (rows, groups): exact also while tracing
    nbytes = _lib.load().tk_segment_workspace_bytes(keys.numel(), num_groups)
    _lib.check(nbytes, 'tk_segment_workspace_bytes')
    return keys.new_empty((nbytes,), dtype=torch.uint8)


@torch.library.custom_op('twinkle_amd::lora_fwd', mutates_args=('y', 'h'))
def lora_fwd(x: torch.Tensor, y: torch.Tensor, h: torch.Tensor, seg_ws: torch.Tensor, a_ptrs: torch.Tensor,
             b_ptrs: torch.Tensor, rank: torch.Tensor, scale: torch.Tensor, max_rank: int, lda: int, ldb: int,
             map_rows: bool) -> None:
    """``y[row] += scale_g (x[row] A_g^T) B_g^T`` in place; ``h`` receives the saved shrink output."""
    for t, n in ((x, 'x'), (y, 'y'), (h, 'h'), (seg_ws, 'seg_ws')):
        _need_gpu(t, n)
    d = _desc(x.shape[0], x.shape[1], y.shape[1], max_rank, x.dtype, map_rows, seg_ws, a_ptrs, b_ptrs, lda, ldb, rank,
              scale)
    need = _lib.load().tk_lora_h_bytes(ctypes.byref(d))
    _lib.check(need, 'tk_lora_h_bytes')
    if h.numel() * h.element_size() < need:
        raise ValueError(f'h holds {h.numel() * h.element_size()} bytes, {need} are needed')
    code = _lib.load().tk_lora_fwd(ctypes.byref(d), x.data_ptr(), x.stride(0), y.data_ptr(), y.stride(0),
                                   h.data_ptr(), _lib.stream_ptr())
    _lib.check(code, 'tk_lora_fwd')


@lora_fwd.register_fake
def _(x, y, h, seg_ws, a_ptrs, b_ptrs, rank, scale, max_rank, lda, ldb, map_rows):
    return None


@torch.library.custom_op('twinkle_amd::lora_bwd', mutates_args=('dx', 'grad_a', 'grad_b', 'workspace'))
def lora_bwd(dy: torch.Tensor, x: torch.Tensor, h: torch.Tensor, dx: torch.Tensor, grad_a: torch.Tensor,
             grad_b: torch.Tensor, grad_a_ptrs: torch.Tensor, grad_b_ptrs: torch.Tensor, workspace: torch.Tensor,
             seg_ws: torch.Tensor, a_ptrs: torch.Tensor,
             b_ptrs: torch.Tensor, rank: torch.Tensor, scale: torch.Tensor, max_rank: int, lda: int, ldb: int,
             map_rows: bool, accumulate: bool) -> None:
    """``dx += ...`` in place; dA / dB are written through ``grad_a_ptrs`` / ``grad_b_ptrs``.

    The pointer arrays (one device pointer per group) must point into ``grad_a`` / ``grad_b``, the flat
    gradient buffers: those two are only named here so that the mutation is visible to the tracer.
    """
    for t, n in ((dy, 'dy'), (x, 'x'), (h, 'h'), (dx, 'dx'), (workspace, 'workspace'), (seg_ws, 'seg_ws')):
        _need_gpu(t, n)
    d = _desc(dy.shape[0], x.shape[1], dy.shape[1], max_rank, dy.dtype, map_rows, seg_ws, a_ptrs, b_ptrs, lda, ldb,
              rank, scale)
    code = _lib.load().tk_lora_bwd(ctypes.byref(d), dy.data_ptr(), dy.stride(0), x.data_ptr(), x.stride(0),
                                   h.data_ptr(), dx.data_ptr(), dx.stride(0), grad_a_ptrs.data_ptr(),
                                   grad_b_ptrs.data_ptr(), 1 if accumulate else 0, workspace.data_ptr(),
                                   workspace.numel() * workspace.element_size(), _lib.stream_ptr())
    _lib.check(code, 'tk_lora_bwd')


@lora_bwd.register_fake
def _(dy, x, h, dx, grad_a, grad_b, grad_a_ptrs, grad_b_ptrs, workspace, seg_ws, a_ptrs, b_ptrs, rank, scale, max_rank,
      lda, ldb, map_rows, accumulate):
    return None


@torch.library.custom_op('twinkle_amd::grouped_linear', mutates_args=('y',))
def grouped_linear(x: torch.Tensor, weight: torch.Tensor, y: torch.Tensor, seg_ws: torch.Tensor,
                   groups_per_expert: int, num_groups: int, map_rows: bool, h: torch.Tensor, a_ptrs: torch.Tensor,
                   b_ptrs: torch.Tensor, rank: torch.Tensor, scale: torch.Tensor, max_rank: int, lda: int,
                   ldb: int) -> None:
    """``y[row] = x[row] @ weight[e].T (+ h[row] @ B_g.T)``, ``weight`` packed ``[E, out, in]`` (``tk_grouped_linear``).

    ``max_rank = 0`` leaves the LoRA term out; ``h`` and the adapter tables are then ignored (pass empty tensors).
    """
    for t, n in ((x, 'x'), (weight, 'weight'), (y, 'y'), (seg_ws, 'seg_ws')):
        _need_gpu(t, n)
    g = _lib.GroupedDesc()
    g.rows, g.num_groups, g.groups_per_expert = x.shape[0], num_groups, groups_per_expert
    g.in_features, g.out_features = weight.shape[2], weight.shape[1]
    g.dtype = _lib.dtype_code(weight.dtype)
    g.map_rows = 1 if map_rows else 0
    g.seg_ws = seg_ws.data_ptr()
    g.weight, g.weight_stride, g.ldw = weight.data_ptr(), weight.stride(0), weight.stride(1)
    lib = _lib.load()
    need = lib.tk_grouped_linear_workspace_bytes(ctypes.byref(g))
    _lib.check(need, 'tk_grouped_linear_workspace_bytes')
    ws = torch.empty(need, dtype=torch.uint8, device=x.device)
    d = None
    if max_rank > 0:
        d = ctypes.byref(_desc(x.shape[0], weight.shape[2], weight.shape[1], max_rank, x.dtype, map_rows, seg_ws,
                               a_ptrs, b_ptrs, lda, ldb, rank, scale))
    code = lib.tk_grouped_linear(ctypes.byref(g), d, x.data_ptr(), x.stride(0), y.data_ptr(), y.stride(0),
                                 h.data_ptr() if max_rank > 0 else None, ws.data_ptr(), ws.numel(), _lib.stream_ptr())
    _lib.check(code, 'tk_grouped_linear')


@grouped_linear.register_fake
def _(x, weight, y, seg_ws, groups_per_expert, num_groups, map_rows, h, a_ptrs, b_ptrs, rank, scale, max_rank, lda,
      ldb):
    return None


# ---- projections that share their input: one op for all of them -------------------------------------------------
# Per-projection tensors arrive as lists; `meta` holds (max_rank, lda, ldb) of every projection.

def _shared_descs(x, outs_like, seg_ws, a_ptrs, b_ptrs, rank, scale, meta, map_rows):
    descs = [_desc(x.shape[0], x.shape[1], o.shape[1], meta[3 * p], x.dtype, map_rows, seg_ws, a_ptrs[p], b_ptrs[p],
                   meta[3 * p + 1], meta[3 * p + 2], rank[p], scale[p]) for p, o in enumerate(outs_like)]
    table = (ctypes.c_void_p * len(descs))(*[ctypes.addressof(d) for d in descs])
    return descs, table


def _host(ctype, values):
    return (ctype * len(values))(*values)


@torch.library.custom_op('twinkle_amd::lora_fwd_shared', mutates_args=('ys', 'hs'))
def lora_fwd_shared(x: torch.Tensor, ys: List[torch.Tensor], hs: List[torch.Tensor], seg_ws: torch.Tensor,
                    a_ptrs: List[torch.Tensor], b_ptrs: List[torch.Tensor], rank: List[torch.Tensor],
                    scale: List[torch.Tensor], meta: List[int], map_rows: bool) -> None:
    """``ys[p][row] += scale (x[row] A_p^T) B_p^T`` for 1..4 projections that read the same ``x``; ``hs[p]``
    receives projection p's saved shrink output (``tk_lora_fwd_shared``)."""
    for t, n in ((x, 'x'), (seg_ws, 'seg_ws'), *((y, 'y') for y in ys), *((h, 'h') for h in hs)):
        _need_gpu(t, n)
    descs, table = _shared_descs(x, ys, seg_ws, a_ptrs, b_ptrs, rank, scale, meta, map_rows)
    code = _lib.load().tk_lora_fwd_shared(table, len(descs), x.data_ptr(), x.stride(0),
                                          _host(ctypes.c_void_p, [y.data_ptr() for y in ys]),
                                          _host(ctypes.c_int64, [y.stride(0) for y in ys]),
                                          _host(ctypes.c_void_p, [h.data_ptr() for h in hs]), _lib.stream_ptr())
    _lib.check(code, 'tk_lora_fwd_shared')


@lora_fwd_shared.register_fake
def _(x, ys, hs, seg_ws, a_ptrs, b_ptrs, rank, scale, meta, map_rows):
    return None


@torch.library.custom_op('twinkle_amd::lora_bwd_shared', mutates_args=('dx', 'grad_a', 'grad_b', 'workspaces'))
def lora_bwd_shared(dys: List[torch.Tensor], x: torch.Tensor, hs: List[torch.Tensor], dx: torch.Tensor,
                    grad_a: List[torch.Tensor], grad_b: List[torch.Tensor], grad_a_ptrs: List[torch.Tensor],
                    grad_b_ptrs: List[torch.Tensor], workspaces: List[torch.Tensor], seg_ws: torch.Tensor,
                    a_ptrs: List[torch.Tensor], b_ptrs: List[torch.Tensor], rank: List[torch.Tensor],
                    scale: List[torch.Tensor], meta: List[int], map_rows: bool, accumulate: bool) -> None:
    """``dx += sum_p dx_p`` in place and every projection's dA / dB through its pointer arrays, which point into
    ``grad_a[p]`` / ``grad_b[p]`` (``tk_lora_bwd_shared``)."""
    for t, n in ((x, 'x'), (dx, 'dx'), (seg_ws, 'seg_ws'), *((d, 'dy') for d in dys)):
        _need_gpu(t, n)
    descs, table = _shared_descs(x, dys, seg_ws, a_ptrs, b_ptrs, rank, scale, meta, map_rows)
    code = _lib.load().tk_lora_bwd_shared(
        table, len(descs), _host(ctypes.c_void_p, [d.data_ptr() for d in dys]),
        _host(ctypes.c_int64, [d.stride(0) for d in dys]), x.data_ptr(), x.stride(0),
        _host(ctypes.c_void_p, [h.data_ptr() for h in hs]), dx.data_ptr(), dx.stride(0),
        _host(ctypes.c_void_p, [t.data_ptr() for t in grad_a_ptrs]),
        _host(ctypes.c_void_p, [t.data_ptr() for t in grad_b_ptrs]), 1 if accumulate else 0,
        _host(ctypes.c_void_p, [w.data_ptr() for w in workspaces]),
        _host(ctypes.c_int64, [w.numel() * w.element_size() for w in workspaces]), _lib.stream_ptr())
    _lib.check(code, 'tk_lora_bwd_shared')


@lora_bwd_shared.register_fake
def _(dys, x, hs, dx, grad_a, grad_b, grad_a_ptrs, grad_b_ptrs, workspaces, seg_ws, a_ptrs, b_ptrs, rank, scale, meta,
      map_rows, accumulate):
    return None
