"""Segmented multi-LoRA linear: torch custom ops over the C ABI, plus autograd.

``y[row] += scale_g * (x[row] A_g^T) B_g^T`` for every adapter ``g`` of a mixed
batch in one pass, and the matching backward.  For the rows of one adapter this
is what the reference's patched forward computes with two ``F.linear`` calls
(src/twinkle/model/multi_lora.py:315-326) and what autograd derives from them.
"""
from __future__ import annotations

import ctypes
import os
from typing import List, Optional, Sequence, Tuple

import torch

from . import _lib
from .segments import SegmentTable


class AdapterGroups:
    """Which weight block, rank and scale every group of a layer uses.

    ``a_tensors`` / ``b_tensors`` are the caller-owned parameters (slot tensors
    ``[max_r, K]`` / ``[M, max_r]``, or packed expert tensors ``[E, max_r, K]`` /
    ``[E, M, max_r]``).  Group ``g`` reads ``a_tensors[a_index[g]]`` starting
    ``a_offset[g]`` elements in (likewise for B); the defaults give one tensor
    per group.  Only pointers are kept: the parameters stay where they are.
    """

    def __init__(self, a_tensors: Sequence[torch.Tensor], b_tensors: Sequence[torch.Tensor], ranks: Sequence[int],
                 scales: Sequence[float], a_index: Optional[Sequence[int]] = None,
                 a_offset: Optional[Sequence[int]] = None, b_index: Optional[Sequence[int]] = None,
                 b_offset: Optional[Sequence[int]] = None, master_a: Optional[Sequence[torch.Tensor]] = None,
                 master_b: Optional[Sequence[torch.Tensor]] = None, act_dtype: Optional[torch.dtype] = None,
                 rank_classes: Optional[bool] = None):
        self.a_tensors = list(a_tensors)
        self.b_tensors = list(b_tensors)
        # mixed precision: the kernels read `a_tensors` / `b_tensors` (compute copies, e.g. bf16) while the
        # parameters autograd knows are `master_a` / `master_b` (same shapes, e.g. fp32)
        self.master_a = list(master_a) if master_a is not None else None
        self.master_b = list(master_b) if master_b is not None else None
        if (self.master_a is None) != (self.master_b is None):
            raise ValueError('master_a and master_b come together')
        if self.master_a is not None and ([t.shape for t in self.master_a] != [t.shape for t in self.a_tensors] or
                                          [t.shape for t in self.master_b] != [t.shape for t in self.b_tensors]):
            raise ValueError('master tensors must have the shapes of the compute copies')
        self.num_groups = len(ranks)
        if self.num_groups == 0:
            raise ValueError('at least one group is needed')
        g = self.num_groups
        self.a_index = list(a_index) if a_index is not None else list(range(g))
        self.b_index = list(b_index) if b_index is not None else list(range(g))
        self.a_offset = list(a_offset) if a_offset is not None else [0] * g
        self.b_offset = list(b_offset) if b_offset is not None else [0] * g
        self.ranks = [int(r) for r in ranks]
        self.scales = [float(s) for s in scales]
        if not (len(self.a_index) == len(self.b_index) == len(self.a_offset) == len(self.b_offset) == len(self.scales)
                == g):
            raise ValueError('per-group lists must have one entry per group')
        a0, b0 = self.a_tensors[0], self.b_tensors[0]
        # `dtype` is the element type of x, y and h; the adapters' own type differs from it in one supported case:
        # fp32 adapters under bf16 activations (tk_lora_desc::weights_f32: the library converts the weights on the
        # fly and writes fp32 gradients)
        self.weight_dtype = a0.dtype
        self.dtype = act_dtype if act_dtype is not None else a0.dtype
        if self.dtype != self.weight_dtype and (self.dtype, self.weight_dtype) != (torch.bfloat16, torch.float32):
            raise ValueError(f'adapters of {self.weight_dtype} under activations of {self.dtype} are not supported')
        self.weights_f32 = self.dtype != self.weight_dtype
        self.device = a0.device
        self.in_features = a0.shape[-1]
        self.out_features = b0.shape[-2]
        self.lda = a0.stride(-2)
        self.ldb = b0.stride(-2)
        for t in self.a_tensors:
            if t.dtype != self.weight_dtype or t.shape[-1] != self.in_features or t.stride(-1) != 1 or \
                    t.stride(-2) != self.lda:
                raise ValueError('all lora_A tensors of a layer must share dtype, width and row stride')
        for t in self.b_tensors:
            if t.dtype != self.weight_dtype or t.shape[-2] != self.out_features or t.stride(-1) != 1 or \
                    t.stride(-2) != self.ldb:
                raise ValueError('all lora_B tensors of a layer must share dtype, height and row stride')
        self.max_rank = max(self.ranks)
        if self.max_rank > _lib.TK_MAX_RANK:
            raise RuntimeError(f'Too big rank for lora: {self.max_rank}')
        # Which padded ranks (16 / 32 / 64 / 128) occur among the live groups (tk_lora_desc::rank_classes).  With
        # more than one of them the backward runs every class of groups on the kernels of its own padded rank, the
        # classes side by side on streams of the library, and only the groups above rank 32 take the two-pass
        # backward (32 adapters of ranks 8 / 16 / 32 / 64 at 4096 -> 14336: backward 645 against 741 us).  The forward
        # is the same either way.  rank_classes=False pads every group to the largest rank in the backward too.
        mask = 0
        for r in self.ranks:
            if r > 0:
                mask |= 1 if r <= 16 else 2 if r <= 32 else 4 if r <= 64 else 8
        if rank_classes is None:
            rank_classes = os.environ.get('TK_RANK_CLASSES', '1') != '0'
        self.rank_classes = mask if (rank_classes and mask & (mask - 1)) else 0
        for i, r in enumerate(self.ranks):
            if r < 0 or r > self.a_tensors[self.a_index[i]].shape[-2] or r > self.b_tensors[self.b_index[i]].shape[-1]:
                raise RuntimeError(f'Too big rank for lora: {r}')
        dev = self.device
        self.rank_dev = torch.tensor(self.ranks, dtype=torch.int32, device=dev)
        self.scale_dev = torch.tensor(self.scales, dtype=torch.float32, device=dev)
        # gradient arena: one flat buffer per side, every live tensor at a fixed element offset.  A tensor is live
        # when a group of positive rank reads it; the others (free slots, tenants that do not target this layer or
        # are not part of the batch) get no gradient at all, like the adapters the reference leaves inactive.
        self.a_live = [False] * len(self.a_tensors)
        self.b_live = [False] * len(self.b_tensors)
        for i, r in enumerate(self.ranks):
            if r > 0:
                self.a_live[self.a_index[i]] = True
                self.b_live[self.b_index[i]] = True
        self._a_arena_off, self.a_arena_elems = self._arena(self.a_tensors, self.a_live)
        self._b_arena_off, self.b_arena_elems = self._arena(self.b_tensors, self.b_live)
        esz = a0.element_size()
        self._grad_a_rel = torch.tensor([(self._a_arena_off[self.a_index[i]] + self.a_offset[i]) * esz
                                         for i in range(g)], dtype=torch.int64, device=dev)
        self._grad_b_rel = torch.tensor([(self._b_arena_off[self.b_index[i]] + self.b_offset[i]) * esz
                                         for i in range(g)], dtype=torch.int64, device=dev)
        self._ptr_key = None
        self._size_cache = {}
        self._desc_template = self._desc_key = None
        self.a_ptrs = self.b_ptrs = None
        self.refresh()

    @staticmethod
    def _arena(tensors, live):
        offs, total = [], 0
        for t, keep in zip(tensors, live):
            offs.append(total if keep else 0)     # groups of rank 0 are never written: any offset will do
            if keep:
                total += (t.numel() + 127) // 128 * 128
        return offs, total

    def refresh(self) -> None:
        """Rebuild the device pointer arrays if a parameter's storage moved."""
        key = [t.data_ptr() for t in self.a_tensors] + [t.data_ptr() for t in self.b_tensors]
        if key == self._ptr_key:
            return
        esz = self.a_tensors[0].element_size()
        g = self.num_groups
        self.a_ptrs = torch.tensor([self.a_tensors[self.a_index[i]].data_ptr() + self.a_offset[i] * esz
                                    for i in range(g)], dtype=torch.int64, device=self.device)
        self.b_ptrs = torch.tensor([self.b_tensors[self.b_index[i]].data_ptr() + self.b_offset[i] * esz
                                    for i in range(g)], dtype=torch.int64, device=self.device)
        self._ptr_key = key

    def grad_views(self, arena: torch.Tensor, side: str) -> List[Optional[torch.Tensor]]:
        """Per-tensor views of a gradient arena; ``None`` for tensors no live group reads."""
        tensors, offs, live = (self.a_tensors, self._a_arena_off, self.a_live) if side == 'a' else \
            (self.b_tensors, self._b_arena_off, self.b_live)
        masters = self.master_a if side == 'a' else self.master_b
        if masters is not None and masters[0].dtype != arena.dtype:
            arena = arena.to(masters[0].dtype)        # one cast for the whole side; the views below share it
        return [arena[o:o + t.numel()].view(t.shape) if keep else None for t, o, keep in zip(tensors, offs, live)]

    def autograd_tensors(self) -> List[torch.Tensor]:
        """The tensors gradients are reported for: the masters where there are any, else the tensors read."""
        if self.master_a is not None:
            return self.master_a + self.master_b
        return self.a_tensors + self.b_tensors

    def sync_masters(self) -> None:
        """Refresh the compute copies from the masters (two multi-tensor copies, whatever changed the masters)."""
        if self.master_a is not None:
            with torch.no_grad():
                torch._foreach_copy_(self.a_tensors + self.b_tensors, self.master_a + self.master_b)


def _desc(seg: SegmentTable, groups: AdapterGroups, map_rows: bool) -> _lib.LoraDesc:
    groups.refresh()
    # a fresh struct per call (callers keep several alive at once), copied from a template that holds everything
    # which is fixed for the AdapterGroups object
    template = groups._desc_template
    if template is None or groups._desc_key is not groups._ptr_key:
        template = _lib.LoraDesc()
        template.in_features = groups.in_features
        template.out_features = groups.out_features
        template.num_groups = groups.num_groups
        template.max_rank = groups.max_rank
        template.dtype = _lib.dtype_code(groups.dtype)
        template.lora_A = groups.a_ptrs.data_ptr()
        template.lora_B = groups.b_ptrs.data_ptr()
        template.lda = groups.lda
        template.ldb = groups.ldb
        template.rank = groups.rank_dev.data_ptr()
        template.scale = groups.scale_dev.data_ptr()
        template.weights_f32 = 1 if groups.weights_f32 else 0
        template.rank_classes = groups.rank_classes
        groups._desc_template, groups._desc_key = template, groups._ptr_key
    d = _lib.LoraDesc.from_buffer_copy(template)
    d.rows = seg.rows
    d.map_rows = 1 if map_rows else 0
    d.seg_ws = seg.workspace.data_ptr()
    return d


def _check_rows(t: torch.Tensor, name: str, rows: int, width: int, dtype: torch.dtype):
    if not t.is_cuda:
        raise RuntimeError(f'{name} must live on the GPU: this path has no CPU implementation')
    if t.dim() != 2 or t.shape[0] != rows or t.shape[1] != width or t.stride(1) != 1:
        raise ValueError(f'{name} must be [{rows}, {width}] with unit inner stride, got {tuple(t.shape)} '
                         f'strides {t.stride()}')
    if t.dtype != dtype:
        raise ValueError(f'{name} has dtype {t.dtype}, adapters have {dtype}')


def _cached_size(seg: SegmentTable, groups: AdapterGroups, which: str) -> int:
    # both sizes are functions of the shapes alone (rows, groups, widths, padded rank, dtype), all of which are
    # fixed for an AdapterGroups object except the row count
    key = (which, seg.rows)
    n = groups._size_cache.get(key)
    if n is None:
        n = getattr(_lib.load(), which)(ctypes.byref(_desc(seg, groups, True)))
        _lib.check(n, which)
        if len(groups._size_cache) > 64:
            groups._size_cache.clear()
        groups._size_cache[key] = n
    return n


def lora_h_bytes(seg: SegmentTable, groups: AdapterGroups) -> int:
    return _cached_size(seg, groups, 'tk_lora_h_bytes')


def lora_bwd_workspace_bytes(seg: SegmentTable, groups: AdapterGroups) -> int:
    return _cached_size(seg, groups, 'tk_lora_bwd_workspace_bytes')


def lora_h_saved_bytes(seg: SegmentTable, groups: AdapterGroups) -> int:
    """The part of ``h`` the backward reads.  With fp32 adapters under bf16 activations the forward also keeps its
    bf16 copies of A and B in the tail of ``h`` (``G * rpad * (K + M)`` elements); the backward makes its own copies
    from the fp32 matrices, so that tail need not stay alive between forward and backward."""
    if not groups.weights_f32:
        return lora_h_bytes(seg, groups)
    key = ('h_saved', seg.rows)
    n = groups._size_cache.get(key)
    if n is None:
        d = _desc(seg, groups, True)
        d.weights_f32 = 0
        n = _lib.load().tk_lora_h_bytes(ctypes.byref(d))
        _lib.check(n, 'tk_lora_h_bytes')
        groups._size_cache[key] = n
    return n


def _h_for_backward(h: torch.Tensor, seg: SegmentTable, groups: AdapterGroups) -> torch.Tensor:
    # fp32 adapters: keep a copy of what the backward reads and let the staged weight copies go with the forward's buffer
    if not groups.weights_f32:
        return h
    return h[:lora_h_saved_bytes(seg, groups)].clone()


def lora_fwd_(x: torch.Tensor, y: torch.Tensor, seg: SegmentTable, groups: AdapterGroups, map_rows: bool = True,
              h: Optional[torch.Tensor] = None) -> torch.Tensor:
    """In place ``y += lora(x)``; returns the saved shrink output ``h`` (opaque bytes)."""
    if groups.num_groups != seg.num_groups:
        raise ValueError(f'segment table has {seg.num_groups} groups, adapters have {groups.num_groups}')
    _check_rows(x, 'x', seg.rows, groups.in_features, groups.dtype)
    _check_rows(y, 'y', seg.rows, groups.out_features, groups.dtype)
    d = _desc(seg, groups, map_rows)
    lib = _lib.load()
    if h is None:
        h = torch.empty(lora_h_bytes(seg, groups), dtype=torch.uint8, device=x.device)
    code = lib.tk_lora_fwd(ctypes.byref(d), x.data_ptr(), x.stride(0), y.data_ptr(), y.stride(0), h.data_ptr(),
                           _lib.stream_ptr())
    _lib.check(code, 'tk_lora_fwd')
    return h


def lora_fwd_noalloc_(x: torch.Tensor, y: torch.Tensor, seg: SegmentTable, groups: AdapterGroups,
                      map_rows: bool = True) -> None:
    """In place ``y += lora(x)`` like :func:`lora_fwd_`, without any device allocation (``tk_lora_fwd_noalloc``):
    the shrink output goes to a buffer the library holds per GPU, so there is no backward after this call.
    ``RuntimeError`` when the problem needs more than ``_lib.TK_NOALLOC_SCRATCH_BYTES``; calls that may overlap on
    one GPU race on that buffer and must be ordered on one stream."""
    if groups.num_groups != seg.num_groups:
        raise ValueError(f'segment table has {seg.num_groups} groups, adapters have {groups.num_groups}')
    _check_rows(x, 'x', seg.rows, groups.in_features, groups.dtype)
    _check_rows(y, 'y', seg.rows, groups.out_features, groups.dtype)
    d = _desc(seg, groups, map_rows)
    code = _lib.load().tk_lora_fwd_noalloc(ctypes.byref(d), x.data_ptr(), x.stride(0), y.data_ptr(), y.stride(0),
                                           _lib.stream_ptr())
    _lib.check(code, 'tk_lora_fwd_noalloc')


def lora_shrink_(x: torch.Tensor, seg: SegmentTable, groups: AdapterGroups, h: torch.Tensor,
                 map_rows: bool = True) -> None:
    """First half of :func:`lora_fwd_`: ``h = scale * x A^T`` (see ``tk_lora_shrink``)."""
    _check_rows(x, 'x', seg.rows, groups.in_features, groups.dtype)
    d = _desc(seg, groups, map_rows)
    _lib.check(_lib.load().tk_lora_shrink(ctypes.byref(d), x.data_ptr(), x.stride(0), h.data_ptr(), _lib.stream_ptr()),
               'tk_lora_shrink')


def lora_expand_(h: torch.Tensor, y: torch.Tensor, seg: SegmentTable, groups: AdapterGroups,
                 map_rows: bool = True) -> None:
    """Second half of :func:`lora_fwd_`: ``y += h B^T`` in place (see ``tk_lora_expand``)."""
    _check_rows(y, 'y', seg.rows, groups.out_features, groups.dtype)
    d = _desc(seg, groups, map_rows)
    _lib.check(_lib.load().tk_lora_expand(ctypes.byref(d), h.data_ptr(), y.data_ptr(), y.stride(0), _lib.stream_ptr()),
               'tk_lora_expand')


def lora_bwd_(dy: torch.Tensor, x: Optional[torch.Tensor], h: Optional[torch.Tensor], dx: Optional[torch.Tensor],
              grad_a_ptrs: Optional[torch.Tensor], grad_b_ptrs: Optional[torch.Tensor], seg: SegmentTable,
              groups: AdapterGroups, map_rows: bool = True, accumulate: bool = False,
              workspace: Optional[torch.Tensor] = None) -> None:
    """``dx += ...`` in place, weight gradients through the pointer arrays (see ``tk_lora_bwd``)."""
    _check_rows(dy, 'dy', seg.rows, groups.out_features, groups.dtype)
    if x is not None:
        _check_rows(x, 'x', seg.rows, groups.in_features, groups.dtype)
    if dx is not None:
        _check_rows(dx, 'dx', seg.rows, groups.in_features, groups.dtype)
    d = _desc(seg, groups, map_rows)
    lib = _lib.load()
    if workspace is None:
        workspace = torch.empty(lora_bwd_workspace_bytes(seg, groups), dtype=torch.uint8, device=dy.device)
    code = lib.tk_lora_bwd(ctypes.byref(d), dy.data_ptr(), dy.stride(0), x.data_ptr() if x is not None else None,
                           x.stride(0) if x is not None else 0, h.data_ptr() if h is not None else None,
                           dx.data_ptr() if dx is not None else None, dx.stride(0) if dx is not None else 0,
                           grad_a_ptrs.data_ptr() if grad_a_ptrs is not None else None,
                           grad_b_ptrs.data_ptr() if grad_b_ptrs is not None else None, 1 if accumulate else 0,
                           workspace.data_ptr(), workspace.numel(), _lib.stream_ptr())
    _lib.check(code, 'tk_lora_bwd')


def grouped_linear_(x: torch.Tensor, weight: torch.Tensor, seg: SegmentTable, groups_per_expert: int = 1,
                    y: Optional[torch.Tensor] = None, groups: Optional[AdapterGroups] = None,
                    h: Optional[torch.Tensor] = None, map_rows: bool = False,
                    workspace: Optional[torch.Tensor] = None, transposed: bool = False) -> torch.Tensor:
    """``y[row] = x[row] @ weight[e].T (+ h[row] @ B_g.T)`` for every row of the table, ``e = g // groups_per_expert``
    (see ``tk_grouped_linear``).  ``weight`` is packed ``[E, out, in]``; with ``groups`` the LoRA term of the
    (expert, tenant) groups is added on the accumulators, from ``h`` as :func:`lora_shrink_` left it.
    ``transposed=True`` computes ``y[row] = x[row] @ weight[e]`` instead (``weight [E, in, out]``): the backward of
    the plain call on the same weights."""
    if not (x.is_cuda and weight.is_cuda):
        raise RuntimeError('x and weight must live on the GPU: this path has no CPU implementation')
    if weight.dim() != 3 or weight.stride(2) != 1 or weight.dtype != x.dtype:
        raise ValueError('weight must be [experts, out, in] with unit inner stride and the dtype of x')
    if transposed and groups is not None:
        raise ValueError('the LoRA term goes with the plain call, not with transposed=True')
    experts, out_f, in_f = weight.shape
    if transposed:
        out_f, in_f = in_f, out_f
    if seg.num_groups != experts * groups_per_expert:
        raise ValueError(f'segment table has {seg.num_groups} groups, weights give {experts} x {groups_per_expert}')
    _check_rows(x, 'x', seg.rows, in_f, weight.dtype)
    if y is None:
        y = torch.empty(seg.rows, out_f, dtype=x.dtype, device=x.device)
    _check_rows(y, 'y', seg.rows, out_f, weight.dtype)
    g = _lib.GroupedDesc()
    g.rows, g.num_groups, g.groups_per_expert = seg.rows, seg.num_groups, groups_per_expert
    g.in_features, g.out_features = in_f, out_f
    g.dtype = _lib.dtype_code(weight.dtype)
    g.map_rows = 1 if map_rows else 0
    g.seg_ws = seg.workspace.data_ptr()
    g.weight, g.weight_stride, g.ldw = weight.data_ptr(), weight.stride(0), weight.stride(1)
    g.weight_layout = 1 if transposed else 0
    lib = _lib.load()
    if workspace is None:
        n = lib.tk_grouped_linear_workspace_bytes(ctypes.byref(g))
        _lib.check(n, 'tk_grouped_linear_workspace_bytes')
        workspace = torch.empty(n, dtype=torch.uint8, device=x.device)
    d = None
    if groups is not None:
        if h is None:
            raise ValueError('the LoRA term needs the h that lora_shrink_ wrote')
        if groups.num_groups != seg.num_groups or groups.in_features != in_f or groups.out_features != out_f:
            raise ValueError('adapters and weights describe different layers')
        d = ctypes.byref(_desc(seg, groups, map_rows))
    code = lib.tk_grouped_linear(ctypes.byref(g), d, x.data_ptr(), x.stride(0), y.data_ptr(), y.stride(0),
                                 h.data_ptr() if h is not None else None, workspace.data_ptr(), workspace.numel(),
                                 _lib.stream_ptr())
    _lib.check(code, 'tk_grouped_linear')
    return y


def _weight_grads(ctx_groups: AdapterGroups, needs_a: bool, needs_b: bool, device):
    groups = ctx_groups
    arena_a = arena_b = pa = pb = None
    if needs_a:
        arena_a = torch.zeros(groups.a_arena_elems, dtype=groups.weight_dtype, device=device)
        pa = groups._grad_a_rel + arena_a.data_ptr()
    if needs_b:
        arena_b = torch.zeros(groups.b_arena_elems, dtype=groups.weight_dtype, device=device)
        pb = groups._grad_b_rel + arena_b.data_ptr()
    return arena_a, arena_b, pa, pb


class _LoraDelta(torch.autograd.Function):
    """``y`` (base output) updated in place; gradients for ``x``, ``y`` and every adapter tensor."""

    @staticmethod
    def forward(ctx, x, y, seg, groups, map_rows, *weights):
        h = _h_for_backward(lora_fwd_(x, y, seg, groups, map_rows), seg, groups)
        ctx.mark_dirty(y)
        ctx.save_for_backward(x, h)
        ctx.seg, ctx.groups, ctx.map_rows = seg, groups, map_rows
        return y

    @staticmethod
    def backward(ctx, dy):
        x, h = ctx.saved_tensors
        seg, groups = ctx.seg, ctx.groups
        dy = dy.contiguous()
        na, nb = len(groups.a_tensors), len(groups.b_tensors)
        needs_a = any(ctx.needs_input_grad[5:5 + na])
        needs_b = any(ctx.needs_input_grad[5 + na:5 + na + nb])
        dx = torch.zeros_like(x) if ctx.needs_input_grad[0] else None
        arena_a, arena_b, pa, pb = _weight_grads(groups, needs_a, needs_b, dy.device)
        lora_bwd_(dy, x, h, dx, pa, pb, seg, groups, ctx.map_rows, accumulate=False)
        ga = groups.grad_views(arena_a, 'a') if needs_a else [None] * na
        gb = groups.grad_views(arena_b, 'b') if needs_b else [None] * nb
        return (dx, dy, None, None, None, *ga, *gb)


class _LoraLinear(torch.autograd.Function):
    """Base ``F.linear`` and the LoRA update as one node: ``dx`` of the base GEMM is updated in place."""

    @staticmethod
    def forward(ctx, x, weight, bias, seg, groups, map_rows, *weights):
        y = torch.nn.functional.linear(x, weight, bias)
        h = _h_for_backward(lora_fwd_(x, y, seg, groups, map_rows), seg, groups)
        ctx.save_for_backward(x, weight, h)
        ctx.has_bias = bias is not None
        ctx.seg, ctx.groups, ctx.map_rows = seg, groups, map_rows
        return y

    @staticmethod
    def backward(ctx, dy):
        x, weight, h = ctx.saved_tensors
        seg, groups = ctx.seg, ctx.groups
        dy = dy.contiguous()
        na, nb = len(groups.a_tensors), len(groups.b_tensors)
        needs_a = any(ctx.needs_input_grad[6:6 + na])
        needs_b = any(ctx.needs_input_grad[6 + na:6 + na + nb])
        dx = dy @ weight if ctx.needs_input_grad[0] else None
        dw = dy.t() @ x if ctx.needs_input_grad[1] else None
        db = dy.sum(0) if ctx.has_bias and ctx.needs_input_grad[2] else None
        arena_a, arena_b, pa, pb = _weight_grads(groups, needs_a, needs_b, dy.device)
        lora_bwd_(dy, x, h, dx, pa, pb, seg, groups, ctx.map_rows, accumulate=False)
        ga = groups.grad_views(arena_a, 'a') if needs_a else [None] * na
        gb = groups.grad_views(arena_b, 'b') if needs_b else [None] * nb
        return (dx, dw, db, None, None, None, *ga, *gb)


class _SwiGLU(torch.autograd.Function):
    """``silu(gate) * up`` for ``gate | up`` side by side in the rows of one tensor (see ``tk_swiglu_fwd``)."""

    @staticmethod
    def forward(ctx, gate_up):
        rows, two_i = gate_up.shape
        inter = two_i // 2
        out = torch.empty(rows, inter, dtype=gate_up.dtype, device=gate_up.device)
        code = _lib.load().tk_swiglu_fwd(gate_up.data_ptr(), gate_up.stride(0), out.data_ptr(), out.stride(0), rows,
                                         inter, _lib.dtype_code(gate_up.dtype), _lib.stream_ptr())
        _lib.check(code, 'tk_swiglu_fwd')
        ctx.save_for_backward(gate_up)
        return out

    @staticmethod
    def backward(ctx, dout):
        gate_up, = ctx.saved_tensors
        dout = dout.contiguous()
        rows, two_i = gate_up.shape
        dgu = torch.empty_like(gate_up)
        code = _lib.load().tk_swiglu_bwd(gate_up.data_ptr(), gate_up.stride(0), dout.data_ptr(), dout.stride(0),
                                         dgu.data_ptr(), dgu.stride(0), rows, two_i // 2,
                                         _lib.dtype_code(gate_up.dtype), _lib.stream_ptr())
        _lib.check(code, 'tk_swiglu_bwd')
        return dgu


def swiglu_applies(gate_up: torch.Tensor) -> bool:
    """Shapes the fused gated activation takes: 2-D, unit inner stride, ``inter`` and the row stride multiples of 8."""
    return (gate_up.is_cuda and gate_up.dim() == 2 and gate_up.stride(1) == 1 and gate_up.shape[1] % 16 == 0 and
            gate_up.stride(0) % 8 == 0 and gate_up.dtype in (torch.float32, torch.bfloat16) and
            gate_up.data_ptr() % (8 * gate_up.element_size()) == 0)


def swiglu(gate_up: torch.Tensor) -> torch.Tensor:
    """``F.silu(gate) * up`` with ``gate, up = gate_up.chunk(2, -1)`` in one pass (and one in backward)."""
    if not gate_up.is_cuda:
        raise RuntimeError('gate_up must live on the GPU: this path has no CPU implementation')
    return _SwiGLU.apply(gate_up)


class _GroupedExpertsLinear(torch.autograd.Function):
    """Frozen packed expert weights and the (expert, tenant) LoRA terms as one node on rows in segment order.

    Forward: shrink, then the grouped GEMM with the LoRA term in its epilogue.  Backward: the grouped GEMM in its
    transposing form on the same weights gives the base part of ``dx``; the segmented backward adds the LoRA part
    onto it in place and yields the adapters' gradients.  The weights get no gradient (the reference freezes them)."""

    @staticmethod
    def forward(ctx, x, weight, seg, groups_per_expert, groups, *weights):
        h = None
        if groups is not None:
            h = torch.empty(lora_h_bytes(seg, groups), dtype=torch.uint8, device=x.device)
            lora_shrink_(x, seg, groups, h, map_rows=False)
        y = grouped_linear_(x, weight, seg, groups_per_expert, groups=groups, h=h, map_rows=False)
        ctx.save_for_backward(x, weight, h)
        ctx.seg, ctx.groups, ctx.groups_per_expert = seg, groups, groups_per_expert
        return y

    @staticmethod
    def backward(ctx, dy):
        x, weight, h = ctx.saved_tensors
        seg, groups = ctx.seg, ctx.groups
        dy = dy.contiguous()
        needs_dx = ctx.needs_input_grad[0]
        dx = grouped_linear_(dy, weight, seg, ctx.groups_per_expert, map_rows=False, transposed=True) \
            if needs_dx else None
        if groups is None:
            return (dx, None, None, None, None)
        na, nb = len(groups.a_tensors), len(groups.b_tensors)
        needs_a = any(ctx.needs_input_grad[5:5 + na])
        needs_b = any(ctx.needs_input_grad[5 + na:5 + na + nb])
        arena_a, arena_b, pa, pb = _weight_grads(groups, needs_a, needs_b, dy.device)
        if needs_dx or needs_a or needs_b:
            lora_bwd_(dy, x, h, dx, pa, pb, seg, groups, False, accumulate=False)
        ga = groups.grad_views(arena_a, 'a') if needs_a else [None] * na
        gb = groups.grad_views(arena_b, 'b') if needs_b else [None] * nb
        return (dx, None, None, None, None, *ga, *gb)


def grouped_experts_linear(x: torch.Tensor, weight: torch.Tensor, seg: SegmentTable, groups_per_expert: int,
                           groups: Optional[AdapterGroups] = None) -> torch.Tensor:
    """``y = x W_e^T`` plus every (expert, tenant) group's LoRA term, for rows in segment order; differentiable in
    ``x`` and the adapters, not in the frozen ``weight [E, out, in]`` (both widths multiples of 128)."""
    extra = groups.autograd_tensors() if groups is not None else []
    if groups is not None:
        groups.sync_masters()
    return _GroupedExpertsLinear.apply(x, weight, seg, groups_per_expert, groups, *extra)


def multi_lora_delta(x: torch.Tensor, base_out: torch.Tensor, seg: SegmentTable, groups: AdapterGroups,
                     map_rows: bool = True) -> torch.Tensor:
    """``base_out`` with every adapter's LoRA term added to its own rows (in place, differentiable)."""
    return _LoraDelta.apply(x, base_out, seg, groups, map_rows, *groups.autograd_tensors())


def multi_lora_linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], seg: SegmentTable,
                      groups: AdapterGroups, map_rows: bool = True) -> torch.Tensor:
    """``F.linear(x, weight, bias)`` plus the segmented LoRA update as one autograd node."""
    return _LoraLinear.apply(x, weight, bias, seg, groups, map_rows, *groups.autograd_tensors())


# ---- projections that share their input (q / k / v, gate / up) ----------------------------------------------

def _host_array(ctype, values):
    return (ctype * len(values))(*values)


def _shared_descs(seg: SegmentTable, groups_list: Sequence[AdapterGroups], map_rows: bool):
    if not 1 <= len(groups_list) <= 4:
        raise ValueError(f'1 to 4 projections can share an input, got {len(groups_list)}')
    g0 = groups_list[0]
    for g in groups_list:
        if g.num_groups != seg.num_groups:
            raise ValueError(f'segment table has {seg.num_groups} groups, adapters have {g.num_groups}')
        if g.in_features != g0.in_features or g.dtype != g0.dtype:
            raise ValueError('projections that share an input must agree in in_features and dtype')
    descs = [_desc(seg, g, map_rows) for g in groups_list]
    table = _host_array(ctypes.c_void_p, [ctypes.addressof(d) for d in descs])
    return descs, table


def lora_fwd_shared_(x: torch.Tensor, ys: Sequence[torch.Tensor], seg: SegmentTable,
                     groups_list: Sequence[AdapterGroups], map_rows: bool = True,
                     hs: Optional[Sequence[torch.Tensor]] = None) -> List[torch.Tensor]:
    """In place ``ys[p] += lora_p(x)`` for projections that read the same ``x``; returns their saved ``h``."""
    descs, table = _shared_descs(seg, groups_list, map_rows)
    _check_rows(x, 'x', seg.rows, groups_list[0].in_features, groups_list[0].dtype)
    for y, g in zip(ys, groups_list):
        _check_rows(y, 'y', seg.rows, g.out_features, g.dtype)
    if hs is None:
        hs = [torch.empty(lora_h_bytes(seg, g), dtype=torch.uint8, device=x.device) for g in groups_list]
    code = _lib.load().tk_lora_fwd_shared(
        table, len(descs), x.data_ptr(), x.stride(0), _host_array(ctypes.c_void_p, [y.data_ptr() for y in ys]),
        _host_array(ctypes.c_int64, [y.stride(0) for y in ys]), _host_array(ctypes.c_void_p, [h.data_ptr() for h in hs]),
        _lib.stream_ptr())
    _lib.check(code, 'tk_lora_fwd_shared')
    return list(hs)


def lora_bwd_shared_(dys: Sequence[torch.Tensor], x: torch.Tensor, hs: Sequence[torch.Tensor], dx: torch.Tensor,
                     grad_a_ptrs: Sequence[torch.Tensor], grad_b_ptrs: Sequence[torch.Tensor], seg: SegmentTable,
                     groups_list: Sequence[AdapterGroups], map_rows: bool = True, accumulate: bool = False,
                     workspaces: Optional[Sequence[torch.Tensor]] = None) -> None:
    """``dx += sum_p dx_p`` in place and every projection's weight gradients (see ``tk_lora_bwd_shared``)."""
    descs, table = _shared_descs(seg, groups_list, map_rows)
    _check_rows(x, 'x', seg.rows, groups_list[0].in_features, groups_list[0].dtype)
    _check_rows(dx, 'dx', seg.rows, groups_list[0].in_features, groups_list[0].dtype)
    for dy, g in zip(dys, groups_list):
        _check_rows(dy, 'dy', seg.rows, g.out_features, g.dtype)
    wss = workspaces
    if wss is None:
        wss = [torch.empty(lora_bwd_workspace_bytes(seg, g), dtype=torch.uint8, device=x.device) for g in groups_list]
    code = _lib.load().tk_lora_bwd_shared(
        table, len(descs), _host_array(ctypes.c_void_p, [t.data_ptr() for t in dys]),
        _host_array(ctypes.c_int64, [t.stride(0) for t in dys]), x.data_ptr(), x.stride(0),
        _host_array(ctypes.c_void_p, [h.data_ptr() for h in hs]), dx.data_ptr(), dx.stride(0),
        _host_array(ctypes.c_void_p, [t.data_ptr() for t in grad_a_ptrs]),
        _host_array(ctypes.c_void_p, [t.data_ptr() for t in grad_b_ptrs]), 1 if accumulate else 0,
        _host_array(ctypes.c_void_p, [w.data_ptr() for w in wss]), _host_array(ctypes.c_int64, [w.numel() for w in wss]),
        _lib.stream_ptr())
    _lib.check(code, 'tk_lora_bwd_shared')


class _LoraDeltaShared(torch.autograd.Function):
    """Several base outputs of one input updated in place by their own adapters, as one node."""

    @staticmethod
    def forward(ctx, x, seg, groups_list, map_rows, n, *rest):
        ys = rest[:n]
        hs = lora_fwd_shared_(x, ys, seg, groups_list, map_rows)
        ctx.mark_dirty(*ys)
        ctx.save_for_backward(x, *hs)
        ctx.seg, ctx.groups_list, ctx.map_rows, ctx.n = seg, groups_list, map_rows, n
        return tuple(ys)

    @staticmethod
    def backward(ctx, *dys):
        x, *hs = ctx.saved_tensors
        seg, groups_list, n = ctx.seg, ctx.groups_list, ctx.n
        dys = [torch.zeros(seg.rows, g.out_features, dtype=g.dtype, device=x.device) if dy is None else dy.contiguous()
               for dy, g in zip(dys, groups_list)]
        dx = torch.zeros_like(x)
        arenas = [_weight_grads(g, True, True, x.device) for g in groups_list]
        lora_bwd_shared_(dys, x, hs, dx, [a[2] for a in arenas], [a[3] for a in arenas], seg, groups_list, ctx.map_rows)
        grads = []
        for g, (arena_a, arena_b, _, _) in zip(groups_list, arenas):
            grads += g.grad_views(arena_a, 'a') + g.grad_views(arena_b, 'b')
        return (dx if ctx.needs_input_grad[0] else None, None, None, None, None, *dys, *grads)


def multi_lora_delta_shared(x: torch.Tensor, base_outs: Sequence[torch.Tensor], seg: SegmentTable,
                            groups_list: Sequence[AdapterGroups], map_rows: bool = True) -> Tuple[torch.Tensor, ...]:
    """:func:`multi_lora_delta` for projections that read the same ``x`` (q / k / v, gate / up).

    ``base_outs[p]`` gets the LoRA term of ``groups_list[p]`` added in place.  ``x`` and, in backward, the
    gradient of ``x`` cross memory once for all projections instead of once per projection.
    """
    weights = []
    for g in groups_list:
        weights += g.autograd_tensors()
    return _LoraDeltaShared.apply(x, seg, tuple(groups_list), map_rows, len(groups_list), *base_outs, *weights)


class _LoraLinearShared(torch.autograd.Function):
    """Base ``F.linear`` of several projections of one input and their LoRA updates as one node: in backward
    the base GEMMs accumulate into one ``dx``, which the shared LoRA backward then updates in place."""

    @staticmethod
    def forward(ctx, x, seg, groups_list, map_rows, n, has_bias, *rest):
        weights, biases = rest[:n], rest[n:2 * n]
        ys = [torch.nn.functional.linear(x, w, b if hb else None) for w, b, hb in zip(weights, biases, has_bias)]
        hs = lora_fwd_shared_(x, ys, seg, groups_list, map_rows)
        ctx.save_for_backward(x, *weights, *hs)
        ctx.seg, ctx.groups_list, ctx.map_rows, ctx.n, ctx.has_bias = seg, groups_list, map_rows, n, has_bias
        return tuple(ys)

    @staticmethod
    def backward(ctx, *dys):
        n, seg, groups_list = ctx.n, ctx.seg, ctx.groups_list
        x, *rest = ctx.saved_tensors
        weights, hs = rest[:n], rest[n:]
        dys = [torch.zeros(seg.rows, g.out_features, dtype=g.dtype, device=x.device) if dy is None else dy.contiguous()
               for dy, g in zip(dys, groups_list)]
        dx = dys[0] @ weights[0]
        for dy, w in zip(dys[1:], weights[1:]):
            dx.addmm_(dy, w)
        dws = [dy.t() @ x if ctx.needs_input_grad[6 + p] else None for p, dy in enumerate(dys)]
        dbs = [dy.sum(0) if ctx.has_bias[p] and ctx.needs_input_grad[6 + n + p] else None for p, dy in enumerate(dys)]
        arenas = [_weight_grads(g, True, True, x.device) for g in groups_list]
        lora_bwd_shared_(dys, x, hs, dx, [a[2] for a in arenas], [a[3] for a in arenas], seg, groups_list, ctx.map_rows)
        grads = []
        for g, (arena_a, arena_b, _, _) in zip(groups_list, arenas):
            grads += g.grad_views(arena_a, 'a') + g.grad_views(arena_b, 'b')
        return (dx if ctx.needs_input_grad[0] else None, None, None, None, None, None, *dws, *dbs, *grads)


def multi_lora_linear_shared(x: torch.Tensor, weights: Sequence[torch.Tensor],
                             biases: Sequence[Optional[torch.Tensor]], seg: SegmentTable,
                             groups_list: Sequence[AdapterGroups], map_rows: bool = True) -> Tuple[torch.Tensor, ...]:
    """:func:`multi_lora_linear` for projections that read the same ``x``: ``F.linear(x, weights[p], biases[p])``
    plus the segmented LoRA update of ``groups_list[p]``, all projections in one autograd node."""
    has_bias = tuple(b is not None for b in biases)
    dummies = [b if b is not None else x.new_zeros(0) for b in biases]
    lora = []
    for g in groups_list:
        lora += g.autograd_tensors()
    return _LoraLinearShared.apply(x, seg, tuple(groups_list), map_rows, len(groups_list), has_bias, *weights, *dummies,
                                   *lora)
