"""The shared library loads and exports every entry point the header declares (no GPU needed)."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, 'include', 'twinkle_amd.h')).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(tk_[a-z_0-9]+)\s*\(', text)))


def test_header_declares_entry_points():
    names = _declared()
    assert 'tk_segment_build' in names and 'tk_lora_fwd' in names and 'tk_lora_bwd' in names
    assert len(names) >= 10


def test_library_exports_every_declared_symbol():
    from twinkle_amd import _lib
    if not os.path.exists(_lib.library_path()):
        pytest.fail(f'{_lib.library_path()} is not built (run __graft_entry__.build())')
    lib = _lib.load()
    for name in _declared():
        assert hasattr(lib, name), f'{name} declared in the header but not exported'
    assert set(_lib.EXPORTS) == set(_declared()), 'ctypes table and header disagree'
    assert lib.tk_version().startswith(b'twinkle_amd')
    assert lib.tk_error_string(-2) == b'workspace too small'


def test_size_queries_run_on_the_host():
    import ctypes
    from twinkle_amd import _lib
    lib = _lib.load()
    small = lib.tk_segment_workspace_bytes(1024, 4)
    big = lib.tk_segment_workspace_bytes(65536, 512)
    assert 0 < small < big
    assert lib.tk_segment_workspace_bytes(-1, 4) == _lib.TK_ERR_INVALID
    d = _lib.LoraDesc()
    d.rows, d.in_features, d.out_features, d.num_groups, d.max_rank, d.dtype = 16384, 4096, 4096, 16, 16, 1
    h = lib.tk_lora_h_bytes(ctypes.byref(d))
    slots = 16384 + 32 * 17 + 64                      # padded slots
    split = (16384 // 32 + 17) * 8 * 32 * 16 * 4       # partial sums of the 8 column slices of a 4096-wide shrink
    assert 2 * 16 * 16384 * 2 <= h <= 2 * 16 * slots * 2 + split + 512
    assert lib.tk_lora_bwd_workspace_bytes(ctypes.byref(d)) > h
    d.max_rank = 1000
    assert lib.tk_lora_h_bytes(ctypes.byref(d)) == _lib.TK_ERR_INVALID


def test_ops_refuse_cpu_tensors():
    import torch
    from twinkle_amd import build_segments
    with pytest.raises(RuntimeError):
        build_segments(torch.zeros(8, dtype=torch.int32), 2)


def test_shared_entry_points_reject_malformed_arguments_on_the_host():
    """Argument checks of tk_lora_fwd_shared / tk_lora_bwd_shared run before any GPU work (fake device pointers)."""
    import ctypes
    from twinkle_amd import _lib
    lib = _lib.load()

    def desc(rows=64, k=2048, m=512):
        d = _lib.LoraDesc()
        d.rows, d.in_features, d.out_features, d.num_groups, d.max_rank, d.dtype = rows, k, m, 2, 16, 1
        d.map_rows, d.lda, d.ldb = 1, k, 16
        d.seg_ws = d.lora_A = d.lora_B = d.rank = d.scale = 0x1000      # never dereferenced by the checks
        return d

    def table(descs):
        return (ctypes.c_void_p * len(descs))(*[ctypes.addressof(d) for d in descs])

    ptrs = (ctypes.c_void_p * 5)(*([0x1000] * 5))
    lds = (ctypes.c_int64 * 5)(*([4096] * 5))
    a, b = desc(), desc()
    bad = _lib.TK_ERR_INVALID
    fwd = lambda t, n, y=ptrs, ld=lds, h=ptrs: lib.tk_lora_fwd_shared(t, n, 0x1000, 2048, y, ld, h, None)  # noqa: E731
    assert fwd(None, 2) == bad                                   # no descriptor table
    assert fwd(table([a, b]), 0) == bad                          # no projection
    assert fwd(table([a] * 5), 5) == bad                         # more than TK_MAX_SHARED
    assert fwd(table([a, desc(rows=65)]), 2) == bad              # projections disagree in rows
    assert fwd(table([a, desc(k=1024)]), 2) == bad               # ... in in_features
    assert fwd(table([a, b]), 2, y=None) == bad                  # no output table
    small = (ctypes.c_int64 * 2)(4096, 100)
    assert fwd(table([a, b]), 2, ld=small) == bad                # a row stride below out_features
    empty = desc(rows=0)
    assert fwd(table([empty, desc(rows=0)]), 2) == _lib.TK_OK    # nothing to do
    assert lib.tk_lora_bwd_shared(table([a, b]), 2, ptrs, lds, 0x1000, 2048, ptrs, 0x1000, 2048, None, ptrs, 0, ptrs,
                                  lds, None) == bad              # no dA table
    assert lib.tk_lora_bwd_shared(table([a, b]), 2, ptrs, lds, 0x1000, 100, ptrs, 0x1000, 2048, ptrs, ptrs, 0, ptrs,
                                  lds, None) == bad              # x row stride below in_features
    tiny = (ctypes.c_int64 * 2)(16, 16)
    assert lib.tk_lora_bwd_shared(table([a, b]), 2, ptrs, lds, 0x1000, 2048, ptrs, 0x1000, 2048, ptrs, ptrs, 0, ptrs,
                                  tiny, None) == _lib.TK_ERR_WORKSPACE


def test_entry_points_reject_malformed_arguments_on_the_host():
    """Every entry point checks its arguments before any GPU work: fake device pointers, only failing calls."""
    import ctypes
    from twinkle_amd import _lib
    lib = _lib.load()
    bad, small, unsupported = _lib.TK_ERR_INVALID, _lib.TK_ERR_WORKSPACE, _lib.TK_ERR_UNSUPPORTED
    P = 0x1000
    # segment builder
    assert lib.tk_segment_build(P, 0, -1, 4, None, None, P, 1 << 20, None) == bad           # negative row count
    assert lib.tk_segment_build(P, 0, 64, 0, None, None, P, 1 << 20, None) == bad           # no groups
    assert lib.tk_segment_build(None, 0, 64, 4, None, None, P, 1 << 20, None) == bad        # no keys
    assert lib.tk_segment_build(P, 7, 64, 4, None, None, P, 1 << 20, None) == bad           # unknown key type
    assert lib.tk_segment_build(P, 0, 64, 1 << 20, None, None, P, 1 << 40, None) == unsupported   # too many groups
    assert lib.tk_segment_build(P, 0, 64, 4, None, None, P, 16, None) == small              # workspace too small
    # row movers
    assert lib.tk_permute_rows(P, 64, P, 64, None, None, 64, 64, 64, 4, 1, None) == bad     # no segment table
    assert lib.tk_permute_rows(P, 64, P, 64, None, P, 65, 64, 64, 4, 1, None) == bad        # rows not k * tokens
    assert lib.tk_unpermute_rows(P, 64, P, 64, None, P, 64, 64, 0, 4, 1, None) == bad       # zero width
    assert lib.tk_unpermute_rows(P, 64, P, 64, None, P, 64, 64, 64, 4, 9, None) == bad      # unknown dtype
    # single-projection LoRA
    d = _lib.LoraDesc()
    d.rows, d.in_features, d.out_features, d.num_groups, d.max_rank, d.dtype = 64, 256, 128, 2, 8, 1
    d.map_rows, d.lda, d.ldb = 1, 256, 8
    d.seg_ws = d.lora_A = d.lora_B = d.rank = d.scale = P
    ref = ctypes.byref(d)
    assert lib.tk_lora_fwd(ref, P, 255, P, 128, P, None) == bad                              # ldx below in_features
    assert lib.tk_lora_fwd(ref, P, 256, P, 64, P, None) == bad                               # ldy below out_features
    assert lib.tk_lora_fwd(ref, P, 256, P, 128, None, None) == bad                           # no h buffer
    assert lib.tk_lora_fwd(None, P, 256, P, 128, P, None) == bad                             # no descriptor
    assert lib.tk_lora_bwd(ref, None, 128, P, 256, P, P, 256, P, P, 0, P, 1 << 30, None) == bad   # no dy
    assert lib.tk_lora_bwd(ref, P, 128, None, 256, P, P, 256, P, P, 0, P, 1 << 30, None) == bad   # dA wanted, no x
    assert lib.tk_lora_bwd(ref, P, 128, P, 256, P, P, 256, P, P, 0, P, 16, None) == small
    d.lda = 100
    assert lib.tk_lora_fwd(ref, P, 256, P, 128, P, None) == bad                              # lda below in_features
    d.lda, d.dtype = 256, 5
    assert lib.tk_lora_h_bytes(ref) == bad                                                   # unknown dtype
    # grouped expert GEMM
    g = _lib.GroupedDesc()
    g.rows, g.num_groups, g.groups_per_expert, g.in_features, g.out_features = 64, 4, 2, 128, 256
    g.dtype, g.map_rows, g.weight_stride, g.ldw = 1, 0, 256 * 128, 128
    g.seg_ws = g.weight = P
    gref = ctypes.byref(g)
    need = lib.tk_grouped_linear_workspace_bytes(gref)
    assert need > 0
    assert lib.tk_grouped_linear(gref, None, P, 128, P, 256, None, P, need - 1, None) == small
    assert lib.tk_grouped_linear(gref, None, P, 127, P, 256, None, P, need, None) == bad      # ldx below in_features
    assert lib.tk_grouped_linear(gref, None, None, 128, P, 256, None, P, need, None) == bad   # no x
    assert lib.tk_grouped_linear(None, None, P, 128, P, 256, None, P, need, None) == bad      # no descriptor
    assert lib.tk_grouped_linear(gref, ref, P, 128, P, 256, P, P, need, None) == bad          # LoRA of another layer
    g.groups_per_expert = 3
    assert lib.tk_grouped_linear_workspace_bytes(gref) == bad                                 # 4 groups, 3 per expert
    g.groups_per_expert, g.in_features, g.ldw = 2, 96, 96
    assert lib.tk_grouped_linear(gref, None, P, 96, P, 256, None, P, need, None) == unsupported   # width not a multiple of 64
    g.in_features, g.ldw, g.dtype = 128, 128, 0
    assert lib.tk_grouped_linear(gref, None, P, 128, P, 256, None, P, need, None) == unsupported  # fp32
    g.dtype, g.weight_stride = 1, 100
    assert lib.tk_grouped_linear(gref, None, P, 128, P, 256, None, P, need, None) == bad      # experts overlap
    g.weight_stride, g.weight_layout = 256 * 128, 2
    assert lib.tk_grouped_linear(gref, None, P, 128, P, 256, None, P, need, None) == bad      # unknown layout
    g.weight_layout = 1
    assert lib.tk_grouped_linear(gref, None, P, 128, P, 256, None, P, need, None) == bad      # ldw below out_features
    g.weight_layout = 0
    g.rows, g.weight_stride = 0, 256 * 128
    assert lib.tk_grouped_linear(gref, None, None, 128, None, 256, None, None, 0, None) == _lib.TK_OK  # nothing to do
    # gated activation
    assert lib.tk_swiglu_fwd(P, 32, P, 16, -1, 16, 1, None) == bad                            # negative rows
    assert lib.tk_swiglu_fwd(P, 31, P, 16, 4, 16, 1, None) == bad                             # ld below 2 * inter
    assert lib.tk_swiglu_fwd(P, 32, None, 16, 4, 16, 1, None) == bad                          # no output
    assert lib.tk_swiglu_fwd(P, 32, P, 16, 4, 16, 7, None) == bad                             # unknown dtype
    assert lib.tk_swiglu_fwd(P, 24, P, 12, 4, 12, 1, None) == unsupported                     # inter not a multiple of 8
    assert lib.tk_swiglu_bwd(P, 32, None, 16, P, 32, 4, 16, 1, None) == bad                   # no d(hidden)
    assert lib.tk_swiglu_bwd(P, 32, P, 16, P, 31, 4, 16, 1, None) == bad                      # ld of d(gate | up)
    assert lib.tk_swiglu_fwd(None, 32, None, 16, 0, 16, 1, None) == _lib.TK_OK                # nothing to do
    # optimizer
    assert lib.tk_opt_workspace_bytes(-1, 10) == bad
    assert lib.tk_opt_grad_norm(P, 4, P, 0, 100, 1, P, P, P, 1 << 20, None) == bad           # no tenants
    assert lib.tk_opt_grad_norm(P, 4, P, 2, 100, 1, None, P, P, 1 << 20, None) == bad        # no norm output
    assert lib.tk_opt_grad_norm(P, 4, P, 2, 100, 1, P, P, P, 0, None) == small
    assert lib.tk_opt_adamw_step(None, 4, P, 2, 100, 1, None, 0, None) == bad                # no tensor table
    assert lib.tk_opt_adamw_step(P, 70000, P, 2, 100, 1, None, 0, None) == bad               # more tensors than a launch takes
    assert lib.tk_opt_adamw_step(P, 0, P, 2, 100, 1, None, 0, None) == _lib.TK_OK            # nothing to do
