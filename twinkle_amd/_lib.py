"""ctypes binding of ``include/twinkle_amd.h``.

The library is loaded after ``torch`` so that it shares torch's HIP runtime
(both name ``libamdhip64.so.7``).  There is no fallback: a missing library is
an error at first use.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_float, c_int32, c_int64, c_void_p

import torch  # noqa: F401  (must come first: brings in the HIP runtime the library binds to)

from ._build import LIB_PATH

TK_OK = 0
TK_ERR_INVALID = -1
TK_ERR_WORKSPACE = -2
TK_ERR_UNSUPPORTED = -3
TK_ERR_LAUNCH = -4
TK_ERR_SCRATCH = -5
TK_NOALLOC_SCRATCH_BYTES = 16 << 20
TK_DTYPE_F32 = 0
TK_DTYPE_BF16 = 1
TK_KEY_I32 = 0
TK_KEY_I64 = 1
TK_TILE_ROWS = 32
TK_CHUNK_ROWS = 128
TK_MAX_GROUPS = 16384
TK_MAX_RANK = 128


class LoraDesc(Structure):
    """Mirror of ``tk_lora_desc``."""
    _fields_ = [
        ('rows', c_int64),
        ('in_features', c_int32),
        ('out_features', c_int32),
        ('num_groups', c_int32),
        ('max_rank', c_int32),
        ('dtype', c_int32),
        ('map_rows', c_int32),
        ('seg_ws', c_void_p),
        ('lora_A', c_void_p),
        ('lora_B', c_void_p),
        ('lda', c_int64),
        ('ldb', c_int64),
        ('rank', c_void_p),
        ('scale', c_void_p),
        ('weights_f32', c_int32),
        ('rank_classes', c_int32),
    ]


class GroupedDesc(Structure):
    """Mirror of ``tk_grouped_desc``."""
    _fields_ = [
        ('rows', c_int64),
        ('num_groups', c_int32),
        ('groups_per_expert', c_int32),
        ('in_features', c_int32),
        ('out_features', c_int32),
        ('dtype', c_int32),
        ('map_rows', c_int32),
        ('seg_ws', c_void_p),
        ('weight', c_void_p),
        ('weight_stride', c_int64),
        ('ldw', c_int64),
        ('weight_layout', c_int32),
        ('reserved', c_int32),
    ]


EXPORTS = {
    'tk_version': (c_char_p, []),
    'tk_error_string': (c_char_p, [c_int32]),
    'tk_segment_workspace_bytes': (c_int64, [c_int64, c_int32]),
    'tk_segment_build': (c_int32, [c_void_p, c_int32, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_int64,
                                   c_void_p]),
    'tk_segment_bad_keys': (c_int32, [c_void_p, c_void_p, POINTER(c_int64)]),
    'tk_segment_validate': (c_int32, [c_void_p, c_int64, c_int32, c_void_p, POINTER(c_int32), POINTER(c_int64)]),
    'tk_permute_rows': (c_int32, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int64, c_int32,
                                  c_int32, c_int32, c_void_p]),
    'tk_unpermute_rows': (c_int32, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int64,
                                    c_int32, c_int32, c_int32, c_void_p]),
    'tk_unpermute_weight_grad': (c_int32, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int64,
                                           c_int32, c_int32, c_int32, c_void_p]),
    'tk_lora_h_bytes': (c_int64, [POINTER(LoraDesc)]),
    'tk_lora_bwd_workspace_bytes': (c_int64, [POINTER(LoraDesc)]),
    'tk_lora_fwd': (c_int32, [POINTER(LoraDesc), c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p]),
    'tk_lora_fwd_noalloc': (c_int32, [POINTER(LoraDesc), c_void_p, c_int64, c_void_p, c_int64, c_void_p]),
    'tk_lora_shrink': (c_int32, [POINTER(LoraDesc), c_void_p, c_int64, c_void_p, c_void_p]),
    'tk_lora_expand': (c_int32, [POINTER(LoraDesc), c_void_p, c_void_p, c_int64, c_void_p]),
    'tk_lora_bwd': (c_int32, [POINTER(LoraDesc), c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_int64,
                              c_void_p, c_void_p, c_int32, c_void_p, c_int64, c_void_p]),
    # arrays indexed by projection are host arrays: pointers to descriptors / device pointers / strides
    'tk_lora_fwd_shared': (c_int32, [c_void_p, c_int32, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    'tk_lora_bwd_shared': (c_int32, [c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p,
                                     c_int64, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p]),
    'tk_grouped_linear_workspace_bytes': (c_int64, [POINTER(GroupedDesc)]),
    'tk_grouped_linear': (c_int32, [POINTER(GroupedDesc), POINTER(LoraDesc), c_void_p, c_int64, c_void_p, c_int64,
                                    c_void_p, c_void_p, c_int64, c_void_p]),
    'tk_swiglu_fwd': (c_int32, [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int32, c_int32, c_void_p]),
    'tk_swiglu_bwd': (c_int32, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int32, c_int32,
                                c_void_p]),
    'tk_yardstick': (c_int32, [c_int32, c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_void_p]),
    'tk_opt_workspace_bytes': (c_int64, [c_int32, c_int64]),
    'tk_opt_grad_norm': (c_int32, [c_void_p, c_int32, c_void_p, c_int32, c_int64, c_int32, c_void_p, c_void_p, c_void_p,
                                   c_int64, c_void_p]),
    'tk_opt_adamw_step': (c_int32, [c_void_p, c_int32, c_void_p, c_int32, c_int64, c_int32, c_void_p, c_int32,
                                    c_void_p]),
}

_lib = None


def library_path() -> str:
    return LIB_PATH


def load() -> ctypes.CDLL:
    """Load the HIP library (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f'{LIB_PATH} is missing: build it with `python -m twinkle_amd._build` '
                           '(or __graft_entry__.build()); there is no fallback path')
    lib = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_LOCAL)
    for name, (res, args) in EXPORTS.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is absent
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(code: int, what: str) -> None:
    """Map a negative return code to the exception type the reference raises for the same misuse."""
    if code >= 0:
        return
    msg = f'{what}: {load().tk_error_string(code).decode()} ({code})'
    if code in (TK_ERR_INVALID, TK_ERR_UNSUPPORTED):
        raise ValueError(msg)
    raise RuntimeError(msg)


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return TK_DTYPE_F32
    if dtype == torch.bfloat16:
        return TK_DTYPE_BF16
    raise ValueError(f'unsupported dtype {dtype}: the kernels take float32 or bfloat16')


def stream_ptr() -> int:
    """The current HIP stream of the current device as an integer handle."""
    # the raw accessor costs a fraction of a microsecond; torch.cuda.current_stream() builds a Stream object (8 us)
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())
