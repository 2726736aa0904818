"""twinkle_amd: the multi-LoRA hot path of modelscope/twinkle on MI355X (gfx950).

Segment builder, segmented LoRA linear forward/backward and the row
permute/unpermute around them run in hand-written HIP kernels behind a C ABI
(``include/twinkle_amd.h``); this package binds them to PyTorch-ROCm tensors
and mirrors the reference's ``MultiLora`` interface on top.  There is no CPU
path: every op raises if the HIP library is missing or a tensor is not on the GPU.
"""
from . import custom_ops  # noqa: F401  (registers torch.ops.twinkle_amd.*)
from .lora_layer import LoraConfig, LoraLinear, LoraModel, inject_adapter  # noqa: F401
from .multi_lora import LoraTenant, MultiLora, batch, forward_shared, share_inputs, unshare_inputs  # noqa: F401
from .integration import use_mi355x_path  # noqa: F401
from .ops import (AdapterGroups, grouped_linear_, swiglu, lora_bwd_, lora_bwd_shared_, lora_bwd_workspace_bytes, lora_expand_,  # noqa: F401
                  lora_fwd_, lora_fwd_noalloc_, lora_fwd_shared_, lora_h_bytes, lora_shrink_, multi_lora_delta, multi_lora_delta_shared,
                  multi_lora_linear, multi_lora_linear_shared)
from .optim import BatchedStep, MultiTenantAdamW, do_grad_sync, trainable_parameters  # noqa: F401
from .segments import (SegmentTable, build_segments, flat_keys_from_topk, packed_cu_seqlens, permute,  # noqa: F401
                       token_groups_from_sequences, unpermute, validate_segment_table)

__version__ = '0.1.0'
