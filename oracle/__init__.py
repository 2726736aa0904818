"""CPU oracle for the multi-LoRA hot path.  TEST INFRASTRUCTURE ONLY.

This package restates, in plain PyTorch on the CPU, the arithmetic that
modelscope/twinkle runs on its multi-LoRA path.  It exists to *check* the HIP
kernels: only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` may import it.  The product package (``twinkle_amd``)
never imports it and has no CPU fallback.

Every function cites the reference lines it follows (paths relative to the
reference checkout).  None of the reference's Python is imported or executed:
the reference's own module imports ``peft`` at module scope, which this image
does not have, and its tests hold no numeric golden vectors for this path, so
each function is pinned by what the mathematics fixes (closed forms in fp64,
``torch.autograd.gradcheck``, brute-force loops on tiny inputs, special cases
that reduce to a library routine, and the behavioural invariants the
reference's tests assert).  ``tests/test_oracle_*.py`` holds those pins.

Pin status per function
-----------------------
segment_build_sort / segment_build_bruteforce / permute_by_mask : pinned
    (two independent constructions + brute force + invariants)
unpermute                                                  : pinned
    (index_add_ closed form; permute∘unpermute identity)
lora_linear_forward / multi_lora_linear / grads            : pinned
    (fp64 closed form, gradcheck, B=0, r<max_r, single segment ≡ F.linear)
swiglu                                                     : pinned (x sigmoid(x) u in closed form, gradcheck)
expert_delta_weight / expert_lora_low_rank / experts_linear : pinned
    (merged-weight form ≡ low-rank form; shape KAT of the reference test; the chunk loop
    against a row-by-row product with each row's own expert and against one F.linear for E = 1)
packed_cu_seqlens                                          : pinned (brute force)
slice_rank_tensor / copy_rank_tensor / match_target_modules : pinned
    (round-trip + hand-written cases from the reference's comments)
normalize_and_clip_grad_norm / TenantAdamW (oracle/optim.py)  : pinned
    (they are torch.nn.utils.clip_grad_norm_ and torch.optim.AdamW themselves, the
    library routines the reference calls; one step also checked against the closed form)
PEFT-side container behaviour (attribute names, adapter dtype autocast)
    : parity unpinned — PEFT is absent from this image; affects dtypes at the
    boundary, not the arithmetic.
"""
from .segments import (  # noqa: F401
    expert_mask_from_topk,
    flat_keys_from_topk,
    packed_cu_seqlens,
    permute_by_mask,
    segment_build_bruteforce,
    segment_build_sort,
    token_ids_from_cu_seqlens,
    unpermute,
    unpermute_rows,
)
from .optim import TenantAdamW, normalize_and_clip_grad_norm, trainable_parameter_names  # noqa: F401
from .lora import (  # noqa: F401
    copy_rank_tensor,
    expert_delta_weight,
    expert_lora_low_rank,
    experts_linear,
    swiglu,
    lora_linear_forward,
    lora_scaling,
    match_target_modules,
    multi_lora_linear,
    multi_lora_linear_grads,
    slice_rank_tensor,
)
