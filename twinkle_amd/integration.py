"""Switching an existing ``MultiLora`` of the reference onto the HIP path.

The reference binds its LoRA arithmetic per layer instance:
``MultiLora._patch_lora_forward(name, base_layer)`` sets ``base_layer.forward``
(src/twinkle/model/multi_lora.py:289-331).  :func:`use_mi355x_path` does the
same binding with the forward of this package, on an object that only has to
offer what the reference's class offers (``loras``, ``find_lora``,
``find_lora_by_tenant``, ``match_target_modules``, ``module``); whatever else the
forward needs it attaches to that object itself the first time it runs.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import multi_lora as _host


def use_mi355x_path(multi_lora, lora_compute_dtype: Optional[torch.dtype] = None):
    """Rebind ``forward`` on every LoRA layer under ``multi_lora.module`` (after its ``patch()`` has run).

    ``multi_lora.adapter(name)`` keeps its meaning: one tenant for every row, computed by the segmented kernels.
    Mixed batches go through ``twinkle_amd.batch(multi_lora, tenant_names, row_tenant)``.  ``lora_compute_dtype``
    is the option of :class:`twinkle_amd.MultiLora` of the same name (fp32 adapters under a bf16 model).
    Returns ``multi_lora``.
    """
    if lora_compute_dtype is not None:
        multi_lora.lora_compute_dtype = lora_compute_dtype
    bound = 0
    for module in _host._modules_of(multi_lora):
        for name, sub in module.named_modules():
            if _host._is_lora_layer(sub) and hasattr(sub, 'in_features'):
                _host.MultiLora._patch_lora_forward(multi_lora, name, sub)
                bound += 1
    if bound == 0:
        raise ValueError('no LoRA layer found under multi_lora.module: call its patch() first')
    return multi_lora
