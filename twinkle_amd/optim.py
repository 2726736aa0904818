"""Per-tenant gradient normalisation, clipping and AdamW, stepped for all tenants at once.

The reference keeps one ``torch.optim`` optimizer per tenant and walks the tenants one
after the other: ``clip_grad_norm`` divides the tenant's gradients by its token count and
clips their norm, ``step`` applies per-call lr / weight decay / eps / betas, ``zero_grad``
clears them (src/twinkle/model/transformers/transformers.py:732-894,
src/twinkle/utils/grad_clip.py:31-96).  With many small adapters that is thousands of tiny
launches per training step.  Here every tenant's adapter tensors sit in one device table and
three launches (two for the norms, one for the update) serve all tenants, each with its own
token count, threshold and hyper-parameters (``tk_opt_grad_norm``, ``tk_opt_adamw_step``).
Moments are fp32 whatever the parameter dtype; arithmetic is fp32.
"""
from __future__ import annotations

import math
import operator
import re
from typing import Dict, Iterable, List, Optional, Sequence

import numpy as np
import torch

from . import _lib

_TENSOR_DTYPE = np.dtype([('param', '<u8'), ('grad', '<u8'), ('exp_avg', '<u8'), ('exp_avg_sq', '<u8'),
                          ('numel', '<i8'), ('tenant', '<i4'), ('reserved', '<i4')])
_TENANT_DTYPE = np.dtype([('lr', '<f4'), ('beta1', '<f4'), ('beta2', '<f4'), ('eps', '<f4'), ('weight_decay', '<f4'),
                          ('one_minus_beta1', '<f4'), ('one_minus_beta2', '<f4'), ('bias_correction1', '<f4'),
                          ('bias_correction2_sqrt', '<f4'), ('grad_scale', '<f4'),
                          ('max_grad_norm', '<f4'), ('norm_type', '<f4'), ('active', '<i4'), ('reserved', '<i4')])
TK_OPT_WRITE_GRADS = 1
TK_OPT_ZERO_GRADS = 2


def trainable_parameters(model: torch.nn.Module, adapter_name: str) -> Dict[str, torch.nn.Parameter]:
    """The parameters of one tenant's slot: names matching ``.lora_<x>.<adapter_name>`` (transformers.py:962-972)."""
    pattern = re.compile(rf'\.lora_\w+\.{re.escape(adapter_name)}')
    return {n: p for n, p in model.named_parameters() if p.requires_grad and pattern.search(n)}


class _Tenant:

    def __init__(self, index, params, lr, betas, eps, weight_decay):
        self.index = index
        self.params: List[torch.nn.Parameter] = list(params)
        self.lr, self.betas, self.eps, self.weight_decay = float(lr), (float(betas[0]), float(betas[1])), float(eps), \
            float(weight_decay)
        self.step = 0
        self.exp_avg: List[Optional[torch.Tensor]] = [None] * len(self.params)
        self.exp_avg_sq: List[Optional[torch.Tensor]] = [None] * len(self.params)
        # rows of the device tensor table, kept while the gradient tensors stay the same objects
        self.grads_seen: Optional[list] = None
        self.rows: Dict[torch.dtype, list] = {}
        self.rows_version = 0

    def table_rows(self) -> Dict[torch.dtype, list]:
        """This tenant's rows of the tensor table per parameter dtype.  Autograd accumulates into an existing
        ``.grad`` in place and the update kernel clears gradients without replacing them, so from the second step
        on the same tensor objects come back and the rows (six pointers and sizes per tensor) are reused; the
        check is one identity comparison per parameter."""
        grads = [p.grad for p in self.params]
        seen = self.grads_seen
        if seen is not None and len(seen) == len(grads) and all(map(operator.is_, grads, seen)):
            return self.rows
        rows: Dict[torch.dtype, list] = {}
        for i, p in enumerate(self.params):
            g = grads[i]
            if g is None:
                continue  # torch optimizers skip parameters without a gradient
            if g.dtype != p.dtype or not g.is_contiguous() or g.shape != p.shape:
                g = grads[i] = p.grad = g.to(p.dtype).contiguous()
            if self.exp_avg[i] is None:
                self.exp_avg[i] = torch.zeros(p.shape, dtype=torch.float32, device=p.device)
                self.exp_avg_sq[i] = torch.zeros(p.shape, dtype=torch.float32, device=p.device)
            rows.setdefault(p.dtype, []).append((p.data_ptr(), g.data_ptr(), self.exp_avg[i].data_ptr(),
                                                 self.exp_avg_sq[i].data_ptr(), p.numel(), self.index, 0))
        self.grads_seen, self.rows = grads, rows
        self.rows_version += 1
        return rows


class MultiTenantAdamW:
    """AdamW (``weight_decay=0``: Adam) for many tenants, one launch set per step."""

    def __init__(self):
        self._tenants: Dict[str, _Tenant] = {}
        self._last_clip: Dict[torch.dtype, torch.Tensor] = {}
        self._last_tables = None
        self._table_cache: Dict[torch.dtype, tuple] = {}
        self._with_grads: List[str] = []

    # ---- tenant management -------------------------------------------------------------------------------
    def add_tenant(self, name: str, params: Iterable[torch.nn.Parameter], lr: float = 1e-3, betas=(0.9, 0.999),
                   eps: float = 1e-8, weight_decay: float = 1e-2) -> None:
        """Register a tenant with its optimizer defaults (``torch.optim.AdamW``'s)."""
        if name in self._tenants:
            raise ValueError(f'tenant {name} already has an optimizer')
        params = list(params)
        for p in params:
            if not p.is_cuda:
                raise RuntimeError('optimizer parameters must live on the GPU: this path has no CPU implementation')
            if p.dtype not in (torch.float32, torch.bfloat16):
                raise ValueError(f'parameters must be float32 or bfloat16, got {p.dtype}')
            if not p.is_contiguous():
                raise ValueError('parameters must be contiguous')
        self._tenants[name] = _Tenant(len(self._tenants), params, lr, betas, eps, weight_decay)

    def remove_tenant(self, name: str) -> None:
        """Drop a tenant and its state (slot released); the remaining tenants keep their rows."""
        self._tenants.pop(name)
        for i, t in enumerate(self._tenants.values()):
            if t.index != i:
                t.index, t.grads_seen = i, None      # its rows carry the index: rebuild them

    def tenants(self) -> List[str]:
        return list(self._tenants)

    def state(self, name: str):
        t = self._tenants[name]
        return {'step': t.step, 'exp_avg': t.exp_avg, 'exp_avg_sq': t.exp_avg_sq}

    # ---- the step ----------------------------------------------------------------------------------------
    def _tables(self, names: Sequence[str], num_tokens, max_grad_norm, norm_type, optim_params, advance: bool):
        """Device tables per parameter dtype for the tenants in ``names``.

        The tensor table only changes when a gradient tensor was replaced (autograd accumulates in place and the
        in-kernel zeroing keeps the tensors), so it is cached on the pointers it holds; the small tenant table
        carries this call's numbers and is rebuilt every time."""
        names = list(names)
        tenant_rows = np.zeros(len(self._tenants), dtype=_TENANT_DTYPE)
        rows: Dict[torch.dtype, list] = {}
        versions = []
        self._with_grads = []
        device = None
        for name in names:
            t = self._tenants[name]
            over = (optim_params or {}).get(name) or {}
            lr = float(over['lr']) if 'lr' in over else t.lr
            # the reference only overrides a weight decay that was positive (transformers.py:862-863)
            wd = float(over['weight_decay']) if (t.weight_decay > 0.0 and over.get('weight_decay') is not None) \
                else t.weight_decay
            eps = float(over['eps']) if over.get('eps') is not None else t.eps
            b1, b2 = over['betas'] if over.get('betas') is not None else t.betas
            step = t.step + 1 if advance else max(t.step, 1)
            tokens = num_tokens.get(name, 1) if isinstance(num_tokens, dict) else num_tokens
            tokens = float(tokens)
            row = tenant_rows[t.index]
            row['lr'], row['beta1'], row['beta2'], row['eps'], row['weight_decay'] = lr, b1, b2, eps, wd
            row['one_minus_beta1'], row['one_minus_beta2'] = 1.0 - float(b1), 1.0 - float(b2)
            row['bias_correction1'] = 1.0 - float(b1)**step
            row['bias_correction2_sqrt'] = math.sqrt(1.0 - float(b2)**step)
            row['grad_scale'] = 1.0 / tokens if tokens > 0 else 1.0   # grad_clip.py:83-84
            row['max_grad_norm'] = max_grad_norm if max_grad_norm is not None else 0.0
            row['norm_type'] = norm_type
            row['active'] = 1
            mine = t.table_rows()
            versions.append((name, t.rows_version))
            if mine:
                self._with_grads.append(name)
                device = t.params[0].device
            for dtype, lst in mine.items():
                rows.setdefault(dtype, []).append(lst)
        out = {}
        if device is None:
            return out, tenant_rows
        tenants_dev = torch.from_numpy(tenant_rows.view(np.uint8).copy()).to(device)
        key = tuple(versions)
        for dtype, lists in rows.items():
            cached = self._table_cache.get(dtype)
            if cached is None or cached[0] != key:
                arr = np.array([r for lst in lists for r in lst], dtype=_TENSOR_DTYPE)
                cached = (key, torch.from_numpy(arr.view(np.uint8).copy()).to(device), int(arr['numel'].max()),
                          len(arr))
                self._table_cache[dtype] = cached
            out[dtype] = (cached[1], cached[3], cached[2], tenants_dev, None)
        return out, tenant_rows

    def _run_norm(self, tables, names, max_grad_norm, norm_type) -> Dict[str, torch.Tensor]:
        lib = _lib.load()
        norms: Dict[str, torch.Tensor] = {}
        self._last_clip = {}
        per_dtype_norms = []
        nt = len(self._tenants)
        for dtype, (tensors_dev, n, max_numel, tenants_dev, _keep) in tables.items():
            norm = torch.empty(nt, dtype=torch.float32, device=tensors_dev.device)
            clip = torch.empty(nt, dtype=torch.float32, device=tensors_dev.device)
            nbytes = lib.tk_opt_workspace_bytes(n, max_numel)
            _lib.check(nbytes, 'tk_opt_workspace_bytes')
            ws = torch.empty(nbytes, dtype=torch.uint8, device=tensors_dev.device)
            code = lib.tk_opt_grad_norm(tensors_dev.data_ptr(), n, tenants_dev.data_ptr(), nt, max_numel,
                                        _lib.dtype_code(dtype), norm.data_ptr(), clip.data_ptr(), ws.data_ptr(),
                                        ws.numel(), _lib.stream_ptr())
            _lib.check(code, 'tk_opt_grad_norm')
            per_dtype_norms.append(norm)
            self._last_clip[dtype] = clip
        if len(per_dtype_norms) > 1:
            # a tenant with parameters of both dtypes: combine the two partial norms and redo the coefficient
            inf = math.isinf(float(norm_type))
            total = torch.maximum(*per_dtype_norms) if inf else torch.sqrt(sum(v * v for v in per_dtype_norms))
            clip = torch.clamp(max_grad_norm / (total + 1e-6), max=1.0) if max_grad_norm and max_grad_norm > 0 \
                else torch.ones_like(total)
            self._last_clip = {dtype: clip for dtype in self._last_clip}
            per_dtype_norms = [total]
        if per_dtype_norms:
            for name in names:
                norms[name] = per_dtype_norms[0][self._tenants[name].index]
        return norms

    def _run_step(self, tables, names, flags: int, use_clip: bool) -> None:
        lib = _lib.load()
        for dtype, (tensors_dev, n, max_numel, tenants_dev, _keep) in tables.items():
            clip = self._last_clip.get(dtype) if use_clip else None
            code = lib.tk_opt_adamw_step(tensors_dev.data_ptr(), n, tenants_dev.data_ptr(), len(self._tenants),
                                         max_numel, _lib.dtype_code(dtype),
                                         clip.data_ptr() if clip is not None else None, flags, _lib.stream_ptr())
            _lib.check(code, 'tk_opt_adamw_step')
        self._last_tables = tables  # keeps the device tables alive until the next call (stream-ordered use)
        self._last_clip = {}
        for name in self._with_grads:      # a tenant without any gradient takes no step (torch optimizers skip
            self._tenants[name].step += 1  # parameters whose grad is None, state and step count included)

    def clip_grad_norm(self, num_tokens, max_grad_norm: float = 1.0, norm_type: float = 2.0,
                       names: Optional[Sequence[str]] = None) -> Dict[str, torch.Tensor]:
        """Norm of every tenant's gradients after division by its token count (device scalars, no host
        synchronisation), as ``clip_grad_norm`` returns it per tenant; the division and the clipping themselves
        are applied inside :meth:`step`, which must follow (``clip_grad_and_step`` does both)."""
        names = list(names) if names is not None else self.tenants()
        tables, _ = self._tables(names, num_tokens, max_grad_norm, float(norm_type), None, advance=False)
        return self._run_norm(tables, names, max_grad_norm, norm_type)

    def step(self, num_tokens=1, optim_params: Optional[Dict[str, dict]] = None,
             names: Optional[Sequence[str]] = None, zero_grad: bool = False, write_grads: bool = False,
             use_clip: bool = True) -> None:
        """AdamW for the tenants in ``names`` (default: all), gradients divided by ``num_tokens`` (an int or a
        dict per tenant) and scaled by the coefficients of the preceding :meth:`clip_grad_norm`.
        ``optim_params[name]`` may carry ``lr``, ``weight_decay``, ``eps``, ``betas`` for this call
        (transformers.py:857-868)."""
        names = list(names) if names is not None else self.tenants()
        tables, _ = self._tables(names, num_tokens, 0.0, 2.0, optim_params, advance=True)
        flags = (TK_OPT_ZERO_GRADS if zero_grad else 0) | (TK_OPT_WRITE_GRADS if write_grads else 0)
        self._run_step(tables, names, flags, use_clip)

    def clip_grad_and_step(self, num_tokens, max_grad_norm: float = 1.0, norm_type: float = 2.0,
                           optim_params: Optional[Dict[str, dict]] = None,
                           names: Optional[Sequence[str]] = None) -> Dict[str, torch.Tensor]:
        """clip_grad_norm, step and zero_grad for every tenant in one go (transformers.py:781-785); the device
        tables are built once and serve both passes."""
        names = list(names) if names is not None else self.tenants()
        tables, _ = self._tables(names, num_tokens, max_grad_norm, float(norm_type), optim_params, advance=True)
        norms = self._run_norm(tables, names, max_grad_norm, norm_type)
        self._run_step(tables, names, TK_OPT_ZERO_GRADS, use_clip=True)
        return norms

    def zero_grad(self, names: Optional[Sequence[str]] = None, set_to_none: bool = True) -> None:
        for name in (names if names is not None else self.tenants()):
            for p in self._tenants[name].params:
                if p.grad is not None:
                    if set_to_none:
                        p.grad = None
                    else:
                        p.grad.zero_()


def do_grad_sync(cur_step: int, gradient_accumulation_steps: int) -> bool:
    """Whether a tenant's optimizer acts after its ``cur_step``-th backward: always without accumulation, else when
    ``(cur_step - 1) % gradient_accumulation_steps == 0 and cur_step > 1`` (model/optimizer_group.py:56-62)."""
    return gradient_accumulation_steps == 1 or ((cur_step - 1) % gradient_accumulation_steps == 0 and cur_step > 1)


class BatchedStep:
    """Loss reduction and accumulation schedule of training steps that serve many tenants per batch.

    The reference runs, per tenant and one tenant at a time, ``forward`` → ``calculate_loss`` (its loss object
    returns the loss and a token count; both are added to the tenant's running ``loss_value`` / ``num_tokens``,
    transformers.py:617-665) → ``backward`` (``cur_step += 1``, :667-709) → ``clip_grad_and_step``, whose four parts
    each do nothing unless the tenant's ``do_grad_sync`` holds (:732-785, :835-894).  Here one forward / backward
    carries rows of many tenants, so this class keeps the same three per-tenant quantities (``cur_step``,
    accumulated ``num_tokens``, gradient-accumulation setting), reduces the per-token losses of a mixed batch to one
    loss per tenant, and hands the tenants that are due to :class:`MultiTenantAdamW` in one call.

    ``reduction`` follows the reference's ``CrossEntropyLoss`` (loss/cross_entropy.py:16-33): ``'sum'`` gives each
    tenant the sum over its unmasked tokens and counts those tokens (the gradients are divided by the count at the
    step); anything else gives the mean over its unmasked tokens and counts 0, which the reference turns into 1 per
    backward (:646-648).  The batch loss that is back-propagated is the sum of the tenants' losses: a tenant's
    adapters only see its own rows, so each tenant gets exactly the gradient of its own loss.
    """

    def __init__(self, optimizer: MultiTenantAdamW, gradient_accumulation_steps=1, reduction: str = 'sum',
                 ignore_index: int = -100):
        self.optimizer = optimizer
        self.gradient_accumulation_steps = gradient_accumulation_steps   # an int, or a dict per tenant
        self.reduction = reduction
        self.ignore_index = ignore_index
        self.cur_step: Dict[str, int] = {}
        self.num_tokens: Dict[str, float] = {}
        self.last_loss: Dict[str, torch.Tensor] = {}
        self._pending = None       # (tenant names, device token counts) of the loss not yet back-propagated
        self._last_batch: List[str] = []

    def _accumulation(self, name: str) -> int:
        g = self.gradient_accumulation_steps
        return int(g.get(name, 1)) if isinstance(g, dict) else int(g)

    def tenant_losses(self, tenant_adapter_names: Sequence[str], row_tenant: torch.Tensor, per_token: torch.Tensor,
                      mask: torch.Tensor):
        """``(loss [n], counts [n])``: every tenant's reduction of ``per_token * mask`` over its own rows and the
        number of its unmasked rows.  The sums are one small matrix product with the tenants' indicator rows, so
        they do not depend on the order in which atomics would land."""
        n = len(tenant_adapter_names)
        rt = row_tenant.reshape(-1)
        onehot = (rt[None, :] == torch.arange(n, device=rt.device)[:, None]).to(torch.float32)
        m = mask.reshape(-1).to(torch.float32)
        sums = onehot @ (per_token.reshape(-1).to(torch.float32) * m)
        counts = onehot @ m
        if self.reduction == 'sum':
            return sums, counts.clamp(min=1)
        return sums / counts.clamp(min=1), torch.zeros_like(counts)

    def loss(self, tenant_adapter_names: Sequence[str], row_tenant: torch.Tensor, labels: torch.Tensor,
             logps: Optional[torch.Tensor] = None, logits: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Cross entropy of a mixed batch, reduced per tenant as the reference's ``CrossEntropyLoss`` reduces one
        tenant's batch; returns the scalar to back-propagate (the sum of the tenants' losses)."""
        labels = labels.reshape(-1)
        if logps is None:
            flat = logits.reshape(-1, logits.shape[-1])
            logps = torch.log_softmax(flat, dim=-1).gather(-1, labels.clamp(min=0).unsqueeze(-1)).squeeze(-1)
        mask = labels != self.ignore_index
        return self.custom_loss(tenant_adapter_names, row_tenant, -logps.reshape(-1), mask)

    def custom_loss(self, tenant_adapter_names: Sequence[str], row_tenant: torch.Tensor, per_token: torch.Tensor,
                    mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The same reduction for any per-row loss (``mask``: rows that count, default all)."""
        if mask is None:
            mask = torch.ones_like(per_token, dtype=torch.bool)
        losses, counts = self.tenant_losses(tenant_adapter_names, row_tenant, per_token, mask)
        names = list(tenant_adapter_names)
        self.last_loss = {name: losses[i].detach() for i, name in enumerate(names)}
        self._pending = (names, counts.detach())
        return losses.sum()

    def backward(self, loss: torch.Tensor) -> None:
        """``loss.backward()`` and the reference's bookkeeping for every tenant of the batch: one more ``cur_step``,
        its token count added to the running ``num_tokens`` (one copy of the counts to the host, where the
        reference reads one ``.item()`` per tenant)."""
        if self._pending is None:
            raise RuntimeError('call loss() / custom_loss() before backward()')
        names, counts = self._pending
        loss.backward()
        for name, c in zip(names, counts.tolist()):
            self.cur_step[name] = self.cur_step.get(name, 0) + 1
            self.num_tokens[name] = self.num_tokens.get(name, 0.0) + (c if c else 1.0)    # "if not counts: 1"
        self._last_batch, self._pending = names, None

    def due(self) -> List[str]:
        """Tenants of the last batch whose optimizer acts now."""
        return [n for n in self._last_batch if do_grad_sync(self.cur_step.get(n, 0), self._accumulation(n))]

    def clip_grad_and_step(self, max_grad_norm: float = 1.0, norm_type: float = 2.0,
                           optim_params: Optional[Dict[str, dict]] = None) -> Dict[str, torch.Tensor]:
        """``clip_grad_norm`` → ``step`` → ``zero_grad`` for the tenants that are due, all in one launch set, each
        with the tokens it accumulated since its last step; the others keep accumulating.  Returns the due tenants'
        gradient norms (device scalars)."""
        names = self.due()
        if not names:
            return {}
        norms = self.optimizer.clip_grad_and_step({n: self.num_tokens[n] for n in names}, max_grad_norm, norm_type,
                                                  optim_params, names=names)
        for n in names:
            self.num_tokens[n] = 0.0
        return norms
