#!/usr/bin/env python3
"""Benchmark of the multi-LoRA hot path on one MI355X.

One step = segment build + segmented LoRA forward + segmented LoRA backward (dX, dA, dB) over one
batch of BASELINE.json's config 2: Llama-3-8B q_proj shape (4096 -> 4096), 16384 tokens, 16 adapters of
rank 16 / alpha 32, adapter ids Zipf(1.1)-distributed and shuffled, bf16 with fp32 accumulation.  The
frozen base GEMM is not part of the step (it is timed once and reported separately).  Inputs are
resident in HBM before the timed region; three buffer sets are rotated so that no activation is served
from the 256 MB last-level cache across steps (the backward of a step runs on the set whose forward ran
one full step earlier).

Prints one JSON line (see the keys below).  `roofline` describes the dominant kernel, the expand
kernel (y += h B^T, a read-modify-write of the whole output), on its forward launches: algorithmic
bytes of one launch over its mean duration, measured with HIP events on the launch stream around runs of 20 launches
in a row (an event record idles the queue for a few microseconds, so a pair of records around every single launch
measures the launch plus that; those intervals, taken inside the steps, are reported next to it).  The `steps` timed
steps behind `value` carry no events.  After the headline leg the default run also measures the other BASELINE shapes
with the same step definition (`other_configs`).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0


TRAFFIC_PROFILE = os.path.join('profiles', 'bench_cfg2_hbm_traffic_pmc.txt')
KERNEL_SOURCES = ('kernels_mfma.hip', 'tk_mfma.h', 'tk_common.h')     # what the expand kernel is compiled from


def kernel_source_digest():
    """sha256 over the sources of the dominant kernel, as the traffic profile records it when it is taken."""
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, 'twinkle_amd', 'csrc', name), 'rb') as f:
            h.update(f.read())
    return h.hexdigest()


def measured_traffic(kernel):
    """HBM bytes per launch of `kernel` from the committed rocprofv3 --pmc summary, with where it comes from.

    The counters need a profiler pass of their own, so a plain run cannot measure them; the committed summary
    records the digest of the kernel's sources it was taken with, and the number is only reported while those
    sources are unchanged (otherwise ``traffic`` is null and the note says why)."""
    value = digest = commit = None
    try:
        with open(os.path.join(ROOT, TRAFFIC_PROFILE)) as f:
            for line in f:
                if line.startswith(f'traffic_bytes_per_launch[{kernel}]:'):
                    value = float(line.split(':')[1])
                elif line.startswith('kernel_source_sha256:'):
                    digest = line.split(':')[1].strip()
                elif line.startswith('source_commit:'):
                    commit = line.split(':')[1].strip()
    except OSError:
        return None, {'profile': TRAFFIC_PROFILE, 'note': 'profile not found'}
    source = {'profile': TRAFFIC_PROFILE, 'source_commit': commit, 'kernel_source_sha256': digest}
    try:
        current = kernel_source_digest()
    except OSError:
        current = None
    if value is None or digest is None or digest != current:
        source['note'] = 'kernel sources changed since the profile was taken: traffic not reported'
        return None, source
    return value, source


TRACE_PROFILE = os.path.join('profiles', 'bench_cfg2_kernel_trace.txt')


def traced_duration_ms(kernel):
    """Average duration of `kernel` in the committed rocprofv3 kernel trace of this benchmark, or None when the
    profile is missing or was taken with other kernel sources (it records their digest like the traffic profile)."""
    avg = digest = None
    try:
        with open(os.path.join(ROOT, TRACE_PROFILE)) as f:
            for line in f:
                if line.startswith(kernel + ' ') and avg is None:
                    avg = float(line[len(kernel):].split()[1]) * 1e-3
                elif line.startswith('kernel_source_sha256:'):
                    digest = line.split(':')[1].strip()
        if avg is None or digest is None or digest != kernel_source_digest():
            return None
    except (OSError, ValueError, IndexError):
        return None
    return avg


def cpu_baseline(w, budget_s=15.0):
    """The reference's CPU path (per-adapter F.linear pairs + autograd, restated in oracle/) on this host."""
    import torch
    import oracle
    threads = torch.get_num_threads()
    x = w.x.bfloat16().float()
    base = w.base_out.bfloat16().float()
    dy = w.dy.bfloat16().float()
    a = [t.bfloat16().float() for t in w.lora_A]
    b = [t.bfloat16().float() for t in w.lora_B]
    oracle.multi_lora_linear_grads(x[:2048], base[:2048], w.ids[:2048], a, b, w.ranks, w.scales, dy[:2048])  # warm-up
    reps, t0 = 0, time.perf_counter()
    while True:
        oracle.multi_lora_linear_grads(x, base, w.ids, a, b, w.ranks, w.scales, dy)
        reps += 1
        el = time.perf_counter() - t0
        if el > budget_s or reps >= 20:
            break
    return {
        'value': w.tokens * reps / el, 'unit': 'tokens/s', 'cores': threads, 'kind': 'port',
        'sample': f'{reps} x the full {w.name} batch ({w.tokens} tokens), bf16-rounded inputs, fp32 math, '
                  f'torch {torch.__version__} CPU, per-adapter F.linear pairs + autograd',
    }


def torch_gpu_loop(w, dev, dt, steps=5):
    """What the reference does today, on the same GPU: tenants one after the other, two F.linear per tenant on the
    tenant's rows (index_select / index_add_) and stock autograd.  Plain torch ops, no kernel of this library."""
    import torch
    import torch.nn.functional as F
    x = w.x.to(dt).to(dev).requires_grad_(True)
    base = w.base_out.to(dt).to(dev)
    dy = w.dy.to(dt).to(dev)
    ids = w.ids.to(dev)
    a = [t.to(dt).to(dev).requires_grad_(True) for t in w.lora_A]
    b = [t.to(dt).to(dev).requires_grad_(True) for t in w.lora_B]
    rows = [torch.nonzero(ids == g).flatten() for g in range(w.num_adapters)]

    def one():
        y = base.clone()
        for g in range(w.num_adapters):
            r = w.ranks[g]
            if rows[g].numel() == 0 or r == 0:
                continue
            xg = x.index_select(0, rows[g])
            y = y.index_add(0, rows[g], F.linear(F.linear(xg, a[g][:r]), b[g][:, :r]) * w.scales[g])
        y.backward(dy)
        for t in [x] + a + b:
            t.grad = None

    one()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        one()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    return {'value': w.tokens / (ms * 1e-3), 'unit': 'tokens/s', 'ms_per_step': ms,
            'kind': 'per-adapter F.linear loop with index_select / index_add_ and autograd on the same GPU (torch ops only)'}


def optimizer_step_bench(dev, steps=10):
    """Multi-tenant clip + AdamW over the q_proj adapters of a 32-layer stack for 8 tenants of rank 64 (512 bf16
    tensors, 134 M elements) in three launches, next to one fused torch.optim.AdamW per tenant (the reference's
    schedule) on the same tensors.  Bytes per element of the update pass: read p, g (2 B each), m, v (4 B each),
    write p, m, v = 22 B; the norm pass reads g = 2 B."""
    import torch
    from twinkle_amd import MultiTenantAdamW
    tenants, layers, r, k = 8, 32, 64, 4096
    opt = MultiTenantAdamW()
    params = {}
    for t in range(tenants):
        ps = []
        for _ in range(layers):
            ps.append(torch.nn.Parameter(torch.randn(r, k, device=dev, dtype=torch.bfloat16) * 0.02))
            ps.append(torch.nn.Parameter(torch.randn(k, r, device=dev, dtype=torch.bfloat16) * 0.02))
        for p in ps:
            p.grad = torch.randn_like(p)
        params[f't{t}'] = ps
        opt.add_tenant(f't{t}', ps, lr=1e-4)
    elements = sum(p.numel() for ps in params.values() for p in ps)
    tokens = {n: 4096 for n in params}
    e = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    ours_ms = 0.0
    for i in range(steps + 2):
        e[0].record()
        opt.clip_grad_and_step(tokens, max_grad_norm=1.0)     # in-kernel zeroing keeps the gradient tensors
        e[1].record()
        torch.cuda.synchronize()
        if i >= 2:
            ours_ms += e[0].elapsed_time(e[1]) / steps
        for ps in params.values():
            for p in ps:
                p.grad.normal_()
    ref = [torch.optim.AdamW(ps, lr=1e-4, fused=True) for ps in params.values()]
    torch_ms = 0.0
    for i in range(steps + 2):
        e[0].record()
        for ps, o in zip(params.values(), ref):
            for p in ps:
                p.grad.div_(4096)
            torch.nn.utils.clip_grad_norm_(ps, 1.0)
            o.step()
            o.zero_grad(set_to_none=False)
        e[1].record()
        torch.cuda.synchronize()
        if i >= 2:
            torch_ms += e[0].elapsed_time(e[1]) / steps
    return {'tensors': tenants * layers * 2, 'elements': elements, 'tenants': tenants,
            'clip_and_adamw_ms': ours_ms, 'GBps': 24.0 * elements / (ours_ms * 1e-3) / 1e9,
            'hbm_frac': 24.0 * elements / (ours_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            'torch_per_tenant_ms': torch_ms,
            'note': 'norm pass (2 B/element) + update pass (22 B/element), host-side table build included; torch: '
                    'per tenant grad.div_, clip_grad_norm_, fused AdamW (bf16 moments), zero_grad'}


def yardstick_bench(dev, reps=12):
    """What this GPU sustains for the memory access patterns of the LoRA kernels, with no arithmetic
    (`tk_yardstick`): contiguous read / copy / in-place update, and the per-tile patterns of the expand, shrink and
    row-contraction kernels over a [16384, 4096] bf16 buffer (config 2's activations, 128 MiB), with the rows taken
    in order, in the sweep order of config 2's segment table (tiles sorted by first row), in the table's own
    group-major order, and fully shuffled.  Three buffers are rotated so that nothing is served from the last-level
    cache; every pattern is launched `reps` times between two HIP events, best of four rounds."""
    import torch
    from twinkle_amd import _lib, build_segments, workloads
    lib = _lib.load()
    T, K = 16384, 4096
    bufs = [torch.full((T, K), 1.0, dtype=torch.bfloat16, device=dev) for _ in range(3)]
    sink = torch.zeros(1 << 16, dtype=torch.uint8, device=dev)
    ids = workloads.zipf_ids(T, 16)
    order = torch.sort(ids.long(), stable=True).indices                      # the table's group-major order
    # sweep order: the same tiles of 32 rows, taken in the order of their first row
    tiles, first = [], []
    for g in range(16):
        rows = order[ids[order] == g]
        for j in range(0, rows.numel(), 32):
            t = rows[j:j + 32]
            if t.numel() == 32:
                tiles.append(t)
                first.append(int(t[0]))
    full = torch.stack(tiles)
    left = torch.tensor(sorted(set(range(T)) - set(full.flatten().tolist())), dtype=torch.long)
    def pad(rows_2d):
        flat = torch.cat([rows_2d.flatten(), left])
        return flat[:T].to(torch.int32).to(dev)
    perms = {
        'rows in order': None,
        'sweep order (tiles by first row)': pad(full[torch.tensor(first).argsort()]),
        'group-major order (segment table)': pad(full),
        'shuffled rows': torch.randperm(T, generator=torch.Generator().manual_seed(1)).to(torch.int32).to(dev),
    }
    stream = _lib.stream_ptr()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def run(kind, perm, factor):
        best = 1e9
        for _ in range(4):
            e0.record()
            for i in range(reps):
                a = bufs[i % 3]
                b = bufs[(i + 1) % 3] if kind == 1 else sink
                code = lib.tk_yardstick(kind, a.data_ptr(), b.data_ptr(), perm.data_ptr() if perm is not None else None,
                                        T, K, stream)
                _lib.check(code, 'tk_yardstick')
            e1.record()
            torch.cuda.synchronize()
            best = min(best, e0.elapsed_time(e1) / reps)
        return {'us': best * 1e3, 'GBps': factor * T * K * 2 / (best * 1e-3) / 1e9}

    out = {'buffer': f'[{T}, {K}] bf16 = {T * K * 2 >> 20} MiB, three rotated', 'reps': reps}
    out['contiguous read'] = run(0, None, 1)
    out['contiguous copy (read + write)'] = run(1, None, 2)
    out['contiguous in-place update'] = run(2, None, 2)
    out['contiguous in-place update, non-temporal'] = run(3, None, 2)
    for kind, name, factor in ((4, 'expand pattern, read', 1), (5, 'expand pattern, in-place non-temporal', 2),
                               (6, 'shrink pattern, read', 1), (7, 'row-contraction pattern, read', 1)):
        for pname, perm in perms.items():
            out[f'{name}: {pname}'] = run(kind, perm, factor)
    # the grouped GEMM's operand path, global memory -> LDS in steps of 64 KB per block with a barrier per step
    out['global -> LDS, 64 KB steps per block: every line from memory'] = run(8, None, 1)
    out['global -> LDS, 64 KB steps per block: every line an L2 hit'] = run(9, None, 16)
    for k in ('global -> LDS, 64 KB steps per block: every line from memory',
              'global -> LDS, 64 KB steps per block: every line an L2 hit'):
        steps = T * K * 2 // 256 // 65536 * (16 if 'L2 hit' in k else 1)
        out[k]['us_per_step'] = out[k]['us'] / steps
    return out


def shared_qkv_bench(dev, steps=20, calibrate_copy=False, rank=16, weights_f32=False):
    """q / k / v of one attention block (4096 -> 4096, 1024, 1024; config 2's tokens, adapters and ids):
    one shared call against one call per projection, forward + backward, segment table built once."""
    import torch
    from twinkle_amd import (AdapterGroups, build_segments, lora_bwd_, lora_bwd_shared_, lora_bwd_workspace_bytes,
                             lora_fwd_, lora_fwd_shared_, lora_h_bytes, workloads)
    w = workloads.config2_qproj()
    dt, T, K, G = torch.bfloat16, w.tokens, w.in_features, w.num_adapters
    outs = (4096, 1024, 1024)
    gen = torch.Generator().manual_seed(11)
    x = w.x.to(dt).to(dev)
    seg = build_segments(w.ids.to(dev), G, want_perm=False, want_offsets=False)
    groups, ys, dys, pas, pbs, keep = [], [], [], [], [], []
    for m in outs:
        wdt = torch.float32 if weights_f32 else dt      # fp32 adapters and gradients under the bf16 activations
        A = [(torch.randn(rank, K, generator=gen) / K**0.5).to(wdt).to(dev) for _ in range(G)]
        B = [(torch.randn(m, rank, generator=gen) * 0.05).to(wdt).to(dev) for _ in range(G)]
        groups.append(AdapterGroups(A, B, w.ranks if rank == 16 else [rank] * G, w.scales, act_dtype=dt))
        ys.append(torch.randn(T, m, generator=gen).to(dt).to(dev))
        dys.append(torch.randn(T, m, generator=gen).to(dt).to(dev))
        ga, gb = [torch.zeros_like(t) for t in A], [torch.zeros_like(t) for t in B]
        keep.append((ga, gb))
        pas.append(torch.tensor([t.data_ptr() for t in ga], dtype=torch.int64, device=dev))
        pbs.append(torch.tensor([t.data_ptr() for t in gb], dtype=torch.int64, device=dev))
    dx = torch.zeros(T, K, dtype=dt, device=dev)
    hs = [torch.empty(lora_h_bytes(seg, g), dtype=torch.uint8, device=dev) for g in groups]
    wss = [torch.empty(lora_bwd_workspace_bytes(seg, g), dtype=torch.uint8, device=dev) for g in groups]

    def separate():
        for y, h, g in zip(ys, hs, groups):
            lora_fwd_(x, y, seg, g, h=h)
        for dy, h, pa, pb, g, ws in zip(dys, hs, pas, pbs, groups, wss):
            lora_bwd_(dy, x, h, dx, pa, pb, seg, g, workspace=ws)

    def shared():
        lora_fwd_shared_(x, ys, seg, groups, hs=hs)
        lora_bwd_shared_(dys, x, hs, dx, pas, pbs, seg, groups, workspaces=wss)

    res = {}
    for name, fn in (('one_call_per_projection_ms', separate), ('shared_ms', shared)):
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        res[name] = (time.perf_counter() - t0) * 1e3 / steps
    if calibrate_copy:
        for _ in range(5):
            dx.copy_(x)                                # a known-size kernel for rocprofv3 --pmc readings
        torch.cuda.synchronize()
    elt = 2
    per_proj = sum(elt * T * (4 * m + 3 * K) for m in outs)            # y rw, dy r | x r (fwd, dA), dx rw
    joint = sum(elt * T * 4 * m for m in outs) + elt * T * 4 * K       # x r twice, dx rw once
    res.update({'workload': f'T={T}, {K} -> {outs}, {G} adapters rank {rank}, fwd + bwd, segment table prebuilt' +
                            (', fp32 adapter weights and gradients' if weights_f32 else ''),
                'algorithmic_bytes_one_call_per_projection': per_proj, 'algorithmic_bytes_shared': joint,
                'speedup': res['one_call_per_projection_ms'] / res['shared_ms'],
                'hbm_frac_shared': joint / (res['shared_ms'] * 1e-3) / 1e9 / HBM_PEAK_GBS})
    return res


def moe_experts_bench(dev, steps=10):
    """BASELINE config 4 as a whole expert block: 8192 tokens x top-8 of 128 experts (65536 routed rows in
    (expert, tenant) order), experts 2048 -> 2 x 768 -> 2048, 4 tenants with rank-8 LoRA on both packed
    parameters, bf16.  experts_forward with the reference's per-expert loop for the frozen weights (plus the
    segmented LoRA kernels) against the grouped GEMMs with the LoRA term in their epilogue; forward alone and
    forward + backward (dx and the adapters' gradients; the frozen weights get none)."""
    import torch
    from twinkle_amd import LoraConfig, build_segments, flat_keys_from_topk, grouped_linear_, workloads
    from twinkle_amd.expert_lora import ExpertLoraSlots, experts_forward
    sel, _, tenant = workloads.moe_routing()
    tokens, top_k = sel.shape
    e, hid, inter, nt = 128, 2048, 768, 4
    dt = torch.bfloat16

    class Experts(torch.nn.Module):
        def __init__(self):
            super().__init__()
            g = torch.Generator().manual_seed(3)
            self.gate_up_proj = torch.nn.Parameter((torch.randn(e, 2 * inter, hid, generator=g) * 0.02).to(dt),
                                                   requires_grad=False)
            self.down_proj = torch.nn.Parameter((torch.randn(e, hid, inter, generator=g) * 0.02).to(dt),
                                                requires_grad=False)
            self.act_fn = torch.nn.functional.silu

    experts = Experts().to(dev)
    names = [f'lora_{i}' for i in range(nt)]
    gu = ExpertLoraSlots(e, hid, 2 * inter, max_loras=nt, max_r=8, dtype=dt, device=dev)
    dn = ExpertLoraSlots(e, inter, hid, max_loras=nt, max_r=8, dtype=dt, device=dev)
    for slots in (gu, dn):
        for name in names:
            slots.configure_slot(name, LoraConfig(r=8, lora_alpha=16))
            with torch.no_grad():
                slots.lora_B[name].normal_(0, 0.02)
    keys = flat_keys_from_topk(sel.to(dev), tenant.to(dev), nt)
    seg = build_segments(keys, e * nt, num_tokens=tokens)
    rows = tokens * top_k
    gen = torch.Generator().manual_seed(4)
    x0 = torch.randn(rows, hid, generator=gen).to(dt).to(dev)
    dy = torch.randn(rows, hid, generator=gen).to(dt).to(dev)

    def fwd(grouped):   # the loop leg keeps the reference's torch ops for the gate as well
        with torch.no_grad():
            experts_forward(experts, x0, seg, names, gu, dn, grouped=grouped, fused_activation=grouped)

    def fwd_bwd(grouped):
        x = x0.detach().requires_grad_(True)
        y = experts_forward(experts, x, seg, names, gu, dn, grouped=grouped, fused_activation=grouped)
        y.backward(dy)

    def base_only():
        y = grouped_linear_(x0, experts.gate_up_proj, seg, nt)
        grouped_linear_(y[:, :inter].contiguous(), experts.down_proj, seg, nt)

    # the whole block from the router's outputs: segment build, permute, experts, weighted unpermute, and back
    from twinkle_amd.expert_lora import moe_experts_block
    tok0 = torch.randn(tokens, hid, generator=gen).to(dt).to(dev)
    dtok = torch.randn(tokens, hid, generator=gen).to(dt).to(dev)
    sel_d, tenant_d = sel.to(dev), tenant.to(dev)
    rw = torch.softmax(torch.randn(tokens, top_k, generator=gen), -1).to(dt).to(dev)

    def block():
        t = tok0.detach().requires_grad_(True)
        out = moe_experts_block(t, sel_d, rw, tenant_d, experts, names, gu, dn)
        out.backward(dtok)

    res = {}
    for name, fn in (('loop_fwd_ms', lambda: fwd(False)), ('grouped_fwd_ms', lambda: fwd(True)),
                     ('loop_fwd_bwd_ms', lambda: fwd_bwd(False)), ('grouped_fwd_bwd_ms', lambda: fwd_bwd(True)),
                     ('grouped_gemms_alone_ms', base_only), ('block_from_router_fwd_bwd_ms', block)):
        # (MFMA-heavy launches run about 12 % slower during a process's first tens of milliseconds of them)
        for _ in range(3 if name.startswith('loop') else 20):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        res[name] = (time.perf_counter() - t0) * 1e3 / steps
    flops_fwd = 2 * rows * hid * (2 * inter) + 2 * rows * inter * hid       # the two base GEMMs
    res.update({'workload': f'{tokens} tokens x top-{top_k} of {e} experts, {hid} -> 2x{inter} -> {hid}, {nt} tenants '
                            'rank 8 on gate_up and down, bf16, rows in (expert, tenant) order',
                'base_gemm_flops_fwd': flops_fwd,
                'grouped_gemms_alone_tflops': flops_fwd / (res['grouped_gemms_alone_ms'] * 1e-3) / 1e12,
                'mfma_frac_grouped_gemms': flops_fwd / (res['grouped_gemms_alone_ms'] * 1e-3) / 1e12 / 2500.0,
                'speedup_fwd': res['loop_fwd_ms'] / res['grouped_fwd_ms'],
                'speedup_fwd_bwd': res['loop_fwd_bwd_ms'] / res['grouped_fwd_bwd_ms'],
                'routed_rows_per_s_fwd_bwd': rows / (res['grouped_fwd_bwd_ms'] * 1e-3),
                'tokens_per_s_block_fwd_bwd': tokens / (res['block_from_router_fwd_bwd_ms'] * 1e-3)})
    return res


def cfg5_layer_bench(dev, steps=5):
    """The seven projections of one Llama-3-8B-shaped layer (4096 hidden, 1024 k/v, 14336 intermediate) with LoRA
    rank 64 on all of them, 8 tenants, one per packed 4096-token sequence (T = 32768), bf16: forward + backward
    of the projection chain with the adapters off, on (one mixed batch), and on with q/k/v and gate/up declared
    as shared inputs.  The attention core has no adapter and is left out (q stands in for its output)."""
    import torch
    from torch import nn
    from twinkle_amd import LoraConfig, MultiLora

    class Projections(nn.Module):
        def __init__(self, d=4096, kv=1024, inter=14336):
            super().__init__()
            self.q_proj, self.k_proj, self.v_proj = nn.Linear(d, d, bias=False), nn.Linear(d, kv, bias=False), \
                nn.Linear(d, kv, bias=False)
            self.o_proj = nn.Linear(d, d, bias=False)
            self.gate_proj, self.up_proj = nn.Linear(d, inter, bias=False), nn.Linear(d, inter, bias=False)
            self.down_proj = nn.Linear(inter, d, bias=False)

        def forward(self, x):
            q, k, v = self.q_proj(x), self.k_proj(x), self.v_proj(x)
            h = x + self.o_proj(q) + (k.sum(-1, keepdim=True) + v.sum(-1, keepdim=True)) * 1e-3
            return h + self.down_proj(nn.functional.silu(self.gate_proj(h)) * self.up_proj(h))

    dt, seqs, toks, d = torch.bfloat16, 8, 4096, 4096
    torch.manual_seed(7)
    ml = MultiLora(max_loras=8, max_r=64, max_length=seqs * toks)
    model = ml.patch(Projections().to(dt).to(dev), target_modules='all-linear')
    for n, p in model.named_parameters():
        if 'lora_' not in n:
            p.requires_grad_(False)
        elif '.lora_B.' in n:
            with torch.no_grad():
                p.normal_(0, 0.02)
    names = [f'tenant_{i}' for i in range(8)]
    for n in names:
        ml.acquire_lora(n, LoraConfig(r=64, lora_alpha=128, target_modules='all-linear'))
    x = torch.randn(seqs * toks, d, device=dev, dtype=dt).requires_grad_(True)
    dy = torch.randn(seqs * toks, d, device=dev, dtype=dt)
    row_tenant = torch.repeat_interleave(torch.arange(8, device=dev), toks)

    def run(mode):
        if mode == 'base':
            with ml.adapter(names[0], disable_lora=True):
                y = model(x)
        else:
            with ml.batch(names, row_tenant):
                y = model(x)
        y.backward(dy)
        x.grad = None
        for p in model.parameters():
            p.grad = None

    res = {}
    for mode in ('base', 'lora', 'lora_shared_inputs'):
        if mode == 'lora_shared_inputs':
            ml.share_inputs([['model.q_proj', 'model.k_proj', 'model.v_proj'], ['model.gate_proj', 'model.up_proj']])
        for _ in range(2):
            run(mode)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            run(mode)
        torch.cuda.synchronize()
        res[mode + '_ms'] = (time.perf_counter() - t0) * 1e3 / steps
    ml.unshare_inputs()
    T = seqs * toks
    res.update({'tokens': T, 'lora_share_of_step': 1 - res['base_ms'] / res['lora_ms'],
                'tokens_per_s_with_lora': T / (res['lora_ms'] * 1e-3),
                'workload': 'Llama-3-8B-shaped projections (q, k, v, o, gate, up, down), rank 64, 8 tenants x 4096 packed '
                            'tokens, fwd + bwd; base weights frozen (dX only), attention core omitted'})
    return res


def cfg5_stack_bench(dev, layers=32, steps=2):
    """BASELINE config 5: a Llama-3-8B-shaped stack (hidden 4096, 32 heads / 8 KV heads, intermediate 14336, random
    init, bf16) with LoRA rank 64 on q, k, v, o, gate, up, down, 8 tenants, 8 packed sequences of 4096 tokens (tenant
    j owns sequence j), dY ~ N(0,1) at the final hidden state; activation checkpointing per layer (as the reference
    enables it).  Forward + backward per step with the adapters off and with all tenants in one mixed batch."""
    import torch
    from torch import nn
    from torch.utils.checkpoint import checkpoint
    from twinkle_amd import LoraConfig, MultiLora

    class RMSNorm(nn.Module):
        def __init__(self, d):
            super().__init__()
            self.weight = nn.Parameter(torch.ones(d))

        def forward(self, x):
            v = x.float()
            return (v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + 1e-5)).to(x.dtype) * self.weight

    class Layer(nn.Module):
        def __init__(self, d=4096, heads=32, kv_heads=8, inter=14336):
            super().__init__()
            self.heads, self.kv_heads, self.hd = heads, kv_heads, d // heads
            self.input_layernorm, self.post_attention_layernorm = RMSNorm(d), RMSNorm(d)
            self.q_proj = nn.Linear(d, d, bias=False)
            self.k_proj = nn.Linear(d, kv_heads * self.hd, bias=False)
            self.v_proj = nn.Linear(d, kv_heads * self.hd, bias=False)
            self.o_proj = nn.Linear(d, d, bias=False)
            self.gate_proj, self.up_proj = nn.Linear(d, inter, bias=False), nn.Linear(d, inter, bias=False)
            self.down_proj = nn.Linear(inter, d, bias=False)

        def forward(self, x):                                      # [sequences, tokens, d], causal per sequence
            b, s, _ = x.shape
            h = self.input_layernorm(x)
            q = self.q_proj(h).view(b, s, self.heads, self.hd).transpose(1, 2)
            k = self.k_proj(h).view(b, s, self.kv_heads, self.hd).transpose(1, 2)
            v = self.v_proj(h).view(b, s, self.kv_heads, self.hd).transpose(1, 2)
            rep = self.heads // self.kv_heads
            a = nn.functional.scaled_dot_product_attention(q, k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1),
                                                           is_causal=True)
            x = x + self.o_proj(a.transpose(1, 2).reshape(b, s, -1))
            h = self.post_attention_layernorm(x)
            return x + self.down_proj(nn.functional.silu(self.gate_proj(h)) * self.up_proj(h))

    class Stack(nn.Module):
        def __init__(self, n):
            super().__init__()
            self.layers = nn.ModuleList(Layer() for _ in range(n))
            self.norm = RMSNorm(4096)

        def forward(self, x):
            for layer in self.layers:
                x = checkpoint(layer, x, use_reentrant=False)
            return self.norm(x)

    dt, seqs, toks, d = torch.bfloat16, 8, 4096, 4096
    torch.manual_seed(7)
    with torch.device(dev):
        model = Stack(layers).to(dt)
    with torch.no_grad():
        for p in model.parameters():
            if p.dim() == 2:
                p.normal_(0, 0.02)
    ml = MultiLora(max_loras=8, max_r=64, max_length=seqs * toks)
    model = ml.patch(model, target_modules='all-linear')
    for n, p in model.named_parameters():
        if 'lora_' not in n:
            p.requires_grad_(False)
        elif '.lora_B.' in n:
            with torch.no_grad():
                p.normal_(0, 0.02)
    names = [f'tenant_{i}' for i in range(8)]
    for n in names:
        ml.acquire_lora(n, LoraConfig(r=64, lora_alpha=128, target_modules='all-linear'))
    x = torch.randn(seqs, toks, d, device=dev, dtype=dt).requires_grad_(True)
    dy = torch.randn(seqs, toks, d, device=dev, dtype=dt)
    row_tenant = torch.repeat_interleave(torch.arange(8, device=dev), toks)

    def run(mode):
        if mode == 'base':
            with ml.adapter(names[0], disable_lora=True):
                model(x).backward(dy)
        else:
            with ml.batch(names, row_tenant):
                model(x).backward(dy)
        x.grad = None
        for p in model.parameters():
            p.grad = None

    res = {}
    for mode in ('base', 'lora'):
        run(mode)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            run(mode)
        torch.cuda.synchronize()
        res[mode + '_ms'] = (time.perf_counter() - t0) * 1e3 / steps
        print(f'{mode}: {res[mode + "_ms"]:.1f} ms per step', file=sys.stderr, flush=True)
    T = seqs * toks
    res.update({'layers': layers, 'tokens': T, 'lora_share_of_step': 1 - res['base_ms'] / res['lora_ms'],
                'tokens_per_s_with_lora': T / (res['lora_ms'] * 1e-3), 'activation_checkpointing': True,
                'peak_memory_GiB': torch.cuda.max_memory_allocated() / 2**30,
                'workload': 'Llama-3-8B-shaped stack, LoRA rank 64 on 7 projections, 8 tenants x 4096 packed tokens, '
                            'fwd + recompute + bwd; base frozen'})
    return res


def build_workload(name, tokens=0, rank=0):
    """The synthetic batch of a named BASELINE configuration (see --workload)."""
    import torch
    from twinkle_amd import workloads
    if name == 'cfg2' and (tokens or rank):
        w = workloads.config2_qproj(tokens=tokens or 16384, r=rank or 16)
        w.name = f'cfg2 shape with T={w.tokens}, rank {max(w.ranks)}'
    elif name == 'cfg2':
        w = workloads.config2_qproj()
    elif name == 'cfg5_q':
        w = workloads.config2_qproj(tokens=32768, n=8, r=64)
        w.ids = torch.repeat_interleave(torch.arange(8, dtype=torch.int32), 4096)
        w.name = 'cfg5_llama8b_q_rank64'
    elif name == 'cfg4_gate_up':
        # expert LoRA shape: 8192 tokens x top-8 = 65536 routed rows, 128 experts x 4 tenants = 512 groups of rank 8,
        # hidden 2048 -> fused gate_up 1536; rows arrive sorted by (expert, tenant) like after the routing permute
        w = workloads.config2_qproj(tokens=65536, features=2048, n=512, r=8)
        w.ids = torch.sort(torch.randint(0, 512, (65536,), generator=torch.Generator().manual_seed(6)).to(torch.int32)).values
        w.lora_B = [b[:1536].contiguous() for b in w.lora_B]
        w.base_out, w.dy, w.out_features = w.base_out[:, :1536].contiguous(), w.dy[:, :1536].contiguous(), 1536
        w.name = 'cfg4_qwen3moe_gate_up_rank8'
    else:
        w = workloads.config3_mlp('up' if name == 'cfg3_up' else 'down')
    return w


class StepHarness:
    """Buffers of one workload on the GPU and its step: segment build + LoRA forward + LoRA backward (dX, dA, dB),
    the forward on one of `n_sets` rotated buffer sets and the backward on the set whose forward ran a step earlier."""

    def __init__(self, w, dev, n_sets, weights_f32=False):
        import torch
        from twinkle_amd import AdapterGroups, build_segments, lora_bwd_workspace_bytes, lora_fwd_, lora_h_bytes
        dt = torch.bfloat16
        self.w, self.dev = w, dev
        T, K, G = w.tokens, w.in_features, w.num_adapters
        self.ids = w.ids.to(dev)
        wdt = torch.float32 if weights_f32 else dt     # fp32 adapters under the bf16 activations (PEFT's default)
        A = [t.to(wdt).to(dev) for t in w.lora_A]
        B = [t.to(wdt).to(dev) for t in w.lora_B]
        self.groups = AdapterGroups(A, B, w.ranks, w.scales, act_dtype=dt)
        self.grad_a = [torch.zeros_like(t) for t in A]
        self.grad_b = [torch.zeros_like(t) for t in B]
        self.pa = torch.tensor([t.data_ptr() for t in self.grad_a], dtype=torch.int64, device=dev)
        self.pb = torch.tensor([t.data_ptr() for t in self.grad_b], dtype=torch.int64, device=dev)
        self.sets = []
        for i in range(n_sets):
            self.sets.append({
                'x': (w.x if i == 0 else torch.roll(w.x, i, 0)).to(dt).to(dev),
                'y': w.base_out.to(dt).to(dev),
                'dy': (w.dy if i == 0 else torch.roll(w.dy, i, 0)).to(dt).to(dev),
                'dx': torch.zeros(T, K, dtype=dt, device=dev),
                'h': None,
            })
        seg = build_segments(self.ids, G, want_perm=False, want_offsets=False)
        for s in self.sets:
            s['h'] = torch.empty(lora_h_bytes(seg, self.groups), dtype=torch.uint8, device=dev)
        self.ws = torch.empty(lora_bwd_workspace_bytes(seg, self.groups), dtype=torch.uint8, device=dev)
        self.seg = seg
        # every set needs a forward before its first backward
        for s in self.sets:
            lora_fwd_(s['x'], s['y'], seg, self.groups, h=s['h'])

    def step(self, i, ev=None):
        from twinkle_amd import build_segments, lora_bwd_, lora_expand_, lora_shrink_
        sets, groups = self.sets, self.groups
        f = sets[i % len(sets)]
        b = sets[(i + 1) % len(sets)]
        seg_i = build_segments(self.ids, self.w.num_adapters, want_perm=False, want_offsets=False)
        self.seg = seg_i
        if ev is not None:
            ev[0].record()
        lora_shrink_(f['x'], seg_i, groups, f['h'])     # tk_lora_fwd == these two calls
        if ev is not None:
            ev[1].record()
        lora_expand_(f['h'], f['y'], seg_i, groups)
        if ev is not None:
            ev[2].record()
        lora_bwd_(b['dy'], b['x'], b['h'], b['dx'], self.pa, self.pb, seg_i, groups, accumulate=False, workspace=self.ws)
        if ev is not None:
            ev[3].record()

    def time_steps(self, steps, warmup, first=0):
        """Wall clock around exactly `steps` steps behind `warmup` untimed ones, device synchronised on both sides."""
        import torch
        for i in range(warmup):
            self.step(first + i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            self.step(first + warmup + i)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps


def other_configs_bench(dev, steps=20, warmup=5):
    """The other single-projection BASELINE shapes, same step definition as the headline (measured, not bench lines)."""
    import gc
    import torch
    out = {}
    for name in ('cfg3_up', 'cfg3_down', 'cfg4_gate_up', 'cfg5_q'):
        w = build_workload(name)
        hs = StepHarness(w, dev, 2)
        ms = hs.time_steps(steps, warmup)
        nbytes = w.algorithmic_bytes(2)
        out[name] = {'workload': w.name, 'tokens': w.tokens, 'in': w.in_features, 'out': w.out_features,
                     'adapters': w.num_adapters, 'ranks': sorted(set(w.ranks)), 'steps': steps, 'ms_per_step': ms,
                     'tokens_per_s': w.tokens / (ms * 1e-3), 'algorithmic_bytes': nbytes,
                     'hbm_frac_step': nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     'tflops': w.flops() / (ms * 1e-3) / 1e12}
        del hs, w
        gc.collect()
        torch.cuda.empty_cache()
    return out


def _side_figure(fn):
    try:
        return fn()
    except Exception as e:  # noqa: BLE001
        return {'error': f'{type(e).__name__}: {e}'}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=10)
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--sets', type=int, default=3, help='rotated buffer sets')
    ap.add_argument('--workload', default='cfg2', choices=['cfg2', 'cfg3_up', 'cfg3_down', 'cfg5_q', 'cfg4_gate_up'],
                    help='cfg2 is the headline configuration; the others are the wider BASELINE shapes '
                         '(cfg3: 4096<->14336, T=32768, 32 adapters of rank 8..64; cfg5_q: 4096->4096, T=32768, 8 tenants '
                         'of rank 64, one per packed 4096-token sequence) for additional measurements')
    ap.add_argument('--tokens', type=int, default=0,
                    help='cfg2 with another number of tokens (a scaling measurement, not the headline configuration)')
    ap.add_argument('--rank', type=int, default=0,
                    help='cfg2 with another adapter rank (alpha = 2 x rank; a scaling measurement like --tokens)')
    ap.add_argument('--weights-f32', action='store_true',
                    help='keep the adapters and their gradients in fp32 under the bf16 activations')
    ap.add_argument('--optimizer-only', action='store_true',
                    help='run only the multi-tenant optimizer micro-benchmark and print its JSON (for profiling)')
    ap.add_argument('--shared-qkv', action='store_true',
                    help='run only the q / k / v micro-benchmark (one shared call against one call per projection)')
    ap.add_argument('--layer-cfg5', action='store_true',
                    help='run only the one-layer measurement of BASELINE config 5 (seven projections, rank 64)')
    ap.add_argument('--stack-cfg5', action='store_true',
                    help='run only the Llama-3-8B-shaped stack of BASELINE config 5 (see --layers)')
    ap.add_argument('--layers', type=int, default=32)
    ap.add_argument('--moe-experts', action='store_true',
                    help='run only the expert block of BASELINE config 4: per-expert loop against the grouped GEMMs')
    ap.add_argument('--yardstick', action='store_true',
                    help='run only the memory yardsticks: what the GPU sustains for the kernels\' access patterns')
    ap.add_argument('--calibrate-copy', action='store_true',
                    help='also run five plain 128 MiB device copies (a known-size kernel to scale rocprofv3 --pmc '
                         'FETCH_SIZE / WRITE_SIZE readings by)')
    args = ap.parse_args()
    if args.gpus != 1:
        print('bench.py measures one GPU: this path has no multi-GPU part (rows are independent and would shard trivially). '
              'Run with --gpus 1.', file=sys.stderr)
        sys.exit(2)

    import torch
    from twinkle_amd import (AdapterGroups, _lib, build_segments, lora_bwd_, lora_bwd_workspace_bytes, lora_expand_,
                             lora_fwd_, lora_h_bytes, lora_shrink_, workloads)
    if not torch.cuda.is_available():
        print('bench.py needs a GPU', file=sys.stderr)
        sys.exit(2)
    _lib.load()
    dev = torch.device('cuda:0')
    if args.optimizer_only:
        print(json.dumps({'optimizer_step': optimizer_step_bench(dev)}))
        return
    if args.yardstick:
        print(json.dumps({'yardstick': yardstick_bench(dev)}, indent=1))
        return
    if args.stack_cfg5:
        print(json.dumps({'cfg5_stack': cfg5_stack_bench(dev, layers=args.layers)}))
        return
    if args.layer_cfg5:
        print(json.dumps({'cfg5_layer': cfg5_layer_bench(dev)}))
        return
    if args.moe_experts:
        print(json.dumps({'moe_experts': moe_experts_bench(dev, steps=max(1, min(args.steps, 10)))}))
        return
    if args.shared_qkv:
        print(json.dumps({'shared_qkv': shared_qkv_bench(dev, calibrate_copy=args.calibrate_copy, rank=args.rank or 16,
                                                         weights_f32=args.weights_f32)}))
        return
    w = build_workload(args.workload, args.tokens, args.rank)
    if args.tokens or args.rank:
        args.tokens = w.tokens
    if args.workload != 'cfg2':
        args.sets = min(args.sets, 2)
    dt = torch.bfloat16
    elt = 2
    T, K, M, G = w.tokens, w.in_features, w.out_features, w.num_adapters
    if args.weights_f32:
        w.name += ', fp32 adapter weights and gradients'
    hs = StepHarness(w, dev, args.sets, weights_f32=args.weights_f32)
    sets, groups, step = hs.sets, hs.groups, hs.step

    # First timed region: exactly `steps` steps behind `warmup` untimed ones, with nothing but the step's own launches
    # on the stream -> ms_per_step.
    ms_per_step = hs.time_steps(args.steps, args.warmup)
    # Second timed region: the same `steps` steps again with HIP events around the kernels of every step (on the
    # launch stream).  An event record costs a few microseconds of idle queue, which is why these steps are not the
    # ones behind `value`; their own rate is reported as ms_per_step_with_events.
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    for i in range(args.steps):
        step(args.steps + i, events[i])
    torch.cuda.synchronize()
    ms_per_step_with_events = (time.perf_counter() - t1) * 1e3 / args.steps
    # What a pair of event records measures with nothing between them (the queue's handling of the two records, about
    # 5 us on this GPU), taken the same way behind a kernel.  Subtracting it from a bracketed interval gives an
    # estimate of the kernels' own duration; it is reported as a side figure only (the interval of the empty pair is
    # quantised and comes out a little above what the records cost around a kernel).
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(200)]
    for a, b in pairs:
        sets[0]['h'].zero_()
        a.record()
        b.record()
    torch.cuda.synchronize()
    pair_ms = sorted(a.elapsed_time(b) for a, b in pairs)[len(pairs) // 2]
    shrink_raw = sum(e[0].elapsed_time(e[1]) for e in events) / len(events)
    expand_raw = sum(e[1].elapsed_time(e[2]) for e in events) / len(events)
    bwd_raw = sum(e[2].elapsed_time(e[3]) for e in events) / len(events)
    shrink_ms, expand_ms, bwd_ms = shrink_raw - pair_ms, expand_raw - pair_ms, bwd_raw - pair_ms
    fwd_ms = shrink_ms + expand_ms
    # Third timed region, the one `roofline` is computed from: the dominant kernel's forward launch `run` times in a
    # row between ONE pair of events (buffer sets rotated, h as the steps above left it), so that what the records
    # cost is spread over `run` launches instead of sitting in every interval; repeated and averaged.
    run, reps = 20, 5
    seg_last = hs.seg
    expand_run_ms = []
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        lora_shrink_(sets[0]['x'], seg_last, groups, sets[0]['h'])
        for s_ in sets[1:]:
            s_['h'].copy_(sets[0]['h'])
        e0.record()
        for j in range(run):
            lora_expand_(sets[j % len(sets)]['h'], sets[j % len(sets)]['y'], seg_last, groups)
        e1.record()
        torch.cuda.synchronize()
        expand_run_ms.append(e0.elapsed_time(e1) / run)
    expand_launch_ms = sum(expand_run_ms) / len(expand_run_ms)

    if args.calibrate_copy:
        for _ in range(5):
            sets[0]['dx'].copy_(sets[1]['x'])      # reads T*K*2 bytes, writes T*K*2 bytes
        torch.cuda.synchronize()

    # base GEMM, reported separately and not part of the step
    wbase = torch.randn(M, K, device=dev, dtype=dt) * 0.02
    xs = sets[0]['x']
    for _ in range(3):
        torch.nn.functional.linear(xs, wbase)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(10):
        torch.nn.functional.linear(xs, wbase)
    e1.record()
    torch.cuda.synchronize()
    base_ms = e0.elapsed_time(e1) / 10

    step_bytes = w.algorithmic_bytes(elt)
    # one forward launch of the expand kernel: read + write y, read the live columns of every B
    expand_bytes = elt * T * 2 * M + elt * sum(r * M for r in w.ranks)
    flops = w.flops()
    # The dominant kernel's launch duration: the interval between the event records around it inside the timed steps,
    # less what the records themselves cost.  Two estimates of that cost exist in this run: the interval of an empty
    # pair of records (a little too much: it lands below the duration a kernel trace shows), and what four records
    # add to a step's wall clock, per record (a little too little).  The first is used, but never below the duration
    # of the same kernel in the committed kernel trace of this command (when that profile matches the sources);
    # the raw interval, both corrections and the back-to-back figure are all reported.
    per_record_ms = max(0.0, (ms_per_step_with_events - ms_per_step) / 4)
    traced_ms = traced_duration_ms('k_expand_mfma<1>') if (args.workload == 'cfg2' and not args.tokens and
                                                            not args.rank and not args.weights_f32) else None
    avg_launch_ms = expand_ms if traced_ms is None else max(expand_ms, traced_ms)
    if traced_ms is None:
        avg_launch_ms = expand_raw - per_record_ms
    achieved = expand_bytes / (avg_launch_ms * 1e-3) / 1e9
    traffic, traffic_source = (None, None)
    if args.workload == 'cfg2' and not args.tokens and not args.weights_f32:
        traffic, traffic_source = measured_traffic('k_expand_mfma<1>')
    out = {
        'metric': 'multi-LoRA fwd+bwd tokens/s + % roofline (HBM/MFMA), 8B proj, 16 adapters',
        'value': T / (ms_per_step * 1e-3),
        'unit': 'tokens/s',
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'ms_per_step': ms_per_step,
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': 'bf16',
        'data': 'synthetic',
        'config': {'workload': ('BASELINE config 2: Llama-3-8B q_proj 4096->4096, T=16384, 16 adapters rank 16 alpha 32, '
                                'Zipf(1.1) ids shuffled' if args.workload == 'cfg2' and not args.tokens else w.name) +
                               '; step = segment build + LoRA fwd + LoRA bwd (dX, dA, dB); base GEMM excluded',
                   'tokens': T, 'in': K, 'out': M, 'adapters': G, 'rank': max(w.ranks)},
        'roofline': {'bound': 'hbm', 'achieved': achieved, 'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
                     'frac': achieved / HBM_PEAK_GBS, 'traffic': traffic, 'traffic_source': traffic_source,
                     'kernel': ('k_expand_mfma<1>' if max(w.ranks) <= 16 else
                                f'k_expand_multi<{2 if max(w.ranks) <= 32 else 4},4>') + ' (y += h B^T in place), forward launch',
                     'algorithmic_bytes_per_launch': expand_bytes, 'avg_launch_ms': avg_launch_ms,
                     'launches_timed': len(events),
                     'timing': 'HIP events around the launch inside every timed step, on the launch stream; avg_launch_ms = '
                               'that interval less an empty pair of records, not below the kernel-trace duration of the '
                               'committed profile' if traced_ms is not None else
                               'HIP events around the launch inside every timed step, on the launch stream; avg_launch_ms = '
                               'that interval less the per-record cost seen in the step time',
                     'in_step_interval_ms': expand_raw, 'frac_from_in_step_interval': expand_bytes / (expand_raw * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     'empty_event_pair_ms': pair_ms, 'in_step_interval_minus_empty_pair_ms': expand_ms,
                     'per_record_cost_in_step_time_ms': per_record_ms,
                     'in_step_interval_minus_one_record_ms': expand_raw - per_record_ms,
                     'kernel_trace_profile_avg_ms': traced_ms, 'kernel_trace_profile': TRACE_PROFILE,
                     'back_to_back_launch_ms': expand_launch_ms,
                     'back_to_back_timing': f'{reps} runs of {run} launches in a row between one pair of events each (a launch '
                                            'right behind another in-place update runs a little slower than inside the step)'},
        'step_detail': {'ms_per_step_with_events': ms_per_step_with_events, 'empty_event_pair_ms': pair_ms, 'shrink_ms': shrink_ms, 'expand_ms': expand_ms, 'fwd_ms': fwd_ms, 'bwd_ms': bwd_ms, 'segment_build_and_gaps_ms': ms_per_step_with_events - fwd_ms - bwd_ms,
                        'algorithmic_bytes_per_step': step_bytes, 'flops_per_step': flops,
                        'tflops': flops / (ms_per_step * 1e-3) / 1e12,
                        'hbm_frac_step': step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
                        'hbm_frac_fwd_plus_bwd_kernels': step_bytes / ((fwd_ms + bwd_ms) * 1e-3) / 1e9 / HBM_PEAK_GBS,
                        'mfma_frac_step': flops / (ms_per_step * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                        'base_gemm_ms_excluded': base_ms},
    }
    if not args.no_cpu_baseline and args.workload == 'cfg2' and not args.tokens and not args.rank and not args.weights_f32:
        # the other BASELINE shapes and the expert block of config 4, after the headline leg (its buffers are freed)
        del hs, sets, groups, step, events, pairs
        import gc
        gc.collect()
        torch.cuda.empty_cache()
        # (side figures: a failure in one of them is reported in its place and does not take the headline line down)
        out['other_configs'] = _side_figure(lambda: other_configs_bench(dev))
        if 'error' not in out['other_configs']:
            out['other_configs']['cfg4_moe_experts_block'] = _side_figure(lambda: moe_experts_bench(dev, steps=2))
    if not args.no_cpu_baseline:
        out['optimizer_step'] = _side_figure(lambda: optimizer_step_bench(dev))
        out['torch_gpu_loop'] = _side_figure(lambda: torch_gpu_loop(w, dev, dt))
        out['cpu_baseline'] = cpu_baseline(w)
    print(json.dumps(out))


if __name__ == '__main__':
    main()
