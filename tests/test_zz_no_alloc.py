"""tk_lora_fwd_noalloc: the forward for callers that cannot allocate, against tk_lora_fwd, through the C ABI."""
import ctypes

import pytest
import torch

from twinkle_amd import AdapterGroups, _lib, build_segments
from twinkle_amd.ops import _desc

pytestmark = pytest.mark.gpu


def _case(dev, dtype, t, k, m, n, max_r, ranks, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(t, k, generator=g).to(dtype).to(dev)
    base = torch.randn(t, m, generator=g).to(dtype).to(dev)
    a = [((torch.rand(max_r, k, generator=g) * 2 - 1) / k**0.5).to(dtype).to(dev) for _ in range(n)]
    b = [(torch.randn(m, max_r, generator=g) * 0.05).to(dtype).to(dev) for _ in range(n)]
    ids = torch.randint(-1, n, (t,), generator=g).to(torch.int32).to(dev)       # some rows without an adapter
    seg = build_segments(ids, n, want_perm=False, want_offsets=False)
    groups = AdapterGroups(a, b, ranks, [2.0 if i % 2 == 0 else 0.5 for i in range(n)])
    return x, base, seg, groups


def _both(lib, x, base, seg, groups):
    """(y of tk_lora_fwd with a caller-owned h, y of tk_lora_fwd_noalloc, free device memory around the latter)."""
    d = _desc(seg, groups, True)
    stream = _lib.stream_ptr()
    need = lib.tk_lora_h_bytes(ctypes.byref(d))
    assert 0 < need <= _lib.TK_NOALLOC_SCRATCH_BYTES
    h = torch.empty(need, dtype=torch.uint8, device=x.device)
    y_ref, y_new = base.clone(), base.clone()
    assert lib.tk_lora_fwd(ctypes.byref(d), x.data_ptr(), x.stride(0), y_ref.data_ptr(), y_ref.stride(0), h.data_ptr(),
                           stream) == _lib.TK_OK
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    assert lib.tk_lora_fwd_noalloc(ctypes.byref(d), x.data_ptr(), x.stride(0), y_new.data_ptr(), y_new.stride(0),
                                   stream) == _lib.TK_OK
    torch.cuda.synchronize()
    free_after = torch.cuda.mem_get_info()[0]
    return y_ref, y_new, free_before, free_after


@pytest.mark.parametrize('dtype,shapes', [
    # two calls in a row on the library's one buffer, the second with a smaller problem
    (torch.bfloat16, [(6000, 2048, 1024, 5, 16, [16, 8, 0, 16, 3]), (700, 512, 256, 3, 16, [16, 4, 9])]),
    (torch.bfloat16, [(3000, 1024, 512, 4, 64, [64, 33, 16, 40]), (33, 256, 128, 2, 32, [32, 20])]),
    (torch.float32, [(900, 200, 72, 3, 8, [8, 3, 5]), (40, 24, 40, 2, 4, [4, 1])]),
])
def test_noalloc_forward_equals_the_forward_with_a_caller_buffer(dev, dtype, shapes):
    lib = _lib.load()
    for i, (t, k, m, n, max_r, ranks) in enumerate(shapes):
        x, base, seg, groups = _case(dev, dtype, t, k, m, n, max_r, ranks, seed=100 + i)
        y_ref, y_new, free_before, free_after = _both(lib, x, base, seg, groups)
        assert torch.equal(y_ref, y_new), f'call {i}: {t} rows'
        assert (y_new.float() - base.float()).abs().max() > 0
        if i > 0:         # the first call on a GPU may load the library's device code; later calls hold nothing new
            assert free_after == free_before, 'the call changed the amount of free device memory'


def test_noalloc_forward_rejects_what_does_not_fit(dev):
    """16384 rows at rank 64 over 8192 input features need more than the built-in buffer: a clear error, y untouched."""
    lib = _lib.load()
    t, k, m, n, r = 16384, 8192, 128, 2, 64
    a = [torch.zeros(r, k, dtype=torch.bfloat16, device=dev) for _ in range(n)]
    b = [torch.zeros(m, r, dtype=torch.bfloat16, device=dev) for _ in range(n)]
    seg = build_segments(torch.zeros(t, dtype=torch.int32, device=dev), n, want_perm=False, want_offsets=False)
    groups = AdapterGroups(a, b, [r] * n, [1.0] * n)
    d = _desc(seg, groups, True)
    assert lib.tk_lora_h_bytes(ctypes.byref(d)) > _lib.TK_NOALLOC_SCRATCH_BYTES
    x = torch.ones(t, k, dtype=torch.bfloat16, device=dev)
    y = torch.ones(t, m, dtype=torch.bfloat16, device=dev)
    code = lib.tk_lora_fwd_noalloc(ctypes.byref(d), x.data_ptr(), x.stride(0), y.data_ptr(), y.stride(0),
                                   _lib.stream_ptr())
    assert code == _lib.TK_ERR_SCRATCH and b'scratch' in lib.tk_error_string(code)
    torch.cuda.synchronize()
    assert torch.all(y == 1)
    from twinkle_amd import lora_fwd_noalloc_
    with pytest.raises(RuntimeError, match='scratch'):
        lora_fwd_noalloc_(x, y, seg, groups)


def test_noalloc_forward_in_a_hip_graph(dev):
    """The caller it is for: a warm-up call outside the capture (the first call on a GPU looks up the address of
    the library's buffer), then the same call captured in a HIP graph and replayed with eager work and
    synchronisations between the replays; every replay equals tk_lora_fwd."""
    lib = _lib.load()
    x, base, seg, groups = _case(dev, torch.bfloat16, 2500, 1024, 512, 4, 16, [16, 8, 16, 5], seed=300)
    d = _desc(seg, groups, True)
    h = torch.empty(lib.tk_lora_h_bytes(ctypes.byref(d)), dtype=torch.uint8, device=dev)
    want = base.clone()
    assert lib.tk_lora_fwd(ctypes.byref(d), x.data_ptr(), x.stride(0), want.data_ptr(), want.stride(0), h.data_ptr(),
                           _lib.stream_ptr()) == _lib.TK_OK
    y = torch.empty_like(base)

    def step():
        y.copy_(base)
        code = lib.tk_lora_fwd_noalloc(ctypes.byref(d), x.data_ptr(), x.stride(0), y.data_ptr(), y.stride(0),
                                       _lib.stream_ptr())
        assert code == _lib.TK_OK

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        step()                                   # warm-up on the capture stream, outside the capture
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            step()
    torch.cuda.current_stream().wait_stream(side)
    for _ in range(3):
        y.fill_(3)                               # eager work between the replays (a fill kernel)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want)
