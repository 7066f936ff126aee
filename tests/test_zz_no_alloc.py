"""ddf_hip_backward_static: the backward entry point that allocates nothing.

Called through the C ABI and held, bit for bit, to ddf_hip_backward with a
caller-allocated workspace (same kernels, same cut of the problem), on two
calls in a row that share the built-in scratch buffer - the second with a
smaller input, so that stale contents of the first would show."""
import ctypes

import pytest
import torch

from ddfnet_amd import _lib
from ddf_testlib import random_case

pytestmark = pytest.mark.gpu

STATIC_BYTES = 16 * 1024 * 1024


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _backward_both_ways(shape, k, d, s, combine, dtype, need=7, seed=0):
    N, C, H, W = shape
    x, cf, sf, go = (t.cuda() for t in random_case(N, C, H, W, k, s, dtype, seed=seed))
    lib = _lib.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    tail = (N, C, H, W, k, d, s, _lib.COMBINE[combine], _lib.DTYPE[dtype])
    want_bytes = _lib.backward_workspace_bytes(shape, k, d, s, combine, dtype, need)
    ws = torch.empty(max(want_bytes, 1), dtype=torch.uint8, device='cuda')
    ref = [torch.full_like(t, float('nan')) for t in (x, cf, sf)]
    rc = lib.ddf_hip_backward(_ptr(go), _ptr(x), _ptr(cf), _ptr(sf), _ptr(ref[0]), _ptr(ref[1]),
                              _ptr(ref[2]), _ptr(ws), want_bytes, *tail, need, 0, stream)
    assert rc == 0, lib.ddf_hip_last_error()
    got = [torch.full_like(t, float('nan')) for t in (x, cf, sf)]
    rc = lib.ddf_hip_backward_static(_ptr(go), _ptr(x), _ptr(cf), _ptr(sf), _ptr(got[0]),
                                     _ptr(got[1]), _ptr(got[2]), *tail, need, 0, stream)
    assert rc == 0, lib.ddf_hip_last_error()
    torch.cuda.synchronize()
    return want_bytes, ref, got


@pytest.mark.parametrize('first,second,k,d,s,combine,dtype', [
    ((8, 64, 14, 14), (3, 24, 14, 14), 3, 1, 1, 'mul', torch.float32),   # one-launch backward, dSF partials
    ((4, 32, 56, 56), (2, 16, 28, 28), 3, 1, 1, 'add', torch.float16),   # dX + filters, dCF partials over strips
    ((4, 32, 28, 28), (2, 8, 12, 12), 5, 2, 1, 'mul', torch.float32),    # tile kernels
    ((4, 32, 57, 57), (2, 9, 30, 30), 3, 1, 2, 'mul', torch.float32),    # stride 2, odd size
])
def test_static_backward_equals_workspace_backward(first, second, k, d, s, combine, dtype):
    used = 0
    for shape, seed in ((first, 1), (second, 2)):   # back to back, the second one smaller
        want_bytes, ref, got = _backward_both_ways(shape, k, d, s, combine, dtype, seed=seed)
        used = max(used, want_bytes)
        assert want_bytes <= STATIC_BYTES
        for name, a, b in zip(('dX', 'dCF', 'dSF'), ref, got):
            assert torch.isfinite(b).all(), name
            assert torch.equal(a, b), name
    assert used > 0, 'no case here exercised the scratch buffer'


def test_static_backward_rejects_what_does_not_fit():
    lib = _lib.lib()
    shape, k, d, s, combine, dtype = (64, 512, 112, 112), 5, 1, 1, 'mul', torch.float32
    need_bytes = _lib.backward_workspace_bytes(shape, k, d, s, combine, dtype, 7)
    assert need_bytes > STATIC_BYTES
    N, C, H, W = shape
    dummy = ctypes.c_void_p(256)   # never dereferenced: the size check comes first
    rc = lib.ddf_hip_backward_static(dummy, dummy, dummy, dummy, dummy, dummy, dummy, N, C, H, W,
                                     k, d, s, 0, _lib.DTYPE[dtype], 7, 0, None)
    assert rc == 3   # DDF_ERR_WORKSPACE
    assert b'ddf_hip_backward_static holds' in lib.ddf_hip_last_error()


def test_static_backward_allocates_nothing_and_replays_in_a_graph():
    """The reason the entry point exists: a call leaves the device's free memory and
    torch's allocator untouched, and it can be recorded into a HIP graph (which
    forbids allocation) and replayed."""
    shape, k, d, s, combine, dtype, need = (8, 64, 14, 14), 3, 1, 1, 'mul', torch.float32, 7
    N, C, H, W = shape
    assert _lib.backward_workspace_bytes(shape, k, d, s, combine, dtype, need) > 0
    x, cf, sf, go = (t.cuda() for t in random_case(N, C, H, W, k, s, dtype, seed=5))
    lib = _lib.lib()
    tail = (N, C, H, W, k, d, s, _lib.COMBINE[combine], _lib.DTYPE[dtype])
    got = [torch.full_like(t, float('nan')) for t in (x, cf, sf)]

    def call(stream):
        rc = lib.ddf_hip_backward_static(_ptr(go), _ptr(x), _ptr(cf), _ptr(sf), _ptr(got[0]),
                                         _ptr(got[1]), _ptr(got[2]), *tail, need, 0,
                                         ctypes.c_void_p(stream.cuda_stream))
        assert rc == 0, lib.ddf_hip_last_error()

    call(torch.cuda.current_stream())        # first call on the device: looks the array up
    torch.cuda.synchronize()
    eager = [t.clone() for t in got]
    free_before, allocated_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
    reserved_before = torch.cuda.memory_reserved()
    call(torch.cuda.current_stream())
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.cuda.memory_allocated() == allocated_before
    assert torch.cuda.memory_reserved() == reserved_before

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(torch.cuda.current_stream())    # (the capture stream)
    for _ in range(3):
        for t in got:
            t.fill_(float('nan'))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(('dX', 'dCF', 'dSF'), eager, got):
            assert torch.equal(a, b), name
