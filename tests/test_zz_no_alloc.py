"""lbt_quantise_gradients_static: the quantiser with its scratch in a device array of the
library, for callers that cannot allocate. Called through the C ABI and compared, bit for bit,
with lbt_quantise_gradients (caller's workspace) on the same inputs: two calls in a row on the
same GPU, the second with a smaller input, so that nothing the first call left in the shared
array may leak into the second."""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _with_workspace(g, h, seed, row_offset):
    from lbtree import _lib

    n, k = g.shape
    ws = torch.empty(_lib.lib.lbt_quantise_gradients_workspace_bytes(n, k), dtype=torch.uint8, device=g.device)
    q = torch.empty((n, k, 2), dtype=torch.int32, device=g.device)
    sums = torch.empty((k, 2), dtype=torch.int64, device=g.device)
    scales = torch.empty(4, dtype=torch.float64, device=g.device)
    _lib.check(_lib.lib.lbt_quantise_gradients(_stream(), g.data_ptr(), h.data_ptr(), n, k, row_offset, seed,
                                               q.data_ptr(), sums.data_ptr(), scales.data_ptr(), ws.data_ptr(),
                                               ws.numel()))
    return q, sums, scales


def _static(g, h, seed, row_offset, out):
    from lbtree import _lib

    n, k = g.shape
    q, sums, scales = out
    return _lib.lib.lbt_quantise_gradients_static(_stream(), g.data_ptr(), h.data_ptr(), n, k, row_offset, seed,
                                                  q.data_ptr(), sums.data_ptr(), scales.data_ptr())


def test_static_scratch_quantiser_equals_the_workspace_one():
    from lbtree import _lib

    rs = np.random.RandomState(5)
    # the first call fills two levels of partial sums (3,000,000 x 3 entries = 2198 chunks of 4096)
    shapes = [(3_000_000, 3, 1234, 0), (70_001, 2, 99, 5_000_000), (1, 1, 7, 0)]
    inputs = []
    for n, k, seed, off in shapes:
        g = torch.from_numpy(rs.normal(size=(n, k))).cuda()
        h = torch.from_numpy(rs.rand(n, k) + 0.05).cuda()
        h[::7] *= -1.0  # hessians of either sign
        inputs.append((g, h, seed, off))
    want = [_with_workspace(*a) for a in inputs]
    # outputs are allocated before the calls: the calls themselves must not allocate
    outs = [(torch.empty_like(w[0]), torch.empty_like(w[1]), torch.empty_like(w[2])) for w in want]
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    for a, o in zip(inputs, outs):  # back to back on one stream, no synchronisation in between
        _lib.check(_static(*a, o))
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    for (q, sums, scales), (wq, wsums, wscales) in zip(outs, want):
        assert torch.equal(q, wq)
        assert torch.equal(sums, wsums)
        assert torch.equal(scales, wscales)
    # once more in the other order: what the larger call left behind does not matter either way
    for a, o, w in reversed(list(zip(inputs, outs, want))):
        for t in o:
            t.zero_()
        _lib.check(_static(*a, o))
        torch.cuda.synchronize()
        assert torch.equal(o[0], w[0]) and torch.equal(o[1], w[1]) and torch.equal(o[2], w[2])


def test_static_scratch_quantiser_rejects_what_it_cannot_hold():
    from lbtree import _lib

    g = torch.zeros((4, 1), dtype=torch.float64, device="cuda")
    q = torch.empty((4, 1, 2), dtype=torch.int32, device="cuda")
    sums = torch.empty((1, 2), dtype=torch.int64, device="cuda")
    scales = torch.empty(4, dtype=torch.float64, device="cuda")
    limit = _lib.LBT_QUANTISE_STATIC_MAX_ENTRIES
    # sizes beyond the array are refused before anything is launched (the pointers are never followed)
    rc = _lib.lib.lbt_quantise_gradients_static(_stream(), g.data_ptr(), g.data_ptr(), limit // 2 + 1, 2, 0, 1,
                                                q.data_ptr(), sums.data_ptr(), scales.data_ptr())
    assert rc == -1
    msg = _lib.lib.lbt_last_error().decode()
    assert str(limit) in msg and "lbt_quantise_gradients" in msg
    with pytest.raises(_lib.LbtError):
        _lib.check(_lib.lib.lbt_quantise_gradients_static(_stream(), None, g.data_ptr(), 4, 1, 0, 1, q.data_ptr(),
                                                          sums.data_ptr(), scales.data_ptr()))
    # and the call still works afterwards
    g.fill_(0.5)
    _lib.check(_lib.lib.lbt_quantise_gradients_static(_stream(), g.data_ptr(), g.data_ptr(), 4, 1, 0, 1, q.data_ptr(),
                                                      sums.data_ptr(), scales.data_ptr()))
    torch.cuda.synchronize()
    wq, wsums, wscales = _with_workspace(g, g, 1, 0)
    assert torch.equal(q, wq) and torch.equal(sums, wsums) and torch.equal(scales, wscales)
