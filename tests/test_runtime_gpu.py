"""The library's per-stream scratch: more distinct streams than it has slots, and a clear error (not a broken
capture) when scratch would have to grow on a stream that is capturing."""
import ctypes
import os

import numpy as np
import pytest
import torch

from tests.gpu_util import dev, host

pytestmark = pytest.mark.gpu


def _hip():
    return ctypes.CDLL(os.path.join(os.path.dirname(torch.__file__), "lib", "libamdhip64.so"))


def test_scratch_slots_are_recycled_beyond_64_streams():
    """Column sums need scratch for their row-slice partial sums. 70 distinct streams each get a working
    buffer: once the 64 slots are taken, the one used longest ago passes on."""
    from deepbind_amd import _lib
    hip = _hip()
    hip.hipStreamCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    hip.hipStreamDestroy.argtypes = [ctypes.c_void_p]
    hip.hipStreamSynchronize.argtypes = [ctypes.c_void_p]
    rng = np.random.default_rng(0)
    A = rng.standard_normal((5000, 48)).astype(np.float32)
    Ad = dev(A)
    want = A.astype(np.float64).sum(axis=0)
    torch.cuda.synchronize()
    streams = []
    try:
        for i in range(70):
            s = ctypes.c_void_p()
            assert hip.hipStreamCreate(ctypes.byref(s)) == 0
            streams.append(s)
            out = torch.full((1, 48), np.nan, dtype=torch.float32, device="cuda")
            torch.cuda.synchronize()
            _lib.call("dbk_colsum", s, _lib.DBK_F32, _lib.ptr(Ad), _lib.ptr(out), 5000, 48)
            assert hip.hipStreamSynchronize(s) == 0
            np.testing.assert_allclose(host(out).ravel(), want, rtol=1e-4, err_msg="stream %d" % i)
        # the first stream lost its slot long ago and gets one again
        out = torch.empty((1, 48), dtype=torch.float32, device="cuda")
        _lib.call("dbk_colsum", streams[0], _lib.DBK_F32, _lib.ptr(Ad), _lib.ptr(out), 5000, 48)
        assert hip.hipStreamSynchronize(streams[0]) == 0
        np.testing.assert_allclose(host(out).ravel(), want, rtol=1e-4)
    finally:
        torch.cuda.synchronize()
        for s in streams:
            hip.hipStreamDestroy(s)


def test_scratch_allocation_under_capture_is_refused_with_a_clear_error():
    """A stream that has no scratch yet cannot get it while capturing (allocating would break the capture):
    the call fails with a message that says so; after one eager call on that stream the capture goes through."""
    from deepbind_amd import _lib, smat as sm
    hip = _hip()
    hip.hipStreamCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    hip.hipStreamDestroy.argtypes = [ctypes.c_void_p]
    raw = ctypes.c_void_p()
    assert hip.hipStreamCreate(ctypes.byref(raw)) == 0
    side = torch.cuda.ExternalStream(raw.value)
    A = torch.ones((5000, 64), dtype=torch.float32, device="cuda")           # several row slices: needs partial sums
    torch.cuda.synchronize()
    try:
        g = torch.cuda.CUDAGraph()
        err = None
        with torch.cuda.graph(g, stream=side, capture_error_mode="thread_local"):
            try:
                sm.sum_axis0(A)
            except _lib.DeepbindError as e:          # caught inside, so that the capture itself ends normally
                err = str(e)
        assert err is not None and "capturing" in err, err
        del g
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            sm.sum_axis0(A)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side, capture_error_mode="thread_local"):
            out = sm.sum_axis0(A)
        for _ in range(2):
            g.replay()
            torch.cuda.synchronize()
            assert np.array_equal(host(out).ravel(), np.full(64, 5000, np.float32))
        del g
    finally:
        torch.cuda.synchronize()
        hip.hipStreamDestroy(raw)


def test_scratch_of_a_captured_graph_survives_slot_recycling():
    """A graph captured on a stream keeps the addresses of that stream's scratch. 70 further streams then ask for
    scratch of their own (more than there are slots): the captured stream's slot is not handed on, and a replay of the
    graph afterwards still gives the right sums. A larger eager call on the captured stream gets a new buffer; the one
    the graph refers to is set aside, not freed: the replay after it is still right."""
    from deepbind_amd import _lib, smat as sm
    hip = _hip()
    hip.hipStreamCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
    hip.hipStreamDestroy.argtypes = [ctypes.c_void_p]
    hip.hipStreamSynchronize.argtypes = [ctypes.c_void_p]
    raw = ctypes.c_void_p()
    assert hip.hipStreamCreate(ctypes.byref(raw)) == 0
    side = torch.cuda.ExternalStream(raw.value)
    rng = np.random.default_rng(1)
    A = rng.standard_normal((5000, 64)).astype(np.float32)
    Ad = dev(A)
    other = dev(rng.standard_normal((5000, 48)).astype(np.float32))
    streams = []
    try:
        with torch.cuda.stream(side):
            first = host(sm.sum_axis0(Ad))                                  # eager: the stream's scratch exists from here on
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side, capture_error_mode="thread_local"):
            out = sm.sum_axis0(Ad)
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(host(out), first)
        for i in range(70):
            s_ = ctypes.c_void_p()
            assert hip.hipStreamCreate(ctypes.byref(s_)) == 0
            streams.append(s_)
            junk = torch.empty((1, 48), dtype=torch.float32, device="cuda")
            _lib.call("dbk_colsum", s_, _lib.DBK_F32, _lib.ptr(other), _lib.ptr(junk), 5000, 48)
            assert hip.hipStreamSynchronize(s_) == 0
        out.fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(host(out), first)
        # a call whose partial sums (5.8 MB) do not fit the stream's first buffer (1 MB), on that stream and on another
        from deepbind_amd import deepity_smat as ds
        n, nb, k, h = 20000, 4, 16, 32
        t = lambda *shape: torch.randn(shape, dtype=torch.float32, device="cuda") * 0.1
        pooled, W1, b1, W2, b2, Y = t(n, k * nb), t(k * nb, h), t(1, h * nb), t(h * nb, 1), t(1, nb), (t(n, nb) > 0).float()
        grads = lambda: (torch.empty_like(W1), torch.empty_like(b1), torch.empty_like(W2), torch.empty_like(b2))
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            Zs, _, _ = ds.head_train(pooled, W1, b1, W2, b2, Y, nb, "nll", *grads())
        torch.cuda.synchronize()
        Z, _, _ = ds.head_train(pooled, W1, b1, W2, b2, Y, nb, "nll", *grads())
        assert bool(torch.isfinite(Z).all()) and torch.equal(Z, Zs)
        out.fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(host(out), first)
        del g
    finally:
        torch.cuda.synchronize()
        for s_ in streams:
            hip.hipStreamDestroy(s_)
        hip.hipStreamDestroy(raw)
