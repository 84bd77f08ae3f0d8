"""Helpers for the GPU parity tests."""
import numpy as np
import torch


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def assert_close(got, ref, rel, what=""):
    """|got - ref| <= rel * max(|ref|, scale) elementwise, scale = largest magnitude in ref.

    Relative error against the array's own scale: sums of signed terms may cancel to values far
    below the terms' size, where a pure elementwise relative bound is meaningless.
    """
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, "%s shape %s vs %s" % (what, got.shape, ref.shape)
    scale = np.abs(ref).max() if ref.size else 0.0
    bound = rel * np.maximum(np.abs(ref), scale)
    err = np.abs(got - ref)
    bad = err > bound + 1e-30
    assert not bad.any(), "%s: %d / %d elements off, worst err %.3e (bound %.3e)" % (
        what, int(bad.sum()), bad.size, float(err.max()), float(bound.flat[err.argmax()]))


def random_codes(rng, N, pn=0.05, p254=0.0):
    X = rng.integers(0, 4, size=N).astype(np.uint8)
    u = rng.random(N)
    X[u < pn] = 255
    X[(u >= pn) & (u < pn + p254)] = 254
    return X
