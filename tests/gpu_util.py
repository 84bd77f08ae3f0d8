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


def model_blocks(a, nmodel, axis):
    """The per-model blocks of an array whose models are laid out along `axis`."""
    return np.split(np.asarray(a), nmodel, axis=axis)


def assert_close_per_model(got, ref, rel, nmodel, axis, what=""):
    """assert_close on every model's own block, with that block's own scale: a model whose values are
    orders of magnitude below its neighbours' is still checked to `rel` of ITS largest magnitude."""
    for b, (g, r) in enumerate(zip(model_blocks(got, nmodel, axis), model_blocks(ref, nmodel, axis))):
        assert_close(g, r, rel, "%s [model %d]" % (what, b))


# Worst elementwise relative errors seen by the parity tests, printed in the run's summary
# (tests/conftest.py) and written as parity_elementwise.json to the run's output folder when there is one.
# err_rel = |got - ref| / max(|ref|, FLOOR_FRAC * max|ref| of the compared block): a pure elementwise ratio
# is meaningless where a sum of signed terms cancels to ~0, so magnitudes below a thousandth of the block's
# largest are measured against that floor; `share_within` is the share of elements inside the stated
# tolerance with NO floor at all.
FLOOR_FRAC = 1e-3
REPORT = {}


def record_error(config, kind, got, ref, tol):
    got = np.asarray(got, dtype=np.float64).ravel()
    ref = np.asarray(ref, dtype=np.float64).ravel()
    if ref.size == 0:
        return
    scale = np.abs(ref).max()
    if scale == 0:
        return
    err = np.abs(got - ref)
    floored = float((err / np.maximum(np.abs(ref), FLOOR_FRAC * scale)).max())
    nz = np.abs(ref) > 0
    within = float(((err[nz] / np.abs(ref[nz])) <= tol).mean()) if nz.any() else 1.0
    e = REPORT.setdefault((config, kind), {"worst_rel_err": 0.0, "share_within": 1.0, "tol": tol, "elements": 0,
                                            "floor": "%g x block max" % FLOOR_FRAC})
    e["worst_rel_err"] = max(e["worst_rel_err"], floored)
    e["share_within"] = (e["share_within"] * e["elements"] + within * ref.size) / (e["elements"] + ref.size)
    e["elements"] += int(ref.size)


def random_codes(rng, N, pn=0.05, p254=0.0):
    X = rng.integers(0, 4, size=N).astype(np.uint8)
    u = rng.random(N)
    X[u < pn] = 255
    X[(u >= pn) & (u < pn + p254)] = 254
    return X
