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


# How far the HIP float32 result is from the float64 truth, next to how far the reference's OWN float32 arithmetic
# (the oracle run in float32: taps ascending as corr1ord.cuh:139-157, rows ascending as poolrgn.cuh:61-112) is from it.
# The reference sums gradients with atomics in no fixed order, so "the reference's bits" do not exist for them; what
# can be stated and tested is that the HIP result is no further from the truth than a float32 evaluation in reference
# order, up to the factor C_F32 (two independent roundings of the same sums differ by a small factor in their worst
# element). Both distances are floored at F32_FLOOR = 2^-22 of the block's largest value, two units in its last place:
# a block that the NumPy evaluation happens to get right to the last bit says nothing about the reference, whose
# device code is built with -use_fast_math (exponential and division each one to two units off) and stores float32.
# C_F32 = 8: over all configurations the worst ratio measured is 5.9, and every ratio above 3 is a bias gradient: ONE sum
# of a hundred-odd signed terms that cancel to a tenth of their size, where the last bits of either float32 evaluation
# are a matter of which order it happened to take; blocks of weights (hundreds of sums each) stay below 3.
C_F32 = 8.0
F32_FLOOR = 2.0 ** -22
VS_F32 = {}


def assert_no_further_than_f32_reference(config, kind, got, ref64, ref32, what="", c=C_F32):
    got = np.asarray(got, dtype=np.float64)
    ref64 = np.asarray(ref64, dtype=np.float64)
    ref32 = np.asarray(ref32, dtype=np.float64)
    assert got.shape == ref64.shape == ref32.shape, "%s shapes %s %s %s" % (what, got.shape, ref64.shape, ref32.shape)
    if ref64.size == 0:
        return
    scale = float(np.abs(ref64).max())
    if scale == 0.0:
        assert not got.any(), "%s: non-zero where the truth is all zero" % what
        return
    e_hip = float(np.abs(got - ref64).max()) / scale
    e_ref = float(np.abs(ref32 - ref64).max()) / scale
    ratio = e_hip / max(e_ref, F32_FLOOR)
    e = VS_F32.setdefault((config, kind), {"worst_ratio": 0.0, "hip_err": 0.0, "f32_ref_err": 0.0, "blocks": 0, "c": c})
    if ratio > e["worst_ratio"]:
        e["worst_ratio"], e["hip_err"], e["f32_ref_err"] = ratio, e_hip, e_ref
    e["blocks"] += 1
    assert ratio <= c, "%s: HIP is %.3e of the block's scale from the float64 result, the float32 reference %.3e (ratio %.1f > %g)" % (
        what, e_hip, e_ref, ratio, c)


# Pooling winners (argmax) that differ from the float32 evaluation in reference order, per configuration.
ARGMAX = {}


def record_argmax(config, got, ref):
    got, ref = np.asarray(got), np.asarray(ref)
    assert got.shape == ref.shape
    e = ARGMAX.setdefault(config, {"moved": 0, "total": 0})
    e["moved"] += int((got != ref).sum())
    e["total"] += int(ref.size)
    return int((got != ref).sum())


def random_codes(rng, N, pn=0.05, p254=0.0):
    X = rng.integers(0, 4, size=N).astype(np.uint8)
    u = rng.random(N)
    X[u < pn] = 255
    X[(u >= pn) & (u < pn + p254)] = 254
    return X
