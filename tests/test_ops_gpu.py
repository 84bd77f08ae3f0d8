"""GPU parity: every operator of the C-ABI library, called through the Python surface, against the
CPU oracle on the same seeded inputs. Tolerances: float32 activations 1e-5 and gradients 1e-4
relative to the array's scale; indices and masks bit-exact; the unfused scan is bit-exact because it
accumulates taps in the reference's order."""
import numpy as np
import pytest
import torch

from oracle import deepbind_oracle as orc
from tests.gpu_util import (assert_close, assert_no_further_than_f32_reference as assert_vs_f32, dev, host, random_codes,
                            record_argmax, record_error)

pytestmark = pytest.mark.gpu

ACT, GRAD = 1e-5, 1e-4


@pytest.fixture(scope="module")
def ks():
    from deepbind_amd import kangaroo_smat
    return kangaroo_smat


@pytest.fixture(scope="module")
def ds():
    from deepbind_amd import deepity_smat
    return deepity_smat


@pytest.fixture(scope="module")
def sm():
    from deepbind_amd import smat
    return smat


# ------------------------------------------------------------------------------------------ scan
@pytest.mark.parametrize("N,m,F", [(300, 24, 16), (1000, 16, 64), (777, 5, 70), (24, 24, 3), (5000, 24, 200), (130, 32, 17),
                                   # many rows of 17-24 taps: the four-filters-per-lane kernel (16-byte stores; scalar stores when
                                   # the filter count is no multiple of four; a last tile with one filter)
                                   (70400, 24, 256), (140100, 19, 70), (263000, 24, 17), (70400, 16, 256), (140100, 9, 70)])
def test_corr1ord_bit_exact(ks, N, m, F):
    rng = np.random.default_rng(N + m + F)
    X = random_codes(rng, N, 0.05, 0.03)
    W = (rng.standard_normal((4 * m, F)) * 0.1).astype(np.float32)
    Zr = np.full((N, F), 5.0, np.float32)
    orc.corr1ord(W, X, Zr)
    Z = dev(np.full((N, F), 5.0, np.float32))
    ks.corr1ord(dev(W), dev(X.reshape(-1, 1)), Z, 4)
    assert np.array_equal(host(Z), Zr)


def test_exact_scan_switch_keeps_the_reference_bits_at_bulk_sizes(ks):
    """With the library's exact-scan switch on, a map of more than 2^25 values comes out with the bits of the
    reference's tap order (what smaller maps always get), the two gradients come from the vector kernels, and the
    same rows give the same bits whether they arrive in a small batch or a bulk one."""
    N, m, F = 140000, 24, 256
    rng = np.random.default_rng(5)
    X = random_codes(rng, N, 0.05, 0.03)
    W = (rng.standard_normal((4 * m, F)) * 0.1).astype(np.float32)
    Zr = np.zeros((N, F), np.float32)
    orc.corr1ord(W, X, Zr)
    Wd, Xd = dev(W), dev(X.reshape(-1, 1))
    Zfast = dev(np.zeros((N, F), np.float32))
    ks.corr1ord(Wd, Xd, Zfast, 4)
    assert not np.array_equal(host(Zfast), Zr)                      # bulk size: the matrix-core kernel, equal to round-off only
    assert_close(host(Zfast), Zr.astype(np.float64), ACT, "bulk map, default path")
    dZ = dev(rng.standard_normal((N, F)).astype(np.float32))
    grads = {}
    assert ks.set_exact_scan(True) is False
    try:
        Z = dev(np.zeros((N, F), np.float32))
        ks.corr1ord(Wd, Xd, Z, 4)
        assert np.array_equal(host(Z), Zr)
        n_small = 3000                                              # the same leading rows as a small batch of their own
        Zs = dev(np.zeros((n_small, F), np.float32))
        ks.corr1ord(Wd, dev(X[:n_small].reshape(-1, 1)), Zs, 4)
        assert np.array_equal(host(Zs)[: n_small - m + 1], Zr[: n_small - m + 1])
        for name, fn, shape in (("dW", lambda out: ks.corr1ord_bprop_W(out, Xd, dZ, 4), W.shape),
                                ("dX", lambda out: ks.corr1ord_bprop_X(out, Wd, dZ, 4), (N, 4))):
            out = dev(np.zeros(shape, np.float32))
            fn(out)
            grads[name] = host(out)
    finally:
        assert ks.set_exact_scan(False) is True
    for name, fn, shape in (("dW", lambda out: ks.corr1ord_bprop_W(out, Xd, dZ, 4), W.shape),
                            ("dX", lambda out: ks.corr1ord_bprop_X(out, Wd, dZ, 4), (N, 4))):
        out = dev(np.zeros(shape, np.float32))
        fn(out)
        fast = host(out)
        assert not np.array_equal(fast, grads[name]), "%s: the switch did not change the kernel" % name
        assert_close(fast, grads[name].astype(np.float64), GRAD, "%s, matrix-core vs vector kernel" % name)
    dWr = np.zeros(W.shape); orc.corr1ord_bprop_W(dWr, X, host(dZ).astype(np.float64))
    assert_close(grads["dW"], dWr, GRAD, "dW with the switch on vs the oracle")


@pytest.mark.parametrize("N,m,F", [(300000, 24, 128), (600001, 11, 70), (1100000, 32, 32)])
def test_corr1ord_bulk_sizes_on_the_matrix_cores(ks, N, m, F):
    """From 2^25 map values on, float32 maps come from the matrix-core kernel: the same sums in another order, so the
    comparison is to round-off; rows past N - m + 1 stay untouched, codes 254 / 255 are in the input."""
    rng = np.random.default_rng(N + m + F)
    X = random_codes(rng, N, 0.05, 0.03)
    W = (rng.standard_normal((4 * m, F)) * 0.1).astype(np.float32)
    Zr = np.full((N, F), 5.0, np.float64)
    orc.corr1ord(W.astype(np.float64), X, Zr)
    Z = dev(np.full((N, F), 5.0, np.float32))
    ks.corr1ord(dev(W), dev(X.reshape(-1, 1)), Z, 4)
    got = host(Z)
    assert np.all(got[N - m + 1:] == 5.0)
    assert_close(got[: N - m + 1], Zr[: N - m + 1], ACT, "map")
    Z2 = dev(np.full((N, F), 5.0, np.float32))
    ks.corr1ord(dev(W), dev(X.reshape(-1, 1)), Z2, 4)
    assert np.array_equal(host(Z2), got)


def test_corr1ord_float64_and_short_input(ks):
    rng = np.random.default_rng(1)
    X = random_codes(rng, 400, 0.1)
    W = rng.standard_normal((4 * 7, 33))
    Zr = np.zeros((400, 33)); orc.corr1ord(W, X, Zr)
    Z = dev(np.zeros((400, 33)))
    ks.corr1ord(dev(W), dev(X), Z, 4)
    assert np.array_equal(host(Z), Zr)
    # fewer symbols than taps: nothing is written
    Z2 = dev(np.ones((3, 33)))
    ks.corr1ord(dev(W), dev(X[:3]), Z2, 4)
    assert np.all(host(Z2) == 1.0)


def test_corr1ord_rejects_bad_arguments(ks):
    from deepbind_amd._lib import DeepbindError
    W = dev(np.zeros((12, 4), np.float32))
    X = dev(np.zeros(20, np.uint8))
    with pytest.raises(DeepbindError):
        ks.corr1ord(W, X, dev(np.zeros((20, 5), np.float32)), 4)       # wrong number of columns
    with pytest.raises(DeepbindError):
        ks.corr1ord(W, X, dev(np.zeros((20, 4), np.float32)), 3)       # no kernel for 3 channels
    with pytest.raises(DeepbindError):
        ks.corr1ord(W, dev(np.zeros(20, np.float32)), dev(np.zeros((20, 4), np.float32)), 4)


@pytest.mark.parametrize("N,m,F,dense,dtype", [(400, 24, 16, True, np.float32), (3000, 16, 100, True, np.float32),
                                               (2000, 24, 64, False, np.float32), (50, 7, 5, True, np.float32),
                                               (70000, 24, 200, True, np.float32), (900, 30, 40, True, np.float32),
                                               (60001, 11, 70, True, np.float32), (40000, 32, 160, True, np.float32),
                                               (33000, 5, 130, False, np.float32),
                                               (600, 24, 33, True, np.float64), (20, 24, 8, True, np.float32)])
def test_corr1ord_bprop_W(ks, N, m, F, dense, dtype):
    """Several chunks per workgroup (N = 70000), the any-length kernel (m = 30), float64, a stream shorter than the
    filter (no row defined: the gradient is zero), and bulk sizes, which go through the matrix-core kernel (from
    4 M gradient values on: tap counts that fill one to four 32-row blocks of dW, filters that do not fill a block)."""
    rng = np.random.default_rng(N + F)
    X = random_codes(rng, N, 0.05, 0.02)
    dZ = rng.standard_normal((N, F)).astype(dtype)
    if not dense:
        dZ[rng.random((N, F)) < 0.98] = 0                              # 1-sparse-like, as after max pooling
    ref = np.zeros((4 * m, F), np.float64)
    orc.corr1ord_bprop_W(ref, X, dZ.astype(np.float64))
    dW = dev(np.ones((4 * m, F), dtype))                               # accumulates onto existing content
    ks.corr1ord_bprop_W(dW, dev(X), dev(dZ), 4)
    assert_close(host(dW), ref + 1.0, GRAD if dtype == np.float32 else 1e-12, "dW")
    # run-to-run bit stability (no float atomics)
    dW2 = dev(np.ones((4 * m, F), dtype))
    ks.corr1ord_bprop_W(dW2, dev(X), dev(dZ), 4)
    assert np.array_equal(host(dW), host(dW2))


@pytest.mark.parametrize("n,m,F,dtype", [(300, 24, 48, np.float32), (1000, 11, 130, np.float32), (97, 5, 64, np.float32),
                                         (5000, 24, 256, np.float32), (3, 16, 7, np.float32), (50, 30, 20, np.float32),
                                         (400, 24, 70, np.float64),
                                         (40000, 24, 256, np.float32), (70001, 11, 130, np.float32), (66000, 32, 64, np.float32),
                                         (33003, 5, 200, np.float32)])
def test_corr1ord_bprop_X(ks, n, m, F, dtype):
    """Row counts around the per-wave block of 96 rows, several filter tiles, fewer rows than taps, the
    any-length kernel (m = 30) and float64; accumulates into dX and is bit-stable. From 4 M gradient values on
    (float32, at least 64 filters) the matrix-core kernel: one to four blocks of taps, filter counts that are no
    multiple of 128 or of 4, row counts that are no multiple of a workgroup's 1024 rows."""
    rng = np.random.default_rng(5 + n)
    W = (rng.standard_normal((4 * m, F)) * 0.1).astype(dtype)
    dZ = rng.standard_normal((n, F)).astype(dtype)
    ref = np.ones((n, 4)); orc.corr1ord_bprop_X(ref, W.astype(np.float64), dZ.astype(np.float64))
    dX = dev(np.ones((n, 4), dtype))
    ks.corr1ord_bprop_X(dX, dev(W), dev(dZ), 4)
    assert_close(host(dX), ref, GRAD if dtype == np.float32 else 1e-12, "dX")
    dX2 = dev(np.ones((n, 4), dtype))
    ks.corr1ord_bprop_X(dX2, dev(W), dev(dZ), 4)
    assert np.array_equal(host(dX), host(dX2))


# ------------------------------------------------------------------------------------------ pooling
def _regions(rng, P, lo, hi, gap=0):
    lens = rng.integers(lo, hi + 1, size=P)
    edges = np.concatenate([[0], np.cumsum(lens + gap)])
    return np.stack([edges[:-1], edges[:-1] + lens], axis=1).astype(np.uint32), int(edges[-1])


@pytest.mark.parametrize("ptype", ["max", "avg", "sum", "all"])
@pytest.mark.parametrize("F", [16, 100])
def test_poolrgn_forward_and_backward(ks, ptype, F):
    rng = np.random.default_rng(F)
    R, N = _regions(rng, 37, 1, 60)
    U = rng.standard_normal((N, F)).astype(np.float32)
    U[3] = U[1]                                                        # exact tie: first row must win
    Zr, Ir = orc.poolrgn(U, R, ptype, want_argmax=True)
    Z, I = ks.poolrgn(dev(U), dev(R), ptype, want_argmax=True)
    if ptype in ("max", "all"):
        assert np.array_equal(host(I), Ir)
        got = host(Z)
        assert np.array_equal(got if ptype == "max" else got[:, 0::2], Zr if ptype == "max" else Zr[:, 0::2])
    else:
        assert I is None
    assert_close(host(Z), Zr, ACT, "pooled")
    Z0, I0 = ks.poolrgn(dev(U), dev(R), ptype, want_argmax=False)
    assert I0 is None and np.array_equal(host(Z0), host(Z))
    dP = rng.standard_normal(Zr.shape).astype(np.float32)
    ref = np.ones((N, F), np.float32); orc.poolrgn_bprop(ref, R, dP, Ir, ptype)
    dU = dev(np.ones((N, F), np.float32))
    ks.poolrgn_bprop(dU, dev(R), dev(dP), I, ptype)
    assert_close(host(dU), ref, ACT, "dU")


def test_poolrgn_step_and_overlapping_regions(ks):
    rng = np.random.default_rng(9)
    U = rng.standard_normal((64, 8)).astype(np.float32)
    R = np.array([[0, 20, 3], [10, 40, 2], [5, 64, 7]], np.uint32)      # strided and overlapping
    for ptype in ("max", "avg", "all"):
        Zr, Ir = orc.poolrgn(U, R, ptype, want_argmax=True)
        Z, I = ks.poolrgn(dev(U), dev(R), ptype, want_argmax=True)
        assert_close(host(Z), Zr, ACT, ptype)
        if Ir is not None:
            assert np.array_equal(host(I), Ir)
        dP = rng.standard_normal(Zr.shape).astype(np.float32)
        ref = np.zeros_like(U); orc.poolrgn_bprop(ref, R, dP, Ir, ptype)
        dU = dev(np.zeros_like(U))
        ks.poolrgn_bprop(dU, dev(R), dev(dP), I, ptype)
        assert_close(host(dU), ref, GRAD, "dU " + ptype)


# ------------------------------------------------------------------------------------------ fused scan + pool
def _chain_oracle(W, b, X, R, ptype):
    Z = np.zeros((X.size, W.shape[1]), W.dtype)
    orc.corr1ord(W, X, Z)
    A = orc.relu_fprop(orc.bias_fprop(Z, b))
    P, I = orc.poolrgn(A, R, ptype, want_argmax=True)
    return A, P, I


def _tied_winners(A, got, ref):
    """The device's pooling winners after checking that each one that differs from the oracle's is a round-off tie:
    same column, and a map value within the activation tolerance of the oracle's winner."""
    moved = got != ref
    F = A.shape[1]
    assert np.array_equal(got[moved] % F, ref[moved] % F), "argmax in another column"
    va, vb = A.ravel()[got[moved]], A.ravel()[ref[moved]]
    assert np.all(np.abs(va - vb) <= ACT * np.abs(A).max()), "argmax differs off a tie"
    assert moved.mean() < 0.01
    return got


def _fused_case(seed, B, lo, hi, m, F, pn=0.03, p254=0.0):
    rng = np.random.default_rng(seed)
    lens = rng.integers(lo, hi + 1, size=B)
    ords = [random_codes(rng, int(n), pn, p254) for n in lens]
    from deepbind_amd import data
    X, R = data.pack_ordinals(ords, m - 1)
    W = (rng.standard_normal((4 * m, F)) * 0.1).astype(np.float32)
    b = (rng.standard_normal((1, F)) * 0.05).astype(np.float32)
    return rng, W, b, X, R


@pytest.mark.parametrize("general", [True, False])
@pytest.mark.parametrize("ptype", ["max", "avg", "all"])
@pytest.mark.parametrize("B,lo,hi,m,F", [(64, 101, 101, 24, 16), (128, 38, 41, 16, 16), (40, 20, 40, 24, 144), (9, 1, 300, 11, 70)])
def test_scanpool_fprop(ks, general, ptype, B, lo, hi, m, F):
    path = "general" if general else "auto"
    rng, W, b, X, R = _fused_case(B + m + F, B, lo, hi, m, F, p254=0.01)
    A, Pr, Ir = _chain_oracle(W, b, X, R, ptype)
    P, I = ks.scanpool_fprop(dev(W), dev(b), dev(X), dev(R), ptype, want_argmax=True, path=path)
    assert_close(host(P), Pr, ACT, "pooled")
    if Ir is not None:
        got = host(I)
        same = got == Ir
        if not same.all():
            # only an exact or round-off tie may move the argmax: the map values must agree to tolerance
            va, vb = A.ravel()[got[~same]], A.ravel()[Ir[~same]]
            assert np.all(np.abs(va - vb) <= ACT * np.abs(A).max()), "argmax differs off a tie"
            assert (~same).mean() < 0.01
        # each index addresses the right column and a row of its own region
        rows, cols = got // F, got % F
        assert np.array_equal(cols, np.tile(np.arange(F), (len(R), 1)))
        assert np.all(rows >= R[:, :1]) and np.all(rows < R[:, 1:2])


@pytest.mark.parametrize("ptype", ["max", "avg", "all"])
@pytest.mark.parametrize("B,lo,hi,m,F", [(64, 101, 101, 24, 16), (40, 20, 40, 24, 144), (23, 0, 300, 17, 70), (300, 30, 70, 20, 64),
                                          (128, 38, 41, 16, 16), (50, 0, 200, 9, 130), (200, 30, 70, 13, 64)])
def test_scanpool_fprop_wide_kernel(ks, ptype, B, lo, hi, m, F):
    """The many-regions forward kernel (four filters per lane, a wave per region), forced on small inputs: against
    the unfused chain, and bit for bit against the one-filter-per-lane kernel where the two add in the same order
    (maxima, argmax, activity masks); regions of 0 to 300 rows, both tap tiers (9-16, 17-24), code 254 and N present, filter counts that leave
    lanes and whole quarters of a tile empty."""
    rng, W, b, X, R = _fused_case(B + m + F + 1, B, lo, hi, m, F, p254=0.01)
    A, Pr, Ir = _chain_oracle(W, b, X, R, ptype)
    Wd, bd, Xd, Rd = dev(W), dev(b), dev(X), dev(R)
    act_w, act_n = ks.activity_words(Xd, Wd), ks.activity_words(Xd, Wd)
    act_w.fill_(-1), act_n.fill_(-1)
    P, I = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=True, path="wide", act=act_w)
    Pn, In = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=True, path="general", act=act_n)   # few regions: the narrow kernel
    keep = R[:, 1] > R[:, 0]                                          # an empty region's average is 0/0
    assert_close(host(P)[keep], Pr[keep], ACT, "pooled")
    got, ref = host(P), host(Pn)
    if ptype == "max":
        assert np.array_equal(got, ref)
    elif ptype == "all":
        assert np.array_equal(got[:, 0::2], ref[:, 0::2])
        assert_close(got[keep][:, 1::2], ref[keep][:, 1::2], ACT, "averages, wide vs narrow")
    if I is not None:
        assert np.array_equal(host(I), host(In))
    # masks: the rows inside regions carry the same bits; every other word is left alone
    aw, an = host(act_w), host(act_n)
    assert np.array_equal(aw, an)
    inside = np.zeros(len(X), bool)
    for a_, b_ in R:
        inside[a_:b_] = True
    assert np.all(aw[~inside] == -1)
    # without argmax and without masks (other template instances)
    P2, _ = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=False, path="wide")
    assert np.array_equal(host(P2)[keep], got[keep])


@pytest.mark.parametrize("m", [24, 16, 30])
def test_scanpool_general_path_picks_the_matrix_core_kernel_for_many_regions(ks, m):
    """From 512 (region, tile) items on, the general path runs the matrix-core kernel: same bits as forcing it."""
    rng, W, b, X, R = _fused_case(5, 1100, 18, 40, m, 40, p254=0.01)
    Wd, bd, Xd, Rd = dev(W), dev(b), dev(X), dev(R)
    for ptype in ("max", "avg", "all"):
        P, I = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=True, path="general")
        Pw, Iw = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=True, path="mfma")
        assert np.array_equal(host(P), host(Pw))
        if I is not None:
            assert np.array_equal(host(I), host(Iw))
        A, Pr, Ir = _chain_oracle(W, b, X, R, ptype)
        assert_close(host(P), Pr, ACT, "pooled " + ptype)


@pytest.mark.parametrize("ptype", ["max", "avg", "all"])
@pytest.mark.parametrize("B,lo,hi,m,F", [(64, 101, 101, 24, 16), (128, 38, 41, 16, 16), (40, 20, 40, 24, 144), (9, 1, 300, 11, 70),
                                          (17, 0, 9, 5, 33), (25, 60, 90, 32, 64), (30, 10, 50, 1, 40), (20, 30, 64, 20, 100)])
def test_scanpool_fprop_matrix_core_kernel(ks, ptype, B, lo, hi, m, F):
    """The scan as a product on the matrix cores (weights as three exact bf16 pieces): pooled values, argmax and the
    activity masks against the operator chain; bits may differ from the lookup kernels' only where values tie to round-off."""
    rng, W, b, X, R = _fused_case(B + m + F + 1, B, lo, hi, m, F, p254=0.01)
    A, Pr, Ir = _chain_oracle(W.astype(np.float64), b.astype(np.float64), X, R, ptype)
    Wd, bd, Xd, Rd = dev(W), dev(b), dev(X), dev(R)
    act = ks.activity_words(Xd, Wd); act.fill_(-1)
    P, I = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=True, path="mfma", act=act)
    assert_close(host(P), Pr, ACT, "pooled")
    scale = np.abs(A).max()
    if Ir is not None:
        got = host(I)
        same = got == Ir
        if not same.all():
            va, vb = A.ravel()[got[~same]], A.ravel()[Ir[~same]]
            assert np.all(np.abs(va - vb) <= ACT * scale), "argmax differs off a tie"
            assert (~same).mean() < 0.01
        rows, cols = got // F, got % F
        assert np.array_equal(cols, np.tile(np.arange(F), (len(R), 1)))
        assert np.all(rows >= R[:, :1]) and np.all((rows < R[:, 1:2]) | (R[:, 1:2] == R[:, :1]))
    # masks: bit f of word (row, tile) <=> rectifier open, for rows inside a region; rows outside stay untouched
    Z = np.zeros((X.size, F)); orc.corr1ord(W.astype(np.float64), X, Z)
    pre = Z + b.astype(np.float64)
    words = host(act).view(np.uint64).reshape(X.size, -1)
    bits = ((words[:, :, None] >> np.arange(64, dtype=np.uint64)[None, None, :]) & np.uint64(1)).reshape(X.size, -1)[:, :F].astype(bool)
    inside = np.zeros(X.size, bool)
    for a_, b_ in R:
        inside[a_:b_] = True
    clear = np.abs(pre) > ACT * scale                                  # away from a round-off tie with zero
    assert np.array_equal(bits[inside][clear[inside]], (pre > 0)[inside][clear[inside]])
    assert np.all(words[~inside] == np.uint64(0xFFFFFFFFFFFFFFFF))
    P2, _ = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=False, path="mfma")
    assert np.array_equal(host(P), host(P2))


@pytest.mark.parametrize("path", ["auto", "mfma"])
def test_scanpool_regions_past_the_end_and_gaps(ks, path):
    """Arbitrary (non-packed) regions, including rows the scan does not define (relu(bias) there), regions that
    overlap, a region longer than the matrix-core kernel's chunk of 192 rows and one of exactly 32 rows."""
    rng = np.random.default_rng(77)
    m, F, N = 8, 20, 520
    X = random_codes(rng, N, 0.1)
    W = rng.standard_normal((4 * m, F)).astype(np.float32)
    b = rng.standard_normal((1, F)).astype(np.float32)
    R = np.array([[0, 10], [50, 51], [30, 90], [100, 120], [5, 6], [120, 520], [200, 232], [500, 520], [64, 257]], np.uint32)
    for ptype in ("max", "avg", "all"):
        A, Pr, Ir = _chain_oracle(W.astype(np.float64), b.astype(np.float64), X, R, ptype)
        P, I = ks.scanpool_fprop(dev(W), dev(b), dev(X), dev(R), ptype, want_argmax=True, path=path)
        assert_close(host(P), Pr, ACT, ptype)
        if Ir is not None:
            got = host(I)
            same = got == Ir
            assert np.all(np.abs(A.ravel()[got[~same]] - A.ravel()[Ir[~same]]) <= ACT * np.abs(A).max())


@pytest.mark.parametrize("ptype", ["max", "avg", "all"])
@pytest.mark.parametrize("B,lo,hi,m,F", [(64, 101, 101, 24, 16), (128, 38, 41, 16, 16), (30, 20, 40, 24, 144), (33, 1, 300, 11, 70),
                                          (17, 0, 9, 5, 33), (25, 200, 300, 7, 64), (12, 480, 520, 30, 40), (40, 90, 110, 2, 8)])
def test_scanpool_bprop(ks, ptype, B, lo, hi, m, F):
    rng, W, b, X, R = _fused_case(B + F, B, lo, hi, m, F)
    A, Pr, Ir = _chain_oracle(W.astype(np.float64), b.astype(np.float64), X, R, ptype)
    dP = rng.standard_normal(Pr.shape).astype(np.float32)
    dA = np.zeros_like(A)
    orc.poolrgn_bprop(dA, R, dP.astype(np.float64), Ir, ptype)
    dZ = orc.relu_bprop(dA, A)
    dbr = orc.bias_bprop(dZ)[1]
    dWr = np.zeros(W.shape); orc.corr1ord_bprop_W(dWr, X, dZ)
    Wd, bd, Xd, Rd = dev(W), dev(b), dev(X), dev(R)
    P, I = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=True)
    if Ir is not None and not np.array_equal(host(I), Ir):
        # a winner moved between rows that tie to round-off: the gradient is checked for the winners the device chose
        Ir = _tied_winners(A, host(I), Ir)
        dA = np.zeros_like(A)
        orc.poolrgn_bprop(dA, R, dP.astype(np.float64), Ir, ptype)
        dZ = orc.relu_bprop(dA, A)
        dbr = orc.bias_bprop(dZ)[1]
        dWr = np.zeros(W.shape); orc.corr1ord_bprop_W(dWr, X, dZ)
    dW = dev(np.ones(W.shape, np.float32)); db = dev(np.full((1, F), 7.0, np.float32))
    ks.scanpool_bprop(Wd, bd, Xd, Rd, ptype, P, I, dev(dP), dW, db)
    assert_close(host(dW), dWr + 1.0, GRAD, "dW")
    assert_close(host(db), dbr, GRAD, "db")                            # written, not accumulated
    dW2 = dev(np.ones(W.shape, np.float32)); db2 = dev(np.zeros((1, F), np.float32))
    ks.scanpool_bprop(Wd, bd, Xd, Rd, ptype, P, I, dev(dP), dW2, db2)
    assert np.array_equal(host(dW), host(dW2)) and np.array_equal(host(db), host(db2))


@pytest.mark.parametrize("ptype,stepped", [("sum", False), ("max", True), ("avg", True), ("sum", True), ("all", True)])
@pytest.mark.parametrize("B,lo,hi,m,F", [(64, 101, 101, 24, 16), (33, 1, 300, 11, 70), (17, 0, 9, 5, 33)])
def test_scanpool_sum_pooling_and_stepped_regions(ks, ptype, stepped, B, lo, hi, m, F):
    """What the fused kernels do not take - sum pooling, a third region column (row step) - goes through the same two
    calls and comes out as the reference's operator chain gives it, forward and backward."""
    rng, W, b, X, R = _fused_case(B + F + 3, B, lo, hi, m, F, p254=0.01)
    if stepped:
        R = np.concatenate([R, rng.integers(1, 5, size=(len(R), 1)).astype(np.uint32)], axis=1)
    A, Pr, Ir = _chain_oracle(W.astype(np.float64), b.astype(np.float64), X, R, ptype)
    Wd, bd, Xd, Rd = dev(W), dev(b), dev(X), dev(R)
    P, I = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=True)
    assert_close(host(P), Pr, ACT, "pooled")
    assert (I is None) == (Ir is None)
    if Ir is not None and not np.array_equal(host(I), Ir):
        Ir = _tied_winners(A, host(I), Ir)                             # (the gradient is checked for the winners the device chose)
    dP = rng.standard_normal(Pr.shape).astype(np.float32)
    dA = np.zeros_like(A)
    orc.poolrgn_bprop(dA, R, dP.astype(np.float64), Ir, ptype)
    dZ = orc.relu_bprop(dA, A)
    dbr = orc.bias_bprop(dZ)[1]
    dWr = np.zeros(W.shape); orc.corr1ord_bprop_W(dWr, X, dZ)
    for overwrite in (False, True):
        dW = dev(np.ones(W.shape, np.float32)); db = dev(np.full((1, F), 7.0, np.float32))
        ks.scanpool_bprop(Wd, bd, Xd, Rd, ptype, P, I, dev(dP), dW, db, overwrite=overwrite)
        assert_close(host(dW), dWr + (0.0 if overwrite else 1.0), GRAD, "dW")
        assert_close(host(db), dbr, GRAD, "db")
    with pytest.raises(Exception, match="operator chain"):
        ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, path="general")


@pytest.mark.parametrize("ptype,stepped", [("max", False), ("avg", False), ("all", False), ("sum", True)])
def test_scanpool_float64(ks, ptype, stepped):
    """The two fused calls with float64 tensors (the reference compiles every operator for both float types): the
    operator kernels in double precision inside the library, forward and backward against the float64 oracle chain
    at float64 accuracy."""
    rng, W, b, X, R = _fused_case(91, 40, 5, 120, 13, 37, p254=0.01)
    if stepped:
        R = np.concatenate([R, rng.integers(1, 4, size=(len(R), 1)).astype(np.uint32)], axis=1)
    W, b = W.astype(np.float64), b.astype(np.float64)
    A, Pr, Ir = _chain_oracle(W, b, X, R, ptype)
    Wd, bd, Xd, Rd = dev(W), dev(b), dev(X), dev(R)
    P, I = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=True)
    assert P.dtype == torch.float64
    assert_close(host(P), Pr, 1e-13, "pooled")
    if Ir is not None:
        assert np.array_equal(host(I), Ir)
    dP = rng.standard_normal(Pr.shape)
    dA = np.zeros_like(A)
    orc.poolrgn_bprop(dA, R, dP, Ir, ptype)
    dZ = orc.relu_bprop(dA, A)
    dWr = np.zeros(W.shape); orc.corr1ord_bprop_W(dWr, X, dZ)
    dW, db = dev(np.ones(W.shape)), dev(np.full((1, W.shape[1]), 7.0))
    ks.scanpool_bprop(Wd, bd, Xd, Rd, ptype, P, I, dev(dP), dW, db)
    assert_close(host(dW), dWr + 1.0, 1e-12, "dW")
    assert_close(host(db), orc.bias_bprop(dZ)[1], 1e-12, "db")
    with pytest.raises(Exception, match="both be float32 or both float64"):
        ks.scanpool_fprop(Wd, dev(b.astype(np.float32)), Xd, Rd, ptype)


def test_scanpool_unfused_chain_agrees_with_the_fused_kernels(ks):
    """Step 1 in the third column is the 2-column case: the chain and the fused kernels then compute the same function."""
    rng, W, b, X, R = _fused_case(77, 40, 20, 60, 16, 48)
    R3 = np.concatenate([R, np.ones((len(R), 1), np.uint32)], axis=1)
    Wd, bd, Xd = dev(W), dev(b), dev(X)
    for ptype in ("max", "avg", "all"):
        P, I = ks.scanpool_fprop(Wd, bd, Xd, dev(R), ptype, want_argmax=True)
        Pc, Ic = ks.scanpool_fprop(Wd, bd, Xd, dev(R3), ptype, want_argmax=True)
        assert_close(host(Pc), host(P), ACT, "pooled " + ptype)
        if I is not None:
            assert (host(I) == host(Ic)).mean() > 0.99
        dP = dev(rng.standard_normal(tuple(P.shape)).astype(np.float32))
        dW, db, dWc, dbc = (dev(np.zeros(s, np.float32)) for s in (W.shape, (1, 48), W.shape, (1, 48)))
        ks.scanpool_bprop(Wd, bd, Xd, dev(R), ptype, P, I, dP, dW, db, overwrite=True)
        ks.scanpool_bprop(Wd, bd, Xd, dev(R3), ptype, P, I, dP, dWc, dbc, overwrite=True)
        assert_close(host(dWc), host(dW), GRAD, "dW " + ptype)
        assert_close(host(dbc), host(db), GRAD, "db " + ptype)


@pytest.mark.parametrize("ptype", ["avg", "all"])
@pytest.mark.parametrize("B,lo,hi,m,F", [(64, 101, 101, 24, 16), (128, 38, 41, 16, 16), (33, 1, 300, 11, 70), (17, 0, 9, 5, 33),
                                          (25, 200, 300, 7, 64), (40, 20, 40, 24, 144), (12, 480, 520, 30, 40)])
def test_scanpool_bprop_with_activity_masks_equals_recomputation(ks, ptype, B, lo, hi, m, F):
    """The forward pass can leave one bit per (row, filter) - rectifier open or not - and the backward pass
    then skips recomputing the map: it counts the open rows per (tap, letter) and multiplies once where the
    recomputing kernel adds the same gradient row by row, so the two agree to rounding. Also
    checks the masks themselves against the oracle's activation map, with letters that contribute nothing
    (code 254) and regions that end where the stream ends."""
    rng, W, b, X, R = _fused_case(3 * B + F, B, lo, hi, m, F, p254=0.02)
    Wd, bd, Xd, Rd = dev(W), dev(b), dev(X), dev(R)
    act = ks.activity_words(Xd, Wd)
    act.fill_(-1)                                                      # rows outside every region keep this
    P0, I0 = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=True, path="general")
    P1, I1 = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=True, act=act)
    assert np.array_equal(host(P0), host(P1))
    if I0 is not None:
        assert np.array_equal(host(I0), host(I1))
    # bit l of word [row, tile] <=> activation of filter 64*tile + l is positive (to round-off: skip values near 0)
    A, _, _ = _chain_oracle(W.astype(np.float64), b.astype(np.float64), X, R, ptype)
    words = host(act).view(np.uint64)
    inside = np.zeros(len(X), bool)
    for a_, b_ in R[:, :2]:
        inside[a_:b_] = True
    assert (words[~inside] == np.uint64(0xFFFFFFFFFFFFFFFF)).all()
    rows = np.nonzero(inside)[0]
    bits = ((words[rows][:, np.arange(F) // 64] >> (np.arange(F) % 64).astype(np.uint64)) & np.uint64(1)).astype(bool)
    Zpre = np.zeros((len(X), F))
    orc.corr1ord(W.astype(np.float64), X, Zpre)
    Zpre += b.astype(np.float64)
    sure = np.abs(Zpre[rows]) > 1e-5
    assert np.array_equal(bits[sure], (Zpre[rows] > 0)[sure])
    if F % 64:
        assert (words[rows][:, -1] >> np.uint64(F % 64) == 0).all()    # lanes past the last filter never report open
    dP = dev(rng.standard_normal(tuple(P0.shape)).astype(np.float32))
    dW0 = dev(np.zeros(W.shape, np.float32)); db0 = dev(np.zeros((1, F), np.float32))
    dW1 = dev(np.ones(W.shape, np.float32)); db1 = dev(np.ones((1, F), np.float32))
    ks.scanpool_bprop(Wd, bd, Xd, Rd, ptype, P0, I0, dP, dW0, db0, overwrite=True)
    ks.scanpool_bprop(Wd, bd, Xd, Rd, ptype, P0, I0, dP, dW1, db1, overwrite=True, act=act)
    assert_close(host(dW1), host(dW0), 1e-5, "dW from masks vs recomputed")
    assert_close(host(db1), host(db0), 1e-5, "db from masks vs recomputed")
    dW2 = dev(np.ones(W.shape, np.float32)); db2 = dev(np.ones((1, F), np.float32))
    ks.scanpool_bprop(Wd, bd, Xd, Rd, ptype, P0, I0, dP, dW2, db2, overwrite=True, act=act)
    assert np.array_equal(host(dW1), host(dW2)) and np.array_equal(host(db1), host(db2))      # run to run: the same bits
    with pytest.raises(Exception):
        ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, path="kmer", act=act)


@pytest.mark.parametrize("ptype", ["avg", "all"])
@pytest.mark.parametrize("B,lo,hi,m,F", [(600, 0, 70, 24, 70), (520, 30, 45, 16, 16), (530, 1, 150, 7, 40), (130, 100, 260, 24, 300)])
def test_scanpool_bprop_many_regions_kernel(ks, ptype, B, lo, hi, m, F):
    """From 512 (region, filter tile) items on, the mask-driven dense backward deals whole regions to waves (no
    barrier per region chunk). A call without masks recomputes them (a second forward pass on the matrix cores from
    9 taps on, the map through the letter table below) and agrees with the call given masks to round-off; it is checked against the float64 chain too, must be deterministic, and
    must leave alone what lies outside its output. Regions of 0 to 260 rows (several 64-row rounds per region), all
    three tap tiers, code 254 and N present."""
    rng, W, b, X, R = _fused_case(7 * B + F, B, lo, hi, m, F, p254=0.02)
    assert len(R) * ((F + 63) // 64) >= 512
    Wd, bd, Xd, Rd = dev(W), dev(b), dev(X), dev(R)
    act = ks.activity_words(Xd, Wd)
    P0, I0 = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=True, act=act)
    dPh = rng.standard_normal(tuple(P0.shape)).astype(np.float32)
    dP = dev(dPh)
    grads = []
    for kw in (dict(), dict(act=act), dict(act=act)):
        dW = dev(np.full(W.shape, 7.0, np.float32)); db = dev(np.full((1, F), 7.0, np.float32))
        ks.scanpool_bprop(Wd, bd, Xd, Rd, ptype, P0, I0, dP, dW, db, overwrite=True, **kw)
        grads.append((host(dW), host(db)))
    assert np.array_equal(grads[1][0], grads[2][0]) and np.array_equal(grads[1][1], grads[2][1])      # deterministic
    assert_close(grads[1][0], grads[0][0], GRAD, "dW, masks vs recomputation")
    assert_close(grads[1][1], grads[0][1], GRAD, "db, masks vs recomputation")
    # against the unfused float64 chain
    A, Pr, Ir = _chain_oracle(W.astype(np.float64), b.astype(np.float64), X, R, ptype)
    dA = np.zeros_like(A)
    orc.poolrgn_bprop(dA, R, dPh.astype(np.float64), host(I0) if I0 is not None else None, ptype)
    dZ = orc.relu_bprop(dA, A)
    dWr = np.zeros(W.shape)
    orc.corr1ord_bprop_W(dWr, X, dZ)
    assert_close(grads[1][0], dWr, GRAD, "dW vs float64 chain")
    assert_close(grads[1][1], dZ.sum(axis=0, keepdims=True), GRAD, "db vs float64 chain")
    # accumulate mode adds to what is there
    dW = dev(np.full(W.shape, 0.5, np.float32)); db = dev(np.zeros((1, F), np.float32))
    ks.scanpool_bprop(Wd, bd, Xd, Rd, ptype, P0, I0, dP, dW, db, overwrite=False, act=act)
    assert_close(host(dW) - 0.5, grads[1][0], GRAD, "accumulating call")


@pytest.mark.parametrize("ptype", ["max", "all"])
def test_scanpool_bprop_bulk_is_linear_and_independent_of_region_order(ks, ptype):
    """Size-independent properties of the fused backward at a bulk size (4096 sequences x 101 nt, 128 filters of
    width 24, through the activity masks for max+avg pooling): the gradient is linear in the pooled gradient,
    and listing the regions in another order changes nothing but the order of the additions."""
    from deepbind_amd import data
    rng = np.random.default_rng(11)
    B, L, m, F = 4096, 101, 24, 128
    codes = rng.integers(0, 4, (B, L), dtype=np.uint8)
    codes[rng.random((B, L)) < 0.01] = 255
    Xh, Rh = data.pack_uniform_ordinals(codes, m - 1)
    X, R = dev(Xh), dev(Rh)
    W = dev((rng.standard_normal((4 * m, F)) * 0.1).astype(np.float32))
    b = dev((rng.standard_normal((1, F)) * 0.05).astype(np.float32))
    act = ks.activity_words(X, W) if ptype == "all" else None
    P, I = ks.scanpool_fprop(W, b, X, R, ptype, want_argmax=True, act=act)

    def grad(dP, regions=R, pooled=P, amax=I):
        dW = torch.empty_like(W); db = torch.empty_like(b)
        ks.scanpool_bprop(W, b, X, regions, ptype, pooled, amax, dP, dW, db, overwrite=True, act=act)
        return host(dW).astype(np.float64), host(db).astype(np.float64)

    d1 = torch.randn_like(P); d2 = torch.randn_like(P)
    (w1, b1), (w2, b2), (w12, b12) = grad(d1), grad(d2), grad(2.0 * d1 + d2)
    assert_close(w12, 2.0 * w1 + w2, GRAD, "dW linear")
    assert_close(b12, 2.0 * b1 + b2, GRAD, "db linear")
    perm = rng.permutation(B)                                          # (on the host: unsigned index tensors cannot be gathered on the device)
    wp, bp = grad(dev(host(d1)[perm]), dev(Rh[perm]), dev(host(P)[perm]), dev(host(I)[perm]))
    assert_close(wp, w1, GRAD, "dW under a permutation of the regions")
    assert_close(bp, b1, GRAD, "db under a permutation of the regions")
    # the bias gradient is the plain sum of the gradients that pass the rectifier: for max pooling, of dP where pooled > 0
    if ptype == "max":
        assert_close(b1, (host(d1).astype(np.float64) * (host(P) > 0)).sum(axis=0, keepdims=True), GRAD, "db closed form")


# ------------------------------------------------------------------------------------------ dense head
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_blockwise_dot_family(ds, dtype):
    rng = np.random.default_rng(3)
    n, k, m, nb = 50, 16, 32, 7
    tol = ACT if dtype == np.float32 else 1e-12
    X = rng.standard_normal((n, k * nb)).astype(dtype)
    W = rng.standard_normal((k * nb, m)).astype(dtype)
    Zr = orc.blockwise_dot(X, W, nb)
    assert_close(host(ds.blockwise_dot(dev(X), dev(W), nb)), Zr, tol, "Z")
    dZ = rng.standard_normal(Zr.shape).astype(dtype)
    assert_close(host(ds.blockwise_dot_nt(dev(dZ), dev(W), nb)), orc.blockwise_dot_nt(dZ, W, nb), tol * 10, "dX")
    assert_close(host(ds.blockwise_dot_tn(dev(X), dev(dZ), nb, dev(W))), orc.blockwise_dot_tn(X, dZ, nb, W), tol * 10, "dW")
    Xs = rng.standard_normal((n, k)).astype(dtype)                     # one input shared by all models
    assert_close(host(ds.blockwise_dot(dev(Xs), dev(W), nb)), orc.blockwise_dot(Xs, W, nb), tol, "Z shared")
    assert_close(host(ds.blockwise_dot_tn(dev(Xs), dev(dZ), nb, dev(W))), orc.blockwise_dot_tn(Xs, dZ, nb, W), tol * 10, "dW shared")
    # nblock == 1 is a plain matrix product
    assert_close(host(ds.blockwise_dot(dev(X), dev(W), 1)), X @ W, tol, "dot")
    # combined: conv features + a shared feature block, as the sequence model's combiner uses them
    k2 = 5
    X2 = rng.standard_normal((n, k2)).astype(dtype)
    Wc = rng.standard_normal(((k + k2) * nb, m)).astype(dtype)
    Xl, bc = [X, X2], [False, True]
    Zc = orc.blockwise_dot_combined(Xl, Wc, nb, bc)
    assert_close(host(ds.blockwise_dot_combined([dev(X), dev(X2)], dev(Wc), nb, bc)), Zc, tol, "Zc")
    dZc = rng.standard_normal(Zc.shape).astype(dtype)
    got = ds.blockwise_dot_nt_combined([dev(X), dev(X2)], dev(dZc), dev(Wc), nb, bc)
    ref = orc.blockwise_dot_nt_combined(Xl, dZc, Wc, nb, bc)
    assert got[1] is None and ref[1] is None
    assert_close(host(got[0]), ref[0], tol * 10, "dXc")
    assert_close(host(ds.blockwise_dot_tn_combined([dev(X), dev(X2)], dev(dZc), dev(Wc), nb, bc)),
                 orc.blockwise_dot_tn_combined(Xl, dZc, Wc, nb, bc), tol * 10, "dWc")
    assert_close(host(ds.blockwise_dot_tn_combined([dev(X), dev(X2)], dev(dZc), dev(Wc), nb, bc, dWmask=[True, False])),
                 orc.blockwise_dot_tn_combined(Xl, dZc, Wc, nb, bc, dWmask=[True, False]), tol * 10, "dWc masked")


def test_head_fprop(ds):
    rng = np.random.default_rng(4)
    n, k, nb, h = 300, 16, 9, 32
    Pl = np.abs(rng.standard_normal((n, k * nb))).astype(np.float32)
    W1 = (rng.standard_normal((k * nb, h)) * 0.3).astype(np.float32); b1 = (rng.standard_normal((1, h * nb)) * 0.1).astype(np.float32)
    W2 = (rng.standard_normal((h * nb, 1)) * 0.3).astype(np.float32); b2 = (rng.standard_normal((1, nb)) * 0.1).astype(np.float32)
    H = orc.relu_fprop(orc.bias_fprop(orc.blockwise_dot(Pl, W1, nb), b1))
    ref = orc.bias_fprop(orc.blockwise_dot(H, W2, nb), b2)
    got = ds.head_fprop(dev(Pl), dev(W1), dev(b1), dev(W2), dev(b2), nblock=nb)
    assert_close(host(got), ref, ACT, "scores")
    got = ds.head_fprop(dev(Pl), dev(W1), dev(b1), dev(W2), dev(b2), nblock=nb, apply_logistic=True)
    assert_close(host(got), orc.logistic(ref), ACT, "probabilities")
    # no hidden layer, with the test-time dropout rescale
    W0 = (rng.standard_normal((k * nb, 1)) * 0.3).astype(np.float32); b0 = (rng.standard_normal((1, nb)) * 0.1).astype(np.float32)
    rate = rng.choice([0.0, 0.25, 0.5], size=nb).astype(np.float32)
    ref0 = orc.bias_fprop(orc.blockwise_dot(orc.dropout_fp_test(Pl, rate), W0, nb), b0)
    got0 = ds.head_fprop(dev(Pl), dev(W0), dev(b0), nblock=nb, in_scale=1 - rate)
    assert_close(host(got0), ref0, ACT, "scores (no hidden)")


@pytest.mark.parametrize("k,h,nb", [(16, 32, 37), (32, 8, 16), (16, 64, 5)])
def test_head_fprop_bulk_rows(ds, k, h, nb):
    """Row counts that take the 16-models-per-workgroup kernel; model count not a multiple of 16; dropout rescale."""
    rng = np.random.default_rng(40 + k + h)
    n = 5001
    Pl = np.abs(rng.standard_normal((n, k * nb))).astype(np.float32)
    W1 = (rng.standard_normal((k * nb, h)) * 0.3).astype(np.float32); b1 = (rng.standard_normal((1, h * nb)) * 0.1).astype(np.float32)
    W2 = (rng.standard_normal((h * nb, 1)) * 0.3).astype(np.float32); b2 = (rng.standard_normal((1, nb)) * 0.1).astype(np.float32)
    rate = rng.choice([0.0, 0.25, 0.5], size=nb).astype(np.float32)
    H = orc.relu_fprop(orc.bias_fprop(orc.blockwise_dot(orc.dropout_fp_test(Pl, rate), W1, nb), b1))
    ref = orc.logistic(orc.bias_fprop(orc.blockwise_dot(H, W2, nb), b2))
    got = ds.head_fprop(dev(Pl), dev(W1), dev(b1), dev(W2), dev(b2), nblock=nb, in_scale=1 - rate, apply_logistic=True)
    assert_close(host(got), ref, ACT, "probabilities")


@pytest.mark.parametrize("n,k,m,nb,dtype", [(2048, 16, 32, 7, np.float32), (5003, 32, 4, 33, np.float32), (3000, 16, 1, 5, np.float32),
                                            (2500, 64, 64, 3, np.float32), (2100, 16, 32, 18, np.float64), (2049, 5, 12, 16, np.float32),
                                            (8200, 32, 64, 6, np.float32), (4100, 48, 16, 5, np.float32), (33000, 16, 32, 64, np.float32)])
def test_blockwise_dot_family_bulk_rows(ds, n, k, m, nb, dtype):
    """Row counts that take the bulk kernels (16 models per workgroup; chunked weight gradient; float32 products with
    multiples of 16 inputs and outputs on the matrix cores, tiles half used and model counts off the group of four
    included), model counts off the group size, output widths that are / are not multiples of four (the latter fall
    back), float64."""
    rng = np.random.default_rng(n + k + m)
    tol = ACT if dtype == np.float32 else 1e-12
    X = rng.standard_normal((n, k * nb)).astype(dtype)
    W = rng.standard_normal((k * nb, m)).astype(dtype)
    dZ = rng.standard_normal((n, m * nb)).astype(dtype)
    X64, W64, dZ64 = X.astype(np.float64), W.astype(np.float64), dZ.astype(np.float64)
    assert_close(host(ds.blockwise_dot(dev(X), dev(W), nb)), orc.blockwise_dot(X64, W64, nb), tol, "Z")
    assert_close(host(ds.blockwise_dot_nt(dev(dZ), dev(W), nb)), orc.blockwise_dot_nt(dZ64, W64, nb), tol * 10, "dX")
    got = host(ds.blockwise_dot_tn(dev(X), dev(dZ), nb, dev(W)))
    assert_close(got, orc.blockwise_dot_tn(X64, dZ64, nb, W64), tol * 10, "dW")
    assert np.array_equal(got, host(ds.blockwise_dot_tn(dev(X), dev(dZ), nb, dev(W))))
    # combined: conv features + a shared feature block
    k2 = 8
    X2 = rng.standard_normal((n, k2)).astype(dtype)
    Wc = rng.standard_normal(((k + k2) * nb, m)).astype(dtype)
    Xl, bc = [X, X2], [False, True]
    assert_close(host(ds.blockwise_dot_combined([dev(X), dev(X2)], dev(Wc), nb, bc)),
                 orc.blockwise_dot_combined([X64, X2.astype(np.float64)], Wc.astype(np.float64), nb, bc), tol * 3, "Zc")
    dXs = ds.blockwise_dot_nt_combined([dev(X), dev(X2)], dev(dZ), dev(Wc), nb, bc)
    dXr = orc.blockwise_dot_nt_combined([X64, X2.astype(np.float64)], dZ64, Wc.astype(np.float64), nb, bc)
    assert_close(host(dXs[0]), dXr[0], tol * 10, "dX combined")
    dWc = host(ds.blockwise_dot_tn_combined([dev(X), dev(X2)], dev(dZ), dev(Wc), nb, bc))
    assert_close(dWc, orc.blockwise_dot_tn_combined([X64, X2.astype(np.float64)], dZ64, Wc.astype(np.float64), nb, bc), tol * 10, "dW combined")


# ------------------------------------------------------------------------------------------ elementwise / optimiser
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_gradstep_and_madd_bcast(ds, dtype):
    rng = np.random.default_rng(6)
    n = 5000
    P0, dP, mP0 = (rng.standard_normal(n).astype(dtype) for _ in range(3))
    drate = (rng.random(n) * 0.1).astype(dtype); mrate = (0.9 + rng.random(n) * 0.09).astype(dtype)
    for nesterov in (False, True):
        Pr, mPr = P0.copy(), mP0.copy()
        if nesterov:
            orc.gradstep_nesterov1(Pr, mPr, mrate); orc.gradstep_nesterov2(Pr, dP, drate, mPr, mrate)
        else:
            orc.gradstep(Pr, dP, drate, mPr, mrate)
        P, mP, called = dev(P0.reshape(-1, 1)), dev(mP0.reshape(-1, 1)), []
        ds.gradstep(P, dev(dP.reshape(-1, 1)), dev(drate.reshape(-1, 1)), mP, dev(mrate.reshape(-1, 1)),
                    grad=lambda: called.append(1), nesterov=nesterov)
        assert called == [1]
        assert np.array_equal(host(P).ravel(), Pr) and np.array_equal(host(mP).ravel(), mPr)
    # the look-ahead kept in a vector of its own: two steps give the bits of nesterov1 / nesterov2 applied in place
    from deepbind_amd import _lib
    Pr, mPr = P0.copy(), mP0.copy()
    col = lambda a: dev(a.reshape(-1, 1))
    P, mP, L, g1, g2, dr, mr = col(P0), col(mP0), col(np.zeros(n, dtype)), col(dP), col(dP * dtype(0.5)), col(drate), col(mrate)
    dt = _lib.dtype_code(P)
    _lib.call("dbk_gradstep_lookahead", _lib.stream(), dt, n, _lib.ptr(L), _lib.ptr(P), _lib.ptr(mP), _lib.ptr(mr))
    for g, gh in ((g1, dP), (g2, dP * dtype(0.5))):
        orc.gradstep_nesterov1(Pr, mPr, mrate)
        assert np.array_equal(host(L).ravel(), Pr)                     # the gradient is taken at these look-ahead parameters
        orc.gradstep_nesterov2(Pr, gh, drate, mPr, mrate)
        _lib.call("dbk_gradstep_nesterov2_lookahead", _lib.stream(), dt, n, _lib.ptr(P), _lib.ptr(L), _lib.ptr(g), _lib.ptr(dr),
                  _lib.ptr(mP), _lib.ptr(mr))
        assert np.array_equal(host(P).ravel(), Pr) and np.array_equal(host(mP).ravel(), mPr)
    A = rng.standard_normal((24, 10)).astype(dtype); b = rng.standard_normal(3).astype(dtype)
    dst = rng.standard_normal((24, 10)).astype(dtype)
    ref = dst.copy(); orc.madd_bcast(A, b, 16, ref)
    d = dev(dst); ds.madd_bcast(dev(A), b, 16, d)
    assert np.array_equal(host(d), ref)
    d = dev(dst); ds.madd_bcast(dev(A), 0.5, 1, d)
    assert np.array_equal(host(d), dst + A * dtype(0.5))


def test_masks_dropout_and_loss_ops(ds, sm, ks):
    rng = np.random.default_rng(8)
    n, nb, k = 64, 5, 16
    X = rng.standard_normal((n, nb * k)).astype(np.float32)
    rate = np.array([0.0, 0.25, 0.5, 0.5, 0.1], np.float32)
    U = rng.random((n, nb * k)).astype(np.float32)
    for match in (False, True):
        Zr, Mr = orc.dropout_fp_train(X, rate, U, matchrows=match)
        Z, M = ds.dropout_fp_train(dev(X), rate, match, U=dev(U))
        assert np.array_equal(host(M), Mr) and np.array_equal(host(Z), Zr)
    assert np.array_equal(host(ds.dropout_bp_tr(dev(X), M)), orc.dropout_bp_tr(X, Mr))
    assert np.array_equal(host(ds.dropout_fp_test(dev(X), rate)), orc.dropout_fp_test(X, rate))
    assert np.array_equal(host(ds.dropout_bp_te(dev(X), rate)), orc.dropout_bp_te(X, rate))
    # the library's own generator: uniforms in [0,1), keep fraction ~ 1-rate, identical to uniform_like
    ds.set_seed(123)
    Z, M = ds.dropout_fp_train(dev(X), rate, False)
    Ug = host(ds.uniform_like(dev(X), 123, 0))
    assert Ug.min() >= 0.0 and Ug.max() < 1.0 and abs(Ug.mean() - 0.5) < 0.02
    assert np.array_equal(host(M), orc.dropout_fp_train(X, rate, Ug)[1])
    Z2, M2 = ds.dropout_fp_train(dev(X), rate, False)
    assert not np.array_equal(host(M2), host(M))                       # the stream advances
    # input-base dropout
    Xo = random_codes(rng, 500, 0.1)
    Uo = rng.random(500).astype(np.float32)
    Zo, Mo = ks.dropoutord_fp_train(dev(Xo), 0.3, U=dev(Uo))
    Zor, Mor = orc.dropoutord_fp_train(Xo, np.float32(0.3), Uo)
    assert np.array_equal(host(Zo), Zor) and np.array_equal(host(Mo), Mor)
    assert host(Mo)[Xo == 255].all()                                   # padding always reports "kept"
    # reverse-complement rows: the reverse strand drops the mirrored letters
    from deepbind_amd import data
    seqs = ["".join("ACGTN"[v] for v in rng.integers(0, 5, int(rng.integers(1, 40)))) for _ in range(30)]
    Xp, Rp = data.pack_sequences(seqs, 7, reverse_complement=True)
    Up = rng.random(Xp.shape).astype(np.float32)
    Zp, Mp = ks.dropoutord_fp_train(dev(Xp), 0.4, U=dev(Up), regions=dev(Rp), padding=7)
    Zpr, Mpr = orc.dropoutord_fp_train(Xp, np.float32(0.4), Up, regions=Rp, reverse_complement=True)
    assert np.array_equal(host(Zp), Zpr) and np.array_equal(host(Mp), Mpr)
    # maskout / zmask
    A = rng.standard_normal((n, nb)).astype(np.float32); A[3, 2] = np.nan
    Mk = rng.random((n, nb)) < 0.7; Mk[3, 2] = False
    ref = A.copy(); orc.maskout(Mk, ref)
    a = dev(A); ds.maskout(dev(Mk), a)
    assert np.array_equal(host(a), ref)
    Zp = rng.standard_normal((n, nb)).astype(np.float32); Zp[4] = Zp[5]
    zm = torch.zeros((n, nb), dtype=torch.bool, device="cuda")
    ds.calc_Zmask(dev(Zp), zm)
    assert np.array_equal(host(zm), orc.calc_zmask(Zp))
    # bias / relu / logistic / loss pieces
    b = rng.standard_normal((1, nb * k)).astype(np.float32)
    assert np.array_equal(host(sm.add_rowvec(dev(X), dev(b))), orc.bias_fprop(X, b))
    assert np.array_equal(host(sm.relu(dev(X))), orc.relu_fprop(X))
    assert np.array_equal(host(sm.mul_sign(dev(U), dev(X))), orc.relu_bprop(U, X))
    assert_close(host(sm.sum_axis0(dev(X))), orc.bias_bprop(X.astype(np.float64))[1], ACT, "colsum")
    assert_close(host(sm.logistic(dev(X))), orc.logistic(X), ACT, "logistic")
    Zl = orc.logistic(A := rng.standard_normal((n, nb)).astype(np.float32))
    Y = (rng.random((n, nb)) < 0.5).astype(np.float32)
    eps = np.float32(1e-15)
    ref = np.log(np.maximum(eps, Zl)) * Y + np.log(np.maximum(eps, 1 - Zl)) * (1 - Y)
    assert_close(host(sm.loss_terms(dev(Zl), dev(Y), "nll")), ref, ACT, "nll terms")
    assert_close(host(sm.loss_terms(dev(A), dev(Y), "mse")), (A - Y) ** 2, ACT, "mse terms")
    assert_close(host(sm.sub_scale(dev(Zl), dev(Y), 1.0 / n)), orc.loss_bprop(Zl, Y), ACT, "dZ")
    # bidirectional hinge (deepity/std/loss.py:157-174): terms and gradient, float32 and float64, kinks included
    for dt in (np.float32, np.float64):
        Ah = (rng.standard_normal((n, nb)) * 2).astype(dt)
        Ah[0, 0], Ah[1, 0], Y[0, 0], Y[1, 0] = 0.0, 1.0, 0.0, 1.0                  # exactly on the kinks: no cost, no gradient
        Yh = Y.astype(dt)
        assert np.array_equal(host(sm.loss_terms(dev(Ah), dev(Yh), "hinge")), np.maximum(0, (1 - Yh) * Ah + Yh * (1 - Ah)).astype(dt))
        assert np.array_equal(host(sm.hinge_grad(dev(Ah), dev(Yh), 1.0 / n)), orc.loss_bprop(Ah, Yh, kind="hinge"))
    assert_close(host(sm.dot(dev(X), dev(X.T.copy()))), X.astype(np.float64) @ X.T.astype(np.float64), ACT, "dot")
    assert_close(host(sm.dot_nt(dev(X), dev(X))), X.astype(np.float64) @ X.T.astype(np.float64), ACT, "dot_nt")
    assert_close(host(sm.dot_tn(dev(X), dev(X))), X.T.astype(np.float64) @ X.astype(np.float64), ACT, "dot_tn")


# ------------------------------------------------------------------------------------------ k-mer table fast path
@pytest.mark.parametrize("B,lo,hi,m,F", [(64, 101, 101, 24, 16), (128, 38, 41, 16, 16), (300, 20, 40, 24, 144), (33, 1, 300, 11, 70),
                                          (50, 500, 500, 24, 64), (17, 0, 9, 5, 33), (700, 30, 60, 20, 40), (40, 90, 110, 2, 8),
                                          (1, 50, 50, 24, 32), (49, 10, 80, 24, 32)])
def test_scanpool_kmer_path_matches_oracle(ks, B, lo, hi, m, F):
    rng, W, b, X, R = _fused_case(1000 + B + m + F, B, lo, hi, m, F, pn=0.04)
    A, Pr, Ir = _chain_oracle(W, b, X, R, "max")
    P, I = ks.scanpool_fprop(dev(W), dev(b), dev(X), dev(R), "max", path="kmer")
    assert I is None
    assert_close(host(P), Pr, ACT, "pooled (kmer path)")
    # and it agrees with the general kernel to the same tolerance
    Pg, _ = ks.scanpool_fprop(dev(W), dev(b), dev(X), dev(R), "max", path="general")
    assert_close(host(P), host(Pg), ACT, "kmer vs general")


def test_scanpool_kmer_path_repeats_its_bits(ks):
    """The table kernel's streams take regions as they become free, so which stream scans a region differs from call to
    call; every region's result must not (same additions in the same order whoever performs them)."""
    rng, W, b, X, R = _fused_case(515, 3000, 5, 200, 24, 96, pn=0.03)
    Wd, bd, Xd, Rd = dev(W), dev(b), dev(X), dev(R)
    for ptype, want in (("max", False), ("max", True), ("all", True), ("avg", False)):
        P0, I0 = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=want, path="kmer")
        for _ in range(3):
            P1, I1 = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=want, path="kmer")
            assert torch.equal(P0, P1) and (I0 is None or torch.equal(I0, I1)), ptype


def test_scanpool_kmer_path_device_side_fallbacks(ks):
    """Code 254 and regions past the scan's last row cannot be expressed in the table: the call must
    still return the right answer (the general kernel runs behind a device flag)."""
    rng, W, b, X, R = _fused_case(4242, 60, 30, 50, 24, 48, pn=0.03, p254=0.02)
    assert (X == 254).any()
    A, Pr, _ = _chain_oracle(W, b, X, R, "max")
    P, _ = ks.scanpool_fprop(dev(W), dev(b), dev(X), dev(R), "max", path="kmer")
    assert_close(host(P), Pr, ACT, "pooled with code 254")
    rng, W, b, X, R = _fused_case(4243, 20, 30, 50, 24, 48)
    R2 = R.copy(); R2[-1, 1] = X.size                                   # last region runs into rows >= n
    A, Pr, _ = _chain_oracle(W, b, X, R2, "max")
    P, _ = ks.scanpool_fprop(dev(W), dev(b), dev(X), dev(R2), "max", path="kmer")
    assert_close(host(P), Pr, ACT, "pooled with a region past the last scan row")
    from deepbind_amd._lib import DeepbindError
    with pytest.raises(DeepbindError):
        ks.scanpool_fprop(dev(W[:, :8].repeat(2, axis=0)[:4 * 30].copy()), dev(b[:, :8].copy()), dev(X), dev(R), "max", path="kmer")   # 30 taps


@pytest.mark.parametrize("ptype", ["max", "avg", "all"])
@pytest.mark.parametrize("B,lo,hi,m,F", [(200, 101, 101, 24, 64), (150, 30, 60, 16, 40), (60, 1, 30, 24, 33), (90, 40, 90, 7, 32)])
def test_scanpool_kmer_path_pooling_variants_and_argmax(ks, ptype, B, lo, hi, m, F):
    """The table kernel's average / max+average pooling and its argmax (winning triple of positions, settled
    exactly at the region's end) against the oracle, with the general kernel as a second opinion."""
    rng, W, b, X, R = _fused_case(7000 + B + m + F, B, lo, hi, m, F, pn=0.04)
    b = b - 0.05                                                    # some filters never fire in some regions: argmax = first row
    A, Pr, Ir = _chain_oracle(W.astype(np.float64), b.astype(np.float64), X, R, ptype)
    want = ptype != "avg"
    P, I = ks.scanpool_fprop(dev(W), dev(b), dev(X), dev(R), ptype, want_argmax=want, path="kmer")
    assert_close(host(P), Pr, ACT, "pooled (%s, table kernel)" % ptype)
    Pg, Ig = ks.scanpool_fprop(dev(W), dev(b), dev(X), dev(R), ptype, want_argmax=want, path="general")
    assert_close(host(P), host(Pg), ACT, "table vs general")
    if want:
        got = host(I)
        agree = got == Ir
        assert agree.mean() > 0.995                                 # float32 round-off can move a near-tie
        # wherever the index differs from the float64 oracle the two rows must be a float32 tie
        rows, cols = np.nonzero(~agree)
        Af = A.astype(np.float32)
        for r_, c_ in zip(rows[:50], cols[:50]):
            i_got, i_ref = got[r_, c_] // F, Ir[r_, c_] // F
            assert got[r_, c_] % F == c_ and R[r_, 0] <= i_got < R[r_, 1]
            assert abs(Af[i_got, c_] - Af[i_ref, c_]) <= 1e-5 * max(1.0, abs(Af[i_ref, c_]))
        zero = Pr[:, ::2] == 0 if ptype == "all" else Pr == 0
        assert zero.any() and np.array_equal(got[zero] // F, np.broadcast_to(R[:, :1], got.shape)[zero])
    else:
        assert I is None


def test_scanpool_kmer_argmax_takes_the_first_of_exactly_equal_rows(ks):
    """A sequence made of one 40-letter unit repeated: every window value recurs bit-for-bit 40 rows later,
    so the maximum is attained several times and the index must be the first occurrence."""
    rng = np.random.default_rng(3)
    m, F = 24, 32
    unit = rng.integers(0, 4, 40, dtype=np.uint8)
    ords = [np.tile(unit, 5), np.tile(unit[::-1].copy(), 3)]
    from deepbind_amd import data
    X, R = data.pack_ordinals(ords, m - 1)
    W = (rng.standard_normal((4 * m, F)) * 0.1).astype(np.float32)
    b = np.zeros((1, F), np.float32)
    A, Pr, Ir = _chain_oracle(W.astype(np.float64), b.astype(np.float64), X, R, "max")
    rows_ref = Ir // F
    # the oracle's maxima really are attained more than once
    repeats = sum(int((A[R[r_, 0]:R[r_, 1], c_] == Pr[r_, c_]).sum() > 1) for r_ in range(2) for c_ in range(F))
    assert repeats > F
    for path in ("kmer", "general"):
        P, I = ks.scanpool_fprop(dev(W), dev(b), dev(X), dev(R), "max", want_argmax=True, path=path)
        assert np.array_equal(host(I) // F, rows_ref), path
        assert np.array_equal(host(I) % F, np.broadcast_to(np.arange(F), (2, F)))


def test_scanpool_auto_path_bulk(ks):
    """A batch large enough for the library to pick the table kernel by itself."""
    rng, W, b, X, R = _fused_case(99, 2500, 100, 100, 24, 256, pn=0.01)
    P, _ = ks.scanpool_fprop(dev(W), dev(b), dev(X), dev(R), "max")
    Pg, _ = ks.scanpool_fprop(dev(W), dev(b), dev(X), dev(R), "max", path="general")
    assert_close(host(P), host(Pg), ACT, "auto vs general")
    from oracle import oracle_c
    Pr, _ = oracle_c.scanpool(W, b, X, R, 0)
    assert_close(host(P), Pr, ACT, "auto vs C oracle")


@pytest.mark.parametrize("B,lo,hi,m,F", [(200, 101, 101, 24, 64), (150, 30, 60, 16, 40), (77, 24, 24, 24, 16), (500, 1, 5, 24, 32),
                                          (300, 60, 200, 16, 64), (100, 500, 500, 12, 32), (400, 40, 70, 5, 16), (64, 101, 101, 18, 96)])
def test_scanpool_kmer_regions_in_any_order(ks, B, lo, hi, m, F):
    """Regions need not be sorted or contiguous for the table kernel: shuffling the region table
    permutes the output rows and nothing else - not a bit. (With filters of up to 18 taps a stream walks through regions
    that follow each other in the text without a fresh start and splits the block in which one ends between the two;
    shuffled, every region gets a fresh start: the two ways must agree exactly.)"""
    rng, W, b, X, R = _fused_case(31 + B + m, B, lo, hi, m, F, pn=0.03)
    A, Pr, _ = _chain_oracle(W, b, X, R, "max")
    P, _ = ks.scanpool_fprop(dev(W), dev(b), dev(X), dev(R), "max", path="kmer")
    assert_close(host(P), Pr, ACT, "packed order")
    perm = rng.permutation(B)
    P2, _ = ks.scanpool_fprop(dev(W), dev(b), dev(X), dev(R[perm]), "max", path="kmer")
    assert_close(host(P2), Pr[perm], ACT, "shuffled order")
    assert np.array_equal(host(P2), host(P)[perm]), "a region's result depends on its neighbours in the region table"


@pytest.mark.parametrize("B,lo,hi,m", [(4000, 20, 60, 16), (13000, 5, 30, 11), (4000, 20, 60, 24), (13000, 1, 40, 20), (5000, 30, 30, 24),
                                        (4500, 101, 101, 18)])
def test_scanpool_kmer_walks_on_through_regions_at_bulk_sizes(ks, B, lo, hi, m):
    """Enough regions per workgroup (1 024 filters: eight workgroups per tile) that every stream of the table kernel
    claims several regions at a time and goes on from one into the next where they follow each other in the text (runs
    of up to eight with at most 18 taps, pairs with 19-24 and for average pooling): the packed table, the same with a third of the regions
    dropped (runs and pairs break off, second halves of claims are scanned alone), with regions cut in two that touch,
    and shuffled (no region follows another) - against the general kernel, against the C oracle on a sample, and the
    shuffled call against the packed one bit for bit."""
    from oracle import oracle_c
    F = 1024
    rng, W, b, X, R = _fused_case(77 + B + m, B, lo, hi, m, F, pn=0.02)
    Wd, bd, Xd = dev(W), dev(b), dev(X)
    cut = []
    for a_, b_ in R:
        if b_ - a_ >= 2 and rng.random() < 0.5:
            c_ = int(rng.integers(a_ + 1, b_))
            cut += [(a_, c_), (c_, b_)]
        else:
            cut.append((a_, b_))
    tables = {"packed": R, "some dropped": np.ascontiguousarray(R[rng.random(B) < 0.67]),
              "cut in two": np.array(cut, dtype=R.dtype).reshape(-1, 2)}
    for name, Rt in tables.items():
        P, _ = ks.scanpool_fprop(Wd, bd, Xd, dev(Rt), "max", path="kmer")
        Pg, _ = ks.scanpool_fprop(Wd, bd, Xd, dev(Rt), "max", path="general")
        assert_close(host(P), host(Pg), ACT, "table vs general kernel, %s" % name)
        for _ in range(2):                                             # which stream takes which regions differs from call to call
            Pagain, _ = ks.scanpool_fprop(Wd, bd, Xd, dev(Rt), "max", path="kmer")
            assert torch.equal(P, Pagain), "two calls, different bits (%s)" % name
        pick = np.sort(rng.choice(len(Rt), 40, replace=False))
        Pr, _ = oracle_c.scanpool(W, b, X, np.ascontiguousarray(Rt[pick]), 0)
        assert_close(host(P)[pick], Pr, ACT, "table kernel vs C oracle, %s" % name)
        perm = rng.permutation(len(Rt))
        P2, _ = ks.scanpool_fprop(Wd, bd, Xd, dev(np.ascontiguousarray(Rt[perm])), "max", path="kmer")
        assert np.array_equal(host(P2), host(P)[perm]), "a region's result depends on its neighbours in the region table (%s)" % name
        # average and max + average pooling go through pairs at every filter length
        for ptype in ("avg", "all"):
            Pa, _ = ks.scanpool_fprop(Wd, bd, Xd, dev(Rt), ptype, path="kmer")
            Pag, _ = ks.scanpool_fprop(Wd, bd, Xd, dev(Rt), ptype, path="general")
            assert_close(host(Pa), host(Pag), ACT, "table vs general kernel, %s, %s" % (ptype, name))
            Pa2, _ = ks.scanpool_fprop(Wd, bd, Xd, dev(np.ascontiguousarray(Rt[perm])), ptype, path="kmer")
            assert np.array_equal(host(Pa2), host(Pa)[perm]), "%s pooling: a region's result depends on its neighbours (%s)" % (ptype, name)


@pytest.mark.parametrize("n,m,dtype", [(1, 5, np.float32), (255, 64, np.float32), (13591, 720, np.float32), (100000, 70, np.float32),
                                       (4097, 1, np.float64), (0, 9, np.float32)])
def test_column_sums(sm, n, m, dtype):
    """One slice and many slices of rows, column counts off the 64-wide tile, bit-stability, zero rows."""
    rng = np.random.default_rng(n + m)
    X = rng.standard_normal((n, m)).astype(dtype)
    got = host(sm.sum_axis0(dev(X)))
    assert got.shape == (1, m)
    assert_close(got, X.astype(np.float64).sum(axis=0, keepdims=True), ACT if dtype == np.float32 else 1e-12, "column sums")
    assert np.array_equal(got, host(sm.sum_axis0(dev(X))))


# ------------------------------------------------------------------------------------------ empty and degenerate inputs
def test_empty_and_degenerate_inputs(ks, ds):
    """Zero regions, streams shorter than the filter, zero rows: every entry point must
    return the defined (empty or all-padding) result without touching memory it does not own."""
    rng = np.random.default_rng(12)
    m, F = 6, 20
    W = (rng.standard_normal((4 * m, F)) * 0.3).astype(np.float32)
    b = (rng.standard_normal((1, F)) * 0.3).astype(np.float32)
    Wd, bd = dev(W), dev(b)
    # no regions at all
    X = random_codes(rng, 40, 0.1)
    R0 = np.zeros((0, 2), np.uint32)
    for ptype in ("max", "avg", "all"):
        P, I = ks.scanpool_fprop(Wd, bd, dev(X), dev(R0), ptype, want_argmax=(ptype != "avg"))
        assert P.shape == (0, F * (2 if ptype == "all" else 1))
        dW, db = dev(np.ones_like(W)), dev(np.full_like(b, 5.0))
        ks.scanpool_bprop(Wd, bd, dev(X), dev(R0), ptype, P, I, torch.zeros_like(P), dW, db)
        assert np.array_equal(host(dW), np.ones_like(W)) and np.array_equal(host(db), np.zeros_like(b))
    # a stream shorter than the filter: the scan defines no row, every row of the map is relu(bias)
    Xs = random_codes(rng, m - 2, 0.0)
    Rs = np.array([[0, m - 2]], np.uint32)
    A, Pr, Ir = _chain_oracle(W.astype(np.float64), b.astype(np.float64), Xs, Rs, "all")
    P, I = ks.scanpool_fprop(Wd, bd, dev(Xs), dev(Rs), "all", want_argmax=True)
    assert_close(host(P), Pr, ACT, "short stream")
    assert np.array_equal(host(I), Ir)
    Z = dev(np.full((m - 2, F), 3.0, np.float32))
    ks.corr1ord(Wd, dev(Xs), Z, 4)
    assert np.array_equal(host(Z), np.full((m - 2, F), 3.0, np.float32))        # rows >= n are left untouched
    # (zero-length regions are outside the reference's domain: its kernels read the region's first row
    # unconditionally, poolrgn.cuh:64-66, and the batcher never produces one; not tested)
    # zero rows through the dense head and the elementwise ops
    e = torch.zeros((0, 16 * 3), dtype=torch.float32, device="cuda")
    W1 = dev(rng.standard_normal((48, 8)).astype(np.float32)); b1 = dev(np.zeros((1, 24), np.float32))
    W2 = dev(rng.standard_normal((24, 1)).astype(np.float32)); b2 = dev(np.zeros((1, 3), np.float32))
    assert ds.head_fprop(e, W1, b1, W2, b2, nblock=3).shape == (0, 3)
    assert ds.blockwise_dot(e, W1, 3).shape == (0, 24)
    Zd, Md = ds.dropout_fp_train(e, dev(np.full(3, 0.5, np.float32)), False)
    assert Zd.shape == e.shape and Md.shape == e.shape
    Ze, Me = ks.dropoutord_fp_train(torch.zeros((0, 1), dtype=torch.uint8, device="cuda"), 0.5)
    assert Ze.numel() == 0 and Me.numel() == 0


@pytest.mark.parametrize("ptype", ["max", "all"])
def test_scanpool_extreme_shapes(ks, ptype):
    """One very long region (a chromosome-scale scan: many staging chunks per region) and very many one-letter
    regions in the same call, against the plain-C oracle; forward on every path and the fused backward."""
    from oracle import oracle_c
    rng = np.random.default_rng(77)
    m, F = 24, 40
    lens = [150001] + [1] * 20000 + [3000] + [2] * 5000
    ords = [rng.integers(0, 4, L, dtype=np.uint8) for L in lens]
    for o in ords[:3]:
        o[rng.random(o.size) < 0.01] = 255
    from deepbind_amd import data
    X, R = data.pack_ordinals(ords, m - 1)
    W = (rng.standard_normal((4 * m, F)) * 0.1).astype(np.float32)
    b = (rng.standard_normal((1, F)) * 0.1).astype(np.float32)
    pt = {"max": 0, "all": 3}[ptype]
    Pr, Ir = oracle_c.scanpool(W, b, X, R, pt, want_argmax=True)
    Wd, bd, Xd, Rd = dev(W), dev(b), dev(X), dev(R)
    P, I = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=True)
    assert_close(host(P), Pr, ACT, "pooled (general, argmax)")
    same = host(I) == Ir
    assert same.mean() > 0.999                                       # the rest are float32 round-off ties between rows
    if ptype == "max":
        Pk, _ = ks.scanpool_fprop(Wd, bd, Xd, Rd, "max", path="kmer")
        assert_close(host(Pk), Pr, ACT, "pooled (table kernel)")
    # backward: linear in dpooled, so two calls with g and 2g must give dW2 = 2 dW1 (bit-exact) and run-to-run identical
    dP = dev(rng.standard_normal(Pr.shape).astype(np.float32))
    outs = []
    for scale in (1.0, 2.0, 1.0):
        dW, db = dev(np.zeros_like(W)), dev(np.zeros_like(b))
        ks.scanpool_bprop(Wd, bd, Xd, Rd, ptype, P, I, dP * scale, dW, db)
        outs.append((host(dW), host(db)))
    assert np.array_equal(outs[0][0], outs[2][0]) and np.array_equal(outs[0][1], outs[2][1])
    assert np.array_equal(outs[1][0], 2 * outs[0][0]) and np.array_equal(outs[1][1], 2 * outs[0][1])
    assert np.isfinite(outs[0][0]).all() and np.abs(outs[0][0]).max() > 0


def test_config5_full_size_against_subsampled_checkers(ks, ds):
    """The full bulk-scoring workload (100 000 x 500 nt, 1024 filters): rows of the table kernel's result are
    checked against the general kernel and the plain-C oracle run on random subsets of the regions (same
    packed stream, region table subsampled), and a permuted region table must permute the rows and nothing else."""
    from deepbind_amd import synth
    from oracle import oracle_c
    cfg = synth.config5(seed=4, nseq=100000)
    p = cfg["params"]
    W, b, X, R = dev(p["Wc"]), dev(p["bc"]), dev(cfg["X"]), dev(cfg["R"])
    P, _ = ks.scanpool_fprop(W, b, X, R, "max")
    assert tuple(P.shape) == (100000, 1024) and bool(torch.isfinite(P).all()) and float(P.min()) >= 0.0
    rng = np.random.default_rng(0)
    pick = np.sort(rng.choice(100000, 1500, replace=False))
    Rs = np.ascontiguousarray(cfg["R"][pick])
    Pg, _ = ks.scanpool_fprop(W, b, X, dev(Rs), "max", path="general")
    sub = host(P[torch.as_tensor(pick, device="cuda")])
    assert_close(sub, host(Pg), ACT, "table kernel vs general kernel on 1500 regions")
    few = pick[:120]
    Pc, _ = oracle_c.scanpool(p["Wc"], p["bc"], cfg["X"], np.ascontiguousarray(cfg["R"][few]), 0)
    assert_close(sub[:120], Pc, ACT, "table kernel vs C oracle on 120 regions")
    perm = rng.permutation(100000)
    Pp, _ = ks.scanpool_fprop(W, b, X, dev(np.ascontiguousarray(cfg["R"][perm])), "max")
    assert torch.equal(Pp, P[torch.as_tensor(perm, device="cuda")])
    # the pooling winners of the table kernel against the float32 evaluation in reference order (the plain-C oracle):
    # at full size row * 1024 + filter does not fit the reference's 32-bit index, so the 120 regions are repacked as
    # a stream of their own (each region starts with its padding: every window reads the same letters as before)
    def repack(which):
        Xr = np.concatenate([cfg["X"].ravel()[a:b_] for a, b_ in cfg["R"][which]] + [np.full(cfg["spec"].m - 1, 255, np.uint8)])
        edges = np.concatenate([[0], np.cumsum(cfg["R"][which][:, 1].astype(np.int64) - cfg["R"][which][:, 0])])
        return Xr.reshape(-1, 1), np.stack([edges[:-1], edges[1:]], axis=1).astype(np.uint32)
    X120, R120 = repack(few)
    Pc2, Ic = oracle_c.scanpool(p["Wc"], p["bc"], X120, R120, 0, want_argmax=True)
    assert np.array_equal(Pc2, Pc)
    Pa, Ia = ks.scanpool_fprop(W, b, dev(X120), dev(R120), "max", want_argmax=True, path="kmer")
    assert np.array_equal(host(Pa), sub[:120])
    moved = record_argmax("config5", host(Ia), Ic)
    assert moved <= 0.001 * Ic.size, "%d of %d pooling winners differ from the reference order's" % (moved, Ic.size)
    del Pp, Pa, Ia
    # the end result of the configuration, the 100000 x 64 score matrix: scan + pool + dense head (16 -> 32 -> 1 per model)
    scores = ds.head_fprop(P, dev(p["W1"]), dev(p["b1"]), dev(p["W2"]), dev(p["b2"]), nblock=64)
    assert tuple(scores.shape) == (100000, 64) and bool(torch.isfinite(scores).all())
    # ... against the float64 oracle's whole forward pass on 40 of the regions (their bytes repacked as a stream of
    # their own: each region starts with its padding, so every window reads the same letters as in the full stream),
    # and next to the same pass in float32 in reference order
    some = few[:40]
    Xs, Rs40 = repack(some)
    p64 = {k: v.astype(np.float64) for k, v in p.items()}
    st = orc.model_forward(p64, Xs, Rs40, 64, "max", 32)
    st32 = orc.model_forward(p, Xs, Rs40, 64, "max", 32)
    got_scores, got_pooled = host(scores[torch.as_tensor(some, device="cuda")]), sub[:40]
    assert_close(got_pooled, st["Pl"], ACT, "config 5 pooled features of 40 regions vs the float64 oracle")
    record_error("config5", "activations", got_pooled, st["Pl"], ACT)
    for j in range(64):
        assert_close(got_scores[:, j], st["A"][:, j], ACT, "config 5 scores of model %d vs the float64 oracle" % j)
        record_error("config5", "activations", got_scores[:, j], st["A"][:, j], ACT)
        assert_vs_f32("config5", "activations", got_scores[:, j], st["A"][:, j], st32["A"][:, j], "scores of model %d" % j)
        assert_vs_f32("config5", "activations", got_pooled[:, 16 * j:16 * j + 16], st["Pl"][:, 16 * j:16 * j + 16],
                      st32["Pl"][:, 16 * j:16 * j + 16], "pooled features of model %d" % j)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_softmax_chunks_and_multiclass_loss_terms(dtype):
    """Output node of a model with several columns per output (deepity/std/softmax.py:58-71, loss.py:147-151)."""
    from deepbind_amd import smat as sm
    rng = np.random.default_rng(13)
    X = (rng.standard_normal((300, 24)) * 4).astype(dtype)
    tol = 1e-6 if dtype == np.float32 else 1e-14
    for nchunk in (1, 3, 24):
        got = host(sm.softmax(dev(X), nchunk))
        ref = orc.softmax(X.astype(np.float64), nchunk)
        assert np.abs(got - ref).max() <= tol
    with pytest.raises(Exception):
        sm.softmax(dev(X), 5)
    Z = orc.softmax(X.astype(np.float64), 3).astype(dtype)
    Z[0, 0] = 0                                                     # log(max(1e-15, 0))
    Y = (rng.random(Z.shape) < 0.3).astype(dtype)
    got = host(sm.loss_terms(dev(Z), dev(Y), "nll_multiclass"))
    ref = orc.nll_multiclass_terms(Z.astype(np.float64), Y.astype(np.float64))
    assert np.abs(got - ref).max() <= (1e-5 if dtype == np.float32 else 1e-13) * np.abs(ref).max()

# ------------------------------------------------------------------------------------------ 16-byte packs
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("n", [1, 3, 4, 5, 1023, 4096, 70001])
def test_elementwise_packs_tails_unaligned_and_in_place(sm, n, dtype):
    """The elementwise kernels take 16 bytes per thread where the arrays allow it: every size (no pack, whole packs, a
    tail), arrays that start off a 16-byte boundary (element by element) and a result written over its input give the
    values of the plain formulas, bit for bit."""
    from deepbind_amd import _lib
    g = torch.Generator(device="cuda").manual_seed(n)
    for off in (0, 1):
        X = torch.randn(n + off, generator=g, device="cuda", dtype=torch.float64).to(dtype)[off:]
        Y = torch.randn(n + off, generator=g, device="cuda", dtype=torch.float64).to(dtype)[off:]
        X[::7] = 0.0                                                      # sign(0) = 0, relu(0) = 0
        zero = torch.zeros((), device="cuda", dtype=dtype)
        assert torch.equal(sm.relu(X), torch.where(X > 0, X, zero))
        assert torch.equal(sm.sign(X), torch.sign(X))
        assert torch.equal(sm.mul_sign(Y, X), Y * torch.sign(X))
        assert torch.equal(sm.sub_scale(X, Y, 0.125), (X - Y) * 0.125)
        assert torch.allclose(sm.logistic(X), torch.sigmoid(X), rtol=1e-6 if dtype == torch.float32 else 1e-14, atol=0)
        # in place: the result over the input
        Z = X.clone()
        _lib.call("dbk_relu", _lib.stream(), _lib.dtype_code(Z), _lib.ptr(Z), _lib.ptr(Z), n)
        assert torch.equal(Z, torch.where(X > 0, X, zero))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("rows,cols", [(1, 1), (5, 3), (7, 4), (33, 6), (129, 16), (1000, 68), (3, 2050)])
def test_add_rowvec_packs_and_plain_rows(sm, rows, cols, dtype):
    """Rows of whole 16-byte packs take the packed kernel, other widths and unaligned arrays the element-wise one: the
    same sums either way."""
    g = torch.Generator(device="cuda").manual_seed(rows * 131 + cols)
    for off in (0, 1):
        X = torch.randn(rows * cols + off, generator=g, device="cuda", dtype=torch.float64).to(dtype)[off:].reshape(rows, cols)
        b = torch.randn(cols, generator=g, device="cuda", dtype=torch.float64).to(dtype)
        assert torch.equal(sm.add_rowvec(X, b), X + b)


@pytest.mark.parametrize("F", [4, 6, 8, 64, 100, 256])
def test_poolrgn_packed_and_plain_columns_agree(ks, F):
    """Maps whose rows are whole packs pool four columns per lane, others one: every column's maximum, first winning
    row, sum and gradient must be what the one-column kernels give (F = 6 and an unaligned map go through them)."""
    rng = np.random.default_rng(F)
    P, lens = 37, rng.integers(1, 40, size=37)
    starts = np.concatenate([[0], np.cumsum(lens)[:-1]])
    R = np.stack([starts, starts + lens], 1).astype(np.uint32)
    N = int(lens.sum())
    U = rng.standard_normal((N, F)).astype(np.float32)
    U[rng.random((N, F)) < 0.2] = 0.5                                      # ties: the first row wins
    Ud, Rd = dev(U), dev(R)
    base = torch.empty(N * F + 1, dtype=torch.float32, device="cuda")
    Uoff = base[1:].reshape(N, F)                                          # the same map off a 16-byte boundary
    Uoff.copy_(Ud)
    for ptype in ("max", "avg", "sum", "all"):
        want = ptype in ("max", "all")
        Pa, Ia = ks.poolrgn(Ud, Rd, ptype, want_argmax=want)
        Pb, Ib = ks.poolrgn(Uoff, Rd, ptype, want_argmax=want)
        assert torch.equal(Pa, Pb), ptype
        if want:
            assert torch.equal(Ia, Ib), ptype
        dP = dev(rng.standard_normal(tuple(Pa.shape)).astype(np.float32))
        dUa = torch.zeros_like(Ud) + 0.25
        dUb = torch.empty_like(base)[1:].reshape(N, F)
        dUb.fill_(0.25)
        ks.poolrgn_bprop(dUa, Rd, dP, Ia if want else None, ptype)
        ks.poolrgn_bprop(dUb, Rd, dP, Ib if want else None, ptype)
        assert torch.equal(dUa, dUb), ptype
