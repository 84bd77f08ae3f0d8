"""The plain-C restatement must agree with the (pinned) NumPy oracle: bit-exact where both
accumulate in the same order, to float32 round-off where the order legitimately differs."""
import numpy as np
import pytest

from oracle import deepbind_oracle as orc
from oracle import oracle_c as oc


def _case(seed, N=300, m=7, F=9):
    rng = np.random.default_rng(seed)
    X = rng.integers(0, 4, size=N).astype(np.uint8)
    u = rng.random(N)
    X[u < 0.1] = 255
    X[(u > 0.1) & (u < 0.13)] = 254
    W = rng.standard_normal((4 * m, F)).astype(np.float32)
    return rng, W, X


def test_corr1ord_bit_exact():
    rng, W, X = _case(0)
    Za = np.full((300, 9), 3.0, np.float32); orc.corr1ord(W, X, Za)
    Zb = np.full((300, 9), 3.0, np.float32); oc.corr1ord(W, X, Zb)
    assert np.array_equal(Za, Zb)


def test_bprop_W_and_X():
    rng, W, X = _case(1)
    dZ = rng.standard_normal((300, 9)).astype(np.float32)
    a = np.zeros_like(W); orc.corr1ord_bprop_W(a, X, dZ)
    b = np.zeros_like(W); oc.corr1ord_bprop_W(b, X, dZ)
    np.testing.assert_allclose(a, b, rtol=1e-4, atol=1e-4)
    a = np.zeros((300, 4), np.float32); orc.corr1ord_bprop_X(a, W, dZ)
    b = np.zeros((300, 4), np.float32); oc.corr1ord_bprop_X(b, W, dZ)
    np.testing.assert_allclose(a, b, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("ptype", ["max", "avg", "sum", "all"])
def test_poolrgn_and_bprop(ptype):
    rng = np.random.default_rng(2)
    U = rng.standard_normal((200, 10)).astype(np.float32)
    R = np.array([[0, 30], [30, 31], [31, 120], [120, 200]], np.uint32)
    pt = orc.STR2POOLTYPE[ptype]
    Za, Ia = orc.poolrgn(U, R, ptype, want_argmax=True)
    Zb, Ib = oc.poolrgn(U, R, pt, want_argmax=True)
    np.testing.assert_allclose(Za, Zb, rtol=1e-6, atol=1e-7)
    if Ia is not None:
        assert np.array_equal(Ia, Ib)
    dP = rng.standard_normal(Za.shape).astype(np.float32)
    a = np.zeros_like(U); orc.poolrgn_bprop(a, R, dP, Ia, ptype)
    b = np.zeros_like(U); oc.poolrgn_bprop(b, R, dP, Ib, pt)
    np.testing.assert_allclose(a, b, rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("ptype", ["max", "avg", "all"])
def test_scanpool_equals_unfused_chain(ptype):
    rng, W, _ = _case(3, m=6, F=8)
    seqs = ["ACGTNNACGTTGCA", "TT", "GATTACAGATTACA" * 3, "C"]
    X, R = orc.pack(seqs, 5)
    bias = rng.standard_normal((1, 8)).astype(np.float32) * 0.3
    Z = np.zeros((X.size, 8), np.float32)
    orc.corr1ord(W, X, Z)
    A = orc.relu_fprop(orc.bias_fprop(Z, bias))
    Pa, Ia = orc.poolrgn(A, R, ptype, want_argmax=True)
    Pb, Ib = oc.scanpool(W, bias, X, R, orc.STR2POOLTYPE[ptype], want_argmax=True)
    np.testing.assert_allclose(Pa, Pb, rtol=1e-6, atol=1e-7)
    if Ia is not None:
        assert np.array_equal(Ia, Ib)
