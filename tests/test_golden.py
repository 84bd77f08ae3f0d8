"""Committed golden vectors: the oracle must still reproduce them (CPU), and the HIP library must
match them (GPU)."""
import os

import numpy as np
import pytest

from oracle import deepbind_oracle as orc

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
SCAN_FILES = ["scan_pool_small.npz", "scan_pool_m24.npz"]


def _load(name):
    return dict(np.load(os.path.join(GOLD, name)))


@pytest.mark.parametrize("name", SCAN_FILES)
def test_oracle_reproduces_scan_pool_fixture(name):
    g = _load(name)
    Z = np.zeros_like(g["Z"]); orc.corr1ord(g["W"], g["X"], Z)
    assert np.array_equal(Z, g["Z"])
    A = orc.relu_fprop(orc.bias_fprop(Z, g["b"]))
    for pt in ("max", "avg", "sum", "all"):
        P, I = orc.poolrgn(A, g["R"], pt, want_argmax=True)
        assert np.array_equal(P, g["pool_" + pt])
        if I is not None:
            assert np.array_equal(I, g["argmax_" + pt])
    dW = np.zeros_like(g["W"]); orc.corr1ord_bprop_W(dW, g["X"], g["dZ"])
    np.testing.assert_allclose(dW, g["dW"], rtol=1e-6, atol=1e-6)


def test_oracle_reproduces_train_fixture():
    g = _load("train_two_steps.npz")
    names = ["Wc", "bc", "W1", "b1", "W2", "b2"]
    q = {a: g["p0_" + a].astype(np.float64) for a in names}
    mP = {a: np.zeros(v.shape) for a, v in q.items()}
    for step in range(2):
        orc.train_step(q, mP, g["X"], g["R"], g["Y"].astype(np.float64), 3, "all", 5, "nll", g["rate"], g["momentum"],
                       decay_conv=np.array([1e-3, 0, 1e-2]), decay_full=np.array([1e-2, 1e-3, 0]), step=step, weight_decay_start=1)
    for a in names:
        np.testing.assert_allclose(q[a], g["p2_" + a], rtol=1e-6, atol=1e-7)


@pytest.mark.gpu
@pytest.mark.parametrize("name", SCAN_FILES)
def test_library_matches_scan_pool_fixture(name):
    from deepbind_amd import kangaroo_smat as ks
    from tests.gpu_util import assert_close, dev, host
    g = _load(name)
    W, b, X, R = dev(g["W"]), dev(g["b"]), dev(g["X"]), dev(g["R"])
    Z = dev(np.zeros_like(g["Z"]))
    ks.corr1ord(W, X, Z, 4)
    assert np.array_equal(host(Z), g["Z"])
    for pt in ("max", "avg", "all"):
        for path in ("general", "kmer") if pt == "max" else ("general",):
            P, I = ks.scanpool_fprop(W, b, X, R, pt, want_argmax=(path == "general"), path=path)
            assert_close(host(P), g["pool_" + pt], 1e-5, "%s %s" % (pt, path))
            if I is not None:
                assert np.array_equal(host(I), g["argmax_" + pt])
    dW = dev(np.zeros_like(g["W"])); ks.corr1ord_bprop_W(dW, X, dev(g["dZ"]), 4)
    assert_close(host(dW), g["dW"], 1e-4, "dW")
    dX = dev(np.zeros_like(g["dX"])); ks.corr1ord_bprop_X(dX, W, dev(g["dZ"]), 4)
    assert_close(host(dX), g["dX"], 1e-4, "dX")


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["fused", "unfused"])
def test_library_matches_train_fixture(mode):
    from deepbind_amd.model import SequenceNet
    from tests.gpu_util import assert_close, dev
    g = _load("train_two_steps.npz")
    names = ["Wc", "bc", "W1", "b1", "W2", "b2"]
    net = SequenceNet(3, 4, 6, pool="all", hidden=5, loss="nll", rate=g["rate"], momentum=g["momentum"],
                      decay_conv=[1e-3, 0, 1e-2], decay_full=[1e-2, 1e-3, 0], weight_decay_start=1, mode=mode)
    net.set_params({a: g["p0_" + a] for a in names})
    X, R, Y = dev(g["X"]), dev(g["R"]), dev(g["Y"])
    for _ in range(2):
        net.train_step(X, R, Y)
    got = net.get_params()
    for a in names:
        assert_close(got[a], g["p2_" + a], 1e-4, a)
