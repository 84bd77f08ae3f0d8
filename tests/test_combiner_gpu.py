"""GPU parity of the reference-shaped first dense layer (pooled features + a broadcast feature matrix stacked along
each model's rows of W1: kangaroo/kangaroo/model.py:101-112, deepity/std/full.py:137-178) and of the scan filters'
constraints (kangaroo/_ext/corr1ord.py:60-77, deepity/sgd.py:103-107,137) against the CPU oracle, in every way a
step can be issued: natively (one call), fused with injected uniforms, layer by layer through the `_combined`
drop-in operators, as shared launches of several architecture groups, and from a captured graph."""
import numpy as np
import pytest
import torch

from oracle import deepbind_oracle as orc
from tests.gpu_util import assert_close, assert_close_per_model, dev, host, record_error

pytestmark = pytest.mark.gpu

ACT, GRAD = 1e-5, 1e-4
NFEAT = 16              # the reference's models carry 16 such columns


def _f64(d):
    return {k: np.asarray(v, dtype=np.float64).copy() for k, v in d.items()}


def _setup(pool, hidden, loss, nm=3, nf=16, m=11, B=70, seed=3, **netkw):
    from deepbind_amd import data
    from deepbind_amd.model import SequenceNet
    rng = np.random.default_rng(seed)
    seqs = ["".join("ACGTN"[c] for c in rng.choice(5, size=int(rng.integers(12, 45)), p=[.24, .24, .24, .24, .04])) for _ in range(B)]
    X, R = data.pack_sequences(seqs, m - 1)
    net = SequenceNet(nm, nf, m, pool=pool, hidden=hidden, loss=loss, feature_columns=NFEAT, **netkw)
    params = {name: (rng.standard_normal(shape) * (0.3 if name.startswith("W") else 0.05)).astype(np.float32) for name, shape, _ in net.layout}
    net.set_params(params)
    Y = rng.random((B, nm)).astype(np.float32) if loss == "mse" else (rng.random((B, nm)) < 0.5).astype(np.float32)
    F = rng.standard_normal((B, NFEAT)).astype(np.float32)
    return net, params, X, R, Y, F, rng


@pytest.mark.parametrize("how", ["native", "fused_u", "unfused"])
@pytest.mark.parametrize("pool,hidden,loss,with_f", [("max", 32, "nll", True), ("all", 0, "mse", True), ("max", 32, "nll", False),
                                                     ("avg", 8, "nll", False)])
def test_feature_columns_train_steps_match_the_oracle(how, pool, hidden, loss, with_f):
    rate, mu, drop = np.array([0.05, 0.02, 0.1]), np.array([0.9, 0.5, 0.8]), np.array([0.5, 0.0, 0.25])
    dfull, dconv = np.array([1e-3, 3e-2, 0.0]), 1e-3
    net, params, X, R, Y, F, rng = _setup(pool, hidden, loss, rate=rate, momentum=mu, dropout=drop, decay_conv=dconv, decay_full=dfull,
                                          weight_decay_start=1, mode="unfused" if how == "unfused" else "fused")
    nm, k = net.ninst, net.k
    assert net.p["W1"].shape[0] == (k + NFEAT) * nm
    Xd, Rd, Yd = dev(X), dev(R), dev(Y)
    Fd = dev(F) if with_f else None
    Fo = F.astype(np.float64) if with_f else np.zeros((len(R), NFEAT))
    ref_p, ref_m = _f64(params), {n: np.zeros(v.shape) for n, v in params.items()}
    from deepbind_amd import deepity_smat as ds
    for step in range(3):
        if how == "native":
            U = host(ds.uniform_like(torch.empty((len(R), k * nm), device="cuda"), net.rng_seed, net._rng_offset))
            net.train_step(Xd, Rd, Yd, F=Fd)
        else:
            U = rng.random((len(R), k * nm)).astype(np.float32)
            net.train_step(Xd, Rd, Yd, U=dev(U), F=Fd)
        _, g = orc.train_step(ref_p, ref_m, X, R, Y.astype(np.float64), nm, pool, hidden, loss, rate, mu, dropout=(drop, U),
                              decay_conv=dconv, decay_full=dfull, step=step, weight_decay_start=1, features=Fo)
        got = net.get_grads()
        for name, _, axis in net.layout:
            assert_close_per_model(got[name], g[name], GRAD, nm, axis, "step %d gradient %s (%s)" % (step, name, how))
            record_error("combiner (%s)" % how, "gradients", got[name], g[name], GRAD)
    got = net.get_params()
    for name, _, axis in net.layout:
        assert_close_per_model(got[name], ref_p[name], GRAD, nm, axis, "parameters %s (%s)" % (name, how))
    # the feature rows did move (decay alone when the features are zeros), and test-mode predictions agree
    for b in range(nm):
        rows = slice(b * (k + NFEAT) + k, (b + 1) * (k + NFEAT))
        if dfull[b] > 0 or with_f:
            assert np.abs(got["W1"][rows] - params["W1"][rows]).max() > 0
    st = orc.model_forward(ref_p, X, R, nm, pool, hidden, out="logistic" if loss == "nll" else "linear",
                           dropout=(drop, None), train=False, features=Fo)
    assert_close(host(net.predict(Xd, Rd, Fd)), st["Zout"], ACT, "predictions (%s)" % how)
    assert_close(host(net.forward(Xd, Rd, F=Fd)["Z"]), st["Zout"], ACT, "layer-by-layer predictions (%s)" % how)
    # the L1 cost covers the feature rows too (deepity/std/full.py:92-109)
    net.step_count = 5
    assert_close(net.penalty_value(), orc.weight_cost(_f64(got), nm, dconv, dfull), 1e-5, "L1 cost")


def test_zero_feature_matrix_equals_no_feature_matrix_bit_for_bit():
    """F = None (the reference's all-zero matrix, skipped by the kernels) and an explicit matrix of zeros give the same bits."""
    outs = []
    for explicit in (False, True):
        net, params, X, R, Y, F, _ = _setup("all", 32, "nll", rate=0.05, momentum=0.9, dropout=0.3, decay_full=1e-2, weight_decay_start=0)
        Fd = torch.zeros((len(R), NFEAT), device="cuda") if explicit else None
        for _ in range(3):
            net.train_step(dev(X), dev(R), dev(Y), F=Fd)
        outs.append((net.get_params(), host(net.predict(dev(X), dev(R), Fd))))
    for name in outs[0][0]:
        assert np.array_equal(outs[0][0][name], outs[1][0][name]), name
    assert np.array_equal(outs[0][1], outs[1][1])


def test_bulk_scoring_head_with_feature_columns():
    """The 16-models-per-workgroup scoring head (>= 4096 rows) with and without a feature matrix."""
    from deepbind_amd import deepity_smat as ds
    rng = np.random.default_rng(11)
    n, nm, k, h = 5000, 20, 16, 32
    pooled = rng.random((n, k * nm)).astype(np.float32)
    F = rng.standard_normal((n, NFEAT)).astype(np.float32)
    p = {"W1": rng.standard_normal(((k + NFEAT) * nm, h)).astype(np.float32) * 0.2, "b1": rng.standard_normal((1, h * nm)).astype(np.float32) * 0.1,
         "W2": rng.standard_normal((h * nm, 1)).astype(np.float32) * 0.2, "b2": rng.standard_normal((1, nm)).astype(np.float32) * 0.1}
    scale = rng.random(nm).astype(np.float32)
    for feats in (F, None):
        Fo = F.astype(np.float64) if feats is not None else np.zeros((n, NFEAT))
        A1 = orc.blockwise_dot_combined([pooled.astype(np.float64) * np.repeat(scale.astype(np.float64), k), Fo], p["W1"].astype(np.float64), nm, [False, True])
        H1 = np.maximum(A1 + p["b1"], 0)
        ref = orc.logistic(orc.blockwise_dot(H1, p["W2"].astype(np.float64), nm) + p["b2"])
        for rows in (n, 300):                    # bulk kernel and the one-model-per-workgroup kernel
            got = ds.head_fprop(dev(pooled[:rows]), dev(p["W1"]), dev(p["b1"]), dev(p["W2"]), dev(p["b2"]), nblock=nm, in_scale=dev(scale),
                                apply_logistic=True, nfeat=NFEAT, feats=None if feats is None else dev(feats[:rows]))
            assert_close(host(got), ref[:rows], ACT, "scoring head, %d rows, feats %s" % (rows, feats is not None))


def test_group_of_architectures_with_feature_columns_shared_launches_and_graph():
    """Several architecture groups with feature columns: the shared launches give each group the bits of its own
    step, and a captured graph replays the same steps."""
    from deepbind_amd import data
    from deepbind_amd.model import ModelGroup
    rng = np.random.default_rng(21)
    m, nf, B = 12, 16, 96
    seqs = ["".join("ACGT"[c] for c in rng.integers(0, 4, int(rng.integers(20, 41)))) for _ in range(B)]
    X, R = data.pack_sequences(seqs, m - 1)
    pools, hiddens = ["max", "all", "max", "all", "max", "all"], [32, 0, 0, 32, 32, 0]
    Y = (rng.random((B, len(pools))) < 0.5).astype(np.float32)
    F = rng.standard_normal((B, NFEAT)).astype(np.float32)
    Xd, Rd, Yd, Fd = dev(X), dev(R), dev(Y), dev(F)

    def make():
        grp = ModelGroup(pools, hiddens, nf, m, loss="nll", rate=0.05, momentum=0.9, dropout=0.25, decay_full=1e-2,
                         weight_decay_start=1, feature_columns=NFEAT, single_launch=False)
        for gi, (_, net) in enumerate(grp.groups):
            net.init_params(init_conv=0.1, init_full=0.1, seed=gi)
            net.rng_seed = 7 + gi
        return grp
    together, alone, graphed = make(), make(), make()
    step = graphed.make_graphed_step(Xd, Rd, Yd, F=Fd)
    for _ in range(3):
        together.train_step(Xd, Rd, Yd, F=Fd)
        for idx, net in alone.groups:
            net.train_step(Xd, Rd, Yd[:, idx].contiguous(), F=Fd)
        step()
        torch.cuda.synchronize()
    for (_, a), (_, b), (_, c) in zip(together.groups, alone.groups, graphed.groups):
        pa, pb, pc = a.get_params(), b.get_params(), c.get_params()
        for name in pa:
            assert np.array_equal(pa[name], pb[name]), "shared launches vs own step: %s" % name
            assert np.array_equal(pa[name], pc[name]), "graph replay vs eager: %s" % name
    one = together.slice_model(3)
    assert one.nfeat == NFEAT and np.array_equal(host(one.predict(Xd, Rd, Fd))[:, 0], host(together.predict(Xd, Rd, Fd))[:, 3])


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("constraint", ["pfm", "psam", (-0.2, 0.35)])
def test_scan_filter_constraint_operator(constraint, dtype):
    from deepbind_amd import kangaroo_smat as ks
    rng = np.random.default_rng(2)
    W = (rng.standard_normal((4 * 24, 150)) * 1.5).astype(dtype)
    ref = orc.enforce_constraints(W.astype(np.float64), constraint)
    Wd = dev(W)
    ks.corr1ord_enforce_constraints(Wd, constraint)
    got = host(Wd)
    if isinstance(constraint, tuple):
        assert np.array_equal(got, np.clip(W, dtype(constraint[0]), dtype(constraint[1])))
    else:
        tol = 2e-6 if dtype == np.float32 else 1e-13
        assert np.abs(got - ref).max() <= tol * max(1.0, np.abs(ref).max())
    with pytest.raises(NotImplementedError):
        ks.corr1ord_enforce_constraints(Wd, "other")
    ks.corr1ord_enforce_constraints(Wd, None)
    assert np.array_equal(host(Wd), got)


@pytest.mark.parametrize("mode", ["fused", "unfused"])
@pytest.mark.parametrize("constraint", ["pfm", (-0.4, 0.5)])       # (a tight clip would make most weights equal and the max pool tie)
def test_constraint_enforced_after_every_step(mode, constraint):
    net, params, X, R, Y, F, _ = _setup("max", 32, "nll", nm=2, rate=0.05, momentum=0.9, mode=mode, constraint=constraint)
    ref_p, ref_m = _f64(params), {n: np.zeros(v.shape) for n, v in params.items()}
    net.enforce_constraints()                                    # the trainer's call before the first step (sgd.py:107)
    orc.enforce_constraints(ref_p["Wc"], constraint)
    Xd, Rd, Yd = dev(X), dev(R), dev(Y)
    for step in range(3):
        net.train_step(Xd, Rd, Yd)
        orc.train_step(ref_p, ref_m, X, R, Y.astype(np.float64), 2, "max", 32, "nll", 0.05, 0.9, step=step,
                       features=np.zeros((len(R), NFEAT)), constraint=constraint)
    got = net.get_params()
    for name, _, axis in net.layout:
        assert_close_per_model(got[name], ref_p[name], GRAD, 2, axis, "parameters %s" % name)
    if constraint == "pfm":
        np.testing.assert_allclose(np.exp(got["Wc"].astype(np.float64)).reshape(-1, 4, got["Wc"].shape[1]).sum(axis=1), 1.0, rtol=1e-5)
    else:
        assert got["Wc"].min() == np.float32(-0.4) and got["Wc"].max() == np.float32(0.5)
