"""Pins for the CPU oracle's whole optimiser step (oracle.train_step): the function every GPU step-parity
test compares against. None of these retypes the function; each fails for a plausible mistake in it
(a model laid out along the wrong axis, an off-by-one gate, a wrong block length in the decay term,
a dropped momentum factor, the gradient taken at the wrong point).

  * a batch of models stepped together == every model stepped alone with its own scalar rates
    (pins the per-element rate / momentum / dense-decay vectors and the model axis of every parameter);
  * two Nesterov steps written out from the reference's docstring recurrence
    (deepity/deepity/_ext/deepity_smat.py:77-98, deepity_smat/gradstep.cu:41-72) with the gradient taken
    by central finite differences of the reported cost (loss + L1 weight cost), never by the oracle's
    backward pass;
  * a hand-written worked case for the scan filters' decay block length rows/ninst
    (kangaroo/kangaroo/_ext/corr1ord.py:126) and the dense layers' size/ninst (deepity/std/full.py:119);
  * the two gates at step = start - 1 and step = start
    (corr1ord.py:124,135 ; full.py:113).
All paths relative to /root/reference/code/libs.
"""
import numpy as np
import pytest

from oracle import deepbind_oracle as orc


def _case(rng, nm, nf, m, hid, pool, seqs=None):
    k = nf * (2 if pool == "all" else 1)
    seqs = seqs or ["ACGTNACGGT", "TTGACA", "GGNNCATTAGC", "CATG", "TGCATGCAAT"]
    X, R = orc.pack(seqs, m - 1)
    p = {"Wc": rng.standard_normal((4 * m, nf * nm)) * 0.7, "bc": rng.standard_normal((1, nf * nm)) * 0.1}
    if hid:
        p.update({"W1": rng.standard_normal((k * nm, hid)), "b1": rng.standard_normal((1, hid * nm)) * 0.1,
                  "W2": rng.standard_normal((hid * nm, 1)), "b2": rng.standard_normal((1, nm)) * 0.1})
    else:
        p.update({"W1": rng.standard_normal((k * nm, 1)), "b1": rng.standard_normal((1, nm)) * 0.1})
    return X, R, p, len(seqs), k


def _model_slice(p, b, nm, nf, k, hid):
    """Model b's own parameters, cut out by hand: filters are columns, dense weights are row blocks."""
    one = {"Wc": p["Wc"][:, b * nf:(b + 1) * nf].copy(), "bc": p["bc"][:, b * nf:(b + 1) * nf].copy()}
    if hid:
        one.update({"W1": p["W1"][b * k:(b + 1) * k].copy(), "b1": p["b1"][:, b * hid:(b + 1) * hid].copy(),
                    "W2": p["W2"][b * hid:(b + 1) * hid].copy(), "b2": p["b2"][:, b:b + 1].copy()})
    else:
        one.update({"W1": p["W1"][b * k:(b + 1) * k].copy(), "b1": p["b1"][:, b:b + 1].copy()})
    return one


@pytest.mark.parametrize("pool,hid,loss", [("max", 4, "nll"), ("all", 0, "mse"), ("all", 3, "nll"), ("avg", 0, "nll")])
def test_models_stepped_together_equal_models_stepped_alone(pool, hid, loss):
    rng = np.random.default_rng(31)
    nm, nf, m = 3, 2, 3
    X, R, p, B, k = _case(rng, nm, nf, m, hid, pool)
    Y = rng.random((B, nm)) if loss == "mse" else (rng.random((B, nm)) < 0.5).astype(np.float64)
    Ymask = rng.random((B, nm)) < 0.8
    rate = np.array([0.3, 0.05, 0.11])
    mu = np.array([0.5, 0.9, 0.7])
    dfull = np.array([0.02, 0.3, 0.0])
    dconv = 0.05                      # one value for all models: a per-model value depends on the grouping (worked case below)
    drop = np.array([0.5, 0.0, 0.25])
    U = rng.random((B, k * nm))
    mom = {n: rng.standard_normal(v.shape) * 0.05 for n, v in p.items()}
    together_p, together_m = {n: v.copy() for n, v in p.items()}, {n: v.copy() for n, v in mom.items()}
    for step in range(2):
        orc.train_step(together_p, together_m, X, R, Y, nm, pool, hid, loss, rate, mu, Ymask=Ymask, dropout=(drop, U),
                       decay_conv=dconv, decay_full=dfull, step=step, weight_decay_start=1)
    for b in range(nm):
        one_p, one_m = _model_slice(p, b, nm, nf, k, hid), _model_slice(mom, b, nm, nf, k, hid)
        for step in range(2):
            orc.train_step(one_p, one_m, X, R, Y[:, b:b + 1], 1, pool, hid, loss, float(rate[b]), float(mu[b]),
                           Ymask=Ymask[:, b:b + 1], dropout=(drop[b:b + 1], U[:, b * k:(b + 1) * k]),
                           decay_conv=dconv, decay_full=float(dfull[b]), step=step, weight_decay_start=1)
        want_p, want_m = _model_slice(together_p, b, nm, nf, k, hid), _model_slice(together_m, b, nm, nf, k, hid)
        for n in one_p:
            np.testing.assert_allclose(one_p[n], want_p[n], rtol=1e-12, atol=1e-14, err_msg="model %d %s" % (b, n))
            np.testing.assert_allclose(one_m[n], want_m[n], rtol=1e-12, atol=1e-14, err_msg="model %d momentum %s" % (b, n))
        # and the step did move this model: its own learning rate was applied to its own block
        assert np.abs(one_p["Wc"] - _model_slice(p, b, nm, nf, k, hid)["Wc"]).max() > 1e-6


def _fd_gradient(cost, p, h=1e-6):
    g = {}
    for n, v in p.items():
        gv = np.zeros(v.size)
        flat = v.reshape(-1)
        for i in range(flat.size):
            old = flat[i]
            flat[i] = old + h; cp = cost(p)
            flat[i] = old - h; cm = cost(p)
            flat[i] = old
            gv[i] = (cp - cm) / (2 * h)
        g[n] = gv.reshape(v.shape)
    return g


@pytest.mark.parametrize("pool,hid,loss,revcomp", [("max", 3, "nll", False), ("all", 0, "mse", False), ("max", 2, "nll", True),
                                                   ("avg", 2, "hinge", False)])
def test_two_nesterov_steps_follow_the_docstring_recurrence_with_finite_difference_gradients(pool, hid, loss, revcomp):
    """P <- P + mu*mP ; g = dCost/dP there ; mP <- mu*mP - eta*g ; P <- P - eta*g, twice from mP = 0,
    where Cost is what the reference reports: per-model loss summed over models + L1 weight cost."""
    rng = np.random.default_rng(32)
    nm, nf, m = 1, 2, 3                       # one model: the L1 term is the plain decay*sign(W) (deepity/std/full.py:114-115)
    seqs = ["ACGTNACGGT", "ACCGTNACGT", "TTGACA", "TGTCAA"] if revcomp else None
    X, R, p, B, k = _case(rng, nm, nf, m, hid, pool, seqs)
    if loss == "mse":
        Y = rng.standard_normal((B, nm))
    else:
        Y = (rng.random((B, nm)) < 0.5).astype(np.float64)
    if revcomp:
        Y = np.repeat(Y[0::2], 2, axis=0)
    Ymask = np.ones((B, nm), bool)
    Ymask[1 if not revcomp else 2] = False
    if revcomp:
        Ymask[3] = False
    eta, mu, dconv, dfull = 0.2, 0.8, 0.03, 0.07
    drop = np.array([0.4])
    U = rng.random((B, k * nm))
    out = "logistic" if loss == "nll" else "linear"

    def cost(q):
        st = orc.model_forward(q, X, R, nm, pool, hid, out=out, dropout=(drop, U), train=True, matchrows=revcomp)
        # the pair rule picks which strand trains from the predictions at the evaluation point and is not
        # differentiated through (deepity/std/loss.py:114-119): freeze it per call site below
        Zmask = cost.zmask
        return float(orc.loss_fprop(st["Zout"], Y, loss, nm, Ymask=Ymask, Zmask=Zmask).sum()
                     + orc.weight_cost(q, nm, dconv, dfull).sum())

    def grad_at(q):
        if revcomp:
            st = orc.model_forward(q, X, R, nm, pool, hid, out=out, dropout=(drop, U), train=True, matchrows=True)
            a, b = st["Zout"][0::2], st["Zout"][1::2]
            zm = np.zeros(st["Zout"].shape, bool)
            zm[0::2], zm[1::2] = a >= b, a < b                 # the larger prediction of each pair trains, ties: the forward strand
            cost.zmask = zm
        else:
            cost.zmask = None
        return _fd_gradient(cost, q)

    P = {n: v.copy() for n, v in p.items()}
    mP = {n: np.zeros(v.shape) for n, v in p.items()}
    got_p, got_m = {n: v.copy() for n, v in p.items()}, {n: np.zeros(v.shape) for n, v in p.items()}
    for step in range(2):
        for n in P:
            P[n] = P[n] + mu * mP[n]
        g = grad_at(P)
        for n in P:
            mP[n] = mu * mP[n] - eta * g[n]
            P[n] = P[n] - eta * g[n]
        orc.train_step(got_p, got_m, X, R, Y, nm, pool, hid, loss, eta, mu, Ymask=Ymask, dropout=(drop, U),
                       decay_conv=dconv, decay_full=dfull, step=step, weight_decay_start=0, reverse_complement=revcomp)
        for n in P:
            np.testing.assert_allclose(got_p[n], P[n], rtol=0, atol=2e-8, err_msg="step %d %s" % (step, n))
            np.testing.assert_allclose(got_m[n], mP[n], rtol=0, atol=2e-8, err_msg="step %d momentum %s" % (step, n))
    # the second step really used the momentum: dropping the mu*mP look-ahead would land elsewhere
    assert max(np.abs(got_m[n]).max() for n in got_m) > 1e-3


def test_l1_decay_block_lengths_worked_case():
    """Two models, one 2-tap filter each: Wc is (8, 2), flattened row-major; the reference calls
    madd_bcast(sign(W), decay, W.shape[0]/ninst = 4, dW), i.e. element i takes decay[(i // 4) % 2]
    (kangaroo/_ext/corr1ord.py:126, deepity_smat/madd_bcast.cu:41-47). Elements 0-3 are rows 0-1 (both columns),
    4-7 rows 2-3, ... so the coefficient alternates every two ROWS, not per column, although models are columns.
    Dense weights use size/ninst: W1 (2 models x 1 feature, 3 hidden) -> elements 0-2 model 0, 3-5 model 1."""
    rng = np.random.default_rng(33)
    nm, nf, m, hid = 2, 1, 2, 3
    X, R, p, B, k = _case(rng, nm, nf, m, hid, "max")
    Y = (rng.random((B, nm)) < 0.5).astype(np.float64)
    dconv, dfull = np.array([10.0, 1000.0]), np.array([3.0, 7.0])
    runs = {}
    for name, start in (("off", 5), ("on", 0)):
        q, mom = {n: v.copy() for n, v in p.items()}, {n: np.zeros(v.shape) for n, v in p.items()}
        _, g = orc.train_step(q, mom, X, R, Y, nm, "max", hid, "nll", 0.1, 0.9, decay_conv=dconv, decay_full=dfull,
                              step=0, weight_decay_start=start)
        runs[name] = g
    want_conv = np.array([[10, 10], [10, 10], [1000, 1000], [1000, 1000], [10, 10], [10, 10], [1000, 1000], [1000, 1000]], float)
    want_w1 = np.array([[3, 3, 3], [7, 7, 7]], float)
    want_w2 = np.array([[3], [3], [3], [7], [7], [7]], float)
    sgn = lambda a: (a > 0).astype(float) - (a < 0).astype(float)
    # momentum starts at zero, so the gradient is taken at the initial parameters
    np.testing.assert_allclose(runs["on"]["Wc"] - runs["off"]["Wc"], sgn(p["Wc"]) * want_conv, rtol=1e-9, atol=1e-12)
    np.testing.assert_allclose(runs["on"]["W1"] - runs["off"]["W1"], sgn(p["W1"]) * want_w1, rtol=1e-9, atol=1e-12)
    np.testing.assert_allclose(runs["on"]["W2"] - runs["off"]["W2"], sgn(p["W2"]) * want_w2, rtol=1e-9, atol=1e-12)
    for n in ("bc", "b1", "b2"):
        assert np.array_equal(runs["on"][n], runs["off"][n]), "biases carry no decay"


def test_decay_and_freeze_gates_at_the_boundary_steps():
    rng = np.random.default_rng(34)
    nm, nf, m, hid = 2, 2, 3, 0
    X, R, p, B, k = _case(rng, nm, nf, m, hid, "all")
    Y = rng.standard_normal((B, nm))

    def run(step, wds, start_training):
        q, mom = {n: v.copy() for n, v in p.items()}, {n: np.zeros(v.shape) for n, v in p.items()}
        _, g = orc.train_step(q, mom, X, R, Y, nm, "all", hid, "mse", 0.1, 0.9, decay_conv=0.5, decay_full=0.25,
                              step=step, weight_decay_start=wds, start_training=start_training)
        return q, g

    _, plain = run(0, 100, 0)
    # weight_decay_start <= step switches the decay on: off at start-1, on at start (corr1ord.py:124, full.py:113)
    _, before = run(6, 7, 0)
    _, at = run(7, 7, 0)
    for n in plain:
        assert np.array_equal(before[n], plain[n]), n
    assert np.abs(at["Wc"] - plain["Wc"]).max() == pytest.approx(0.5) and np.abs(at["W1"] - plain["W1"]).max() == pytest.approx(0.25)
    # start_training > step zeroes the scan filters' gradient (after the decay was added): frozen at start-1, free at start
    # (corr1ord.py:135-136); biases and dense weights train from the first step
    q_frozen, frozen = run(2, 0, 3)
    q_free, free = run(3, 0, 3)
    assert not frozen["Wc"].any() and np.array_equal(q_frozen["Wc"], p["Wc"])
    assert np.array_equal(free["Wc"], at["Wc"]) and not np.array_equal(q_free["Wc"], p["Wc"])
    assert np.array_equal(frozen["bc"], free["bc"]) and frozen["bc"].any() and np.array_equal(frozen["W1"], free["W1"])
