"""Pins for the oracle's restatement of the reference-shaped first dense layer (the "combiner": pooled features
plus a broadcast feature matrix stacked along each model's rows of W1; kangaroo/kangaroo/model.py:101-112,
deepity/std/full.py:137-178) and of the scan filters' constraints (kangaroo/_ext/corr1ord.py:60-77).
None of these retypes the functions:

  * forward: the pre-activations equal a hand-made concatenation [pooled_b | F] times model b's rows of W1;
  * an all-zero feature matrix (what the reference's data source supplies, kangaroo/data.py:59-69): the step of
    every live parameter equals the step of the model built WITHOUT the input, and the 16 dead rows move by the
    L1 term alone, written out from the Nesterov recurrence (deepity_smat.py:77-98) by hand;
  * a non-zero feature matrix: the gradient of the extra rows equals central finite differences of the loss;
  * constraints: closed-form properties (probabilities sum to one, shift invariance, largest letter at zero,
    np.clip, idempotence).
All paths relative to /root/reference/code/libs.
"""
import numpy as np
import pytest

from oracle import deepbind_oracle as orc


def _case(rng, nm, nf, m, hid, pool, q):
    k = nf * (2 if pool == "all" else 1)
    seqs = ["ACGTNACGGT", "TTGACA", "GGNNCATTAGC", "CATG", "TGCATGCAAT", "ACCA"]
    X, R = orc.pack(seqs, m - 1)
    h1 = hid if hid else 1
    p = {"Wc": rng.standard_normal((4 * m, nf * nm)) * 0.7, "bc": rng.standard_normal((1, nf * nm)) * 0.1,
         "W1": rng.standard_normal(((k + q) * nm, h1)), "b1": rng.standard_normal((1, h1 * nm)) * 0.1}
    if hid:
        p.update({"W2": rng.standard_normal((hid * nm, 1)), "b2": rng.standard_normal((1, nm)) * 0.1})
    return X, R, p, len(seqs), k


def _without_feature_rows(p, nm, k, q):
    """The same model built without the feature input: every model's last q rows of W1 cut away."""
    out = {n: v.copy() for n, v in p.items()}
    out["W1"] = np.concatenate([p["W1"][b * (k + q):b * (k + q) + k] for b in range(nm)], axis=0)
    return out


@pytest.mark.parametrize("pool,hid", [("max", 3), ("all", 0)])
def test_forward_equals_hand_concatenation(pool, hid):
    rng = np.random.default_rng(5)
    nm, nf, m, q = 3, 2, 3, 4
    X, R, p, B, k = _case(rng, nm, nf, m, hid, pool, q)
    F = rng.standard_normal((B, q))
    st = orc.model_forward(p, X, R, nm, pool, hid, features=F)
    h1 = hid if hid else 1
    for b in range(nm):
        stacked = np.concatenate([st["Pl"][:, b * k:(b + 1) * k], F], axis=1)           # [pooled_b | F]
        A1 = stacked @ p["W1"][b * (k + q):(b + 1) * (k + q)] + p["b1"][:, b * h1:(b + 1) * h1]
        A = np.maximum(A1, 0) @ p["W2"][b * hid:(b + 1) * hid] + p["b2"][:, b:b + 1] if hid else A1
        np.testing.assert_allclose(st["A"][:, b:b + 1], A, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("pool,hid,loss", [("max", 3, "nll"), ("all", 0, "mse")])
def test_zero_features_step_live_rows_as_without_and_dead_rows_by_decay_alone(pool, hid, loss):
    rng = np.random.default_rng(6)
    nm, nf, m, q = 2, 2, 3, 16
    X, R, p, B, k = _case(rng, nm, nf, m, hid, pool, q)
    Y = rng.random((B, nm))
    rate, mu, dfull = np.array([0.3, 0.05]), np.array([0.5, 0.9]), np.array([0.02, 0.3])
    kw = dict(decay_conv=0.01, decay_full=dfull, weight_decay_start=1)
    with_f = {n: v.copy() for n, v in p.items()}
    mom_f = {n: np.zeros_like(v) for n, v in p.items()}
    plain = _without_feature_rows(p, nm, k, q)
    mom_p = {n: np.zeros_like(v) for n, v in plain.items()}
    dead0 = [p["W1"][b * (k + q) + k:(b + 1) * (k + q)].copy() for b in range(nm)]
    dead, dead_m = [d.copy() for d in dead0], [np.zeros_like(d) for d in dead0]
    for step in range(3):
        orc.train_step(with_f, mom_f, X, R, Y, nm, pool, hid, loss, rate, mu, step=step, features=np.zeros((B, q)), **kw)
        orc.train_step(plain, mom_p, X, R, Y, nm, pool, hid, loss, rate, mu, step=step, **kw)
        for b in range(nm):                      # P += mu*mP ; g = decay*sign(P) once switched on ; mP = mu*mP - eta*g ; P -= eta*g
            look = dead[b] + mu[b] * dead_m[b]
            g = dfull[b] * np.sign(look) if step >= 1 else 0.0 * look
            dead_m[b] = mu[b] * dead_m[b] - rate[b] * g
            dead[b] = look - rate[b] * g
    live = _without_feature_rows(with_f, nm, k, q)
    for n in plain:
        np.testing.assert_allclose(live[n], plain[n], rtol=1e-13, atol=1e-15, err_msg=n)
    for b in range(nm):
        np.testing.assert_allclose(with_f["W1"][b * (k + q) + k:(b + 1) * (k + q)], dead[b], rtol=1e-13, atol=1e-15)
        assert np.abs(dead[b] - dead0[b]).max() > 0


def test_feature_rows_gradient_matches_finite_differences():
    rng = np.random.default_rng(7)
    nm, nf, m, q, hid, pool = 2, 2, 3, 3, 3, "all"
    X, R, p, B, k = _case(rng, nm, nf, m, hid, pool, q)
    F = rng.standard_normal((B, q))
    Y = (rng.random((B, nm)) < 0.5).astype(np.float64)

    def cost(params):
        st = orc.model_forward(params, X, R, nm, pool, hid, out="logistic", features=F)
        return orc.loss_fprop(st["Zout"], Y, "nll", nm).sum()

    work = {n: v.copy() for n, v in p.items()}
    mom = {n: np.zeros_like(v) for n, v in p.items()}
    _, g = orc.train_step(work, mom, X, R, Y, nm, pool, hid, "nll", 0.0, 0.0, features=F)      # rate 0: gradient at p itself
    eps = 1e-6
    for b in range(nm):
        for r in range(k + q):                   # the model's own rows and the feature rows alike
            for c in range(hid):
                i = b * (k + q) + r
                up = {n: v.copy() for n, v in p.items()}
                dn = {n: v.copy() for n, v in p.items()}
                up["W1"][i, c] += eps
                dn["W1"][i, c] -= eps
                fd = (cost(up) - cost(dn)) / (2 * eps)
                assert abs(fd - g["W1"][i, c]) <= 1e-6 * max(1.0, abs(fd)), (b, r, c, fd, g["W1"][i, c])


def test_constraints_closed_form_properties():
    rng = np.random.default_rng(8)
    m, F = 5, 6
    W0 = rng.standard_normal((4 * m, F)) * 2
    # pfm: every tap's four letters become log-probabilities; differences between letters are untouched
    W = orc.enforce_constraints(W0.copy(), "pfm")
    taps = W.reshape(m, 4, F)
    np.testing.assert_allclose(np.exp(taps).sum(axis=1), 1.0, rtol=1e-12)
    np.testing.assert_allclose(taps - taps[:, :1], W0.reshape(m, 4, F) - W0.reshape(m, 4, F)[:, :1], atol=1e-12)
    np.testing.assert_allclose(orc.enforce_constraints(W.copy(), "pfm"), W, atol=1e-12)
    # psam: the largest letter of every tap lands on 0, differences untouched
    W = orc.enforce_constraints(W0.copy(), "psam")
    taps = W.reshape(m, 4, F)
    np.testing.assert_allclose(taps.max(axis=1), 0.0, atol=1e-12)
    np.testing.assert_allclose(taps - taps[:, :1], W0.reshape(m, 4, F) - W0.reshape(m, 4, F)[:, :1], atol=1e-12)
    # a tap of one filter must not leak into its neighbours: change one filter, the others keep their values
    W1 = W0.copy()
    W1[:, 2] += rng.standard_normal(4 * m)
    np.testing.assert_array_equal(np.delete(orc.enforce_constraints(W1, "pfm"), 2, axis=1),
                                  np.delete(orc.enforce_constraints(W0.copy(), "pfm"), 2, axis=1))
    # clip
    np.testing.assert_array_equal(orc.enforce_constraints(W0.copy(), (-0.5, 0.25)), np.clip(W0, -0.5, 0.25))
    assert orc.enforce_constraints(W0.copy(), None) is not None and np.array_equal(orc.enforce_constraints(W0.copy(), None), W0)
    with pytest.raises(NotImplementedError):
        orc.enforce_constraints(W0.copy(), "other")


def test_constraint_is_applied_after_the_update():
    rng = np.random.default_rng(9)
    nm, nf, m, hid, pool = 2, 2, 3, 0, "max"
    X, R, p, B, k = _case(rng, nm, nf, m, hid, pool, 0)
    Y = rng.random((B, nm))
    a = {n: v.copy() for n, v in p.items()}
    b = {n: v.copy() for n, v in p.items()}
    ma, mb = ({n: np.zeros_like(v) for n, v in p.items()} for _ in range(2))
    orc.train_step(a, ma, X, R, Y, nm, pool, hid, "mse", 0.1, 0.9, constraint="pfm")
    orc.train_step(b, mb, X, R, Y, nm, pool, hid, "mse", 0.1, 0.9)
    np.testing.assert_allclose(a["Wc"], orc.enforce_constraints(b["Wc"].copy(), "pfm"), atol=1e-14)
    for n in ("bc", "W1", "b1"):
        np.testing.assert_array_equal(a[n], b[n])
