"""Pins for the oracle's prediction-time functions (CPU only): checks that do not retype the formula."""
import numpy as np
import pytest

from oracle import deepbind_oracle as orc


def _params(rng, m, F, pool, hidden, scale=0.6):
    k = F * (2 if pool == "all" else 1)
    p = {"Wc": rng.standard_normal((4 * m, F)) * scale, "bc": rng.standard_normal((1, F)) * 0.2}
    if hidden:
        p.update(W1=rng.standard_normal((k, hidden)) * scale, b1=rng.standard_normal((1, hidden)) * 0.1,
                 W2=rng.standard_normal((hidden, 1)) * scale, b2=rng.standard_normal((1, 1)) * 0.1)
    else:
        p.update(W1=rng.standard_normal((k, 1)) * scale, b1=rng.standard_normal((1, 1)) * 0.1)
    return p


def _random_seqs(rng, n, lo, hi, p_n=0.05):
    out = []
    for _ in range(n):
        L = int(rng.integers(lo, hi + 1))
        s = "".join("ACGT"[v] for v in rng.integers(0, 4, L))
        out.append("".join("N" if rng.random() < p_n else ch for ch in s))
    return out


def _dense_objective(p, Xd, R, pool, hidden, out, rate, keep_rows):
    """Scalar whose derivative w.r.t. the pre-activation output is Z on the kept rows: softplus(A) for the
    logistic output, Z^2/2 for the linear one. The scan is written as a dense correlation of a real
    (N, 4) input, nothing shared with the oracle's gather formulation."""
    m = p["Wc"].shape[0] // 4
    N = Xd.shape[0]
    n = N - m + 1
    Wt = p["Wc"].reshape(m, 4, -1)
    Z0 = np.zeros((N, Wt.shape[2]))
    for j in range(m):
        Z0[:n] += Xd[j:j + n] @ Wt[j]
    A0 = np.maximum(Z0 + p["bc"], 0)
    feats = []
    for a, b in R:
        mx, av = A0[a:b].max(axis=0), A0[a:b].mean(axis=0)
        feats.append(mx if pool == "max" else (av if pool == "avg" else np.stack([mx, av], 1).ravel()))
    H = np.array(feats) * (1.0 - rate)
    A = H @ p["W1"] + p["b1"]
    if hidden:
        A = np.maximum(A, 0) @ p["W2"] + p["b2"]
    A = A[:, 0]
    val = np.logaddexp(0, A) if out == "logistic" else 0.5 * A * A
    return float(val[keep_rows].sum())


@pytest.mark.parametrize("pool,hidden,out,rc", [("max", 6, "logistic", False), ("all", 0, "linear", False),
                                                ("max", 0, "logistic", True), ("avg", 5, "linear", True)])
def test_input_gradients_match_finite_differences(pool, hidden, out, rc):
    rng = np.random.default_rng(11)
    m, F, rate = 4, 5, 0.25
    p = _params(rng, m, F, pool, hidden)
    seqs = _random_seqs(rng, 4, 6, 11)
    rows = orc.insert_reverse_complements(seqs) if rc else seqs
    X, R = orc.pack(rows, m - 1)
    X, R = X.ravel(), R.astype(np.int64)
    Z, dX = orc.eval_with_input_gradients(p, X, R, 1, pool, hidden, out, dropout_rate=[rate], reverse_complement=rc)
    keep = orc.calc_zmask(Z).ravel() if rc else np.ones(len(R), bool)
    Xd = np.zeros((X.size, 4))
    for i, c in enumerate(X):
        Xd[i] = np.eye(4)[c] if c < 4 else 0.25
    h = 1e-6
    idx = [(int(i), int(c)) for i, c in zip(rng.integers(0, X.size, 40), rng.integers(0, 4, 40))]
    for i, c in idx:
        Xp, Xm = Xd.copy(), Xd.copy()
        Xp[i, c] += h
        Xm[i, c] -= h
        fd = (_dense_objective(p, Xp, R, pool, hidden, out, rate, keep) - _dense_objective(p, Xm, R, pool, hidden, out, rate, keep)) / (2 * h)
        assert abs(fd - dX[i, c]) <= 1e-6 * max(1.0, abs(fd)), (i, c, fd, dX[i, c])
    assert np.abs(dX).max() > 1e-3


@pytest.mark.parametrize("rc", [False, True])
def test_finite_difference_map_equals_single_mutant_rescoring(rc):
    """Equal-length batch: entry (i, j) of a sequence's map must be score(sequence with letter i := j) -
    score(sequence), gated to 0 when both scores are <= 0, each mutant scored on its own."""
    rng = np.random.default_rng(5)
    m, F = 5, 4
    p = _params(rng, m, F, "max", 3)
    p["b2"] -= 0.3                                   # some scores below zero so that the gate matters
    seqs = _random_seqs(rng, 3, 9, 9, p_n=0.1)
    Z, maps = orc.gen_predictions(p, seqs, "max", 3, "linear", reverse_complement=rc, want_gmaps="finite_diff")

    def score(s):
        return float(orc.gen_predictions(p, [s], "max", 3, "linear", reverse_complement=rc)[0][0, 0])

    assert len(maps) == len(seqs)
    gated = 0
    for k, s in enumerate(seqs):
        assert maps[k][0] == s and maps[k][1].shape == (len(s), 4)
        z0 = score(s)
        assert abs(z0 - Z[k, 0]) < 1e-12
        for i in range(len(s)):
            for j in range(4):
                z1 = score(s[:i] + "ACGT"[j] + s[i + 1:])
                want = (z1 - z0) if max(z0, z1) > 0 else 0.0
                gated += max(z0, z1) <= 0
                assert abs(maps[k][1][i, j] - want) < 1e-12, (k, i, j)
    assert gated > 0


def test_gradient_maps_keep_the_winning_strand():
    rng = np.random.default_rng(8)
    m, F = 4, 3
    p = _params(rng, m, F, "max", 0)
    seqs = _random_seqs(rng, 5, 7, 12, p_n=0.0)
    Z, maps = orc.gen_predictions(p, seqs, "max", 0, "logistic", reverse_complement=True, want_gmaps=True)
    assert Z.shape == (5, 1) and len(maps) == 5
    for k, s in enumerate(seqs):
        zf = orc.gen_predictions(p, [s], "max", 0, "logistic")[0][0, 0]
        zr = orc.gen_predictions(p, [orc.revcomp_string(s)], "max", 0, "logistic")[0][0, 0]
        assert abs(Z[k, 0] - max(zf, zr)) < 1e-12
        assert maps[k][0] == (s if zf >= zr else orc.revcomp_string(s))


@pytest.mark.parametrize("stride", [1, 3])
def test_prediction_maps_are_per_window_scores(stride):
    rng = np.random.default_rng(3)
    m, F, w = 4, 3, 6
    p = _params(rng, m, F, "max", 0)
    seqs = _random_seqs(rng, 2, 8, 13)
    # (the reference's window-averaged gradient map only lines up for stride 1: other strides raise in its slicing)
    pmaps, gmaps = orc.gen_predictionmaps(p, seqs, "max", 0, "linear", stride=stride, windowsize=w, want_gmaps=(stride == 1))
    for s, pm, gm in zip(seqs, pmaps, gmaps or [None] * len(seqs)):
        padded = "N" * (w - 1) + s + "N" * (w - 1)
        starts = list(range(0, len(padded) - w + 1, stride))
        assert len(pm) == len(starts)
        for t, i0 in enumerate(starts):
            z = orc.gen_predictions(p, [padded[i0:i0 + w]], "max", 0, "linear")[0][0, 0]
            assert abs(pm[t] - z) < 1e-12
        if gm is None:
            continue
        assert gm.shape == (len(s) + w - 1, 4) and np.isfinite(gm).all()
        # stride 1: every map row is the mean over the windows covering it of that window's own gradient row
        if stride == 1:
            acc, cnt = np.zeros_like(gm), np.zeros(len(gm))
            for t, i0 in enumerate(starts):
                g = orc.gen_predictions(p, [padded[i0:i0 + w]], "max", 0, "linear", want_gmaps=True)[1][0][1]
                rows = min(w, len(starts) - t)
                acc[i0:i0 + rows] += g[:rows]
                cnt[i0:i0 + rows] += 1
            assert np.allclose(gm, acc / cnt[:, None], atol=1e-12)
