"""Seeded random sweeps over shapes the hand-picked cases of the other GPU tests leave between them: ragged, empty,
overlapping, touching and shuffled regions, filter counts that fill no tile, tap counts from 1 to 40, both float types.
Every case is printed before it runs, so a failure names its shape."""
import numpy as np
import pytest

from oracle import deepbind_oracle as orc
from tests.gpu_util import dev, host

pytestmark = pytest.mark.gpu

ACT, GRAD = 1e-5, 1e-4


@pytest.fixture(scope="module")
def ks():
    from deepbind_amd import kangaroo_smat
    return kangaroo_smat


def _close(got, ref, rel, floor=0.0, slack=0.0):
    """|got - ref| <= rel * max(|ref|, scale) + slack with scale = max(largest |ref|, floor); NaNs must coincide.
    floor: the size of the terms where the result cancels to far less. slack: see _kink_slack."""
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    assert got.shape == ref.shape
    nan = np.isnan(ref)
    if not np.array_equal(np.isnan(got), nan):
        return False, float("nan")
    if nan.all():
        return True, 0.0
    scale = max(np.abs(ref[~nan]).max(), floor)
    err = np.abs(got - ref)
    bound = rel * np.maximum(np.abs(ref), scale) + 1e-30 + slack
    return bool(np.all((err <= bound)[~nan])), float(err[~nan].max())


def _kink_slack(dA, S):
    """What rows whose rectifier input lies within float32 round-off of zero may add to a column's gradients: there
    the float32 device and the float64 oracle can legitimately disagree on open / shut (per filter, as a row vector)."""
    return (np.abs(dA) * (np.abs(S) < 5e-7)).sum(axis=0)[None, :]


def _sequences(rng, kind, m, p254=0.0, cap=None):
    from deepbind_amd import data
    if kind == 0:   B, lo, hi = int(rng.integers(1, 60)), 0, int(rng.integers(1, 700))
    elif kind == 1: B, lo, hi = int(rng.integers(500, 3000)), 0, int(rng.integers(1, 40))
    elif kind == 2: L = int(rng.integers(1, 300)); B, lo, hi = int(rng.integers(50, 1000)), L, L
    elif kind == 3: B, lo, hi = int(rng.integers(100, 1500)), int(rng.integers(0, 50)), int(rng.integers(50, 250))
    else:           B, lo, hi = int(rng.integers(1, 9)), 1, int(rng.integers(500, 3000))
    if cap:                                                      # about `cap` rows at most (the oracle's map is rows x filters in float64)
        B = max(1, min(B, cap // ((lo + hi) // 2 + m)))
    ords = []
    for n in rng.integers(lo, hi + 1, size=B):
        x = rng.integers(0, 4, int(n)).astype(np.uint8)
        u = rng.random(int(n))
        x[u < 0.03] = 255
        x[u > 1.0 - p254] = 254
        ords.append(x)
    X, R = data.pack_ordinals(ords, m - 1)
    return X, R, (B, lo, hi)


def _region_variant(rng, R, variant):
    """0: as packed; 1: shuffled; 2: some dropped; 3: regions split in two that touch; 4: starts pulled back into the neighbour."""
    if variant == 1:
        R = R[rng.permutation(len(R))]
    elif variant == 2:
        R = R[rng.random(len(R)) < 0.7]
    elif variant == 3:
        parts = []
        for a, b in R:
            if b - a >= 2 and rng.random() < 0.5:
                c = int(rng.integers(a + 1, b))
                parts += [(a, c), (c, b)]
            else:
                parts.append((a, b))
        R = np.array(parts, dtype=R.dtype).reshape(-1, 2)
    elif variant == 4 and len(R) > 1:
        R = R.copy()
        k = rng.random(len(R) - 1) < 0.3
        R[1:][k, 0] = np.maximum(R[:-1][k, 0], R[1:][k, 0] - rng.integers(0, 20, k.sum()).astype(R.dtype))
    return np.ascontiguousarray(R)


def test_table_kernel_against_the_general_kernel_over_random_shapes(ks):
    """1-24 taps, any pooling, with and without argmax, empty regions included (their average is 0/0 on both paths):
    the table kernel agrees with the general kernel, and the same regions in another order give the same bits."""
    bad = []
    for case in range(120):
        rng = np.random.default_rng(100000 + case)
        m = int(rng.integers(1, 25))
        F = int(rng.choice([1, 2, 7, 16, 31, 32, 33, 64, 96, 100, 130]))
        X, R, shape = _sequences(rng, int(rng.integers(0, 5)), m)
        variant = int(rng.integers(0, 5))
        R = _region_variant(rng, R, variant)
        if len(R) == 0:
            continue
        ptype = str(rng.choice(["max", "max", "avg", "all"]))
        want = bool(rng.random() < 0.4) and ptype != "avg"
        W = (rng.standard_normal((4 * m, F)) * 0.1).astype(np.float32)
        b = (rng.standard_normal((1, F)) * 0.05 - 0.03).astype(np.float32)
        what = "case %d: m=%d F=%d sequences %s variant=%d regions=%d %s argmax=%s" % (case, m, F, shape, variant, len(R), ptype, want)
        print(what, flush=True)
        Wd, bd, Xd, Rd = dev(W), dev(b), dev(X), dev(R)
        P, I = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=want, path="kmer")
        Pg, Ig = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=want, path="general")
        P, Pg = host(P), host(Pg)
        ok, err = _close(P, Pg, ACT, floor=float(np.abs(W).max()))
        if want:
            I, Ig = host(I), host(Ig)
            ne = R[:, 1] > R[:, 0]
            rows = I // F
            ok = ok and (I != Ig).mean() < 0.01 and np.array_equal(I % F, np.broadcast_to(np.arange(F), I.shape))
            ok = ok and np.all(rows[ne] >= R[ne, :1]) and np.all(rows[ne] < R[ne, 1:2])
        perm = rng.permutation(len(R))
        P2, I2 = ks.scanpool_fprop(Wd, bd, Xd, dev(R[perm]), ptype, want_argmax=want, path="kmer")
        same = np.array_equal(host(P2), P[perm], equal_nan=True) and (not want or np.array_equal(host(I2), I[perm]))
        if not (ok and same):
            bad.append("%s: err %.3e, same bits in another order: %s" % (what, err, same))
    assert not bad, "\n".join(bad)


def test_fused_paths_against_the_oracle_chain_over_random_shapes(ks):
    """Every forward kernel the shape allows (library's choice, general, matrix cores, four filters per lane, table) and
    the backward with and without activity masks, 1-32 taps, codes 254 and 255, against the float64 operator chain."""
    bad = []
    for case in range(70):
        rng = np.random.default_rng(200000 + case)
        m = int(rng.integers(1, 33))
        F = int(rng.choice([1, 3, 16, 31, 32, 33, 64, 70, 100, 144]))
        kind = int(rng.integers(0, 5))
        X, R, shape = _sequences(rng, kind, m, p254=0.01, cap=40000)
        variant = int(rng.integers(0, 4))
        R = _region_variant(rng, R, variant)
        R = np.ascontiguousarray(R[R[:, 1] > R[:, 0]])           # (the oracle's max pooling takes no empty region)
        if len(R) == 0:
            continue
        ptype = str(rng.choice(["max", "avg", "all"]))
        W = (rng.standard_normal((4 * m, F)) * 0.1).astype(np.float32)
        b = (rng.standard_normal((1, F)) * 0.05 - 0.02).astype(np.float32)
        what = "case %d: m=%d F=%d sequences %s variant=%d regions=%d rows=%d %s" % (case, m, F, shape, variant, len(R), X.size, ptype)
        print(what, flush=True)
        Z = np.zeros((X.size, F))
        orc.corr1ord(W.astype(np.float64), X, Z)
        S = Z + b.astype(np.float64)
        A = orc.relu_fprop(S)
        Pr, Ir = orc.poolrgn(A, R, ptype, want_argmax=True)
        Wd, bd, Xd, Rd = dev(W), dev(b), dev(X), dev(R)
        for path in ["auto", "general", "mfma"] + (["wide"] if 9 <= m <= 24 else []) + (["kmer"] if m <= 24 else []):
            P, I = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=True, path=path)
            ok, err = _close(host(P), Pr, ACT, floor=float(np.abs(W).max()))
            if not ok:
                bad.append("%s: pooled[%s] err %.3e" % (what, path, err))
            if Ir is not None:
                got = host(I)
                moved = got != Ir
                if moved.any():                                  # only between rows that tie to round-off, in the same column
                    va, vb = A.ravel()[got[moved]], A.ravel()[Ir[moved]]
                    if not (np.all(np.abs(va - vb) <= ACT * np.abs(A).max()) and np.array_equal(got[moved] % F, Ir[moved] % F)):
                        bad.append("%s: argmax[%s] differs off a tie" % (what, path))
        dP = rng.standard_normal(Pr.shape).astype(np.float32)
        for use_act in (False, True):
            if use_act and ptype == "max":
                continue
            act = ks.activity_words(Xd, Wd) if use_act else None
            P, I = ks.scanpool_fprop(Wd, bd, Xd, Rd, ptype, want_argmax=True, path="general" if use_act else "auto", act=act)
            dA = np.zeros_like(A)
            orc.poolrgn_bprop(dA, R, dP.astype(np.float64), host(I) if I is not None else None, ptype)   # the device's winners
            slack = _kink_slack(dA, S)
            dZ = orc.relu_bprop(dA, A)
            dbr = orc.bias_bprop(dZ)[1]
            dWr = np.zeros(W.shape)
            orc.corr1ord_bprop_W(dWr, X, dZ)
            dW, db = dev(np.ones(W.shape, np.float32)), dev(np.full((1, F), 7.0, np.float32))
            ks.scanpool_bprop(Wd, bd, Xd, Rd, ptype, P, I, dev(dP), dW, db, act=act)
            ok, err = _close(host(dW), dWr + 1.0, GRAD, slack=slack)
            if not ok:
                bad.append("%s: dW (masks %s) err %.3e" % (what, use_act, err))
            ok, err = _close(host(db).reshape(1, -1), np.asarray(dbr).reshape(1, -1), GRAD, slack=slack)
            if not ok:
                bad.append("%s: db (masks %s) err %.3e" % (what, use_act, err))
    assert not bad, "\n".join(bad)


def _codes(rng, n):
    x = rng.integers(0, 4, n).astype(np.uint8)
    u = rng.random(n)
    x[u < 0.04] = 255
    x[u > 0.985] = 254
    return x


def test_drop_in_operators_against_the_oracle_over_random_shapes(ks):
    """corr1ord, its two gradients (1-40 taps, stream lengths on both sides of the kernels' size switches, float32 and
    float64) and poolrgn with its gradient (max / avg / sum / all, gaps, overlaps, a step column, shuffled tables)."""
    bad = []
    for case in range(200):
        rng = np.random.default_rng(300000 + case)
        which = int(rng.integers(0, 4))
        f64 = bool(rng.random() < 0.15)
        dt = np.float64 if f64 else np.float32
        tol_a, tol_g = (1e-12, 1e-12) if f64 else (ACT, GRAD)
        if which < 3:
            m = int(rng.integers(1, 41)) if rng.random() < 0.2 else int(rng.integers(1, 33))
            F = int(rng.choice([1, 2, 5, 16, 31, 32, 33, 64, 70, 128, 130, 200, 256]))
            big = rng.random() < 0.25 and not f64
            N = int(rng.integers(1 << 14, 1 << 16)) if big else int(rng.integers(1, 3000))
            if big:
                F = int(rng.choice([64, 70, 128, 200, 256]))
            X = _codes(rng, N)
            what = "case %d: %s N=%d m=%d F=%d %s" % (case, ("corr1ord", "corr1ord_bprop_W", "corr1ord_bprop_X")[which], N, m, F, dt.__name__)
            print(what, flush=True)
            if which == 0:
                W = (rng.standard_normal((4 * m, F)) * 0.1).astype(dt)
                Zr = np.full((N, F), 3.0)
                orc.corr1ord(W.astype(np.float64), X, Zr)
                Z = dev(np.full((N, F), 3.0, dt))
                ks.corr1ord(dev(W), dev(X), Z, 4)
                ok, err = _close(host(Z), Zr, tol_a)
            elif which == 1:
                dZ = rng.standard_normal((N, F)).astype(dt)
                if rng.random() < 0.4:
                    dZ[rng.random((N, F)) < 0.98] = 0
                ref = np.zeros((4 * m, F))
                orc.corr1ord_bprop_W(ref, X, dZ.astype(np.float64))
                dW, dW2 = dev(np.ones((4 * m, F), dt)), dev(np.ones((4 * m, F), dt))
                ks.corr1ord_bprop_W(dW, dev(X), dev(dZ), 4)
                ks.corr1ord_bprop_W(dW2, dev(X), dev(dZ), 4)
                ok, err = _close(host(dW), ref + 1.0, tol_g)
                ok = ok and np.array_equal(host(dW), host(dW2))
            else:
                W = (rng.standard_normal((4 * m, F)) * 0.1).astype(dt)
                dZ = rng.standard_normal((N, F)).astype(dt)
                ref = np.ones((N, 4))
                orc.corr1ord_bprop_X(ref, W.astype(np.float64), dZ.astype(np.float64))
                dX, dX2 = dev(np.ones((N, 4), dt)), dev(np.ones((N, 4), dt))
                ks.corr1ord_bprop_X(dX, dev(W), dev(dZ), 4)
                ks.corr1ord_bprop_X(dX2, dev(W), dev(dZ), 4)
                ok, err = _close(host(dX), ref, tol_g)
                ok = ok and np.array_equal(host(dX), host(dX2))
            if not ok:
                bad.append("%s: err %.3e" % (what, err))
            continue
        F = int(rng.choice([1, 2, 3, 4, 6, 8, 12, 16, 31, 32, 64, 100, 130, 256]))
        P = int(rng.integers(1, 400))
        ptype = str(rng.choice(["max", "avg", "sum", "all"]))
        layout = int(rng.integers(0, 4))
        lens = rng.integers(1, int(rng.choice([4, 30, 120, 700])) + 1, size=P)
        gap = int(rng.integers(0, 4)) if layout == 1 else 0
        edges = np.concatenate([[0], np.cumsum(lens + gap)])
        R = np.stack([edges[:-1], edges[:-1] + lens], axis=1).astype(np.uint32)
        N = int(edges[-1])
        if layout == 2:                                          # overlapping: starts pulled back
            R[1:, 0] = np.maximum(0, R[1:, 0].astype(np.int64) - rng.integers(0, 10, P - 1)).astype(np.uint32)
        if layout == 3:                                          # a step column
            R = np.concatenate([R, rng.integers(1, 5, size=(P, 1)).astype(np.uint32)], axis=1)
        if rng.random() < 0.3:
            R = np.ascontiguousarray(R[rng.permutation(P)])
        what = "case %d: poolrgn N=%d F=%d P=%d %s layout=%d %s" % (case, N, F, P, ptype, layout, dt.__name__)
        print(what, flush=True)
        U = rng.standard_normal((N, F)).astype(dt)
        if N > 4:
            U[3] = U[1]                                          # an exact tie: the first row wins
        Zr, Ir = orc.poolrgn(U, R, ptype, want_argmax=True)
        Z, I = ks.poolrgn(dev(U), dev(R), ptype, want_argmax=True)
        ok, err = _close(host(Z), Zr, tol_a)
        ok = ok and (Ir is None or np.array_equal(host(I), Ir))
        dP = rng.standard_normal(Zr.shape).astype(dt)
        ref = np.ones((N, F), np.float64)
        orc.poolrgn_bprop(ref, R, dP.astype(np.float64), Ir, ptype)
        dU = dev(np.ones((N, F), dt))
        ks.poolrgn_bprop(dU, dev(R), dev(dP), I, ptype)
        ok2, err2 = _close(host(dU), ref, tol_g)
        if not (ok and ok2):
            bad.append("%s: pooled err %.3e, gradient err %.3e" % (what, err, err2))
    assert not bad, "\n".join(bad)


def test_dense_family_against_the_oracle_over_random_shapes():
    """blockwise_dot, _nt, _tn and the scoring head: row counts on both sides of the bulk kernels' switch, block sizes
    that are / are not multiples of 4 and 16, one to 70 models, shared inputs, both float types."""
    from deepbind_amd import deepity_smat as ds
    bad = []
    for case in range(120):
        rng = np.random.default_rng(400000 + case)
        f64 = bool(rng.random() < 0.15)
        dt = np.float64 if f64 else np.float32
        tol = 1e-12 if f64 else ACT
        n = int(rng.choice([1, 3, 50, 300, 2047, 2049, 5001, 9000]))
        k = int(rng.choice([1, 3, 4, 5, 12, 16, 17, 32, 48, 64]))
        h = int(rng.choice([1, 2, 4, 7, 8, 16, 32, 33, 64]))
        nb = int(rng.choice([1, 2, 3, 4, 5, 16, 17, 37, 70]))
        X = rng.standard_normal((n, k * nb)).astype(dt)
        W = rng.standard_normal((k * nb, h)).astype(dt)
        dZ = rng.standard_normal((n, h * nb)).astype(dt)
        X64, W64, dZ64 = X.astype(np.float64), W.astype(np.float64), dZ.astype(np.float64)
        what = "case %d: n=%d k=%d h=%d models=%d %s" % (case, n, k, h, nb, dt.__name__)
        print(what, flush=True)
        fails = []
        ok, err = _close(host(ds.blockwise_dot(dev(X), dev(W), nb)), orc.blockwise_dot(X64, W64, nb), tol)
        if not ok: fails.append("dot %.3e" % err)
        ok, err = _close(host(ds.blockwise_dot_nt(dev(dZ), dev(W), nb)), orc.blockwise_dot_nt(dZ64, W64, nb), tol * 10)
        if not ok: fails.append("dot_nt %.3e" % err)
        got = host(ds.blockwise_dot_tn(dev(X), dev(dZ), nb, dev(W)))
        ok, err = _close(got, orc.blockwise_dot_tn(X64, dZ64, nb, W64), tol * 10)
        if not ok: fails.append("dot_tn %.3e" % err)
        if not np.array_equal(got, host(ds.blockwise_dot_tn(dev(X), dev(dZ), nb, dev(W)))): fails.append("dot_tn not repeatable")
        Xs = rng.standard_normal((n, k)).astype(dt)                   # one input shared by all models
        ok, err = _close(host(ds.blockwise_dot(dev(Xs), dev(W), nb)), orc.blockwise_dot(Xs.astype(np.float64), W64, nb), tol)
        if not ok: fails.append("dot shared %.3e" % err)
        ok, err = _close(host(ds.blockwise_dot_tn(dev(Xs), dev(dZ), nb, dev(W))), orc.blockwise_dot_tn(Xs.astype(np.float64), dZ64, nb, W64), tol * 10)
        if not ok: fails.append("dot_tn shared %.3e" % err)
        if not f64:
            # the scoring head: rescale -> dense -> rectifier -> dense (-> logistic), or one dense layer
            Pl = np.abs(X)
            W1, b1 = (W * 0.3).astype(np.float32), (rng.standard_normal((1, h * nb)) * 0.1).astype(np.float32)
            W2, b2 = (rng.standard_normal((h * nb, 1)) * 0.3).astype(np.float32), (rng.standard_normal((1, nb)) * 0.1).astype(np.float32)
            rate = rng.choice([0.0, 0.25, 0.5], size=nb).astype(np.float32)
            logistic = bool(rng.random() < 0.5)
            Hd = orc.relu_fprop(orc.bias_fprop(orc.blockwise_dot(orc.dropout_fp_test(Pl.astype(np.float64), rate), W1.astype(np.float64), nb), b1))
            ref = orc.bias_fprop(orc.blockwise_dot(Hd, W2.astype(np.float64), nb), b2)
            ref = orc.logistic(ref) if logistic else ref
            out = ds.head_fprop(dev(Pl), dev(W1), dev(b1), dev(W2), dev(b2), nblock=nb, in_scale=1 - rate, apply_logistic=logistic)
            ok, err = _close(host(out), ref, ACT * 3)
            if not ok: fails.append("head %.3e" % err)
            W0, b0 = (rng.standard_normal((k * nb, 1)) * 0.3).astype(np.float32), (rng.standard_normal((1, nb)) * 0.1).astype(np.float32)
            ref0 = orc.bias_fprop(orc.blockwise_dot(orc.dropout_fp_test(Pl.astype(np.float64), rate), W0.astype(np.float64), nb), b0)
            ok, err = _close(host(ds.head_fprop(dev(Pl), dev(W0), dev(b0), nblock=nb, in_scale=1 - rate)), ref0, ACT * 3)
            if not ok: fails.append("head without hidden layer %.3e" % err)
        if fails:
            bad.append(what + ": " + "; ".join(fails))
    assert not bad, "\n".join(bad)
