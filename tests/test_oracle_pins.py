"""Pins for the CPU oracle: every check here fails for a plausible transcription mistake
(dropped term, wrong sign/index, transposed operand) and none of them retypes the oracle's formula."""
import numpy as np
import pytest
import torch

from oracle import deepbind_oracle as orc


def _rand_case(rng, N=60, m=5, F=7, pn=0.1, p254=0.0, dtype=np.float64):
    X = rng.integers(0, 4, size=N).astype(np.uint8)
    u = rng.random(N)
    X[u < pn] = 255
    X[(u >= pn) & (u < pn + p254)] = 254
    W = rng.standard_normal((4 * m, F)).astype(dtype)
    return W, X.reshape(-1, 1)


def _onehot5(X):
    """(4, N) one-hot with N/pad columns = 1/4 and 254 columns = 0."""
    x = X.ravel()
    oh = np.zeros((4, x.size))
    for c in range(4):
        oh[c, x == c] = 1.0
    oh[:, (x >= 4) & (x != 254)] = 0.25
    return oh


def test_pack_worked_example():
    # "AC","G" with m=3: two pad bytes before, between and after the sequences
    X, R = orc.pack(["AC", "G"], 2)
    assert X.ravel().tolist() == [255, 255, 0, 1, 255, 255, 2, 255, 255]
    assert R.tolist() == [[0, 4], [4, 7]]
    assert X.dtype == np.uint8 and R.dtype == np.uint32
    # lower case, U == T, anything else is 255
    assert orc.acgt2ord("acgtuN.x").tolist() == [0, 1, 2, 3, 3, 255, 255, 255]
    # n = N-m+1 equals the end of the last region, so every pooled row is computed
    assert X.size - 3 + 1 == R[-1, 1]


def test_corr1ord_equals_conv1d_on_onehot():
    rng = np.random.default_rng(10)
    W, X = _rand_case(rng, N=80, m=6, F=5, pn=0.15, p254=0.05)
    m, F, N = 6, 5, 80
    Z = np.full((N, F), 7.0)
    orc.corr1ord(W, X, Z)
    # library routine: cross-correlation of the 4-channel one-hot with kernels W[f][c][j]
    inp = torch.from_numpy(_onehot5(X))[None]                        # (1, 4, N)
    ker = torch.from_numpy(W.reshape(m, 4, F).transpose(2, 1, 0).copy())  # (F, 4, m)
    ref = torch.nn.functional.conv1d(inp, ker)[0].numpy().T          # (n, F)
    n = N - m + 1
    np.testing.assert_allclose(Z[:n], ref, rtol=1e-12, atol=1e-12)
    assert np.all(Z[n:] == 7.0)                                      # rows >= n untouched


def test_corr1ord_bruteforce_and_float32_order():
    rng = np.random.default_rng(11)
    W, X = _rand_case(rng, N=40, m=4, F=3, pn=0.2, p254=0.1, dtype=np.float32)
    Z = np.zeros((40, 3), np.float32)
    orc.corr1ord(W, X, Z)
    # the scalar loop accumulates j ascending in float32: bit-identical, not merely close
    assert np.array_equal(Z, orc.corr1ord_bruteforce(W, X))


def test_corr1ord_invariants():
    rng = np.random.default_rng(12)
    m, F, N = 5, 4, 30
    W = rng.standard_normal((4 * m, F))
    # all-N input: every output is the sum over taps of the channel mean
    X = np.full((N, 1), 255, np.uint8)
    Z = np.zeros((N, F))
    orc.corr1ord(W, X, Z)
    expect = W.reshape(m, 4, F).mean(axis=1).sum(axis=0)
    np.testing.assert_allclose(Z[:N - m + 1], np.tile(expect, (N - m + 1, 1)), rtol=1e-12)
    # adding c to all four channels of tap j adds c to every output (also at N positions)
    W2, X2 = _rand_case(rng, N=N, m=m, F=F, pn=0.3)
    Za = np.zeros((N, F)); orc.corr1ord(W2, X2, Za)
    W3 = W2.copy(); W3[4 * 2:4 * 3] += 1.5
    Zb = np.zeros((N, F)); orc.corr1ord(W3, X2, Zb)
    np.testing.assert_allclose(Zb[:N - m + 1] - Za[:N - m + 1], 1.5, rtol=1e-9)
    # code 254 is the same as deleting that tap's term
    X4 = X2.copy(); X4[10] = 254
    Zc = np.zeros((N, F)); orc.corr1ord(W2, X4, Zc)
    lut = W2.reshape(m, 4, F)
    for i in range(N - m + 1):
        j = 10 - i
        if 0 <= j < m:
            k = int(X2[10, 0])
            term = lut[j, k] if k < 4 else lut[j].mean(axis=0)
            np.testing.assert_allclose(Za[i] - Zc[i], term, rtol=1e-9, atol=1e-12)
        else:
            np.testing.assert_allclose(Za[i], Zc[i])


def test_bprop_W_is_exact_adjoint_and_matches_fd():
    rng = np.random.default_rng(13)
    W, X = _rand_case(rng, N=70, m=6, F=5, pn=0.15, p254=0.05)
    N, F = 70, 5
    n = N - 6 + 1
    dZ = rng.standard_normal((N, F))
    Z = np.zeros((N, F)); orc.corr1ord(W, X, Z)
    dW = np.zeros_like(W); orc.corr1ord_bprop_W(dW, X, dZ)
    # <corr1ord(W,X), dZ> == <W, bprop_W(X,dZ)> because the op is linear in W (rows >= n excluded)
    np.testing.assert_allclose((Z[:n] * dZ[:n]).sum(), (W * dW).sum(), rtol=1e-11)
    # central differences on a few entries
    for (r, c) in [(0, 0), (7, 3), (23, 4), (13, 1)]:
        Wp = W.copy(); Wp[r, c] += 1e-6
        Wm = W.copy(); Wm[r, c] -= 1e-6
        Zp = np.zeros((N, F)); orc.corr1ord(Wp, X, Zp)
        Zm = np.zeros((N, F)); orc.corr1ord(Wm, X, Zm)
        fd = ((Zp[:n] - Zm[:n]) * dZ[:n]).sum() / 2e-6
        np.testing.assert_allclose(dW[r, c], fd, rtol=1e-6, atol=1e-8)
    # accumulates into dW rather than overwriting
    dW2 = np.ones_like(W); orc.corr1ord_bprop_W(dW2, X, dZ)
    np.testing.assert_allclose(dW2, dW + 1.0, rtol=1e-12)


def test_bprop_X_bruteforce_and_adjoint():
    rng = np.random.default_rng(14)
    m, F, n = 4, 3, 25
    W = rng.standard_normal((4 * m, F))
    dZ = rng.standard_normal((n, F))
    dX = np.zeros((n, 4)); orc.corr1ord_bprop_X(dX, W, dZ)
    # the reference's host loop, literally: i over rows, filters, taps k<=i
    ref = np.zeros((n, 4))
    for i in range(n):
        for f in range(F):
            for k in range(m):
                if i < k:
                    continue
                for c in range(4):
                    ref[i, c] += dZ[i - k, f] * W[4 * k + c, f]
    np.testing.assert_allclose(dX, ref, rtol=1e-12, atol=1e-12)
    # adjoint of the dense (soft one-hot) convolution: <conv(S), dZ> == <S, dX> with S any (n,4) input,
    # restricted to outputs whose window lies inside S
    S = rng.standard_normal((n, 4))
    inp = torch.from_numpy(S.T.copy())[None]
    ker = torch.from_numpy(W.reshape(m, 4, F).transpose(2, 1, 0).copy())
    conv = torch.nn.functional.conv1d(inp, ker)[0].numpy().T         # (n-m+1, F)
    dZ0 = dZ.copy(); dZ0[n - m + 1:] = 0
    dX0 = np.zeros((n, 4)); orc.corr1ord_bprop_X(dX0, W, dZ0)
    np.testing.assert_allclose((conv * dZ0[:n - m + 1]).sum(), (S * dX0).sum(), rtol=1e-11)


@pytest.mark.parametrize("ptype", ["max", "avg", "sum", "all"])
def test_poolrgn_against_numpy_slices(ptype):
    rng = np.random.default_rng(15)
    N, F = 50, 6
    U = rng.standard_normal((N, F)).astype(np.float32)
    U[12] = U[10]                       # exact ties inside region 1: first one must win
    R = np.array([[0, 7], [7, 20], [20, 21], [21, 50]], np.uint32)
    Zp, I = orc.poolrgn(U, R, ptype, want_argmax=True)
    for r, (a, b) in enumerate(R):
        blk = U[a:b]
        if ptype in ("max", "all"):
            mx = Zp[r] if ptype == "max" else Zp[r, 0::2]
            assert np.array_equal(mx, blk.max(axis=0))
            assert np.array_equal(I[r], (a + blk.argmax(axis=0)) * F + np.arange(F))
            assert np.array_equal(U.ravel()[I[r]], mx)
        if ptype in ("avg", "all"):
            av = Zp[r] if ptype == "avg" else Zp[r, 1::2]
            np.testing.assert_allclose(av, blk.mean(axis=0, dtype=np.float64), rtol=2e-6, atol=1e-7)
        if ptype == "sum":
            np.testing.assert_allclose(Zp[r], blk.sum(axis=0, dtype=np.float64), rtol=2e-6, atol=1e-6)
    if ptype in ("avg", "sum"):
        assert I is None
    assert Zp.shape == (4, F * (2 if ptype == "all" else 1))


def test_poolrgn_step_column():
    rng = np.random.default_rng(16)
    U = rng.standard_normal((30, 3))
    R = np.array([[0, 10, 3], [10, 30, 4]], np.uint32)     # rows 0,3,6,9 and 10,14,...,26
    Zp, I = orc.poolrgn(U, R, "all", want_argmax=True)
    for r, (a, b, s) in enumerate(R):
        blk = U[a:b:s]
        np.testing.assert_allclose(Zp[r, 0::2], blk.max(axis=0))
        np.testing.assert_allclose(Zp[r, 1::2], blk.mean(axis=0), rtol=1e-12)


@pytest.mark.parametrize("ptype", ["max", "avg", "sum", "all"])
def test_poolrgn_bprop_is_adjoint(ptype):
    rng = np.random.default_rng(17)
    N, F = 40, 5
    U = rng.standard_normal((N, F))
    R = np.array([[0, 9], [9, 25], [25, 40]], np.uint32)
    Zp, I = orc.poolrgn(U, R, ptype, want_argmax=True)
    dP = rng.standard_normal(Zp.shape)
    dU = np.zeros_like(U)
    orc.poolrgn_bprop(dU, R, dP, I, ptype)
    # directional derivative of <pool(U), dP> along a random direction D equals <dU, D>
    D = rng.standard_normal(U.shape)
    eps = 1e-7
    Zq, _ = orc.poolrgn(U + eps * D, R, ptype)
    Zm, _ = orc.poolrgn(U - eps * D, R, ptype)
    fd = ((Zq - Zm) * dP).sum() / (2 * eps)
    np.testing.assert_allclose((dU * D).sum(), fd, rtol=1e-6)
    # accumulates
    dU2 = np.ones_like(U); orc.poolrgn_bprop(dU2, R, dP, I, ptype)
    np.testing.assert_allclose(dU2, dU + 1, rtol=1e-12)


def test_elementwise_closed_forms():
    rng = np.random.default_rng(18)
    A = rng.standard_normal((9, 4)).astype(np.float32)
    b = rng.standard_normal((1, 4)).astype(np.float32)
    assert np.array_equal(orc.bias_fprop(A, b), A + b)
    assert np.array_equal(orc.relu_fprop(A), np.where(A > 0, A, 0))
    assert np.array_equal(orc.sign(A), np.sign(A))
    dZ = rng.standard_normal(A.shape).astype(np.float32)
    assert np.array_equal(orc.relu_bprop(dZ, orc.relu_fprop(A)), np.where(A > 0, dZ, 0))
    np.testing.assert_allclose(orc.bias_bprop(dZ)[1].ravel(), dZ.astype(np.float64).sum(axis=0), rtol=1e-6)
    # logistic: symmetric about 0.5 and the inverse of the logit
    Z = orc.logistic(A)
    np.testing.assert_allclose(Z + orc.logistic(-A), 1.0, rtol=1e-6)
    np.testing.assert_allclose(np.log(Z / (1 - Z)), A, rtol=1e-4, atol=1e-5)


def test_loss_closed_forms_and_gradient():
    rng = np.random.default_rng(19)
    n, ninst = 12, 3
    A = rng.standard_normal((n, ninst))
    Y = (rng.random((n, ninst)) < 0.5).astype(np.float64)
    Ymask = rng.random((n, ninst)) < 0.8
    Z = orc.logistic(A)
    L = orc.loss_fprop(Z, Y, "nll", ninst, Ymask=Ymask)
    # textbook binary cross-entropy over unmasked rows, mean over ALL rows
    bce = -(Y * np.log(Z) + (1 - Y) * np.log(1 - Z)) * Ymask
    np.testing.assert_allclose(L.ravel(), bce.sum(axis=0) / n, rtol=1e-12)
    # d(sum_j L_j)/dA == loss_bprop (the logistic's derivative cancels, softmax bprop is identity)
    dA = orc.loss_bprop(Z, Y, Ymask=Ymask)
    eps = 1e-6
    for (i, j) in [(0, 0), (5, 2), (11, 1)]:
        Ap = A.copy(); Ap[i, j] += eps
        Am = A.copy(); Am[i, j] -= eps
        fd = (orc.loss_fprop(orc.logistic(Ap), Y, "nll", ninst, Ymask=Ymask).sum()
              - orc.loss_fprop(orc.logistic(Am), Y, "nll", ninst, Ymask=Ymask).sum()) / (2 * eps)
        np.testing.assert_allclose(dA[i, j], fd, rtol=1e-6, atol=1e-10)
    # mse: 0.5*mean((Z-Y)^2), gradient (Z-Y)/n
    Yr = rng.standard_normal((n, ninst))
    Lm = orc.loss_fprop(A, Yr, "mse", ninst)
    np.testing.assert_allclose(Lm.ravel(), 0.5 * ((A - Yr) ** 2).mean(axis=0), rtol=1e-12)
    np.testing.assert_allclose(orc.loss_bprop(A, Yr), (A - Yr) / n, rtol=1e-12)


def test_hinge_loss_worked_values_and_gradient():
    """The bidirectional hinge (deepity/std/loss.py:157-174): a label-0 row costs its output where that is positive, a
    label-1 row costs 1 - output where that is positive. Hand-worked rows on both sides of both kinks, then the
    gradient against central finite differences of the loss at points away from the kinks."""
    Z = np.array([[-0.5], [0.25], [2.0], [0.75], [1.5], [-1.0]])
    Y = np.array([[0.0], [0.0], [0.0], [1.0], [1.0], [1.0]])
    terms = np.array([0.0, 0.25, 2.0, 0.25, 0.0, 2.0])                # by hand: max(0, Z) for Y = 0, max(0, 1 - Z) for Y = 1
    np.testing.assert_allclose(orc.loss_fprop(Z, Y, "hinge", 1).ravel(), [terms.mean()], rtol=1e-15)
    slopes = np.array([0.0, 1.0, 1.0, -1.0, 0.0, -1.0])               # d term / dZ, by hand
    np.testing.assert_allclose(orc.loss_bprop(Z, Y, kind="hinge").ravel(), slopes / len(Z), rtol=1e-15)
    # masks drop rows from loss and gradient alike
    Ymask = np.array([[True], [False], [True], [True], [True], [False]])
    np.testing.assert_allclose(orc.loss_fprop(Z, Y, "hinge", 1, Ymask=Ymask).ravel(), [(terms * Ymask.ravel()).sum() / len(Z)], rtol=1e-15)
    np.testing.assert_allclose(orc.loss_bprop(Z, Y, Ymask=Ymask, kind="hinge").ravel(), slopes * Ymask.ravel() / len(Z), rtol=1e-15)
    rng = np.random.default_rng(31)
    n, ninst = 40, 3
    A = rng.standard_normal((n, ninst)) * 2
    Yb = (rng.random((n, ninst)) < 0.5).astype(np.float64)
    A[np.abs(A) < 0.05] = 0.3                                         # keep clear of the kinks at 0 (Y = 0) and 1 (Y = 1)
    A[np.abs(A - 1) < 0.05] = 1.4
    dA = orc.loss_bprop(A, Yb, kind="hinge")
    eps = 1e-4
    for i in range(n):
        for j in range(ninst):
            Ap = A.copy(); Ap[i, j] += eps
            Am = A.copy(); Am[i, j] -= eps
            fd = (orc.loss_fprop(Ap, Yb, "hinge", ninst).sum() - orc.loss_fprop(Am, Yb, "hinge", ninst).sum()) / (2 * eps)
            np.testing.assert_allclose(dA[i, j], fd, rtol=1e-9, atol=1e-12)


def test_zmask_and_maskout():
    Z = np.array([[1.0, 5.0], [2.0, 5.0], [3.0, -1.0], [0.0, np.nan]])
    M = orc.calc_zmask(Z)
    assert M.tolist() == [[False, True], [True, False], [True, False], [False, True]]
    A = np.array([1.0, np.nan, 3.0])
    orc.maskout(np.array([True, False, False]), A)
    assert A.tolist() == [1.0, 0.0, 0.0]            # NaN is replaced, unlike A *= M


def test_blockwise_dot_family_against_block_diagonal_matmul():
    rng = np.random.default_rng(20)
    n, k, m, nb = 7, 3, 4, 5
    X = rng.standard_normal((n, k * nb))
    W = rng.standard_normal((k * nb, m))
    # one big matmul with a block-diagonal weight matrix
    Wbd = np.zeros((k * nb, m * nb))
    for b in range(nb):
        Wbd[b * k:(b + 1) * k, b * m:(b + 1) * m] = W[b * k:(b + 1) * k]
    Z = orc.blockwise_dot(X, W, nb)
    np.testing.assert_allclose(Z, X @ Wbd, rtol=1e-12)
    dZ = rng.standard_normal(Z.shape)
    np.testing.assert_allclose(orc.blockwise_dot_nt(dZ, W, nb), dZ @ Wbd.T, rtol=1e-12)
    dWbd = X.T @ dZ
    dW = orc.blockwise_dot_tn(X, dZ, nb, W)
    for b in range(nb):
        np.testing.assert_allclose(dW[b * k:(b + 1) * k], dWbd[b * k:(b + 1) * k, b * m:(b + 1) * m], rtol=1e-12)
    # shared (broadcast) input: every model multiplies the same X
    Xs = rng.standard_normal((n, k))
    Zs = orc.blockwise_dot(Xs, W, nb)
    np.testing.assert_allclose(Zs, np.tile(Xs, (1, nb)) @ Wbd, rtol=1e-12)
    # combined: two inputs stacked inside each model's row block == concatenating per model
    k2 = 2
    X2 = rng.standard_normal((n, k2 * nb))
    p = k + k2
    Wc = rng.standard_normal((p * nb, m))
    Zc = orc.blockwise_dot_combined([X, X2], Wc, nb, [False, False])
    for b in range(nb):
        Xcat = np.hstack([X[:, b * k:(b + 1) * k], X2[:, b * k2:(b + 1) * k2]])
        np.testing.assert_allclose(Zc[:, b * m:(b + 1) * m], Xcat @ Wc[b * p:(b + 1) * p], rtol=1e-12)
    dZc = rng.standard_normal(Zc.shape)
    dXs = orc.blockwise_dot_nt_combined([X, X2], dZc, Wc, nb, [False, False])
    dWc = orc.blockwise_dot_tn_combined([X, X2], dZc, Wc, nb, [False, False])
    for b in range(nb):
        Xcat = np.hstack([X[:, b * k:(b + 1) * k], X2[:, b * k2:(b + 1) * k2]])
        full = dZc[:, b * m:(b + 1) * m] @ Wc[b * p:(b + 1) * p].T
        np.testing.assert_allclose(dXs[0][:, b * k:(b + 1) * k], full[:, :k], rtol=1e-12)
        np.testing.assert_allclose(dXs[1][:, b * k2:(b + 1) * k2], full[:, k:], rtol=1e-12)
        np.testing.assert_allclose(dWc[b * p:(b + 1) * p], Xcat.T @ dZc[:, b * m:(b + 1) * m], rtol=1e-12)


def test_gradstep_closed_forms():
    rng = np.random.default_rng(21)
    n = 11
    P0, dP, mP0 = rng.standard_normal((3, n))
    drate = rng.random(n) * 0.1
    mrate = 0.9 + rng.random(n) * 0.09
    # nesterov: P += mu*mP ; (grad) ; mP = mu*mP - eta*g ; P -= eta*g   -- unrolled per element
    P, mP = P0.copy(), mP0.copy()
    orc.gradstep_nesterov1(P, mP, mrate)
    orc.gradstep_nesterov2(P, dP, drate, mP, mrate)
    for i in range(n):
        p = P0[i] + mrate[i] * mP0[i]
        v = mrate[i] * mP0[i] - drate[i] * dP[i]
        p = p - drate[i] * dP[i]
        assert abs(P[i] - p) < 1e-14 and abs(mP[i] - v) < 1e-14
    # both phases together equal the classical momentum update P0 + v when the gradient is fixed
    np.testing.assert_allclose(P, P0 + mP, rtol=1e-12)
    P, mP = P0.copy(), mP0.copy()
    orc.gradstep(P, dP, drate, mP, mrate)
    np.testing.assert_allclose(mP, mrate * mP0 - drate * dP, rtol=1e-14)
    np.testing.assert_allclose(P, P0 + mP, rtol=1e-14)
    # madd_bcast: per-model scalars over blocks of k consecutive elements, wrapping modulo b.size
    A = rng.standard_normal(12); b = np.array([2.0, -1.0, 0.5]); dst = np.ones(12)
    orc.madd_bcast(A, b, 2, dst)
    expect = np.ones(12) + A * np.array([2, 2, -1, -1, .5, .5, 2, 2, -1, -1, .5, .5])
    np.testing.assert_allclose(dst, expect, rtol=1e-14)


def test_dropout_semantics():
    rng = np.random.default_rng(22)
    X = rng.standard_normal((6, 8)).astype(np.float32)
    rate = np.array([0.25, 0.5], np.float32)           # two models, 4 columns each
    U = rng.random((6, 8)).astype(np.float32)
    Z, M = orc.dropout_fp_train(X, rate, U)
    assert np.array_equal(M[:, :4], U[:, :4] >= 0.25) and np.array_equal(M[:, 4:], U[:, 4:] >= 0.5)
    assert np.array_equal(Z, np.where(M, X, 0))
    Zm, Mm = orc.dropout_fp_train(X, rate, U, matchrows=True)
    assert np.array_equal(Mm[0::2], Mm[1::2])
    np.testing.assert_allclose(orc.dropout_fp_test(X, rate)[:, :4], X[:, :4] * 0.75)
    np.testing.assert_allclose(orc.dropout_bp_te(X, rate)[:, 4:], X[:, 4:] * 0.5)
    assert np.array_equal(orc.dropout_bp_tr(X, M), np.where(M, X, 0))
    Xo = np.array([0, 1, 255, 3, 2], np.uint8)
    Zo, Mo = orc.dropoutord_fp_train(Xo, 0.5, np.array([0.9, 0.1, 0.1, 0.1, 0.7]))
    assert Zo.tolist() == [0, 254, 255, 254, 2]
    assert Mo.tolist() == [True, False, True, False, True]            # padding reports "kept" (dropoutord.cu:47-49)
    # reverse complements: "ACG" and its reverse complement "CGT", padding 2: the reverse row drops the mirrored letters
    Xp, Rp = orc.pack(["ACG", "CGT"], 2)
    Up = np.array([.9, .9, .1, .9, .9, .9, .9, .9, .9, .1, .9, .9])[:, None]      # drops fwd letter 0 (A); rev letter 1 drawn low too
    Zp, Mp = orc.dropoutord_fp_train(Xp, 0.5, Up, regions=Rp, reverse_complement=True)
    assert Zp.ravel().tolist() == [255, 255, 254, 1, 2, 255, 255, 1, 2, 254, 255, 255]   # rev "CGT" loses its T (pairs with A), keeps G
    assert Mp.ravel().tolist() == [True, True, False, True, True, True, True, True, True, False, True, True]


def test_whole_model_gradient_matches_finite_differences():
    """Mirrors the reference's own gradient check (deepity/deepity/gradcheck.py:42-130) in float64."""
    rng = np.random.default_rng(23)
    nm, nf, m, hid = 2, 3, 4, 5
    for pool in ("max", "all"):
        k = nf * (2 if pool == "all" else 1)
        seqs = ["ACGTNACGGT", "TTGACA", "GGNNCATTAGC"]
        X, R = orc.pack(seqs, m - 1)
        B = len(seqs)
        params = {
            "Wc": rng.standard_normal((4 * m, nf * nm)), "bc": rng.standard_normal((1, nf * nm)) * 0.1,
            "W1": rng.standard_normal((k * nm, hid)), "b1": rng.standard_normal((1, hid * nm)) * 0.1,
            "W2": rng.standard_normal((hid * nm, 1)), "b2": rng.standard_normal((1, nm)) * 0.1,
        }
        Y = (rng.random((B, nm)) < 0.5).astype(np.float64)

        def cost(p):
            st = orc.model_forward(p, X, R, nm, pool, hid, out="logistic")
            return orc.loss_fprop(st["Zout"], Y, "nll", nm).sum()

        st = orc.model_forward(params, X, R, nm, pool, hid, out="logistic")
        g = orc.model_backward(params, X, R, st, orc.loss_bprop(st["Zout"], Y), nm, pool, hid)
        for name in params:
            flat = params[name].reshape(-1)
            for idx in rng.choice(flat.size, size=min(6, flat.size), replace=False):
                old = flat[idx]
                flat[idx] = old + 1e-6; cp = cost(params)
                flat[idx] = old - 1e-6; cm = cost(params)
                flat[idx] = old
                np.testing.assert_allclose(g[name].reshape(-1)[idx], (cp - cm) / 2e-6, rtol=2e-5, atol=1e-8,
                                           err_msg="%s[%d] pool=%s" % (name, idx, pool))


def test_weight_cost_is_the_per_model_l1_norm_times_decay():
    """Scalar loops over each model's own weights (scan filters lie along columns, dense weights in row blocks)."""
    rng = np.random.default_rng(4)
    nm, nf, m, hid = 3, 2, 4, 5
    p = {"Wc": rng.standard_normal((4 * m, nf * nm)), "W1": rng.standard_normal((nf * nm, hid)), "W2": rng.standard_normal((hid * nm, 1))}
    dc, df = np.array([0.1, 0.2, 0.3]), np.array([1.0, 2.0, 3.0])
    want = np.zeros(nm)
    for b in range(nm):
        conv = sum(abs(p["Wc"][r, c]) for r in range(4 * m) for c in range(nf * b, nf * (b + 1)))
        full = sum(abs(v) for v in p["W1"][nf * b:nf * (b + 1)].ravel()) + sum(abs(v) for v in p["W2"][hid * b:hid * (b + 1)].ravel())
        want[b] = dc[b] * conv + df[b] * full
    np.testing.assert_allclose(orc.weight_cost(p, nm, dc, df).ravel(), want, rtol=1e-12)


def test_softmax_chunks_and_multiclass_terms():
    """softmax per chunk == scipy's softmax on each chunk; the multiclass term's sum is the cross entropy, whose
    gradient w.r.t. the pre-activations is Z - Y (what the loss node back-propagates, deepity/std/loss.py:98-112)."""
    from scipy.special import softmax as sp_softmax
    rng = np.random.default_rng(12)
    X = rng.standard_normal((7, 12)) * 3
    for nchunk in (1, 3, 4):
        Z = orc.softmax(X, nchunk)
        w = 12 // nchunk
        for c in range(nchunk):
            np.testing.assert_allclose(Z[:, c * w:(c + 1) * w], sp_softmax(X[:, c * w:(c + 1) * w], axis=1), rtol=1e-12)
    Y = np.eye(4)[rng.integers(0, 4, 7)]
    A = rng.standard_normal((7, 4))
    cost = lambda a: -orc.nll_multiclass_terms(orc.softmax(a), Y).sum()
    g = np.zeros_like(A)
    for i in range(7):
        for j in range(4):
            up, dn = A.copy(), A.copy()
            up[i, j] += 1e-6
            dn[i, j] -= 1e-6
            g[i, j] = (cost(up) - cost(dn)) / 2e-6
    np.testing.assert_allclose(g, orc.softmax(A) - Y, atol=1e-8)
