"""CPU restatement (NumPy) of the reference's motif-scan hot path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this module: it exists so that tests,
the smoke check and the CPU-baseline leg of the benchmark can compare the HIP
kernels with the reference's operator semantics.  The reference's own code cannot
run here (CUDA-only kernels, Python-2 host code), so every function below restates
the arithmetic of the reference lines it cites, with the same accumulation order
where the reference's order is deterministic.

Pinning status (what, other than a retyped formula, checks each function; the
checks live in tests/test_oracle_pins.py):
  corr1ord            - torch conv1d on a 4-channel one-hot (N rows = 1/4), brute-force
                        triple loop, all-N closed form, channel-shift invariant, 254 == tap deleted
  corr1ord_bprop_W    - exact adjoint identity <corr1ord(W,X),dZ> == <W,bprop_W(X,dZ)> in
                        float64 and central finite differences
  corr1ord_bprop_X    - adjoint of the one-hot convolution w.r.t. its input, brute force
  poolrgn / _bprop    - np.max / np.argmax / np.mean per slice; scatter / uniform-spread adjoints
  bias/relu/logistic/nll/mse/maskout/calc_zmask - NumPy closed forms the reference's own
                        unit tests compare against (smat/tests/unittest.py:425-471,531-623)
  hinge loss          - hand-worked values on both sides of both kinks (Y = 0: cost Z above 0; Y = 1: cost 1 - Z
                        below 1), gradient against central finite differences of the loss away from the kinks
  softmax             - scipy.special.softmax per chunk (the reference's own test compares with a NumPy softmax,
                        smat/py/smat/tests/unittest.py:601-603); rows sum to one per chunk
  blockwise_dot*      - np.dot per block; no reference test exists at that boundary
                        (closed form only): PARITY UNPINNED beyond the per-block np.dot identity
  weight_cost         - scalar loops over each model's own weights
  gradstep*           - three-line closed form (gradstep.cu:41-72) vs. an unrolled scalar loop
  train_step          - (tests/test_oracle_train_step.py) models stepped together == each model stepped alone
                        with scalar rates; two Nesterov steps written out from the docstring recurrence with
                        central-finite-difference gradients of loss + L1 cost; a hand-written worked case of
                        the decay block lengths rows/ninst and size/ninst; both gates at start-1 and start
  model_forward/_backward/train_step with features= (the combiner's second, broadcast input) - equal to the same
                        functions without it on a model whose pooled features are widened by the feature columns
                        (block-concatenation identity) and finite differences of the loss w.r.t. the extra W1 rows
  enforce_constraints - pfm: each tap's four exp(w) sum to one and differences of w across letters are kept
                        (softmax shift invariance); psam: the largest of the four becomes 0, differences kept;
                        clip: np.clip; all three idempotent
  dropout masks       - the reference draws them from cuRAND (not reproducible without the
                        CUDA SDK): masks are INPUTS here (uniforms U supplied by the caller);
                        the random stream itself is PARITY UNPINNED
  pack (asbatches)    - worked example "AC","G", m=3 from the reference's packing code
  eval_with_input_gradients - central finite differences of softplus(A) (nll) / Z^2/2 (mse) w.r.t. a
                        real-valued 4-channel input, through a dense-correlation restatement
  gen_predictions / gen_predictionmaps - glue loops restated from predict.py; the finite-difference
                        map is checked against brute-force single-mutant rescoring, the window
                        scan against scoring each window by hand
All paths in the comments are relative to /root/reference/code/libs.
"""
import numpy as np

PT_MAX, PT_AVG, PT_SUM, PT_ALL = 0, 1, 2, 3
STR2POOLTYPE = {"max": PT_MAX, "avg": PT_AVG, "sum": PT_SUM, "all": PT_ALL}


# ----------------------------------------------------------------------------------------------
# a1  packing: kangaroo/kangaroo/util.py:50-56,68-74 ; kangaroo/kangaroo/data.py:309-354
# ----------------------------------------------------------------------------------------------
def acgt2ord(s):
    table = {"a": 0, "c": 1, "g": 2, "t": 3, "u": 3}
    return np.array([table.get(ch.lower(), 255) for ch in s], dtype=np.uint8)


def pack(seqs, padding):
    """X = pad|s0|pad|s1|...|pad (255 = pad), R[i] = cumulative [start,end) over (pad+len)."""
    pieces = []
    edges = [0]
    for s in seqs:
        pieces.append(np.full(padding, 255, np.uint8))
        pieces.append(acgt2ord(s))
        edges.append(edges[-1] + padding + len(s))
    pieces.append(np.full(padding, 255, np.uint8))
    X = np.concatenate(pieces).reshape(-1, 1)
    R = np.array([[edges[i], edges[i + 1]] for i in range(len(seqs))], dtype=np.uint32).reshape(-1, 2)
    return X, R


# ----------------------------------------------------------------------------------------------
# a2  corr1ord fprop: kangaroo_smat/corr1ord.cuh:139-157, kangaroo_smat.cpp:98-111
# ----------------------------------------------------------------------------------------------
def _letter_table(W, nchannel):
    """(m, 256, F) lookup: rows 0..C-1 = W taps, 254 = 0, everything else = ((W0+W1)+W2+W3)*(1/C)."""
    W = np.asarray(W)
    m = W.shape[0] // nchannel
    F = W.shape[1]
    Wt = W.reshape(m, nchannel, F)
    mean = Wt[:, 0, :].copy()
    for k in range(1, nchannel):
        mean = mean + Wt[:, k, :]
    mean = mean * W.dtype.type(1.0 / nchannel)
    lut = np.empty((m, 256, F), W.dtype)
    lut[:, :, :] = mean[:, None, :]
    lut[:, :nchannel, :] = Wt
    lut[:, 254, :] = 0
    return lut


def corr1ord(W, X, Z, nchannel=4):
    """Z[i,f] = sum_j w(j, X[i+j], f) for i < n = N-m+1, j ascending, same dtype as W; rows >= n untouched."""
    X = np.asarray(X).ravel()
    m = W.shape[0] // nchannel
    n = X.size - m + 1
    if n <= 0:
        return Z
    lut = _letter_table(W, nchannel)
    acc = np.zeros((n, W.shape[1]), W.dtype)
    for j in range(m):
        acc += lut[j][X[j:j + n]]
    Z[:n] = acc
    return Z


def corr1ord_bruteforce(W, X, nchannel=4):
    """Scalar triple loop straight from the kernel text; for tiny inputs only."""
    X = np.asarray(X).ravel()
    m = W.shape[0] // nchannel
    F = W.shape[1]
    n = X.size - m + 1
    Z = np.zeros((X.size, F), W.dtype)
    inv = W.dtype.type(1.0 / nchannel)
    for i in range(max(n, 0)):
        for f in range(F):
            z = W.dtype.type(0)
            for j in range(m):
                k = int(X[i + j])
                if k < nchannel:
                    z = z + W[nchannel * j + k, f]
                elif k != 254:
                    s = W[nchannel * j, f]
                    for kk in range(1, nchannel):
                        s = s + W[nchannel * j + kk, f]
                    z = z + s * inv
            Z[i, f] = z
    return Z


# ----------------------------------------------------------------------------------------------
# a3  corr1ord bprop_W: kangaroo_smat/corr1ord_bprop.cuh:91-137 (accumulates into dW)
# ----------------------------------------------------------------------------------------------
def corr1ord_bprop_W(dW, X, dZ, nchannel=4):
    X = np.asarray(X).ravel()
    m = dW.shape[0] // nchannel
    n = X.size - m + 1
    if n <= 0:
        return dW
    dZ = np.asarray(dZ)[:n]
    inv = dW.dtype.type(1.0 / nchannel)
    for j in range(m):
        xj = X[j:j + n]
        for k in range(nchannel):
            sel = xj == k
            if sel.any():
                dW[nchannel * j + k] += dZ[sel].sum(axis=0, dtype=dW.dtype)
        other = (xj >= nchannel) & (xj != 254)
        if other.any():
            s = (dZ[other] * inv).sum(axis=0, dtype=dW.dtype)
            for k in range(nchannel):
                dW[nchannel * j + k] += s
    return dW


# ----------------------------------------------------------------------------------------------
# a4  corr1ord bprop_X: host loop kangaroo_smat/corr1ord_bprop.cu:191-201 (accumulates into dX)
# ----------------------------------------------------------------------------------------------
def corr1ord_bprop_X(dX, W, dZ, nchannel=4):
    """dX[i,c] += sum_f sum_{k<m, k<=i} dZ[i-k,f] * W[(C*k+c),f], over ALL n = dX.shape[0] rows of dZ."""
    n = dX.shape[0]
    m = W.shape[0] // nchannel
    Wt = np.asarray(W).reshape(m, nchannel, -1)
    dZ = np.asarray(dZ)
    for k in range(min(m, n)):
        # rows i >= k take dZ[i-k]
        dX[k:] += dZ[:n - k] @ Wt[k].T
    return dX


# ----------------------------------------------------------------------------------------------
# a8/a9  poolrgn: kangaroo_smat/poolrgn.cuh:44-160 ; poolrgn_bprop.cuh:45-127
# ----------------------------------------------------------------------------------------------
def poolrgn(unpooled, regions, ptype, want_argmax=False):
    """Returns (pooled, argmax|None). argmax = flat index row*F+f of the first strict maximum."""
    U = np.asarray(unpooled)
    R = np.asarray(regions)
    F = U.shape[1]
    P = R.shape[0]
    pt = STR2POOLTYPE[ptype] if isinstance(ptype, str) else ptype
    per_step = R.shape[1] == 3
    nout = 2 if pt == PT_ALL else 1
    pooled = np.empty((P, F * nout), U.dtype)
    amax = np.empty((P, F), np.uint32) if (want_argmax and pt in (PT_MAX, PT_ALL)) else None
    for r in range(P):
        a, b = int(R[r, 0]), int(R[r, 1])
        step = int(R[r, 2]) if per_step else 1
        rows = np.arange(a, b, step)
        blk = U[rows]
        cnt = (b - a + step - 1) // step
        if pt in (PT_MAX, PT_ALL):
            am = blk.argmax(axis=0)                      # first maximum == strict '>' scan
            mx = blk[am, np.arange(F)]
            if amax is not None:
                amax[r] = rows[am] * F + np.arange(F)
        if pt in (PT_AVG, PT_SUM, PT_ALL):
            s = blk[0].copy()
            for t in range(1, blk.shape[0]):
                s += blk[t]                              # sequential, same order as the kernel
            if pt != PT_SUM:
                s = s / U.dtype.type(cnt)
        if pt == PT_MAX:
            pooled[r] = mx
        elif pt == PT_ALL:
            pooled[r, 0::2] = mx
            pooled[r, 1::2] = s
        else:
            pooled[r] = s
    return pooled, amax


def poolrgn_bprop(unpooled, regions, pooled, pooled_argmax, ptype):
    """Accumulates into `unpooled` (N,F): max scatters to argmax, avg/sum spread over the region."""
    dX = unpooled
    R = np.asarray(regions)
    dP = np.asarray(pooled)
    F = dX.shape[1]
    pt = STR2POOLTYPE[ptype] if isinstance(ptype, str) else ptype
    per_step = R.shape[1] == 3
    flat = dX.reshape(-1)
    for r in range(R.shape[0]):
        a, b = int(R[r, 0]), int(R[r, 1])
        step = int(R[r, 2]) if per_step else 1
        cnt = (b - a + step - 1) // step
        if pt == PT_MAX:
            np.add.at(flat, pooled_argmax[r].astype(np.int64), dP[r])
        elif pt in (PT_AVG, PT_SUM):
            v = dP[r] / dX.dtype.type(cnt) if pt == PT_AVG else dP[r]
            dX[a:b:step] += v
        else:
            dmax = dP[r, 0::2]
            davg = dP[r, 1::2] / dX.dtype.type(cnt)
            dX[a:b:step] += davg
            np.add.at(flat, pooled_argmax[r].astype(np.int64), dmax)
    return dX


# ----------------------------------------------------------------------------------------------
# a6/a7  bias, relu: deepity/deepity/std/elemwise.py:71-82,162-180 ; smat_cuda/elemwise2.cu:42,77
# ----------------------------------------------------------------------------------------------
def bias_fprop(X, b):
    return X + b.reshape(1, -1)


def bias_bprop(dZ):
    """db = column sums, rows added one after the other in dZ's dtype: the order of the reference's column reduction,
    one thread walking down a column (smat/src/smat_cuda/reduce_y.cuh:57-78). (ndarray.sum would add a single column
    pairwise, which rounds less than the reference does.)"""
    if dZ.shape[0] == 0:
        return dZ, np.zeros((1, dZ.shape[1]), dZ.dtype)
    return dZ, np.cumsum(dZ, axis=0, dtype=dZ.dtype)[-1].reshape(1, -1)


def relu_fprop(X):
    return np.maximum(X.dtype.type(0), X)


def sign(Z):
    return ((Z > 0).astype(Z.dtype) - (Z < 0).astype(Z.dtype))


def relu_bprop(dZ, Z):
    return dZ * sign(Z)


# ----------------------------------------------------------------------------------------------
# a10  dropout on pooled features: deepity_smat/dropout.cu:41-109 (uniforms U are inputs)
# ----------------------------------------------------------------------------------------------
def _rate_per_column(rate, ncol):
    rate = np.asarray(rate).ravel()
    k = ncol // rate.size
    return rate[(np.arange(ncol) // k) % rate.size]


def dropout_fp_train(X, rate, U, matchrows=False):
    """M = (U >= rate[col's model]); Z = X*M. With matchrows each fwd/rev row pair shares row 2i's draw."""
    p = _rate_per_column(rate, X.shape[1]).astype(X.dtype)
    U = np.asarray(U)
    if matchrows:
        U = np.repeat(U[0::2], 2, axis=0)[:X.shape[0]]
    M = U >= p[None, :]
    return X * M.astype(X.dtype), M


def dropout_fp_test(X, rate):
    p = _rate_per_column(rate, X.shape[1]).astype(X.dtype)
    return X * (X.dtype.type(1) - p)[None, :]


def dropout_bp_tr(dZ, M):
    return dZ * M.astype(dZ.dtype)


def dropout_bp_te(dZ, rate):
    p = _rate_per_column(rate, dZ.shape[1]).astype(dZ.dtype)
    return dZ * (dZ.dtype.type(1) - p)[None, :]


def dropoutord_fp_train(X, rate, U, regions=None, reverse_complement=False):
    """kangaroo_smat/dropoutord.cu:41-52: M = (X == 255) or (U >= rate); Z = M ? X : 254.
    With reverse complements (kangaroo/_ext/dropoutord.py:55-68) the reverse row's mask is the forward
    row's flipped over the sequence part and Z is rebuilt as X with 254 wherever M is false."""
    X = np.asarray(X)
    M = (X == 255) | (np.asarray(U).reshape(X.shape) >= rate)
    Z = np.where(M, X, np.uint8(254)).astype(np.uint8)
    if reverse_complement:
        M = M.copy()
        R = np.asarray(regions).astype(np.int64)
        padsize = M.size - int(R[-1, -1])
        Mf = M.reshape(-1)
        for i in range(0, len(R), 2):
            a, b = R[i]
            c, d = R[i + 1]
            Mf[c + padsize:d] = Mf[a + padsize:b][::-1]
        Z = X.copy()
        Z.reshape(-1)[~Mf] = 254
    return Z, M


# ----------------------------------------------------------------------------------------------
# a11  blockwise dot: deepity/_ext/deepity_smat.py:169-251 ; deepity_smat/blockwise_dot.cu:42-260
# ----------------------------------------------------------------------------------------------
def blockwise_dot(X, W, nblock):
    """Z[:, b*m:(b+1)*m] = X_b . W[b*k:(b+1)*k, :]; X_b = X[:, b*k:(b+1)*k] or all of X when shared."""
    k = W.shape[0] // nblock
    m = W.shape[1]
    bcast = X.shape[1] * nblock == W.shape[0] and nblock > 1
    Z = np.empty((X.shape[0], m * nblock), X.dtype)
    for b in range(nblock):
        Xb = X if bcast else X[:, b * k:(b + 1) * k]
        Z[:, b * m:(b + 1) * m] = Xb @ W[b * k:(b + 1) * k]
    return Z


def blockwise_dot_nt(dZ, W, nblock):
    k = W.shape[0] // nblock
    m = W.shape[1]
    dX = np.empty((dZ.shape[0], W.shape[0]), dZ.dtype)
    for b in range(nblock):
        dX[:, b * k:(b + 1) * k] = dZ[:, b * m:(b + 1) * m] @ W[b * k:(b + 1) * k].T
    return dX


def blockwise_dot_tn(X, dZ, nblock, W):
    k = W.shape[0] // nblock
    m = W.shape[1]
    bcast = X.shape[1] * nblock == W.shape[0] and nblock > 1
    dW = np.empty_like(W)
    for b in range(nblock):
        Xb = X if bcast else X[:, b * k:(b + 1) * k]
        dW[b * k:(b + 1) * k] = Xb.T @ dZ[:, b * m:(b + 1) * m]
    return dW


def blockwise_dot_combined(Xs, W, nblock, Xbroadcast):
    """Several inputs stacked along W's rows inside each model's block of p rows."""
    n = [x for x in Xs if x is not None][0].shape[0]
    p = W.shape[0] // nblock
    m = W.shape[1]
    Z = np.zeros((n, m * nblock), W.dtype)
    off = 0
    for X, bc in zip(Xs, Xbroadcast):
        if X is None:
            continue
        k = X.shape[1] if bc else X.shape[1] // nblock
        for b in range(nblock):
            Xb = X if bc else X[:, b * k:(b + 1) * k]
            Z[:, b * m:(b + 1) * m] += Xb @ W[b * p + off:b * p + off + k]
        off += k
    return Z


def blockwise_dot_nt_combined(Xs, dZ, W, nblock, Xbroadcast):
    p = W.shape[0] // nblock
    m = W.shape[1]
    out = []
    off = 0
    for X, bc in zip(Xs, Xbroadcast):
        if X is None:
            out.append(None)
            continue
        k = X.shape[1] if bc else X.shape[1] // nblock
        if bc:
            out.append(None)
        else:
            dX = np.zeros_like(X)
            for b in range(nblock):
                dX[:, b * k:(b + 1) * k] = dZ[:, b * m:(b + 1) * m] @ W[b * p + off:b * p + off + k].T
            out.append(dX)
        off += k
    return out


def blockwise_dot_tn_combined(Xs, dZ, W, nblock, Xbroadcast, dWmask=None):
    p = W.shape[0] // nblock
    m = W.shape[1]
    dW = np.zeros_like(W)
    off = 0
    for i, (X, bc) in enumerate(zip(Xs, Xbroadcast)):
        if X is None:
            continue
        k = X.shape[1] if bc else X.shape[1] // nblock
        if dWmask is None or dWmask[i]:
            for b in range(nblock):
                Xb = X if bc else X[:, b * k:(b + 1) * k]
                dW[b * p + off:b * p + off + k] = Xb.T @ dZ[:, b * m:(b + 1) * m]
        off += k
    return dW


# ----------------------------------------------------------------------------------------------
# a12  output non-linearity and loss: deepity/std/softmax.py:58-77 ; loss.py:52-154 ; maskout.cu:41-67
# ----------------------------------------------------------------------------------------------
def logistic(A):
    return (1 / (1 + np.exp(-A.astype(np.float64)))).astype(A.dtype)


def softmax(X, nchunk=1):
    """deepity/std/softmax.py:58-71: rows split into nchunk = ngroup * ninst chunks, each normalised on its own."""
    A = X.reshape((-1, X.shape[1] // nchunk))
    Z = np.exp(A - A.max(axis=1, keepdims=True))
    Z = Z / Z.sum(axis=1, keepdims=True)
    return Z.reshape(X.shape)


def nll_multiclass_terms(Z, Y):
    """deepity/std/loss.py:147-151."""
    return np.log(np.maximum(Z.dtype.type(1e-15), Z)) * Y


def maskout(M, A):
    A[~np.asarray(M, dtype=bool)] = 0
    return A


def calc_zmask(Z):
    """Rows come in (fwd, rev) pairs; keep the row with the larger Z (ties keep the first)."""
    M = np.zeros(Z.shape, bool)
    a = Z[0::2]
    b = Z[1::2]
    first = a >= b
    M[0::2] = first
    M[1::2] = ~first
    return M


def loss_fprop(Z, Y, kind, ninst, Ymask=None, Zmask=None):
    """Per-model mean loss, shape (1, ninst). kind in {"nll", "mse", "hinge"}; one output column per model.
    hinge: max(0, (1-Y)Z + Y(1-Z)), the reference's bidirectional hinge (deepity/std/loss.py:157-174)."""
    if kind == "nll":
        eps = Z.dtype.type(1e-15)
        L = np.log(np.maximum(eps, Z)) * Y + np.log(np.maximum(eps, 1 - Z)) * (1 - Y)
    elif kind == "hinge":
        L = np.maximum(0, (1 - Y) * Z + Y * (1 - Z))
    else:
        L = (Z - Y) ** 2
    L = L.astype(Z.dtype)
    if Ymask is not None:
        maskout(Ymask, L)
    if Zmask is not None:
        maskout(Zmask, L)
    L = L.mean(axis=0, dtype=Z.dtype)
    L = L.reshape(ninst, -1).sum(axis=1).reshape(1, -1)
    return -L if kind == "nll" else (L if kind == "hinge" else Z.dtype.type(0.5) * L)


def loss_bprop(Z, Y, Ymask=None, Zmask=None, kind="nll"):
    """dLoss/d(output): Z - Y for nll (through the logistic) and mse (deepity/std/loss.py:98-112); for the hinge
    1 - 2Y where its argument is positive, else 0 (loss.py:165-169); then the masks and the 1/rows factor."""
    if kind == "hinge":
        dZ = ((1 - 2 * Y) * (((1 - Y) * Z + Y * (1 - Z)) > 0)).astype(Z.dtype)
    else:
        dZ = (Z - Y).astype(Z.dtype)
    if Ymask is not None:
        maskout(Ymask, dZ)
    if Zmask is not None:
        maskout(Zmask, dZ)
    return dZ * Z.dtype.type(1.0 / Z.shape[0])


# ----------------------------------------------------------------------------------------------
# a13  optimiser: deepity_smat/gradstep.cu:41-72 ; madd_bcast.cu:41-47
# ----------------------------------------------------------------------------------------------
def gradstep(P, dP, drate, mP, mrate):
    delta = mP * mrate - dP * drate
    mP[...] = delta
    P += delta


def gradstep_nesterov1(P, mP, mrate):
    P[...] = P + mrate * mP


def gradstep_nesterov2(P, dP, drate, mP, mrate):
    delta = dP * drate
    mP[...] = mP * mrate - delta
    P -= delta


def madd_bcast(A, b, k, dst):
    """dst[i] += A[i] * b[(i // k) % b.size] over the flattened arrays."""
    b = np.asarray(b).ravel()
    idx = (np.arange(A.size) // int(k)) % b.size
    flat = dst.reshape(-1)
    flat += A.reshape(-1) * b[idx].astype(A.dtype)
    return dst


# ----------------------------------------------------------------------------------------------
# whole-model forward / backward for a homogeneous batch of models on the model axis
# layer order: kangaroo/kangaroo/model.py:45-132 ; deepity/_io_/load.py:51-72 ; cfg/*/M{1,2}.cfg
# ----------------------------------------------------------------------------------------------
def model_forward(params, X, R, nmodel, pool, hidden, out="linear", dropout=None, train=False, matchrows=False, input_keep=1.0,
                  features=None):
    """scan (-> * input_keep: the test-time side of input dropout, kangaroo/_ext/corr1ord.py:104-109) -> bias ->
    relu -> pool -> dropout -> dense(+bias[,relu,dense,bias]) -> (logistic).
    features: the (rows, nfeat) matrix that the reference's first dense layer (its "combiner") takes as a second,
    broadcast input after the pooled features (kangaroo/kangaroo/model.py:101-112, deepity/std/full.py:154-160);
    W1 then has k + nfeat rows per model. None = a model built without that input."""
    m = params["Wc"].shape[0] // 4
    N = np.asarray(X).size
    st = {}
    Z0 = np.zeros((N, params["Wc"].shape[1]), params["Wc"].dtype)
    corr1ord(params["Wc"], X, Z0)
    if input_keep != 1.0:
        Z0 *= input_keep
    st["A0"] = relu_fprop(bias_fprop(Z0, params["bc"]))
    st["Pl"], st["I"] = poolrgn(st["A0"], R, pool, want_argmax=True)
    H = st["Pl"]
    if dropout is not None:
        rate, U = dropout
        if train:
            H, st["M"] = dropout_fp_train(H, rate, U, matchrows=matchrows)
        else:
            H = dropout_fp_test(H, rate)
    st["H0"] = H
    st["F"] = features
    if features is None:
        A1 = blockwise_dot(H, params["W1"], nmodel)
    else:
        A1 = blockwise_dot_combined([H, features], params["W1"], nmodel, [False, True])
    A1 = bias_fprop(A1, params["b1"])
    if hidden:
        st["H1"] = relu_fprop(A1)
        A2 = bias_fprop(blockwise_dot(st["H1"], params["W2"], nmodel), params["b2"])
    else:
        A2 = A1
    st["A"] = A2
    st["Zout"] = logistic(A2) if out == "logistic" else A2
    return st


def model_backward(params, X, R, st, dA, nmodel, pool, hidden, dropout=None, train=True):
    """Gradients of sum(dA * A) w.r.t. every parameter; dA is dLoss/d(pre-activation output)."""
    g = {}
    if hidden:
        g["b2"] = bias_bprop(dA)[1]
        g["W2"] = blockwise_dot_tn(st["H1"], dA, nmodel, params["W2"])
        dH1 = blockwise_dot_nt(dA, params["W2"], nmodel)
        dA1 = relu_bprop(dH1, st["H1"])
    else:
        dA1 = dA
    g["b1"] = bias_bprop(dA1)[1]
    if st.get("F") is None:
        g["W1"] = blockwise_dot_tn(st["H0"], dA1, nmodel, params["W1"])
        dH0 = blockwise_dot_nt(dA1, params["W1"], nmodel)
    else:                                                          # deepity/std/full.py:162-178
        Xs = [st["H0"], st["F"]]
        g["W1"] = blockwise_dot_tn_combined(Xs, dA1, params["W1"], nmodel, [False, True])
        dH0 = blockwise_dot_nt_combined(Xs, dA1, params["W1"], nmodel, [False, True])[0]
    if dropout is not None:
        dH0 = dropout_bp_tr(dH0, st["M"]) if train else dropout_bp_te(dH0, dropout[0])
    dA0 = np.zeros_like(st["A0"])
    poolrgn_bprop(dA0, R, dH0, st["I"], pool)
    dZ0 = relu_bprop(dA0, st["A0"])
    g["bc"] = bias_bprop(dZ0)[1]
    g["Wc"] = np.zeros_like(params["Wc"])
    corr1ord_bprop_W(g["Wc"], X, dZ0)
    return g


# ----------------------------------------------------------------------------------------------
# one optimiser step on a homogeneous batch of models
# deepity/deepity/sgd.py:121-147,287-354 ; deepity/_ext/deepity_smat.py:77-117 ;
# kangaroo/_ext/corr1ord.py:120-138 ; deepity/std/full.py:111-119
# ----------------------------------------------------------------------------------------------
def _per_element(values, shape, nmodel, axis):
    """Spread one value per model over a parameter whose models lie along `axis`."""
    values = np.broadcast_to(np.asarray(values, dtype=np.float64), (nmodel,))
    out = np.empty(shape)
    per = shape[axis] // nmodel
    for b in range(nmodel):
        if axis == 0:
            out[b * per:(b + 1) * per, :] = values[b]
        else:
            out[:, b * per:(b + 1) * per] = values[b]
    return out


PARAM_AXIS = {"Wc": 1, "bc": 1, "W1": 0, "b1": 1, "W2": 0, "b2": 1}


def train_step(params, mom, X, R, Y, nmodel, pool, hidden, loss, rate, momentum, Ymask=None, dropout=None,
               decay_conv=0.0, decay_full=0.0, step=0, weight_decay_start=100, reverse_complement=False, start_training=0,
               features=None, constraint=None):
    """Nesterov step in place on params / mom (dicts of arrays). dropout = (rates, U) or None.
    features: see model_forward. constraint: enforced on the scan filters after the update (deepity/sgd.py:137)."""
    names = [n for n in ("Wc", "bc", "W1", "b1", "W2", "b2") if n in params]
    eta = {n: _per_element(rate, params[n].shape, nmodel, PARAM_AXIS[n]).astype(params[n].dtype) for n in names}
    mu = {n: _per_element(momentum, params[n].shape, nmodel, PARAM_AXIS[n]).astype(params[n].dtype) for n in names}
    for n in names:
        gradstep_nesterov1(params[n], mom[n], mu[n])
    out = "logistic" if loss == "nll" else "linear"
    st = model_forward(params, X, R, nmodel, pool, hidden, out=out, dropout=dropout, train=True, matchrows=reverse_complement,
                       features=features)
    Zmask = calc_zmask(st["Zout"]) if reverse_complement else None      # deepity/std/loss.py:114-119
    dA = loss_bprop(st["Zout"], Y, Ymask=Ymask, Zmask=Zmask, kind=loss)
    g = model_backward(params, X, R, st, dA, nmodel, pool, hidden, dropout=dropout, train=True)
    if weight_decay_start <= step:
        # scan filters: the reference indexes its per-model decay with block length rows/ninst over the
        # flattened (4m, F) matrix (kangaroo/_ext/corr1ord.py:126), kept literally
        W = params["Wc"]
        kq = max(1, W.shape[0] // nmodel)
        madd_bcast(sign(W), np.broadcast_to(np.asarray(decay_conv, dtype=W.dtype), (nmodel,)), kq, g["Wc"])
        for n in ("W1", "W2"):
            if n in params:
                Wn = params[n]
                madd_bcast(sign(Wn), np.broadcast_to(np.asarray(decay_full, dtype=Wn.dtype), (nmodel,)), Wn.size // nmodel, g[n])
    if start_training > step:
        g["Wc"] = g["Wc"] * 0                                      # kangaroo/_ext/corr1ord.py:135-136
    for n in names:
        gradstep_nesterov2(params[n], g[n].astype(params[n].dtype), eta[n], mom[n], mu[n])
    enforce_constraints(params["Wc"], constraint)
    return st, g


def enforce_constraints(W, constraint):
    """corr1ord.enforce_constraints (kangaroo/_ext/corr1ord.py:60-77), in place on W (4*fsize, filters)."""
    if constraint is None:
        return W
    if constraint in ("pfm", "psam"):
        F = np.exp(W)
        for i in range(W.shape[0] // 4):
            Fi = F[i * 4:(i + 1) * 4, :]
            if constraint == "pfm":
                Fi[:] = Fi / np.sum(Fi, axis=0)
            else:
                Fi[:] = Fi / np.max(Fi, axis=0)
        W[:] = np.log(F)
    elif type(constraint) == tuple:
        lo, hi = constraint
        W[:] = np.minimum(W, hi)
        W[:] = np.maximum(W, lo)
    else:
        raise NotImplementedError("constraint \"%s\" not implemented" % str(constraint))
    return W


def weight_cost(params, nmodel, decay_conv, decay_full):
    """Per-model L1 cost added to the reported loss (kangaroo/_ext/corr1ord.py:111-115, deepity/std/full.py:92-109)."""
    C = np.abs(params["Wc"]).sum(axis=0).reshape((nmodel, -1)).sum(axis=1) * np.broadcast_to(decay_conv, (nmodel,))
    for n in ("W1", "W2"):
        if n in params:
            C = C + np.abs(params[n]).reshape((nmodel, -1)).sum(axis=1) * np.broadcast_to(decay_full, (nmodel,))
    return C.reshape(1, nmodel)


# ----------------------------------------------------------------------------------------------
# prediction-time callers of the path: kangaroo/kangaroo/predict.py:145-345 ;
# deepity/deepity/node.py:298-341 (eval with want_bprop_inputs) ; kangaroo/_ext/corr1ord.py:129-133
# The loops below are the reference's loops, one forward pass per mutated (position, base).
# ----------------------------------------------------------------------------------------------
_COMPLEMENT = {"A": "T", "C": "G", "G": "C", "T": "A", "U": "A", "N": "N"}


def revcomp_string(s):
    """kangaroo/kangaroo/util.py:29-37,76-80: complement of the reversed string; unknown letters -> N."""
    return "".join(_COMPLEMENT.get(ch.upper(), "N") for ch in reversed(s))


def insert_reverse_complements(seqs):
    """kangaroo/kangaroo/data.py:274-284: rows become fwd0, rev0, fwd1, rev1, ..."""
    out = []
    for s in seqs:
        out += [s, revcomp_string(s)]
    return out


def ord2acgt(x):
    return "".join("ACGT"[v] if v < 4 else "N" for v in np.asarray(x).ravel())


def maskout_revcomp(Z, reverse_complement):
    """predict.py:145-164: of each (fwd, rev) pair of rows keep the larger prediction (ties: fwd)."""
    if not reverse_complement:
        return Z, None
    Zc = Z.reshape((-1, 2))
    Zmask = np.zeros_like(Zc, dtype=bool)
    Zmask[:, 0] = Zc[:, 0] >= Zc[:, 1]
    Zmask[:, 1] = Zc[:, 0] < Zc[:, 1]
    Zmask = Zmask.reshape((-1, 1))
    return Z[Zmask.ravel()], Zmask


def eval_with_input_gradients(params, X, R, nmodel, pool, hidden, out, dropout_rate=None, reverse_complement=False, input_keep=1.0):
    """Test-mode forward pass, then back-propagation of dA = Z (targets 0, no batch mean, only
    output column 0, reverse-complement losers masked) down to the one-hot inputs: dX (N, 4).
    node.py:317-339, loss.py:98-109, elemwise.py:148-157 (test-mode dropout bprop), corr1ord.py:129-133."""
    dropout = None if dropout_rate is None else (np.asarray(dropout_rate, dtype=params["Wc"].dtype), None)
    st = model_forward(params, X, R, nmodel, pool, hidden, out=out, dropout=dropout, train=False, input_keep=input_keep)
    Z = st["Zout"]
    dA = Z.copy()
    if reverse_complement:
        maskout(calc_zmask(Z), dA)
    if dA.shape[1] > 1:
        dA[:, 1:] = 0
    if hidden:
        dA1 = relu_bprop(blockwise_dot_nt(dA, params["W2"], nmodel), st["H1"])
    else:
        dA1 = dA
    dH0 = blockwise_dot_nt(dA1, params["W1"], nmodel)
    if dropout is not None:
        dH0 = dropout_bp_te(dH0, dropout[0])
    dA0 = np.zeros_like(st["A0"])
    poolrgn_bprop(dA0, R, dH0, st["I"], pool)
    dZ0 = relu_bprop(dA0, st["A0"])
    dX = np.zeros((np.asarray(X).size, 4), dtype=params["Wc"].dtype)
    corr1ord_bprop_X(dX, params["Wc"], dZ0)
    return Z, dX


def gen_predictions(params, seqs, pool, hidden, out, dropout_rate=None, reverse_complement=False, want_gmaps=False, input_keep=1.0):
    """predict.py:168-260 for one model and one batch. Returns (predictions (nseq, 1), gmaps) where
    gmaps is None, or a list of (sequence string, (len, 4) map): the back-propagated input gradient
    (want_gmaps=True; with reverse complements only the winning strand's entry is kept), or the
    finite-difference mutation map (want_gmaps="finite_diff"; forward strands only)."""
    m = params["Wc"].shape[0] // 4
    pad = m - 1
    rows = insert_reverse_complements(seqs) if reverse_complement else list(seqs)
    X, R = pack(rows, pad)
    X = X.ravel()
    R = R.astype(np.int64)

    def predict(Xb):
        dropout = None if dropout_rate is None else (np.asarray(dropout_rate, dtype=params["Wc"].dtype), None)
        return model_forward(params, Xb, R, 1, pool, hidden, out=out, dropout=dropout, train=False, input_keep=input_keep)["Zout"]

    if not want_gmaps:
        Z, _ = maskout_revcomp(predict(X), reverse_complement)
        return Z, None
    Zall, dX = eval_with_input_gradients(params, X, R, 1, pool, hidden, out, dropout_rate, reverse_complement, input_keep)
    Z, Zmask = maskout_revcomp(Zall, reverse_complement)
    if want_gmaps == "finite_diff":
        rcindex = [3, 2, 1, 0]
        Xlen = R[:, 1] - R[:, 0]
        for i in range(int(Xlen.max())):
            for j in range(4):
                mtX = X.copy()
                for k in range(len(R)):
                    a, b = R[k]
                    if i < b - a:
                        if (k % 2 == 0) or not reverse_complement:
                            mtX[pad + a + i] = j
                        else:
                            mtX[b - i - 1] = rcindex[j]
                mtZ, _ = maskout_revcomp(predict(mtX), reverse_complement)
                dZ = mtZ - Z
                dZ = dZ * np.maximum(0, np.sign(np.maximum(Z, mtZ)))
                for k in range(len(R)):
                    if (k % 2 == 0) or not reverse_complement:
                        a, b = R[k]
                        if i < b - a:
                            dX[pad + a + i, j] = dZ[(k // 2) if reverse_complement else k, 0]
        fwd = R[np.arange(0, len(R), 2)] if reverse_complement else R
        return Z, [(ord2acgt(X[a + pad:b]), dX[a + pad:b].copy()) for a, b in fwd]
    maps = [(ord2acgt(X[a + pad:b]), dX[a + pad:b].copy()) for a, b in R]
    if Zmask is not None:
        maps = [maps[i] for i in range(len(maps)) if Zmask[i]]
    return Z, maps


def gen_predictionmaps(params, seqs, pool, hidden, out, dropout_rate=None, reverse_complement=False, stride=1, windowsize=20,
                       want_gmaps=False, input_keep=1.0):
    """predict.py:263-345: every sequence is N-padded by windowsize-1 on both sides and cut into windows
    of `windowsize` every `stride` letters; each window is scored as a sequence of its own. Returns
    (list of per-sequence prediction maps, list of (len+windowsize-1, 4) averaged gradient maps | None)."""
    pmaps, gmaps = [], []
    for raw in seqs:
        padseq = "N" * (windowsize - 1) + raw + "N" * (windowsize - 1)
        windows = [padseq[i:i + windowsize] for i in range(0, max(1, len(padseq) - windowsize + 1), stride)]
        Z, wmaps = gen_predictions(params, windows, pool, hidden, out, dropout_rate, reverse_complement, want_gmaps=want_gmaps,
                                   input_keep=input_keep)
        pmaps.append(Z.ravel().copy())
        if want_gmaps:
            gmap = np.zeros((len(raw) + windowsize - 1, 4), Z.dtype)
            denom = np.zeros_like(gmap)
            nwin = len(windows)
            for j in range(nwin):
                dXj = wmaps[j][1][:min(windowsize, (nwin - j) * stride)]
                gmap[j * stride:j * stride + windowsize] += dXj
                denom[j * stride:j * stride + windowsize] += np.ones_like(dXj)
            with np.errstate(invalid="ignore", divide="ignore"):
                gmap /= denom
            gmaps.append(np.nan_to_num(gmap))
    return pmaps, (gmaps if want_gmaps else None)
