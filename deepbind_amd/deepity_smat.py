"""Dense-head and optimiser operators over device tensors: same names, argument order and
conventions as the reference's shim (reference: code/libs/deepity/deepity/_ext/deepity_smat.py:77-254),
plus the fused scoring head. All arithmetic happens in libdeepbind_hip.so on the current HIP stream.
"""
import numbers

import numpy as np
import torch

from ._lib import LOSS_KIND, call, dtype_code, ptr, require, stream

_rng_seed = 0
_rng_offset = 0


def set_seed(seed):
    """Seeds the generator behind dropout_fp_train (and resets its stream position)."""
    global _rng_seed, _rng_offset
    _rng_seed, _rng_offset = int(seed), 0


def _vec(b, like):
    """Per-model vector argument: ndarray / list -> device tensor of like's dtype."""
    if isinstance(b, torch.Tensor):
        return b.to(device=like.device, dtype=like.dtype).contiguous()
    return torch.as_tensor(np.asarray(b), dtype=like.dtype, device=like.device).contiguous()


def gradstep(P, dP, drate, mP, mrate, grad, nesterov=False):
    """One momentum step on P with per-element rates.
         nesterov=False:  grad(); mP = mrate*mP - drate*dP; P += mP
         nesterov=True:   P += mrate*mP; grad(); mP = mrate*mP - drate*dP; P -= drate*dP
    grad() must fill dP with the gradient at the current P. reference: deepity_smat.py:77-117,
    deepity_smat/gradstep.cu:41-72"""
    assert callable(grad)
    n = P.numel()
    for t in (dP, drate, mP, mrate):
        require(t.numel() == n and t.dtype == P.dtype, "ValueError: P, dP, drate, mP, mrate must match in size and dtype")
    dt = dtype_code(P)
    if nesterov:
        call("dbk_gradstep_nesterov1", stream(), dt, n, ptr(P), ptr(mP), ptr(mrate))
        grad()
        call("dbk_gradstep_nesterov2", stream(), dt, n, ptr(P), ptr(dP), ptr(drate), ptr(mP), ptr(mrate))
    else:
        grad()
        call("dbk_gradstep", stream(), dt, n, ptr(P), ptr(dP), ptr(drate), ptr(mP), ptr(mrate))


def madd_bcast(A, b, k, dst):
    """dst[i] += A[i] * b[(i/k) % b.size] over the flattened arrays. reference: deepity_smat.py:121-131"""
    require(A.numel() == dst.numel() and A.dtype == dst.dtype, "ValueError: A and dst must match in size and dtype")
    if isinstance(b, numbers.Number) or (isinstance(b, np.ndarray) and b.ndim == 0):
        b = [float(b)]
    b = _vec(b, A)
    require(A.numel() % b.numel() == 0, "ValueError: A.size must be a multiple of b.size")
    call("dbk_madd_bcast", stream(), dtype_code(A), ptr(A), ptr(b), ptr(dst), A.numel(), b.numel(), int(k))


def maskout(M, A):
    """A[i] = A[i] if M[i] else 0 (NaN becomes 0, unlike A *= M). reference: deepity_smat.py:135-140"""
    require(M.dtype == torch.bool and M.numel() == A.numel(), "ValueError: M must be a bool array of A's size")
    call("dbk_maskout", stream(), dtype_code(A), ptr(M), ptr(A), A.numel())


def calc_Zmask(Z, Zmask):
    """Marks, in each (fwd, rev) row pair, the row with the larger prediction. reference: deepity_smat.py:253-254"""
    require(Zmask.dtype == torch.bool and Zmask.numel() == Z.numel(), "ValueError: Zmask must be a bool array of Z's size")
    call("dbk_calc_zmask", stream(), dtype_code(Z), ptr(Z), ptr(Zmask), Z.shape[0], Z.shape[1])


def pair_max(Z):
    """Row-pair maximum: the score kept from each (forward, reverse-complement) pair; (n/2 x ncol)."""
    out = torch.empty((Z.shape[0] // 2, Z.shape[1]), dtype=Z.dtype, device=Z.device)
    call("dbk_pair_max", stream(), dtype_code(Z), ptr(Z), ptr(out), Z.shape[0], Z.shape[1])
    return out


def dropout_fp_train(X, rate, matchrows, U=None):
    """Z = X*M with M = (u >= rate[model of the column]); matchrows shares the draw inside each
    (fwd, rev) row pair. U (optional float32, X's shape) supplies the uniforms. Returns (Z, M).
    reference: deepity_smat.py:144-150, deepity_smat/dropout.cu:41-77"""
    global _rng_offset
    rate = _vec(rate, X)
    require(X.shape[1] % rate.numel() == 0, "ValueError: columns must divide evenly among the rates")
    Z = torch.empty_like(X)
    M = torch.empty(X.shape, dtype=torch.bool, device=X.device)
    n, m = X.numel(), rate.numel()
    k = X.shape[1] // m
    if U is not None:
        require(U.dtype == torch.float32 and U.numel() == n, "ValueError: U must be float32 with one value per element")
        call("dbk_dropout_fp_tr_u", stream(), dtype_code(X), ptr(X), ptr(rate), ptr(Z), ptr(M), n, m, k, int(bool(matchrows)), ptr(U))
    else:
        call("dbk_dropout_fp_tr", stream(), dtype_code(X), ptr(X), ptr(rate), ptr(Z), ptr(M), n, m, k, int(bool(matchrows)),
             _rng_seed, _rng_offset)
        _rng_offset += (n + 3) // 4
    return Z, M


def dropout_fp_test(X, rate):
    rate = _vec(rate, X)
    Z = torch.empty_like(X)
    call("dbk_dropout_fp_te", stream(), dtype_code(X), ptr(X), ptr(rate), ptr(Z), X.numel(), rate.numel(), X.shape[1] // rate.numel())
    return Z


def dropout_bp_tr(dZ, M):
    dX = torch.empty_like(dZ)
    call("dbk_dropout_bp_tr", stream(), dtype_code(dZ), ptr(dZ), ptr(M), ptr(dX), dZ.numel())
    return dX


def dropout_bp_te(dZ, rate):
    rate = _vec(rate, dZ)
    dX = torch.empty_like(dZ)
    call("dbk_dropout_bp_te", stream(), dtype_code(dZ), ptr(dZ), ptr(rate), ptr(dX), dZ.numel(), rate.numel(), dZ.shape[1] // rate.numel())
    return dX


def _check_dot(X, W, Z, nblock):
    require(X.dtype == W.dtype == Z.dtype, "TypeError: X, W and Z must share a dtype")
    require(X.shape[0] == Z.shape[0], "ValueError: X and Z must have the same number of rows")
    require(Z.shape[1] == W.shape[1] * nblock and W.shape[0] % nblock == 0, "ValueError: Z must be n x (W.ncol*nblock)")


def blockwise_dot(X, W, nblock):
    """Z[:, i] = dot(X[:, i], W[i, :]) per block i; if X has only one block's columns it is shared
    by all blocks. reference: deepity_smat.py:169-180, deepity_smat.cpp:275-300"""
    Z = torch.empty((X.shape[0], W.shape[1] * nblock), dtype=X.dtype, device=X.device)
    _check_dot(X, W, Z, nblock)
    bcast = nblock > 1 and X.shape[1] * nblock == W.shape[0]
    require(bcast or X.shape[1] == W.shape[0], "ValueError: X columns must equal W rows (or W rows / nblock)")
    call("dbk_blockwise_dot", stream(), dtype_code(X), nblock, X.shape[0], W.shape[1], W.shape[0] // nblock, int(bcast),
         ptr(X), ptr(W), ptr(Z))
    return Z


def blockwise_dot_nt(dZ, W, nblock):
    """dX[:, i] = dot_nt(dZ[:, i], W[i, :]). reference: deepity_smat.py:182-191"""
    dX = torch.empty((dZ.shape[0], W.shape[0]), dtype=dZ.dtype, device=dZ.device)
    _check_dot(dX, W, dZ, nblock)
    call("dbk_blockwise_dot_nt", stream(), dtype_code(dZ), nblock, dZ.shape[0], W.shape[1], W.shape[0] // nblock,
         ptr(dZ), ptr(W), ptr(dX))
    return dX


def blockwise_dot_tn(X, dZ, nblock, W):
    """dW[i, :] = dot_tn(X[:, i], dZ[:, i]). reference: deepity_smat.py:193-202"""
    dW = torch.empty_like(W)
    _check_dot(X, dW, dZ, nblock)
    bcast = nblock > 1 and X.shape[1] * nblock == W.shape[0]
    require(bcast or X.shape[1] == W.shape[0], "ValueError: X columns must equal W rows (or W rows / nblock)")
    call("dbk_blockwise_dot_tn", stream(), dtype_code(X), nblock, X.shape[0], W.shape[1], W.shape[0] // nblock, int(bcast),
         ptr(X), ptr(dZ), ptr(dW))
    return dW


def _xk(X, bcast, nblock):
    return X.shape[1] if bcast else X.shape[1] // nblock


def blockwise_dot_combined(X, W, nblock, Xbroadcast):
    """blockwise_dot over a LIST of inputs stacked along each block's rows of W.
    reference: deepity_smat.py:204-215"""
    first = [x for x in X if x is not None][0]
    Z = torch.empty((first.shape[0], W.shape[1] * nblock), dtype=first.dtype, device=first.device)
    p = W.shape[0] // nblock
    Xoffset = 0
    for x, bc in zip(X, Xbroadcast):
        if x is None:
            continue
        _check_dot(x, W, Z, nblock)
        k = _xk(x, bc, nblock)
        call("dbk_blockwise_dot_combined", stream(), dtype_code(x), nblock, Xoffset, int(bool(bc)), x.shape[0], W.shape[1], k, p,
             ptr(x), ptr(W), ptr(Z))
        Xoffset += k
    return Z


def blockwise_dot_nt_combined(X, dZ, W, nblock, Xbroadcast):
    """List of dX, one per non-broadcast input (None for broadcast inputs). reference: deepity_smat.py:217-235"""
    p = W.shape[0] // nblock
    dX = []
    Xoffset = 0
    for x, bc in zip(X, Xbroadcast):
        if x is None:
            dX.append(None)
            continue
        k = _xk(x, bc, nblock)
        if bc:
            dX.append(None)
        else:
            d = torch.zeros_like(x)
            call("dbk_blockwise_dot_nt_combined", stream(), dtype_code(x), nblock, Xoffset, x.shape[0], W.shape[1], k, p,
                 ptr(d), ptr(W), ptr(dZ))
            dX.append(d)
        Xoffset += k
    return dX


def blockwise_dot_tn_combined(X, dZ, W, nblock, Xbroadcast, dWmask=None):
    """dW rows filled input by input; masked-out inputs leave zeros. reference: deepity_smat.py:237-251"""
    dW = torch.empty_like(W)
    if dWmask is not None:
        assert len(dWmask) == len(X)
        dW.zero_()
    p = W.shape[0] // nblock
    Xoffset = 0
    for i, (x, bc) in enumerate(zip(X, Xbroadcast)):
        if x is None:
            continue
        k = _xk(x, bc, nblock)
        if dWmask is None or dWmask[i]:
            call("dbk_blockwise_dot_tn_combined", stream(), dtype_code(x), nblock, Xoffset, int(bool(bc)), x.shape[0], W.shape[1], k, p,
                 ptr(x), ptr(dW), ptr(dZ))
        Xoffset += k
    return dW


def uniform_like(X, seed, offset):
    """The float32 uniforms dropout_fp_train would draw for X at (seed, offset)."""
    U = torch.empty(X.shape, dtype=torch.float32, device=X.device)
    call("dbk_uniform_fill", stream(), ptr(U), U.numel(), int(seed), int(offset))
    return U


def head_fprop(pooled, W1, b1, W2=None, b2=None, nblock=1, in_scale=None, apply_logistic=False, nfeat=0, feats=None):
    """Scores (n x nblock) of nblock independent heads on pooled (n x k*nblock): one dense layer
    (W2 is None) or dense -> bias -> ReLU -> dense -> bias, optional logistic. float32 only.
    nfeat: feature columns shared by all models, entering after each model's own inputs (W1 has k + nfeat
    rows per model); feats (n, nfeat) or None for all zeros."""
    require(pooled.dtype == torch.float32, "TypeError: the fused head is float32 only")
    n = pooled.shape[0]
    k = pooled.shape[1] // nblock
    hidden = 0 if W2 is None else W1.shape[1]
    require(W1.shape[0] == (k + nfeat) * nblock, "ValueError: W1 must have (k + nfeat) * nblock rows")
    require(feats is None or (feats.dtype == torch.float32 and tuple(feats.shape) == (n, nfeat)), "ValueError: feats must be float32 (n, nfeat)")
    scores = torch.empty((n, nblock), dtype=torch.float32, device=pooled.device)
    sc = None if in_scale is None else _vec(in_scale, pooled)
    call("dbk_head_fprop", stream(), n, nblock, k, hidden, ptr(pooled), int(nfeat), ptr(feats), ptr(sc), ptr(W1), ptr(b1), ptr(W2), ptr(b2),
         int(bool(apply_logistic)), ptr(scores))
    return scores


def head_train(pooled, W1, b1, W2, b2, Y, nblock, loss, dW1, db1, dW2=None, db2=None, Ymask=None, rate=None, U=None,
               seed=0, offset=0, counter=None, counter_advance=0, reverse_complement=False, want_loss=False,
               nfeat=0, feats=None):
    """Forward and backward of nblock dense heads. Returns (Z, dpooled, loss|None); the weight gradients
    are written into dW1, db1, dW2, db2. With `counter` (device int64) the dropout generator position is
    read from it and moved on by `counter_advance` once the masks are drawn. float32 only.
    nfeat: feature columns shared by all models that enter the first layer after each model's pooled
    features (W1 has k + nfeat rows per model); feats (n, nfeat) or None for all zeros."""
    require(pooled.dtype == torch.float32, "TypeError: the fused head is float32 only")
    n = pooled.shape[0]
    k = pooled.shape[1] // nblock
    hidden = 0 if W2 is None else W1.shape[1]
    require(W1.shape[0] == (k + nfeat) * nblock, "ValueError: W1 must have (k + nfeat) * nblock = %d rows, got %d" % ((k + nfeat) * nblock, W1.shape[0]))
    require(feats is None or (feats.dtype == torch.float32 and tuple(feats.shape) == (n, nfeat)), "ValueError: feats must be float32 (n, nfeat)")
    Z = torch.empty((n, nblock), dtype=torch.float32, device=pooled.device)
    dpooled = torch.empty_like(pooled)
    L = torch.empty((1, nblock), dtype=torch.float32, device=pooled.device) if want_loss else None
    r = None if rate is None else _vec(rate, pooled)
    call("dbk_head_train", stream(), n, nblock, k, hidden, LOSS_KIND[loss], int(bool(reverse_complement)),
         ptr(pooled), int(nfeat), ptr(feats), ptr(r), ptr(U), int(seed), int(offset), ptr(counter), int(counter_advance), ptr(W1), ptr(b1), ptr(W2), ptr(b2), ptr(Y), ptr(Ymask),
         ptr(Z), ptr(dpooled), ptr(dW1), ptr(db1), ptr(dW2), ptr(db2), ptr(L))
    return Z, dpooled, L


def l1_decay(P, decay, dP):
    """dP += sign(P) * decay, elementwise over a whole flat parameter vector (decay: one coefficient per element)."""
    require(P.shape == dP.shape == decay.shape and P.dtype == dP.dtype == decay.dtype, "ValueError: P, decay and dP must match")
    call("dbk_l1_decay", stream(), dtype_code(P), ptr(P), ptr(decay), ptr(dP), P.numel())


def counter_add(counter, delta):
    """counter[0] += delta on the device (int64 tensor of one element)."""
    call("dbk_counter_add", stream(), ptr(counter), int(delta))
