"""Sequence operators over device tensors: same names, argument order and in-place conventions
as the reference's operator shim (reference: code/libs/kangaroo/kangaroo/_ext/kangaroo_smat.py:86-146),
plus the fused scan+pool entry points. Arrays are torch tensors on the GPU; all arithmetic happens
in libdeepbind_hip.so on the current HIP stream.
"""
import torch

from . import _lib
from ._lib import DeepbindError, call, dtype_code, ptr, require, str2pooltype, stream

uindex = torch.uint32

_rng_seed = 0
_rng_offset = 0


def set_seed(seed):
    """Seeds the generator behind dropoutord_fp_train (and resets its stream position)."""
    global _rng_seed, _rng_offset
    _rng_seed, _rng_offset = int(seed), 0


def _u8(X):
    require(X.dtype == torch.uint8, "TypeError: X must be uint8, got %s" % X.dtype)
    return X


def _regions(R):
    require(R.dtype in (torch.uint32, torch.int32), "TypeError: regions must be uint32, got %s" % R.dtype)
    require(R.dim() == 2 and R.shape[1] in (2, 3), "ValueError: regions array must have 2 or 3 columns.")
    return R


def set_exact_scan(on):
    """on: corr1ord, corr1ord_bprop_W and corr1ord_bprop_X keep to the kernels that sum in one fixed order at every
    size (corr1ord: the reference's own order, so its bits whatever the batch size). Off (the default) float32 calls
    switch to the faster matrix-core kernels at bulk sizes, whose results equal these to round-off. Process-wide;
    returns the previous setting."""
    from ._lib import dll
    return bool(dll().dbk_set_exact_scan(int(bool(on))))


def corr1ord(W, X, Z, nchannel):
    """Cross-correlates the filter bank W ((M*nchannel) x P) with the ordinal vector X (N uint8,
    values 0..nchannel-1, 255 = all ordinals, 254 = none) into Z (N x P). The final M-1 rows of Z
    are left untouched. reference: kangaroo_smat.py:86-99, kangaroo_smat.cpp:98-124"""
    _u8(X)
    require(W.shape[0] % nchannel == 0, "ValueError: W rows must be a multiple of nchannel")
    require(W.dtype == Z.dtype, "TypeError: W dtype must match Z dtype")
    require(Z.shape[1] == W.shape[1], "ValueError: Z must have one column per filter")
    require(Z.shape[0] == X.numel(), "ValueError: Z must have one row per element of X")
    m = W.shape[0] // nchannel
    n = X.numel() - m + 1
    if n <= 0:
        return
    call("dbk_corr1ord", stream(), dtype_code(Z), ptr(W), m, W.shape[1], ptr(X), n, nchannel, ptr(Z))


def corr1ord_bprop_W(dW, X, dZ, nchannel):
    """Accumulates the filter gradient of corr1ord into dW. reference: kangaroo_smat.py:101-109"""
    _u8(X)
    require(dW.shape[0] % nchannel == 0, "ValueError: dW rows must be a multiple of nchannel")
    require(dW.dtype == dZ.dtype, "TypeError: dW dtype must match dZ dtype")
    require(dZ.shape[1] == dW.shape[1] and dZ.shape[0] == X.numel(), "ValueError: dZ must be N x P")
    m = dW.shape[0] // nchannel
    n = X.numel() - m + 1
    if n <= 0:
        return
    call("dbk_corr1ord_bprop_W", stream(), dtype_code(dZ), ptr(dW), m, dW.shape[1], ptr(X), n, nchannel, ptr(dZ))


def corr1ord_bprop_X(dX, W, dZ, nchannel):
    """Accumulates the input gradient of corr1ord into dX (N x nchannel). reference: kangaroo_smat.py:111-119,
    kangaroo_smat.cpp:141-168"""
    require(W.shape[0] % nchannel == 0, "ValueError: W rows must be a multiple of nchannel")
    require(W.dtype == dZ.dtype and dX.dtype == dZ.dtype, "TypeError: dX, W and dZ must share a dtype")
    require(dX.shape[1] == nchannel, "ValueError: dX must have nchannel columns")
    require(dZ.shape[1] == W.shape[1] and dZ.shape[0] == dX.shape[0], "ValueError: dZ must be N x P")
    m = W.shape[0] // nchannel
    call("dbk_corr1ord_bprop_X", stream(), dtype_code(dZ), ptr(dX), dX.shape[0], nchannel, ptr(W), m, W.shape[1], ptr(dZ))


def poolrgn(unpooledmaps, regions, ptype, want_argmax=False):
    """Pools rows of unpooledmaps (N x M) per region. Returns (pooled, argmax|None); "all" gives
    (P x 2M) with (max, avg) at columns (2j, 2j+1). reference: kangaroo_smat.py:121-132"""
    _regions(regions)
    noutputs = 2 if ptype == "all" else 1
    nregion, nfeaturemap = regions.shape[0], unpooledmaps.shape[1]
    pooledmaps = torch.empty((nregion, nfeaturemap * noutputs), dtype=unpooledmaps.dtype, device=unpooledmaps.device)
    argmax = None
    if ptype in ("max", "all") and want_argmax:
        argmax = torch.empty((nregion, nfeaturemap), dtype=uindex, device=unpooledmaps.device)
    call("dbk_poolrgn", stream(), dtype_code(unpooledmaps), ptr(unpooledmaps), nfeaturemap, ptr(regions), nregion,
         int(regions.shape[1] == 3), ptr(pooledmaps), ptr(argmax), str2pooltype[ptype])
    return pooledmaps, argmax


def poolrgn_bprop(unpooledmaps, regions, pooledmaps, pooledmaps_argmax, ptype):
    """Accumulates the pooling gradient into unpooledmaps. reference: kangaroo_smat.py:134-138"""
    _regions(regions)
    nregion, nfeaturemap = regions.shape[0], unpooledmaps.shape[1]
    noutputs = 2 if ptype == "all" else 1
    require(unpooledmaps.dtype == pooledmaps.dtype, "TypeError: unpooledmaps dtype must match pooledmaps dtype.")
    require(tuple(pooledmaps.shape) == (nregion, nfeaturemap * noutputs),
            "ValueError: pooledmaps must be (regions x feature maps%s)." % (" x 2" if noutputs == 2 else ""))
    amax = pooledmaps_argmax if (pooledmaps_argmax is not None and ptype in ("max", "all")) else None
    if amax is not None:
        require(tuple(amax.shape) == (nregion, nfeaturemap) and amax.dtype in (torch.uint32, torch.int32),
                "ValueError: pooledmaps_argmax must be a (regions x feature maps) uint32 array.")
    call("dbk_poolrgn_bprop", stream(), dtype_code(unpooledmaps), ptr(unpooledmaps), nfeaturemap, ptr(regions), nregion,
         int(regions.shape[1] == 3), ptr(pooledmaps), ptr(amax), str2pooltype[ptype])


def dropoutord_fp_train(X, rate, U=None, regions=None, padding=None, seed=None, offset=None, counter=None):
    """Input-base dropout: returns (Z, M) with dropped bases replaced by 254 (padding always passes and
    reports True in M). U (optional, float32, same shape) supplies the uniforms instead of the
    library's generator; `offset` / `counter` (device int64 tensor) supply the generator position
    instead of the module's host-side one. With `regions` (pairs of fwd/rev rows) and `padding` the reverse
    strand's mask is the forward strand's mirrored, as in reverse-complement training.
    reference: kangaroo_smat.py:140-146, kangaroo/_ext/dropoutord.py:50-70"""
    global _rng_offset
    _u8(X)
    Z = torch.empty_like(X)
    M = torch.empty(X.shape, dtype=torch.bool, device=X.device)
    n = X.numel()
    if U is not None:
        require(U.dtype == torch.float32 and U.numel() == n, "ValueError: U must be float32 with one value per element")
        call("dbk_dropoutord_fp_tr_u", stream(), ptr(X), ptr(Z), ptr(M), n, float(rate), ptr(U))
    elif counter is not None:
        call("dbk_dropoutord_fp_tr", stream(), ptr(X), ptr(Z), ptr(M), n, float(rate), _rng_seed if seed is None else int(seed), 0, ptr(counter))
    elif offset is not None:
        call("dbk_dropoutord_fp_tr", stream(), ptr(X), ptr(Z), ptr(M), n, float(rate), _rng_seed if seed is None else int(seed), int(offset), None)
    else:
        call("dbk_dropoutord_fp_tr", stream(), ptr(X), ptr(Z), ptr(M), n, float(rate), _rng_seed if seed is None else int(seed), _rng_offset, None)
        _rng_offset += (n + 3) // 4
    if regions is not None:
        _regions(regions)
        require(regions.shape[1] == 2 and padding is not None, "ValueError: mirroring needs 2-column regions and the padding length")
        call("dbk_dropoutord_mirror", stream(), ptr(X), ptr(Z), ptr(M), ptr(regions), regions.shape[0], int(padding))
    return Z, M


def corr1ord_enforce_constraints(W, constraint, nchannel=4):
    """Applies the scan filters' constraint to W (4*m, nfilter) in place: "pfm" (each tap's letter weights become
    log-probabilities), "psam" (log of the weights relative to the tap's largest), a (lo, hi) tuple (clip), or
    None (nothing). reference: corr1ord.enforce_constraints, kangaroo/_ext/corr1ord.py:60-77"""
    if constraint is None:
        return
    require(nchannel == 4, "NotImplementedError: only the 4-letter alphabet is supported")
    require(W.dim() == 2 and W.shape[0] % 4 == 0 and W.is_contiguous(), "ValueError: W must be a contiguous (4*m, nfilter) matrix")
    if constraint in ("pfm", "psam"):
        kind, lo, hi = (0 if constraint == "pfm" else 1), 0.0, 0.0
    elif type(constraint) == tuple:
        kind, (lo, hi) = 2, constraint
    else:
        raise NotImplementedError("constraint \"%s\" not implemented" % str(constraint))
    call("dbk_corr1ord_constraint", stream(), dtype_code(W), ptr(W), W.shape[0] // 4, W.shape[1], kind, float(lo), float(hi))


# ------------------------------------------------------------------------------------------------
# fused scan + bias + ReLU + pool
# ------------------------------------------------------------------------------------------------
def activity_words(X, W):
    """Empty buffer for the activity masks of scanpool_fprop: one 64-bit word per row of X and tile of 64 filters."""
    return torch.empty((X.numel(), (W.shape[1] + 63) // 64), dtype=torch.int64, device=W.device)


def scanpool_fprop(W, b, X, regions, ptype, want_argmax=False, path="auto", act=None, out=None):
    """pool(relu(corr1ord(W, X) + b)) per region without storing the (N x P) map.
    Returns (pooled, argmax|None) laid out exactly as poolrgn's. float32; float64 tensors run the operator kernels in
    double precision one after another inside the library (no fused float64 kernel).
    path: "auto" lets the library choose; "general" / "mfma" / "wide" / "kmer" force the general path (which picks its
    kernel by size), its matrix-core kernel for many regions (filters of up to 32 taps; sums in another order than
    the lookup kernels', equal to round-off), the four-filters-per-lane lookup kernel (9-24 taps; the bits of the
    one-filter-per-lane kernel) or the table kernel; "kmer_static" is the table kernel
    with the scratch buffer that is built into the library (no allocation inside the call; at most 64 MiB of
    sequence bytes; calls that overlap on one GPU must not use it together).
    out (optional): (pooled, argmax|None) tensors to write into instead of new ones, so that the call allocates nothing.
    act (optional, from activity_words): receives 1 bit per row and filter - rectifier open or not - which
    scanpool_bprop takes in place of recomputing the map (general kernel only).
    Sum pooling and 3-column regions (row step) run the operator kernels one after another inside the library, with
    the map in its scratch: same results as the reference's chain; path must be "auto" and no masks are written."""
    _u8(X)
    _regions(regions)
    f64 = W.dtype == torch.float64
    unfused = regions.shape[1] == 3 or ptype == "sum" or f64
    require(not unfused or (path == "auto" and act is None),
            "ValueError: sum pooling, stepped regions and float64 run the operator chain: no kernel choice, no activity masks")
    require(W.dtype in (torch.float32, torch.float64) and b.dtype == W.dtype, "TypeError: W and b must both be float32 or both float64")
    require(W.shape[0] % 4 == 0 and b.numel() == W.shape[1], "ValueError: W must be (4m x P) and b must have P entries")
    m, F, P = W.shape[0] // 4, W.shape[1], regions.shape[0]
    want_argmax = want_argmax and ptype in ("max", "all")
    if out is not None:
        pooled, argmax = out
        require(pooled.dtype == W.dtype and tuple(pooled.shape) == (P, F * (2 if ptype == "all" else 1)),
                "ValueError: out[0] must be (regions x pooled features) of W's dtype")
        require((argmax is not None) == bool(want_argmax), "ValueError: out[1] must be given exactly when argmax is wanted")
        require(argmax is None or (argmax.dtype == uindex and tuple(argmax.shape) == (P, F)), "ValueError: out[1] must be (regions x filters) indices")
    else:
        pooled = torch.empty((P, F * (2 if ptype == "all" else 1)), dtype=W.dtype, device=W.device)
        argmax = torch.empty((P, F), dtype=uindex, device=W.device) if want_argmax else None
    if unfused:
        # (float64: the operator kernels in double precision, as the reference compiles every operator for both types)
        call("dbk_scanpool_fprop_f64" if f64 else "dbk_scanpool_fprop_unfused", stream(), ptr(W), ptr(b), m, F, ptr(X), X.numel(),
             ptr(regions), P, regions.shape[1], str2pooltype[ptype], ptr(pooled), ptr(argmax))
        return pooled, argmax
    entry = {"auto": "dbk_scanpool_fprop", "general": "dbk_scanpool_fprop_general", "wide": "dbk_scanpool_fprop_wide", "mfma": "dbk_scanpool_fprop_mfma",
             "kmer": "dbk_scanpool_fprop_kmer", "kmer_static": "dbk_scanpool_fprop_kmer_static"}[path]
    args = [stream(), ptr(W), ptr(b), m, F, ptr(X), X.numel(), ptr(regions), P, str2pooltype[ptype], ptr(pooled), ptr(argmax)]
    if path not in ("kmer", "kmer_static"):
        args.append(_act(act, X, F))
    else:
        require(act is None, "ValueError: the table kernel does not write activity masks")
    call(entry, *args)
    return pooled, argmax


def _act(act, X, F):
    if act is None:
        return None
    require(act.dtype == torch.int64 and act.numel() == X.numel() * ((F + 63) // 64),
            "ValueError: act must hold one 64-bit word per row of X and tile of 64 filters")
    return ptr(act)


def scanpool_bprop(W, b, X, regions, ptype, pooled, argmax, dpooled, dW, db, overwrite=False, act=None):
    """Backward of scanpool_fprop: dW += filter gradient (dW[:] = with overwrite), db[:] = bias gradient.
    act: the activity masks the forward call filled (same W, b, X, regions), if it was given any."""
    _u8(X)
    _regions(regions)
    f64 = W.dtype == torch.float64
    require(W.dtype in (torch.float32, torch.float64) and all(t.dtype == W.dtype for t in (b, dpooled, dW, db)),
            "TypeError: W, b, dpooled, dW and db must all be float32 or all float64")
    require(dW.shape == W.shape and db.numel() == W.shape[1], "ValueError: dW / db shapes must match W / b")
    require(dpooled.shape == pooled.shape, "ValueError: dpooled must have pooled's shape")
    m, F, P = W.shape[0] // 4, W.shape[1], regions.shape[0]
    if regions.shape[1] == 3 or ptype == "sum" or f64:
        require(act is None, "ValueError: sum pooling, stepped regions and float64 take no activity masks")
        call("dbk_scanpool_bprop_f64" if f64 else "dbk_scanpool_bprop_unfused", stream(), ptr(W), ptr(b), m, F, ptr(X), X.numel(),
             ptr(regions), P, regions.shape[1], str2pooltype[ptype], ptr(argmax), ptr(dpooled), ptr(dW), ptr(db), int(bool(overwrite)))
        return
    call("dbk_scanpool_bprop", stream(), ptr(W), ptr(b), m, F, ptr(X), X.numel(), ptr(regions), P, str2pooltype[ptype],
         ptr(pooled), ptr(argmax), ptr(dpooled), ptr(dW), ptr(db), int(bool(overwrite)), _act(act, X, F))
