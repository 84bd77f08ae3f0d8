"""Seeded synthetic workloads for the five benchmark / parity configurations.

Everything is drawn from ``numpy.random.default_rng(seed)`` (PCG64) with seeds
0..4 for configs 1..5. "N(0, s)" means standard deviation s, matching the
reference's ``randn * init_scale`` initialisation
(reference: code/libs/deepity/deepity/sgd.py:340-341). The filter bank layout is
[tap][channel][filter] with filter fastest, i.e. a (4*m, F) row-major matrix
(reference: code/libs/kangaroo/kangaroo_smat/corr1ord.cuh:126-132); dense weights
are (rows_per_model * nmodel, ncol) with model-major rows
(reference: code/libs/deepity/deepity/std/full.py:57).

The combiner of the reference's sequence model has 16 extra, always-zero
"dinucleotide feature" input columns (reference: code/libs/kangaroo/kangaroo/data.py:59-69);
they multiply zeros and never change the output, so the synthetic benchmark models here
leave them out (SequenceNet(feature_columns=16) builds the reference-shaped layer).
"""
import numpy as np

from . import data as _data


class ModelSpec(object):
    """Shapes and per-model options for a batch of independent models on the model axis."""

    def __init__(self, nmodel, nfilter, m, pool, hidden, loss):
        self.nmodel = int(nmodel)
        self.nfilter = int(nfilter)          # motif detectors per model
        self.m = int(m)                      # motif width
        # pool / hidden may be a single value or one per model
        self.pool = list(pool) if isinstance(pool, (list, tuple)) else [pool] * self.nmodel
        self.hidden = list(hidden) if isinstance(hidden, (list, tuple)) else [int(hidden)] * self.nmodel
        self.loss = loss                     # "nll" | "mse" | None (forward only)

    @property
    def F(self):
        return self.nmodel * self.nfilter

    def nfeat(self, i):
        return self.nfilter * (2 if self.pool[i] == "all" else 1)


def _init_params(rng, spec, w_std, dense_std, dtype=np.float32):
    """Random parameters for a homogeneous batch of models (same pool/hidden for all)."""
    nm, nf, m = spec.nmodel, spec.nfilter, spec.m
    assert len(set(spec.pool)) == 1 and len(set(spec.hidden)) == 1
    k = spec.nfeat(0)
    h = spec.hidden[0]
    p = {}
    p["Wc"] = (rng.standard_normal((4 * m, nf * nm)) * w_std).astype(dtype)
    p["bc"] = np.zeros((1, nf * nm), dtype)
    if h > 0:
        p["W1"] = (rng.standard_normal((k * nm, h)) * dense_std).astype(dtype)
        p["b1"] = np.zeros((1, h * nm), dtype)
        p["W2"] = (rng.standard_normal((h * nm, 1)) * dense_std).astype(dtype)
        p["b2"] = np.zeros((1, nm), dtype)
    else:
        p["W1"] = (rng.standard_normal((k * nm, 1)) * dense_std).astype(dtype)
        p["b1"] = np.zeros((1, nm), dtype)
    return p


def _random_codes(rng, B, L, n_rate):
    codes = rng.integers(0, 4, size=(B, L), dtype=np.uint8)
    if n_rate > 0:
        codes[rng.random((B, L)) < n_rate] = _data.PAD_CODE
    return codes


def config1(seed=0, B=64, L=101):
    """Forward scoring, 1 model: 16 motifs x width 24, global max pool, 16->32 ReLU->1."""
    rng = np.random.default_rng(seed)
    spec = ModelSpec(1, 16, 24, "max", 32, None)
    codes = _random_codes(rng, B, L, 0.02)
    X, R = _data.pack_uniform_ordinals(codes, spec.m - 1)
    params = _init_params(rng, spec, 0.01, 0.01)
    return dict(spec=spec, X=X, R=R, params=params)


def config2(seed=1, B=128):
    """RNA probe regression train step: 16 motifs x width 16, max+avg pool -> 32 feats -> 1, mse."""
    rng = np.random.default_rng(seed)
    spec = ModelSpec(1, 16, 16, "all", 0, "mse")
    lens = rng.integers(38, 42, size=B)
    ords = [rng.integers(0, 4, size=int(n), dtype=np.uint8) for n in lens]
    X, R = _data.pack_ordinals(ords, spec.m - 1)
    y = rng.lognormal(0.0, 1.0, size=(B, 1))
    y = ((y - y.mean()) / y.std()).astype(np.float32)
    params = _init_params(rng, spec, 0.01, 0.01)
    return dict(spec=spec, X=X, R=R, Y=y, params=params, rate=0.01, momentum=0.9)


def dinuc_shuffle(codes, rng):
    """Dinucleotide-preserving shuffle (Altschul-Erickson Euler-path construction).

    Returns a permutation of ``codes`` with the same first and last letter and the
    same multiset of adjacent pairs (reference use: code/deepbind_util.py:326-340
    builds shuffled negatives the same way).
    """
    codes = np.asarray(codes)
    n = len(codes)
    if n < 3:
        return codes.copy()
    letters = sorted(set(int(c) for c in codes))
    last = int(codes[-1])
    succ = {a: [] for a in letters}
    for a, b in zip(codes[:-1], codes[1:]):
        succ[int(a)].append(int(b))
    while True:
        # choose for every letter except the final one a "last edge"; accept if all reach `last`
        last_edge = {}
        for a in letters:
            if a != last and succ[a]:
                last_edge[a] = succ[a][int(rng.integers(len(succ[a])))]
        ok = True
        for a in letters:
            seen = set()
            v = a
            while v != last:
                if v in seen or v not in last_edge:
                    ok = False
                    break
                seen.add(v)
                v = last_edge[v]
            if not ok:
                break
        if ok:
            break
    out = [int(codes[0])]
    pools = {}
    for a in letters:
        lst = list(succ[a])
        if a in last_edge:
            lst.remove(last_edge[a])
            perm = rng.permutation(len(lst))
            lst = [lst[i] for i in perm] + [last_edge[a]]
        else:
            perm = rng.permutation(len(lst))
            lst = [lst[i] for i in perm]
        pools[a] = lst[::-1]   # pop() from the end = consume in order
    v = out[0]
    for _ in range(n - 1):
        v = pools[v].pop()
        out.append(v)
    return np.asarray(out, dtype=codes.dtype)


def config3(seed=2, B=128, L=101):
    """Binary peak classification train step: 16 x width 24, max pool, 16->32->1, logistic + nll."""
    rng = np.random.default_rng(seed)
    spec = ModelSpec(1, 16, 24, "max", 32, "nll")
    npos = B // 2
    pwm = rng.dirichlet(0.5 * np.ones(4), size=12)          # (12, 4) column distributions
    pos = rng.integers(0, 4, size=(npos, L), dtype=np.uint8)
    for i in range(npos):
        off = int(rng.integers(0, L - 12 + 1))
        motif = np.array([rng.choice(4, p=pwm[j]) for j in range(12)], dtype=np.uint8)
        pos[i, off:off + 12] = motif
    neg = np.stack([dinuc_shuffle(pos[i], rng) for i in range(npos)])
    codes = np.concatenate([pos, neg], axis=0)
    y = np.concatenate([np.ones((npos, 1)), np.zeros((B - npos, 1))]).astype(np.float32)
    X, R = _data.pack_uniform_ordinals(codes, spec.m - 1)
    params = _init_params(rng, spec, 0.01, 0.01)
    U = rng.random((B, spec.nfeat(0))).astype(np.float32)     # dropout uniforms, keep iff U >= rate
    return dict(spec=spec, X=X, R=R, Y=y, params=params, dropout_rate=0.5, U=U, rate=0.01, momentum=0.9)


def _loguniform(rng, lo, hi, size=None):
    return np.exp(rng.uniform(np.log(lo), np.log(hi), size=size))


def _powuniform(rng, lo, hi, p, size=None):
    # reference: code/libs/deepity/deepity/hpsearch.py:141-161 (uniform in x**p space)
    return rng.uniform(lo ** p, hi ** p, size=size) ** (1.0 / p)


def config4(seed=3, B=256, ndraw=30, nfold=3):
    """Calibration batch: 90 independent models (30 hyper-parameter draws x 3 folds), one shared batch."""
    rng = np.random.default_rng(seed)
    nm = ndraw * nfold
    lens = rng.integers(20, 41, size=B)
    ords = [rng.integers(0, 4, size=int(n), dtype=np.uint8) for n in lens]
    m = 24
    X, R = _data.pack_ordinals(ords, m - 1)
    Y1 = (rng.random((B, 1)) < 0.5).astype(np.float32)
    pool_d = [("max", "all")[int(rng.integers(2))] for _ in range(ndraw)]
    hidden_d = [(0, 32)[int(rng.integers(2))] for _ in range(ndraw)]
    hp = dict(
        init_conv=_loguniform(rng, 1e-7, 1e-3, ndraw), decay_conv=_loguniform(rng, 1e-15, 1e-3, ndraw),
        init_full=_loguniform(rng, 1e-5, 1e-2, ndraw), decay_full=_loguniform(rng, 1e-10, 1e-3, ndraw),
        dropout=rng.choice([0.0, 0.0, 0.25, 0.5], size=ndraw),
        rate=_loguniform(rng, 0.0005, 0.05, ndraw), momentum=_powuniform(rng, 0.95, 0.99, 0.5, ndraw),
    )
    rep = lambda v: np.repeat(np.asarray(v), nfold)
    pool = [p for p in pool_d for _ in range(nfold)]
    hidden = [h for h in hidden_d for _ in range(nfold)]
    spec = ModelSpec(nm, 16, m, pool, hidden, "nll")
    hp = {k: rep(v).astype(np.float32) for k, v in hp.items()}
    # fold f of draw d trains on the rows whose index mod nfold != f
    Ymask = np.zeros((B, nm), dtype=bool)
    for j in range(nm):
        Ymask[:, j] = (np.arange(B) % nfold) != (j % nfold)
    Y = np.repeat(Y1, nm, axis=1)
    # per-model parameters, drawn model by model
    models = []
    for j in range(nm):
        s1 = ModelSpec(1, 16, m, pool[j], hidden[j], "nll")
        models.append(_init_params(rng, s1, float(hp["init_conv"][j]), float(hp["init_full"][j])))
    return dict(spec=spec, X=X, R=R, Y=Y, Ymask=Ymask, hp=hp, models=models)


def config5(seed=4, nseq=100000, L=500, nmodel=64):
    """Bulk forward scoring: 64 models x 16 motifs x width 24, max pool, 16->32->1, over nseq x L DNA."""
    rng = np.random.default_rng(seed)
    spec = ModelSpec(nmodel, 16, 24, "max", 32, None)
    codes = _random_codes(rng, nseq, L, 0.01)
    X, R = _data.pack_uniform_ordinals(codes, spec.m - 1)
    params = _init_params(rng, spec, 0.05, 0.05)
    return dict(spec=spec, X=X, R=R, params=params)


def positions(R):
    """Scan positions of a region table: sum over regions of (end - start) = sum(len + m - 1)."""
    R = np.asarray(R, dtype=np.int64)
    return int((R[:, 1] - R[:, 0]).sum())
