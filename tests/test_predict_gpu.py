"""Prediction-time callers on the GPU (scores, gradient maps, mutation maps, window scans) against the oracle."""
import numpy as np
import pytest
import torch

from oracle import deepbind_oracle as orc
from tests.gpu_util import assert_close

pytestmark = pytest.mark.gpu

ACT, GRAD = 1e-5, 1e-4


def _params(rng, m, F, pool, hidden, scale=0.5):
    # dense weights small enough that the logistic output stays away from saturation: two strands that
    # both round to 1.0f would be a tie in float32 but not in the float64 oracle
    k = F * (2 if pool == "all" else 1)
    f = lambda *s: (rng.standard_normal(s) * scale).astype(np.float32)
    p = {"Wc": f(4 * m, F), "bc": f(1, F) * 0.3}
    if hidden:
        p.update(W1=f(k, hidden) * 0.3, b1=f(1, hidden) * 0.2, W2=f(hidden, 1) * 0.3, b2=f(1, 1) * 0.2 - 0.2)
    else:
        p.update(W1=f(k, 1) * 0.2, b1=f(1, 1) * 0.2 - 0.2)
    return p


def _seqs(rng, n, lo, hi, p_n=0.04):
    out = []
    for _ in range(n):
        s = "".join("ACGT"[v] for v in rng.integers(0, 4, int(rng.integers(lo, hi + 1))))
        out.append("".join("N" if rng.random() < p_n else ch for ch in s))
    return out


def _net(p, m, F, pool, hidden, loss, rc, rate):
    from deepbind_amd.model import SequenceNet
    net = SequenceNet(1, F, m, pool=pool, hidden=hidden, loss=loss, dropout=rate, reverse_complement=rc)
    net.set_params(p)
    return net


CASES = [("max", 8, "nll", False, 0.0, 24, 16), ("all", 0, "mse", False, 0.3, 16, 16), ("max", 0, "mse", True, 0.0, 11, 5),
         ("max", 32, "nll", True, 0.5, 24, 16), ("avg", 4, "mse", False, 0.0, 6, 7)]


@pytest.mark.parametrize("pool,hidden,loss,rc,rate,m,F", CASES)
@pytest.mark.parametrize("mode", [False, True, "finite_diff"])
def test_gen_predictions(pool, hidden, loss, rc, rate, m, F, mode):
    from deepbind_amd import predict
    rng = np.random.default_rng(1000 * m + 10 * hidden + int(rc))
    p = _params(rng, m, F, pool, hidden)
    seqs = _seqs(rng, 7, 18, 30)                       # ragged: includes the pad-mutation quirk of short sequences
    out = "logistic" if loss == "nll" else "linear"
    p64 = {k: v.astype(np.float64) for k, v in p.items()}
    Zr, mr = orc.gen_predictions(p64, seqs, pool, hidden, out, dropout_rate=[rate] if rate else None, reverse_complement=rc, want_gmaps=mode)
    net = _net(p, m, F, pool, hidden, loss, rc, rate)
    # two batches, to cover the batch loop
    Z, maps = predict.gen_predictions(net, seqs, want_gmaps=mode, batchsize=4)
    Zr2 = [orc.gen_predictions(p64, seqs[s:s + 4], pool, hidden, out, dropout_rate=[rate] if rate else None, reverse_complement=rc,
                               want_gmaps=mode) for s in (0, 4)]
    Zr = np.vstack([z for z, _ in Zr2])
    assert Z.shape == (len(seqs), 1)
    assert_close(Z, Zr, ACT, "Z")
    if not mode:
        assert maps is None
        return
    mr = sum([mm for _, mm in Zr2], [])
    assert len(maps) == len(mr) == len(seqs)
    scale = max(np.abs(b).max() for _, b in mr) + 1e-30
    for (sa, a), (sb, b) in zip(maps, mr):
        assert sa == sb and a.shape == b.shape
        assert np.abs(a - b).max() <= GRAD * scale, (np.abs(a - b).max(), scale)


@pytest.mark.parametrize("rc", [False, True])
@pytest.mark.parametrize("stride,want", [(1, True), (1, False), (4, False)])
def test_gen_predictionmaps(rc, stride, want):
    from deepbind_amd import predict
    rng = np.random.default_rng(17)
    m, F, pool, hidden = 8, 6, "max", 5
    p = _params(rng, m, F, pool, hidden)
    p64 = {k: v.astype(np.float64) for k, v in p.items()}
    seqs = _seqs(rng, 3, 25, 40)
    pr, gr = orc.gen_predictionmaps(p64, seqs, pool, hidden, "logistic", reverse_complement=rc, stride=stride, windowsize=12, want_gmaps=want)
    net = _net(p, m, F, pool, hidden, "nll", rc, 0.0)
    pm, gm = predict.gen_predictionmaps(net, seqs, stride=stride, windowsize=12, want_gmaps=want)
    assert len(pm) == len(pr) == 3
    for a, b in zip(pm, pr):
        assert a.shape == b.shape
        assert_close(a, b, ACT, "pmap")
    if want:
        scale = max(np.abs(b).max() for b in gr) + 1e-30
        for a, b in zip(gm, gr):
            assert a.shape == b.shape and np.abs(a - b).max() <= GRAD * scale
    else:
        assert gm is None
    with pytest.raises(ValueError):
        predict.gen_predictionmaps(net, seqs, stride=2, windowsize=12, want_gmaps=True)
