"""Prediction-time callers of the motif-scan path: scores, gradient maps, finite-difference
mutation maps and sliding-window scans for one trained model.

Mirrors the reference's prediction module (code/libs/kangaroo/kangaroo/predict.py:145-345):
`maskout_revcomp`, `gen_convnet_predictions` and `gen_convnet_predictionmaps`, with the model
evaluation replaced by `SequenceNet` calls. The mutation map re-scores the batch once per
(position, base) as the reference does, but mutates the packed stream and collects the
differences on the device, so a batch costs 4 x (longest region) small launches and one copy
back instead of as many host round trips.
"""
import numpy as np
import torch

from . import data as _data

_RCINDEX = (3, 2, 1, 0)


def maskout_revcomp(Z, reverse_complement):
    """Host version of the pair selection (predict.py:145-164): Z holds fwd,rev,fwd,rev rows; keeps
    the larger of each pair (ties keep fwd). Returns (selected rows, Zmask | None)."""
    if not reverse_complement:
        return Z, None
    Zc = Z.reshape((-1, 2))
    Zmask = np.zeros_like(Zc, dtype=bool)
    Zmask[:, 0] = Zc[:, 0] >= Zc[:, 1]
    Zmask[:, 1] = Zc[:, 0] < Zc[:, 1]
    Zmask = Zmask.reshape((-1, 1))
    return Z[Zmask.ravel()], Zmask


def _finite_diff(net, Xd, Rd, R, Z, dX):
    """Overwrites dX (N, 4, device) with mtZ - Z for every single-base change, the reference's way
    (predict.py:201-240): pass (i, j) sets letter i of EVERY region to base j (reverse rows: the
    mirrored letter to the complement), regions being leading pad + sequence, so passes with i past
    the end of a short sequence write into the pad that follows it exactly as the reference does."""
    rc = net.reverse_complement
    pad = net.m - 1
    a = torch.as_tensor(R[:, 0].astype(np.int64), device=Xd.device)
    b = torch.as_tensor(R[:, 1].astype(np.int64), device=Xd.device)
    length = b - a
    k = torch.arange(len(R), device=Xd.device)
    fwd = (k % 2 == 0) if rc else torch.ones_like(k, dtype=torch.bool)
    # only passes that can reach a reported row matter: i below the longest sequence
    longest = int((R[:, 1].astype(np.int64) - R[:, 0].astype(np.int64)).max()) - pad
    Xflat = Xd.view(-1)
    for i in range(max(longest, 0)):
        live = length > i
        at_f = (pad + a + i)[live & fwd]
        at_r = (b - i - 1)[live & ~fwd]
        for j in range(4):
            mt = Xflat.clone()
            mt[at_f] = j
            if rc:
                mt[at_r] = _RCINDEX[j]
            mtZ = net.predict(mt.view(-1, 1), Rd)       # pair maximum included
            dZ = (mtZ - Z) * torch.clamp(torch.sign(torch.maximum(Z, mtZ)), min=0)
            rows = (live & fwd).nonzero().ravel()
            dX[(pad + a + i)[rows], j] = dZ[(rows // 2) if rc else rows, 0]


def gen_predictions(net, seqs, want_gmaps=False, batchsize=2048):
    """Scores a list of sequence strings with a single-model SequenceNet.

    Returns (predictions (nseq, 1) float32, gmaps). gmaps is None, or a list of
    (sequence string, (len, 4) float32 map): with want_gmaps=True the back-propagated input
    gradient (with reverse complements only the winning strand's entry, whose string is that
    strand's), with want_gmaps="finite_diff" the mutation map of the forward strand.
    (reference: predict.py:168-260)"""
    assert net.ninst == 1, "prediction maps are defined for one model at a time"
    rc, pad = net.reverse_complement, net.m - 1
    preds, gmaps = [], ([] if want_gmaps else None)
    for s0 in range(0, len(seqs), batchsize):
        X, R = _data.pack_sequences(seqs[s0:s0 + batchsize], pad, reverse_complement=rc)
        Xd = torch.from_numpy(X).to(net.device)
        Rd = torch.from_numpy(R).to(net.device)
        if not want_gmaps:
            preds.append(net.predict(Xd, Rd).cpu().numpy())
            continue
        Zall, dX = net.input_gradients(Xd, Rd)
        Zh, Zmask = maskout_revcomp(Zall.cpu().numpy(), rc)
        preds.append(Zh)
        Ri = R.astype(np.int64)
        if want_gmaps == "finite_diff":
            _finite_diff(net, Xd, Rd, Ri, torch.from_numpy(Zh).to(net.device), dX)
            dXh = dX.cpu().numpy()
            fwd = Ri[::2] if rc else Ri
            gmaps += [(_data.ord2acgt(X[a + pad:b]), dXh[a + pad:b].copy()) for a, b in fwd]
        else:
            dXh = dX.cpu().numpy()
            maps = [(_data.ord2acgt(X[a + pad:b]), dXh[a + pad:b].copy()) for a, b in Ri]
            if Zmask is not None:
                maps = [mp for mp, keep in zip(maps, Zmask.ravel()) if keep]
            gmaps += maps
    return np.vstack(preds), gmaps


def gen_predictionmaps(net, seqs, stride=1, windowsize=20, want_gmaps=False):
    """Sliding-window scan (reference: predict.py:263-345): every sequence is padded with
    windowsize-1 N on both sides and cut into windows of `windowsize` letters every `stride`;
    all windows of up to 32 sequences are scored in one batch. Returns (list of per-sequence
    prediction maps, list of (len+windowsize-1, 4) window-averaged gradient maps | None)."""
    if want_gmaps and stride != 1:
        # the reference's aggregation (predict.py:330-340) slices rows that only line up for stride 1
        raise ValueError("window-averaged gradient maps need stride 1 (got %d)" % stride)
    pmaps, gmaps = [], ([] if want_gmaps else None)
    chunk = 32
    for c0 in range(0, len(seqs), chunk):
        raws = list(seqs[c0:c0 + chunk])
        windows, nwin = [], []
        for raw in raws:
            padseq = "N" * (windowsize - 1) + raw + "N" * (windowsize - 1)
            w = [padseq[i:i + windowsize] for i in range(0, max(1, len(padseq) - windowsize + 1), stride)]
            windows += w
            nwin.append(len(w))
        Z, wmaps = gen_predictions(net, windows, want_gmaps=want_gmaps, batchsize=len(windows))
        edges = np.cumsum([0] + nwin)
        for i, raw in enumerate(raws):
            pmaps.append(Z[edges[i]:edges[i + 1]].ravel().copy())
            if want_gmaps:
                gmap = np.zeros((len(raw) + windowsize - 1, 4), Z.dtype)
                denom = np.zeros_like(gmap)
                for j in range(nwin[i]):
                    dXj = wmaps[edges[i] + j][1][:min(windowsize, (nwin[i] - j) * stride)]
                    gmap[j * stride:j * stride + windowsize] += dXj
                    denom[j * stride:j * stride + windowsize] += 1
                with np.errstate(invalid="ignore", divide="ignore"):
                    gmap /= denom
                gmaps.append(np.nan_to_num(gmap))
    return pmaps, gmaps
