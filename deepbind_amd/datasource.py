"""Host-side reader and batcher for the sequence files the training scripts consume.

Mirrors the part of the reference's datasource that feeds the motif-scan path
(code/libs/kangaroo/kangaroo/data.py:87-131 `fromtxt`, :168-171 `extract_fold`, :274-306
reverse-complement interleave, :309-354 `asbatches`, :524-558 `loadtxt`): tab-separated text,
optionally gzipped, first row = column names; an optional leading `FoldID EventID` column pair; a
trailing `Bound` column is the target when no target file is given. The dinucleotide side
features of the reference are not produced (they are constant zero there, data.py:66-69, and are
not part of the scan path).
"""
import csv
import gzip
import io
import os

import numpy as np

from . import data as _data


def loadtxt(txtfile, usecols=None, maxrows=None, colnames=None):
    """Reads a (possibly .gz) tab-separated file. Returns (colnames, rows); each row a list of strings.
    Without `colnames` the first line is the header."""
    if txtfile is None:
        return None, None
    if not os.path.exists(txtfile):
        raise IOError('Could not open "%s"' % txtfile)
    opener = gzip.open if txtfile.endswith(".gz") else open
    with opener(txtfile, "rb") as raw:
        reader = csv.reader(io.TextIOWrapper(raw, encoding="latin-1", newline=""), delimiter="\t")
        if colnames is None:
            colnames = next(reader)
        if not usecols:
            usecols = range(len(colnames))
        colnames = [colnames[i] for i in usecols]
        rows = []
        for row in reader:
            rows.append([row[i] for i in usecols])
            if maxrows and len(rows) >= maxrows:
                break
    return colnames, rows


class SequenceData(object):
    """Rows of (sequence string, targets, fold id). Y / Ymask follow the reference: float32 targets and the
    mask of non-NaN entries."""

    def __init__(self, sequences, targets=None, targetnames=None, foldids=None, rowidx=None):
        n = len(sequences)
        self.sequences = list(sequences)
        self.targetnames = list(targetnames) if targetnames else []
        self.Y = None if targets is None else np.asarray(targets, dtype=np.float32).reshape((n, -1))
        self.Ymask = None if self.Y is None else ~np.isnan(self.Y)
        self.foldids = list(foldids) if foldids is not None else ["A"] * n
        self.rowidx = np.arange(n, dtype=np.uint32).reshape((-1, 1)) if rowidx is None else np.asarray(rowidx, np.uint32).reshape((-1, 1))

    @staticmethod
    def fromtxt(sequencefile, targetfile=None, foldfilter=None, maxrows=None, targetcols=None):
        names, rows = loadtxt(sequencefile, maxrows=maxrows)
        tnames, targets = loadtxt(targetfile, maxrows=maxrows, usecols=targetcols)
        if targets is None and names[-1].lower() == "bound":
            tnames = [names.pop()]
            targets = [[row[-1]] for row in rows]
            rows = [row[:-1] for row in rows]
        rowidx = np.arange(len(rows), dtype=np.uint32)
        if foldfilter:
            idx = [i for i in range(len(rows)) if rows[i][0] in foldfilter]
            rows = [rows[i] for i in idx]
            rowidx = rowidx[idx]
            if targets is not None:
                targets = [targets[i] for i in idx]
        if names and names[0].lower() in ("fold", "foldid", "fold id"):
            names = names[2:]
            foldids = [row[0] for row in rows]
            rows = [row[2:] for row in rows]
        else:
            foldids = None
        if len(names) != 1:
            raise ValueError("expected one sequence column, found %r" % (names,))
        if targets is not None:
            targets = [[float(v) if v not in ("", "nan", "NaN", "NA") else np.nan for v in row] for row in targets]
        return SequenceData([row[0] for row in rows], targets, tnames, foldids, rowidx)

    def __len__(self):
        return len(self.sequences)

    def __getitem__(self, idx):
        idx = np.arange(len(self))[idx] if isinstance(idx, slice) else np.asarray(idx, dtype=np.int64).ravel()
        return SequenceData([self.sequences[i] for i in idx], None if self.Y is None else self.Y[idx], self.targetnames,
                            [self.foldids[i] for i in idx], self.rowidx[idx])

    def extract_fold(self, foldid):
        return self[[i for i in range(len(self)) if self.foldids[i] == foldid]]

    def asbatches(self, batchsize=64, padding=0, reverse_complement=False):
        """Yields dicts with the packed stream X (N,1) uint8, the region table R (rows,2) uint32 and, when
        there are targets, Y / Ymask; with reverse complements every row appears as fwd,rev and Y / Ymask
        rows are duplicated."""
        n = len(self)
        assert n > 0
        for s0 in range(0, n, batchsize):
            sl = slice(s0, min(n, s0 + batchsize))
            X, R = _data.pack_sequences(self.sequences[sl], padding, reverse_complement=reverse_complement)
            batch = {"X": X, "R": R, "rowidx": self.rowidx[sl]}
            if self.Y is not None:
                rep = 2 if reverse_complement else 1
                batch["Y"] = np.repeat(self.Y[sl], rep, axis=0)
                batch["Ymask"] = np.repeat(self.Ymask[sl], rep, axis=0)
            yield batch
