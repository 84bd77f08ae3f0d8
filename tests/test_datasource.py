"""Host reader / batcher (CPU only): the reference's file formats and batch layout."""
import gzip
import os

import numpy as np
import pytest

from deepbind_amd import datasource, data
from oracle import deepbind_oracle as orc

ENCODE = "/root/reference/data/encode/ELK1_GM12878_ELK1_(1277-1)_Stanford_AC.seq.gz"
PBM = "/root/reference/data/dream5/pbm/sequences.tsv.gz"


def _write(path, text):
    opener = gzip.open if str(path).endswith(".gz") else open
    with opener(path, "wt") as f:
        f.write(text)
    return str(path)


def test_encode_style_file_with_bound_column(tmp_path):
    p = _write(tmp_path / "x.seq.gz", "FoldID\tEventID\tseq\tBound\nA\te1\tACGT\t1\nB\te2\tGGNA\t0\nA\te3\tTTTTT\t1\n")
    d = datasource.SequenceData.fromtxt(p)
    assert d.sequences == ["ACGT", "GGNA", "TTTTT"] and d.foldids == ["A", "B", "A"] and d.targetnames == ["Bound"]
    assert d.Y.dtype == np.float32 and d.Y.ravel().tolist() == [1, 0, 1] and d.Ymask.all()
    a = d.extract_fold("A")
    assert a.sequences == ["ACGT", "TTTTT"] and a.rowidx.ravel().tolist() == [0, 2]
    only_b = datasource.SequenceData.fromtxt(p, foldfilter="B")
    assert only_b.sequences == ["GGNA"] and only_b.rowidx.ravel().tolist() == [1]
    assert len(datasource.SequenceData.fromtxt(p, maxrows=2)) == 2


def test_plain_file_with_separate_targets_and_missing_values(tmp_path):
    s = _write(tmp_path / "s.tsv", "Fold ID\tEvent ID\tseq\nB\tp1\tACGTAC\nB\tp2\tCCC\n")
    t = _write(tmp_path / "t.tsv", "TF_1\tTF_2\n0.5\tnan\n\t2.0\n")
    d = datasource.SequenceData.fromtxt(s, targetfile=t)
    assert d.targetnames == ["TF_1", "TF_2"] and d.Y.shape == (2, 2)
    assert d.Ymask.tolist() == [[True, False], [False, True]]
    one = datasource.SequenceData.fromtxt(s, targetfile=t, targetcols=[1])
    assert one.targetnames == ["TF_2"] and one.Y.shape == (2, 1)


@pytest.mark.parametrize("rc", [False, True])
def test_batches_match_the_reference_layout(tmp_path, rc):
    seqs = ["ACGTTGCA", "GG", "NACGT", "T", "CATCATCAT"]
    p = _write(tmp_path / "b.seq", "seq\tBound\n" + "".join("%s\t%d\n" % (s, i % 2) for i, s in enumerate(seqs)))
    d = datasource.SequenceData.fromtxt(p)
    batches = list(d.asbatches(batchsize=2, padding=3, reverse_complement=rc))
    assert len(batches) == 3
    for bi, b in enumerate(batches):
        rows = seqs[2 * bi:2 * bi + 2]
        rows = orc.insert_reverse_complements(rows) if rc else rows
        Xr, Rr = orc.pack(rows, 3)
        assert np.array_equal(b["X"], Xr) and np.array_equal(b["R"], Rr) and b["R"].dtype == np.uint32
        assert b["Y"].shape == (len(rows), 1) and b["Ymask"].all()
        if rc:
            assert np.array_equal(b["Y"][0::2], b["Y"][1::2])


@pytest.mark.skipif(not os.path.exists(ENCODE), reason="reference data files are not present on this machine")
def test_reads_the_reference_data_files():
    d = datasource.SequenceData.fromtxt(ENCODE, maxrows=500)
    assert len(d) == 500 and all(len(s) == 101 for s in d.sequences) and set(d.foldids) <= set("ABC")
    assert set(np.unique(d.Y)) <= {0.0, 1.0}
    b = next(d.asbatches(batchsize=64, padding=23, reverse_complement=True))
    assert b["X"].shape == (128 * 124 + 23, 1) and b["R"].shape == (128, 2)
    fwd = data.ord2acgt(b["X"][23:124])
    assert fwd == d.sequences[0] and data.ord2acgt(b["X"][124 + 23:248]) == orc.revcomp_string(fwd)
    pbm = datasource.SequenceData.fromtxt(PBM, maxrows=100)
    assert len(pbm) == 100 and pbm.Y is None and all(len(s) == 40 for s in pbm.sequences) and pbm.foldids[0] == "B"
