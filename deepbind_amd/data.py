"""Host-side sequence packing for the motif-scan path.

Mirrors the layout the reference's batcher hands to the scan operator
(reference: code/libs/kangaroo/kangaroo/util.py:50-56,68-74 for the letter
mapping, code/libs/kangaroo/kangaroo/data.py:274-306 for the reverse-complement
interleave and data.py:309-354 for the packed stream + region table).

A batch of strings s_0..s_{B-1} with padding p = m-1 becomes

    X = pad | s_0 | pad | s_1 | ... | s_{B-1} | pad      (uint8, pad = p bytes of 255)
    R[i] = [sum_{k<i}(p+len_k), sum_{k<=i}(p+len_k))     (uint32, half-open rows)

so region i is the leading pad plus sequence i (len_i + m - 1 rows: the "full"
correlation) and N = sum(p+len) + p.
"""
import numpy as np

PAD_CODE = 255      # 'N', '.', padding: contributes the mean of the four channels
DROP_CODE = 254     # input-dropout marker: contributes nothing

_ACGT2ORD = np.full(256, PAD_CODE, dtype=np.uint8)
for _ch, _v in (("a", 0), ("c", 1), ("g", 2), ("t", 3), ("u", 3)):
    _ACGT2ORD[ord(_ch)] = _v
    _ACGT2ORD[ord(_ch.upper())] = _v

_COMPLEMENT = np.full(256, ord("N"), dtype=np.uint8)
for _a, _b in (("a", "T"), ("c", "G"), ("g", "C"), ("t", "A"), ("u", "A"), ("n", "N")):
    _COMPLEMENT[ord(_a)] = ord(_b)
    _COMPLEMENT[ord(_a.upper())] = ord(_b)

_ORD2ACGT = np.full(256, ord("N"), dtype=np.uint8)
_ORD2ACGT[:4] = [ord(c) for c in "ACGT"]


def acgt2ord(s):
    """String -> uint8 ordinals: A,C,G,T/U -> 0,1,2,3 (either case), anything else -> 255."""
    if isinstance(s, str):
        s = s.encode("latin-1")
    return _ACGT2ORD[np.frombuffer(s, dtype=np.uint8)]


def ord2acgt(x):
    """uint8 ordinals -> string; values outside 0..3 become 'N'."""
    return _ORD2ACGT[np.asarray(x, dtype=np.uint8).ravel()].tobytes().decode("latin-1")


def revcomp(s):
    """Reverse complement of a DNA/RNA string (U pairs to A, unknown letters to N)."""
    b = np.frombuffer(s.encode("latin-1"), dtype=np.uint8)
    return _COMPLEMENT[b[::-1]].tobytes().decode("latin-1")


def insert_reverse_complements(seqs):
    """fwd,rev,fwd,rev,... interleave used when the reverse_complement flag is on."""
    out = []
    for s in seqs:
        out.append(s)
        out.append(revcomp(s))
    return out


def pack_ordinals(ords, padding):
    """Pack a list of uint8 ordinal arrays into (X, R) as described in the module docstring.

    Returns X with shape (N, 1) uint8 and R with shape (B, 2) uint32.
    """
    padding = int(padding)
    B = len(ords)
    lens = np.fromiter((len(o) for o in ords), dtype=np.int64, count=B)
    edges = np.concatenate([[0], np.cumsum(lens + padding)])
    N = int(edges[-1]) + padding
    X = np.full(N, PAD_CODE, dtype=np.uint8)
    for i, o in enumerate(ords):
        a = int(edges[i]) + padding
        X[a:a + len(o)] = o
    R = np.stack([edges[:-1], edges[1:]], axis=1).astype(np.uint32)
    return X.reshape(-1, 1), R


def pack_uniform_ordinals(codes, padding):
    """Vectorised pack for a (B, L) uint8 matrix of equal-length sequences."""
    codes = np.asarray(codes, dtype=np.uint8)
    B, L = codes.shape
    padding = int(padding)
    row = np.full((B, padding + L), PAD_CODE, dtype=np.uint8)
    row[:, padding:] = codes
    X = np.concatenate([row.ravel(), np.full(padding, PAD_CODE, dtype=np.uint8)])
    edges = np.arange(B + 1, dtype=np.int64) * (padding + L)
    R = np.stack([edges[:-1], edges[1:]], axis=1).astype(np.uint32)
    return X.reshape(-1, 1), R


def pack_sequences(seqs, padding, reverse_complement=False):
    """Strings -> (X, R). With reverse_complement the rows are interleaved fwd,rev,..."""
    if reverse_complement:
        seqs = insert_reverse_complements(seqs)
    return pack_ordinals([acgt2ord(s) for s in seqs], padding)
