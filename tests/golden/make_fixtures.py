"""Writes the small golden vectors under tests/golden/ from the CPU oracle.

    python tests/golden/make_fixtures.py

The reference ships no stored vectors for this path and cannot be executed here (CUDA-only kernels,
Python-2 host code), so these files pin the pinned oracle's outputs: the CPU suite checks the oracle
still reproduces them, the GPU suite checks the HIP library against them.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import deepbind_oracle as orc  # noqa: E402


def scan_pool_case(seed, seqs, m, F):
    rng = np.random.default_rng(seed)
    X, R = orc.pack(seqs, m - 1)
    W = (rng.standard_normal((4 * m, F)) * 0.2).astype(np.float32)
    b = (rng.standard_normal((1, F)) * 0.1).astype(np.float32)
    Z = np.zeros((X.size, F), np.float32)
    orc.corr1ord(W, X, Z)
    A = orc.relu_fprop(orc.bias_fprop(Z, b))
    out = dict(X=X, R=R, W=W, b=b, Z=Z)
    for pt in ("max", "avg", "sum", "all"):
        P, I = orc.poolrgn(A, R, pt, want_argmax=True)
        out["pool_" + pt] = P
        if I is not None:
            out["argmax_" + pt] = I
    dZ = rng.standard_normal(Z.shape).astype(np.float32)
    dW = np.zeros_like(W)
    orc.corr1ord_bprop_W(dW, X, dZ)
    dX = np.zeros((X.size, 4), np.float32)
    orc.corr1ord_bprop_X(dX, W, dZ)
    out.update(dZ=dZ, dW=dW, dX=dX)
    return out


def train_case(seed):
    rng = np.random.default_rng(seed)
    nm, nf, m, hid = 3, 4, 6, 5
    seqs = ["ACGTNACGGTAC", "TTGACA", "GGNNCATTAGCAT", "C", "ACGUACGUACGUAACC"]
    X, R = orc.pack(seqs, m - 1)
    k = 2 * nf
    p = {"Wc": rng.standard_normal((4 * m, nf * nm)) * 0.3, "bc": rng.standard_normal((1, nf * nm)) * 0.1,
         "W1": rng.standard_normal((k * nm, hid)) * 0.3, "b1": rng.standard_normal((1, hid * nm)) * 0.1,
         "W2": rng.standard_normal((hid * nm, 1)) * 0.3, "b2": rng.standard_normal((1, nm)) * 0.1}
    p = {a: v.astype(np.float32) for a, v in p.items()}
    Y = (rng.random((len(seqs), nm)) < 0.5).astype(np.float32)
    rate = np.array([0.05, 0.02, 0.1]); mom = np.array([0.9, 0.95, 0.5])
    out = {"X": X, "R": R, "Y": Y, "rate": rate, "momentum": mom}
    out.update({"p0_" + a: v for a, v in p.items()})
    q = {a: v.astype(np.float64) for a, v in p.items()}
    mP = {a: np.zeros(v.shape) for a, v in q.items()}
    for step in range(2):
        orc.train_step(q, mP, X, R, Y.astype(np.float64), nm, "all", hid, "nll", rate, mom,
                       decay_conv=np.array([1e-3, 0, 1e-2]), decay_full=np.array([1e-2, 1e-3, 0]), step=step, weight_decay_start=1)
    out.update({"p2_" + a: v.astype(np.float32) for a, v in q.items()})
    return out


def main():
    np.savez_compressed(os.path.join(HERE, "scan_pool_small.npz"),
                        **scan_pool_case(7, ["ACGTNNACGTTGCA", "TT", "GATTACAGATTACA", "C", "NNNN", "ACGU.acgu"], 5, 7))
    np.savez_compressed(os.path.join(HERE, "scan_pool_m24.npz"),
                        **scan_pool_case(8, ["ACGT" * 13 + "N", "TTGACAGCTAGCTAGCTAGCATCGATCGATGCATGCAT", "GG"], 24, 16))
    np.savez_compressed(os.path.join(HERE, "train_two_steps.npz"), **train_case(9))


if __name__ == "__main__":
    main()
