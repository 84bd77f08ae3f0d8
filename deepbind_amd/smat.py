"""The few array operations the bias / ReLU / dense / loss nodes call, over device tensors.
Names follow the reference's array module (reference: code/libs/smat/py/smat/smat.py), but only the
operations on the motif-scan path exist here, each backed by a kernel in libdeepbind_hip.so.
torch supplies device memory and the stream; it does no arithmetic on this path.
"""
import torch

from ._lib import call, dtype_code, ptr, require, stream
from . import deepity_smat as _ds


def zeros(shape, dtype=torch.float32, device="cuda"):
    return torch.zeros(shape, dtype=dtype, device=device)


def zeros_like(A):
    return torch.zeros_like(A)


def empty(shape, dtype=torch.float32, device="cuda"):
    return torch.empty(shape, dtype=dtype, device=device)


def empty_like(A):
    return torch.empty_like(A)


def asarray(a, dtype=None, device="cuda"):
    return torch.as_tensor(a, dtype=dtype).to(device).contiguous()


def randn(nrow, ncol, dtype=torch.float32, seed=0, offset=0, device="cuda"):
    """(nrow x ncol) standard normal deviates from the library's counter-based generator at (seed, offset).
    reference: smat.randn (cuRAND there; the streams differ, the distribution does not)"""
    Z = torch.empty((nrow, ncol), dtype=dtype, device=device)
    call("dbk_normal_fill", stream(), dtype_code(Z), ptr(Z), Z.numel(), int(seed), int(offset))
    return Z


def sync():
    call("dbk_sync", stream())


def dot(A, B):
    """A (n x k) . B (k x m). reference: smat_cuda/dot.cu:50-67"""
    return _ds.blockwise_dot(A, B, 1)


def dot_nt(A, B):
    """A (n x m) . B (k x m)^T -> (n x k)."""
    return _ds.blockwise_dot_nt(A, B, 1)


def dot_tn(A, B):
    """A (n x k)^T . B (n x m) -> (k x m)."""
    W = torch.empty((A.shape[1], B.shape[1]), dtype=A.dtype, device=A.device)
    return _ds.blockwise_dot_tn(A, B, 1, W)


def add_rowvec(X, b):
    """X + b with the row vector b broadcast down the rows (the bias node's forward)."""
    require(b.numel() == X.shape[1] and b.dtype == X.dtype, "ValueError: b must have one entry per column of X")
    Z = torch.empty_like(X)
    call("dbk_add_rowvec", stream(), dtype_code(X), ptr(X), ptr(b), ptr(Z), X.shape[0], X.shape[1])
    return Z


def sum_axis0(X):
    """Column sums as a (1 x ncol) row (the bias node's gradient)."""
    out = torch.empty((1, X.shape[1]), dtype=X.dtype, device=X.device)
    call("dbk_colsum", stream(), dtype_code(X), ptr(X), ptr(out), X.shape[0], X.shape[1])
    return out


def relu(X):
    """maximum(0, X)."""
    Z = torch.empty_like(X)
    call("dbk_relu", stream(), dtype_code(X), ptr(X), ptr(Z), X.numel())
    return Z


def mul_sign(dZ, Z):
    """dZ * sign(Z): the ReLU node's gradient."""
    dX = torch.empty_like(dZ)
    call("dbk_mul_sign", stream(), dtype_code(dZ), ptr(dZ), ptr(Z), ptr(dX), dZ.numel())
    return dX


def sign(X):
    """(x > 0) - (x < 0)."""
    Z = torch.empty_like(X)
    call("dbk_sign", stream(), dtype_code(X), ptr(X), ptr(Z), X.numel())
    return Z


def logistic(X):
    Z = torch.empty_like(X)
    call("dbk_logistic", stream(), dtype_code(X), ptr(X), ptr(Z), X.numel())
    return Z


def softmax(X, nchunk=1):
    """Row-wise softmax of a 2-D matrix; with nchunk > 1 every row is split into nchunk equal chunks that are
    normalised separately (reference: deepity/std/softmax.py:58-71 with nchunk = ngroup * ninst)."""
    require(X.dim() == 2 and X.shape[1] % nchunk == 0, "ValueError: the number of columns must be divisible by nchunk")
    Z = torch.empty_like(X)
    call("dbk_softmax", stream(), dtype_code(X), ptr(X), ptr(Z), X.numel(), X.shape[1] // nchunk)
    return Z


def loss_terms(Z, Y, kind):
    """Elementwise loss terms before masking / averaging; kind is "nll", "mse", "nll_multiclass"
    (several columns per output: log(max(1e-15, Z)) * Y, reference: deepity/std/loss.py:147-151) or "hinge"
    (max(0, (1-Y)Z + Y(1-Z)), loss.py:162-163)."""
    L = torch.empty_like(Z)
    call("dbk_loss_terms", stream(), dtype_code(Z), {"nll": 0, "mse": 1, "nll_multiclass": 2, "hinge": 3}[kind], ptr(Z), ptr(Y), ptr(L), Z.numel())
    return L


def hinge_grad(Z, Y, scale=1.0):
    """Gradient of the hinge loss at the outputs: (1 - 2Y) * scale where (1-Y)Z + Y(1-Z) > 0, else 0
    (reference: hinge._calc_dZ, deepity/std/loss.py:165-169)."""
    dZ = torch.empty_like(Z)
    call("dbk_hinge_grad", stream(), dtype_code(Z), ptr(Z), ptr(Y), float(scale), ptr(dZ), Z.numel())
    return dZ


def sub_scale(Z, Y, scale):
    """(Z - Y) * scale."""
    dZ = torch.empty_like(Z)
    call("dbk_sub_scale", stream(), dtype_code(Z), ptr(Z), ptr(Y), float(scale), ptr(dZ), Z.numel())
    return dZ
