"""ctypes binding of libdeepbind_hip.so.

The library is the only compute path: if it cannot be loaded, importing an operator module
raises. After every call the thread's last-error text is polled and turned into an exception,
the convention of the reference's Python shim (reference: code/libs/smat/py/smat/smat_dll.py:166-183).
"""
import ctypes
import os
from ctypes import c_char_p, c_double, c_float, c_int, c_size_t, c_uint64, c_void_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdeepbind_hip.so")


class DeepbindError(RuntimeError):
    """Raised when a library call reports a failure (counterpart of the reference's SmatException)."""


DBK_F32, DBK_F64 = 0, 1
PT_MAX, PT_AVG, PT_SUM, PT_ALL = 0, 1, 2, 3
str2pooltype = {"max": PT_MAX, "avg": PT_AVG, "sum": PT_SUM, "all": PT_ALL}
# loss_kind of dbk_head_train / dbk_train_step*: output non-linearity + loss (reference: deepity/std/loss.py:131-174)
LOSS_KIND = {"nll": 0, "mse": 1, "hinge": 2}

_P, _Z, _I, _U64, _F, _D = c_void_p, c_size_t, c_int, c_uint64, c_float, c_double

# name -> argument types; every function returns int except the two noted below
_SIGNATURES = {
    "dbk_version": [],
    "dbk_device_count": [],
    "dbk_set_exact_scan": [_I],
    "dbk_sync": [_P],
    "dbk_corr1ord": [_P, _I, _P, _Z, _Z, _P, _Z, _Z, _P],
    "dbk_corr1ord_bprop_W": [_P, _I, _P, _Z, _Z, _P, _Z, _Z, _P],
    "dbk_corr1ord_bprop_X": [_P, _I, _P, _Z, _Z, _P, _Z, _Z, _P],
    "dbk_poolrgn": [_P, _I, _P, _Z, _P, _Z, _I, _P, _P, _I],
    "dbk_poolrgn_bprop": [_P, _I, _P, _Z, _P, _Z, _I, _P, _P, _I],
    "dbk_dropoutord_fp_tr": [_P, _P, _P, _P, _Z, _F, _U64, _U64, _P],
    "dbk_corr1ord_constraint": [_P, _I, _P, _Z, _Z, _I, _D, _D],
    "dbk_dropoutord_mirror": [_P, _P, _P, _P, _P, _Z, _Z],
    "dbk_dropoutord_fp_tr_u": [_P, _P, _P, _P, _Z, _F, _P],
    "dbk_scanpool_fprop": [_P, _P, _P, _Z, _Z, _P, _Z, _P, _Z, _I, _P, _P, _P],
    "dbk_scanpool_fprop_general": [_P, _P, _P, _Z, _Z, _P, _Z, _P, _Z, _I, _P, _P, _P],
    "dbk_scanpool_fprop_wide": [_P, _P, _P, _Z, _Z, _P, _Z, _P, _Z, _I, _P, _P, _P],
    "dbk_scanpool_fprop_mfma": [_P, _P, _P, _Z, _Z, _P, _Z, _P, _Z, _I, _P, _P, _P],
    "dbk_scanpool_fprop_kmer": [_P, _P, _P, _Z, _Z, _P, _Z, _P, _Z, _I, _P, _P],
    "dbk_scanpool_fprop_kmer_static": [_P, _P, _P, _Z, _Z, _P, _Z, _P, _Z, _I, _P, _P],
    "dbk_scanpool_bprop": [_P, _P, _P, _Z, _Z, _P, _Z, _P, _Z, _I, _P, _P, _P, _P, _P, _I, _P],
    "dbk_scanpool_fprop_unfused": [_P, _P, _P, _Z, _Z, _P, _Z, _P, _Z, _I, _I, _P, _P],
    "dbk_scanpool_bprop_unfused": [_P, _P, _P, _Z, _Z, _P, _Z, _P, _Z, _I, _I, _P, _P, _P, _P, _I],
    "dbk_scanpool_fprop_f64": [_P, _P, _P, _Z, _Z, _P, _Z, _P, _Z, _I, _I, _P, _P],
    "dbk_scanpool_bprop_f64": [_P, _P, _P, _Z, _Z, _P, _Z, _P, _Z, _I, _I, _P, _P, _P, _P, _I],
    "dbk_blockwise_dot": [_P, _I, _I, _I, _I, _I, _I, _P, _P, _P],
    "dbk_blockwise_dot_nt": [_P, _I, _I, _I, _I, _I, _P, _P, _P],
    "dbk_blockwise_dot_tn": [_P, _I, _I, _I, _I, _I, _I, _P, _P, _P],
    "dbk_blockwise_dot_combined": [_P, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P, _P],
    "dbk_blockwise_dot_nt_combined": [_P, _I, _I, _I, _I, _I, _I, _I, _P, _P, _P],
    "dbk_blockwise_dot_tn_combined": [_P, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P, _P],
    "dbk_gradstep": [_P, _I, _Z, _P, _P, _P, _P, _P],
    "dbk_gradstep_nesterov1": [_P, _I, _Z, _P, _P, _P],
    "dbk_gradstep_nesterov2": [_P, _I, _Z, _P, _P, _P, _P, _P],
    "dbk_gradstep_lookahead": [_P, _I, _Z, _P, _P, _P, _P],
    "dbk_gradstep_nesterov2_lookahead": [_P, _I, _Z, _P, _P, _P, _P, _P, _P],
    "dbk_madd_bcast": [_P, _I, _P, _P, _P, _Z, _Z, _Z],
    "dbk_maskout": [_P, _I, _P, _P, _Z],
    "dbk_calc_zmask": [_P, _I, _P, _P, _Z, _Z],
    "dbk_pair_max": [_P, _I, _P, _P, _Z, _Z],
    "dbk_dropout_fp_tr": [_P, _I, _P, _P, _P, _P, _Z, _Z, _Z, _I, _U64, _U64],
    "dbk_dropout_fp_tr_u": [_P, _I, _P, _P, _P, _P, _Z, _Z, _Z, _I, _P],
    "dbk_dropout_fp_te": [_P, _I, _P, _P, _P, _Z, _Z, _Z],
    "dbk_dropout_bp_tr": [_P, _I, _P, _P, _P, _Z],
    "dbk_dropout_bp_te": [_P, _I, _P, _P, _P, _Z, _Z, _Z],
    "dbk_uniform_fill": [_P, _P, _Z, _U64, _U64],
    "dbk_normal_fill": [_P, _I, _P, _Z, _U64, _U64],
    "dbk_philox4x32_10": [_P, _P, _P],
    "dbk_add_rowvec": [_P, _I, _P, _P, _P, _Z, _Z],
    "dbk_colsum": [_P, _I, _P, _P, _Z, _Z],
    "dbk_relu": [_P, _I, _P, _P, _Z],
    "dbk_mul_sign": [_P, _I, _P, _P, _P, _Z],
    "dbk_sign": [_P, _I, _P, _P, _Z],
    "dbk_logistic": [_P, _I, _P, _P, _Z],
    "dbk_loss_terms": [_P, _I, _I, _P, _P, _P, _Z],
    "dbk_sub_scale": [_P, _I, _P, _P, _D, _P, _Z],
    "dbk_hinge_grad": [_P, _I, _P, _P, _D, _P, _Z],
    "dbk_head_train": [_P, _Z, _I, _I, _I, _I, _I, _P, _I, _P, _P, _P, _U64, _U64, _P, _U64, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P],
    "dbk_softmax": [_P, _I, _P, _P, _Z, _Z],
    "dbk_counter_add": [_P, _P, _U64],
    "dbk_l1_decay": [_P, _I, _P, _P, _P, _Z],
    "dbk_head_fprop": [_P, _Z, _I, _I, _I, _P, _I, _P, _P, _P, _P, _P, _P, _I, _P],
    "dbk_train_step": [_P, _P],
    "dbk_train_steps": [_P, _Z, _P],
    "dbk_train_step_single_workspace": [_P, _P],
    "dbk_train_step_single": [_P, _P, _P, _Z],
    "dbk_train_step_args_size": [],
}


class TrainStepArgs(ctypes.Structure):
    """dbk_train_step_args of the public header, field for field."""
    _fields_ = [
        ("nmodel", _Z), ("nfilter", _Z), ("m", _Z), ("hidden", _Z),
        ("ptype", _I), ("loss_kind", _I), ("reverse_complement", _I), ("nesterov", _I),
        ("nparam", _Z),
        ("P", _P), ("dP", _P), ("mP", _P), ("drate", _P), ("mrate", _P),
        ("off_Wc", _Z), ("off_bc", _Z), ("off_W1", _Z), ("off_b1", _Z), ("off_W2", _Z), ("off_b2", _Z),
        ("X", _P), ("N", _Z), ("regions", _P), ("nregion", _Z), ("Y", _P), ("Ymask", _P),
        ("input_rate", _F), ("Xdrop", _P), ("Mdrop", _P),
        ("rate", _P), ("seed", _U64), ("counter", _P),
        ("decay", _P), ("freeze_scan", _I),
        ("pooled", _P), ("argmax", _P), ("Z", _P), ("dpooled", _P), ("loss", _P), ("act", _P),
        ("L", _P), ("L_ready", _I),
        ("nfeat", _Z), ("feats", _P),
    ]

_dll = None


def dll():
    """The loaded shared library; raises if it has not been built."""
    global _dll
    if _dll is None:
        if not os.path.exists(LIB_PATH):
            raise DeepbindError("libdeepbind_hip.so is missing (%s): build it with `python -m deepbind_amd.build`; "
                                "there is no fallback path" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        lib.dbk_last_error.restype = c_char_p
        lib.dbk_last_error.argtypes = []
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = c_int
            fn.argtypes = argtypes
        _dll = lib
    return _dll


def exported_names():
    return ["dbk_last_error"] + sorted(_SIGNATURES)


def call(name, *args):
    """Calls lib.<name>(*args) and raises DeepbindError with the library's message on failure."""
    lib = dll()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        msg = lib.dbk_last_error()
        raise DeepbindError("%s: %s" % (name, msg.decode("utf-8", "replace") if msg else "error %d" % rc))
    return rc


def stream():
    """The current HIP stream of the current device, as the void* the library expects."""
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def ptr(t):
    """Device pointer of a contiguous tensor (None -> NULL)."""
    if t is None:
        return None
    if not t.is_cuda:
        raise DeepbindError("TypeError: expected a device tensor, got a host tensor")
    if not t.is_contiguous():
        raise DeepbindError("ValueError: tensors passed to the library must be contiguous (full stride)")
    return c_void_p(t.data_ptr())


def dtype_code(t):
    if t.dtype == torch.float32:
        return DBK_F32
    if t.dtype == torch.float64:
        return DBK_F64
    raise DeepbindError("TypeError: expected a float32 or float64 tensor, got %s" % t.dtype)


def require(cond, msg):
    if not cond:
        raise DeepbindError(msg)
