"""The C-ABI library loads without a GPU and exports every symbol the public header declares."""
import ctypes
import os
import re

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_functions():
    text = open(os.path.join(ROOT, "include", "deepbind_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dbk_[a-zA-Z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    from deepbind_amd import _lib
    names = _header_functions()
    assert len(names) >= 40
    lib = _lib.dll()
    for name in names:
        assert hasattr(lib, name), "header declares %s but the library does not export it" % name
    # the Python binding covers the header and nothing else
    assert sorted(_lib.exported_names()) == names
    assert lib.dbk_version() == 3
    assert lib.dbk_last_error() == b""


def test_argument_errors_surface_through_last_error():
    from deepbind_amd import _lib
    lib = _lib.dll()
    # nchannel != 4 has no compiled kernel: rejected on the host before anything touches a device
    rc = lib.dbk_corr1ord(None, 0, None, 5, 16, None, 10, 3, None)
    assert rc != 0
    assert b"NotImplementedError" in lib.dbk_last_error()
    rc = lib.dbk_poolrgn(None, 7, None, 4, None, 4, 0, None, None, 0)
    assert rc != 0 and b"TypeError" in lib.dbk_last_error()
    rc = lib.dbk_poolrgn_bprop(None, 0, None, 4, None, 4, 0, None, None, 0)
    assert rc != 0 and b"pooledmaps_argmax must be specified" in lib.dbk_last_error()
    # the 32-bit argmax index cannot address 2^26 rows x 1024 filters: refused before any launch
    one = ctypes.c_void_p(1)
    rc = lib.dbk_scanpool_fprop(None, one, one, 24, 1024, one, 1 << 26, one, 10, 0, one, one, None)
    assert rc != 0 and b"overflow the 32-bit argmax index" in lib.dbk_last_error()
    # empty work succeeds and clears the error text
    assert lib.dbk_corr1ord(None, 0, None, 5, 16, None, 0, 4, None) == 0
    assert lib.dbk_last_error() == b""
    try:
        _lib.call("dbk_blockwise_dot", None, 0, 0, 4, 4, 4, 0, None, None, None)
    except _lib.DeepbindError as e:
        assert "nblock" in str(e)
    else:
        raise AssertionError("expected DeepbindError")


def test_train_step_argument_block_layout_matches_the_header():
    """The ctypes mirror of dbk_train_step_args is read field for field by the library's own checks,
    which run on the host before anything touches a device."""
    from deepbind_amd import _lib
    lib = _lib.dll()
    assert lib.dbk_train_step(None, None) != 0 and b"null argument block" in lib.dbk_last_error()
    assert lib.dbk_train_step_args_size() == ctypes.sizeof(_lib.TrainStepArgs)
    a = _lib.TrainStepArgs()
    a.nmodel, a.nfilter, a.m, a.hidden = 3, 5, 7, 2
    a.ptype, a.loss_kind, a.reverse_complement, a.nesterov = _lib.PT_ALL, 0, 0, 1
    for f in ("P", "dP", "mP", "drate", "mrate", "X", "regions", "Y", "pooled", "Z", "dpooled", "argmax"):
        setattr(a, f, 1)
    a.nparam = 1000
    # blocks: Wc 4*7*15 = 420, bc 15, W1 (10*3)*2 = 60, b1 6, W2 6, b2 3
    a.off_Wc, a.off_bc, a.off_W1, a.off_b1, a.off_W2, a.off_b2 = 0, 420, 435, 495, 501, 998
    assert lib.dbk_train_step(None, ctypes.addressof(a)) != 0
    assert b"reaches past the flat vector (1001 > 1000)" in lib.dbk_last_error()        # off_b2 + nmodel
    a.off_b2, a.off_W1 = 507, 941
    assert lib.dbk_train_step(None, ctypes.addressof(a)) != 0
    assert b"(1001 > 1000)" in lib.dbk_last_error()                                     # off_W1 + k*nmodel*hidden
    a.off_W1, a.ptype = 435, 2
    assert lib.dbk_train_step(None, ctypes.addressof(a)) != 0 and b"max, avg or all pooling" in lib.dbk_last_error()
    a.ptype, a.argmax = _lib.PT_MAX, None
    assert lib.dbk_train_step(None, ctypes.addressof(a)) != 0 and b"argmax work buffer" in lib.dbk_last_error()
    a.argmax, a.input_rate = 1, 0.25
    assert lib.dbk_train_step(None, ctypes.addressof(a)) != 0 and b"Xdrop and Mdrop" in lib.dbk_last_error()
    a.Xdrop, a.Mdrop = 1, 1
    assert lib.dbk_train_step(None, ctypes.addressof(a)) != 0 and b"generator position" in lib.dbk_last_error()
    a.input_rate, a.rate = 0.0, 1
    assert lib.dbk_train_step(None, ctypes.addressof(a)) != 0 and b"generator position" in lib.dbk_last_error()
    a.rate, a.dpooled = None, None
    assert lib.dbk_train_step(None, ctypes.addressof(a)) != 0 and b"null batch or work buffer" in lib.dbk_last_error()
    # the several-groups form checks every block of its list the same way, before any launch
    good = _lib.TrainStepArgs()
    ctypes.memmove(ctypes.addressof(good), ctypes.addressof(a), ctypes.sizeof(a))
    good.dpooled = 1
    blocks = (ctypes.c_void_p * 2)(ctypes.addressof(good), ctypes.addressof(a))
    assert lib.dbk_train_steps(None, 2, blocks) != 0 and b"null batch or work buffer" in lib.dbk_last_error()
    assert lib.dbk_train_steps(None, 2, None) != 0 and b"null argument list" in lib.dbk_last_error()
    blocks[1] = None
    assert lib.dbk_train_steps(None, 2, blocks) != 0 and b"null argument block" in lib.dbk_last_error()
    assert lib.dbk_train_steps(None, 0, None) == 0


def test_philox_known_answers():
    """Published Philox4x32-10 vectors (Random123 kat_vectors)."""
    from deepbind_amd import _lib
    lib = _lib.dll()

    def run(ctr, key):
        c = (ctypes.c_uint32 * 4)(*ctr)
        k = (ctypes.c_uint32 * 2)(*key)
        o = (ctypes.c_uint32 * 4)()
        assert lib.dbk_philox4x32_10(c, k, o) == 0
        return [int(v) for v in o]

    assert run([0, 0, 0, 0], [0, 0]) == [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]
    assert run([0xffffffff] * 4, [0xffffffff] * 2) == [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]
    assert run([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0]) == \
        [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]


def test_host_packing_matches_oracle():
    from deepbind_amd import data
    from oracle import deepbind_oracle as orc
    seqs = ["ACGTNacgu", "G", "", "TTTTGGGGCCCCAAAA.N"]
    for pad in (0, 3, 23):
        X, R = data.pack_sequences(seqs, pad)
        Xo, Ro = orc.pack(seqs, pad)
        assert np.array_equal(X, Xo) and np.array_equal(R, Ro)
    X, R = data.pack_sequences(["ACGTN"], 2, reverse_complement=True)
    assert data.ord2acgt(X.ravel()[2:7]) == "ACGTN" and data.ord2acgt(X.ravel()[9:14]) == "NACGT"
    codes = np.array([[0, 1, 2], [3, 255, 0]], np.uint8)
    Xu, Ru = data.pack_uniform_ordinals(codes, 4)
    Xv, Rv = data.pack_ordinals([codes[0], codes[1]], 4)
    assert np.array_equal(Xu, Xv) and np.array_equal(Ru, Rv)
