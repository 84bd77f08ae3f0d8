"""GPU parity of the single-launch training step (dbk_train_step_single: forward, dense head, backward and the
Nesterov update of a small model group in one kernel) against the CPU oracle's whole step, run-to-run bit
stability, agreement with the multi-launch step, graph replays, and the shapes it hands back to the multi-launch step."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import deepbind_oracle as orc
from tests.gpu_util import assert_close_per_model, assert_no_further_than_f32_reference as assert_vs_f32, dev, host, model_blocks, record_error

pytestmark = pytest.mark.gpu

ACT, GRAD = 1e-5, 1e-4


def _f64(d):
    return {k: np.asarray(v, dtype=np.float64).copy() for k, v in d.items()}


def _batch(rng, B, m, lo, hi, pn=0.03, reverse_complement=False):
    from deepbind_amd import data
    seqs = ["".join("ACGTN"[c] for c in rng.choice(5, size=int(rng.integers(lo, hi + 1)), p=[(1 - pn) / 4] * 4 + [pn])) for _ in range(B)]
    return data.pack_sequences(seqs, m - 1, reverse_complement=reverse_complement)


def _net(rng, nm, nf, m, pool, hidden, loss, scale=0.3, **kw):
    from deepbind_amd.model import SequenceNet
    net = SequenceNet(nm, nf, m, pool=pool, hidden=hidden, loss=loss, **kw)
    params = {name: (rng.standard_normal(shape) * (scale if name.startswith("W") else 0.05)).astype(np.float32) for name, shape, _ in net.layout}
    net.set_params(params)
    return net, params


def _used_single(net):
    return any(buf.get("work") is not None for buf in net._step_bufs.values())


CASES = [
    # pool, hidden, loss, nm, nf, m, B, lengths, rc, nfeat
    ("max", 32, "nll", 1, 16, 24, 128, (101, 101), False, 0),      # config 3's shape
    ("all", 0, "mse", 1, 16, 16, 128, (38, 41), False, 0),         # config 2's shape
    ("avg", 8, "nll", 2, 16, 11, 60, (12, 70), False, 0),
    ("all", 32, "nll", 4, 16, 24, 50, (20, 40), False, 16),
    ("max", 0, "mse", 3, 12, 9, 33, (5, 30), False, 0),            # 36 filters: padded to 64 lanes
    ("all", 16, "nll", 2, 16, 20, 64, (30, 200), True, 0),         # reverse-complement pairs (a pair's rows in neighbouring workgroups), regions up to 219 rows
    ("all", 16, "nll", 2, 16, 20, 150, (30, 120), True, 0),        # reverse-complement pairs, two regions (one pair) per workgroup
    ("max", 32, "nll", 1, 16, 24, 64, (30, 101), True, 0),         # one model, reverse-complement pairs, one region per workgroup
    ("max", 32, "nll", 1, 16, 24, 200, (20, 60), False, 0),        # 200 workgroups
    ("max", 32, "nll", 1, 16, 32, 600, (20, 60), False, 16),       # three regions per workgroup
    # one 16-filter model, one region per workgroup (the instance with that shape compiled in), its other branches:
    ("all", 32, "nll", 1, 16, 24, 100, (20, 90), False, 0),        # 32 pooled features into a hidden layer (two lane groups per feature)
    ("avg", 20, "mse", 1, 12, 32, 77, (8, 50), False, 16),         # 12 filters in 16 lanes, 32 taps, shared feature columns, a hidden width the lane groups do not divide
    ("max", 64, "nll", 1, 16, 8, 128, (30, 60), False, 0),         # 64 hidden units
]


@pytest.mark.parametrize("pool,hidden,loss,nm,nf,m,B,lengths,rc,nfeat", CASES)
def test_single_launch_step_matches_the_oracle(pool, hidden, loss, nm, nf, m, B, lengths, rc, nfeat):
    from deepbind_amd import deepity_smat as ds
    rng = np.random.default_rng(17)
    X, R = _batch(rng, B, m, lengths[0], lengths[1], reverse_complement=rc)
    rows = len(R)
    rate, mu = rng.uniform(0.01, 0.1, nm), rng.uniform(0.5, 0.95, nm)
    drop = np.where(np.arange(nm) % 2 == 0, 0.5, 0.0) if nm > 1 else np.array([0.5])
    dfull, dconv = rng.uniform(0, 1e-2, nm), 1e-3
    net, params = _net(rng, nm, nf, m, pool, hidden, loss, rate=rate, momentum=mu, dropout=drop, decay_conv=dconv, decay_full=dfull,
                       weight_decay_start=1, reverse_complement=rc, feature_columns=nfeat, start_training=1)
    Y = rng.random((rows, nm)).astype(np.float32) if loss == "mse" else (rng.random((rows, nm)) < 0.5).astype(np.float32)
    Ymask = rng.random((rows, nm)) < 0.85
    F = rng.standard_normal((rows, nfeat)).astype(np.float32) if nfeat else None
    Xd, Rd, Yd, Md, Fd = dev(X), dev(R), dev(Y), dev(Ymask), (dev(F) if nfeat else None)
    ref_p, ref_m = _f64(params), {n: np.zeros(v.shape) for n, v in params.items()}
    f32_p, f32_m = {n: v.copy() for n, v in params.items()}, {n: np.zeros(v.shape, np.float32) for n, v in params.items()}
    name = "single launch (%s/%d, %d x %d filters x %d taps)" % (pool, hidden, nm, nf, m)
    f32 = lambda v: np.asarray(v, dtype=np.float32)
    blocks = lambda a, axis: model_blocks(a, nm, axis)
    for step in range(3):
        U = host(ds.uniform_like(torch.empty((rows // (2 if rc else 1), net.k * nm), device="cuda"), net.rng_seed, net._rng_offset))
        if rc:
            U = np.repeat(U, 2, axis=0)                            # a (fwd, rev) pair shares its draw
        net.train_step(Xd, Rd, Yd, Md, F=Fd)
        st, g = orc.train_step(ref_p, ref_m, X, R, Y.astype(np.float64), nm, pool, hidden, loss, rate, mu, Ymask=Ymask, dropout=(drop, U),
                               decay_conv=dconv, decay_full=dfull, step=step, weight_decay_start=1, reverse_complement=rc, start_training=1,
                               features=None if F is None else F.astype(np.float64))
        st32, g32 = orc.train_step(f32_p, f32_m, X, R, Y, nm, pool, hidden, loss, f32(rate), f32(mu), Ymask=Ymask, dropout=(f32(drop), U),
                                   decay_conv=dconv, decay_full=f32(dfull), step=step, weight_decay_start=1, reverse_complement=rc,
                                   start_training=1, features=F)
        got = net.get_grads()
        for pname, _, axis in net.layout:
            assert_close_per_model(got[pname], g[pname], GRAD, nm, axis, "step %d gradient %s" % (step, pname))
            record_error(name, "gradients", got[pname], g[pname], GRAD)
            for b, (a64, a32, ag) in enumerate(zip(blocks(g[pname], axis), blocks(g32[pname], axis), blocks(got[pname], axis))):
                assert_vs_f32(name, "gradients", ag, a64, a32, "step %d gradient %s [model %d]" % (step, pname, b))
        Z = host(net._step_bufs[(Xd.numel(), rows)]["Z"])
        assert_close_per_model(Z, st["Zout"], ACT, nm, 1, "step %d predictions" % step)
        record_error(name, "activations", Z, st["Zout"], ACT)
        for b in range(nm):
            assert_vs_f32(name, "activations", Z[:, b], st["Zout"][:, b], st32["Zout"][:, b], "step %d predictions [model %d]" % (step, b))
    assert _used_single(net), "the step did not go through the single-launch kernel"
    got = net.get_params()
    for pname, _, axis in net.layout:
        assert_close_per_model(got[pname], ref_p[pname], GRAD, nm, axis, "parameters %s" % pname)
        record_error(name, "parameters", got[pname], ref_p[pname], GRAD)
        for b, (a64, a32, ag) in enumerate(zip(blocks(ref_p[pname], axis), blocks(f32_p[pname], axis), blocks(got[pname], axis))):
            assert_vs_f32(name, "parameters", ag, a64, a32, "parameters %s [model %d]" % (pname, b))


@pytest.mark.parametrize("pool,hidden,loss", [("max", 32, "nll"), ("all", 0, "mse")])
def test_single_launch_step_is_bit_stable_and_agrees_with_the_multi_launch_step(pool, hidden, loss):
    rng = np.random.default_rng(5)
    m, B = 24, 128
    X, R = _batch(rng, B, m, 30, 101)
    Y = rng.random((B, 2)).astype(np.float32)
    Xd, Rd, Yd = dev(X), dev(R), dev(Y)
    outs = []
    for single in (True, True, False):
        r2 = np.random.default_rng(6)
        net, _ = _net(r2, 2, 16, m, pool, hidden, loss, rate=0.05, momentum=0.9, dropout=0.4, decay_full=1e-3, weight_decay_start=0,
                      single_launch=single)
        losses = []
        for _ in range(4):
            net.train_step(Xd, Rd, Yd)
        assert _used_single(net) == single
        outs.append(net.get_params())
    for pname in outs[0]:
        assert np.array_equal(outs[0][pname], outs[1][pname]), "run-to-run difference in %s" % pname
        assert_close_per_model(outs[0][pname], outs[2][pname], GRAD, 1, 0, "single vs multi launch %s" % pname)


def test_single_launch_step_in_a_graph_and_loss_output():
    rng = np.random.default_rng(8)
    m, B = 16, 128
    X, R = _batch(rng, B, m, 38, 41)
    Y = rng.standard_normal((B, 1)).astype(np.float32)
    Xd, Rd, Yd = dev(X), dev(R), dev(Y)
    nets = []
    for _ in range(2):
        r2 = np.random.default_rng(9)
        nets.append(_net(r2, 1, 16, m, "all", 0, "mse", rate=0.02, momentum=0.9, dropout=0.25)[0])
    eager, graphed = nets
    step = graphed.make_graphed_step(Xd, Rd, Yd, force_graph=True)
    for i in range(4):
        eager.train_step(Xd, Rd, Yd)
        step()
        torch.cuda.synchronize()
        a, b = eager.get_params(), graphed.get_params()
        for pname in a:
            assert np.array_equal(a[pname], b[pname]), "replay %d differs from the eager step in %s" % (i, pname)
    assert _used_single(eager) and _used_single(graphed)
    assert eager.step_count == graphed.step_count == 4 and eager._rng_offset == graphed._rng_offset
    # without force_graph such a net gets its one launch issued directly (a graph of one node replays slower)
    direct = graphed.make_graphed_step(Xd, Rd, Yd)
    eager.train_step(Xd, Rd, Yd)
    direct()
    a, b = eager.get_params(), graphed.get_params()
    for pname in a:
        assert np.array_equal(a[pname], b[pname])
    assert graphed.step_count == 5


def test_shapes_the_single_launch_step_does_not_take_fall_back():
    """A region longer than 256 rows, or more than four models: the multi-launch step runs (same bits as with the
    single-launch step switched off); calling the entry point directly on an unsupported shape is refused."""
    from deepbind_amd import _lib
    rng = np.random.default_rng(10)
    m = 12
    X, R = _batch(rng, 16, m, 280, 300)
    Y = rng.random((16, 1)).astype(np.float32)
    outs = []
    for single in (True, False):
        net, _ = _net(np.random.default_rng(11), 1, 16, m, "max", 8, "nll", rate=0.05, single_launch=single)
        net.train_step(dev(X), dev(R), dev(Y))
        assert not _used_single(net) or single
        outs.append(net.get_params())
    for pname in outs[0]:
        assert np.array_equal(outs[0][pname], outs[1][pname])
    X, R = _batch(rng, 16, m, 20, 30)
    net, _ = _net(np.random.default_rng(12), 6, 16, m, "max", 8, "nll", rate=0.05)
    net.train_step(dev(X), dev(R), dev(rng.random((16, 6)).astype(np.float32)))
    assert not _used_single(net)
    work = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    with pytest.raises(_lib.DeepbindError, match="NotImplementedError"):
        _lib.call("dbk_train_step_single", _lib.stream(), ctypes.addressof(net._step_args), _lib.ptr(work), work.numel())


def test_region_longer_than_the_kernel_takes_is_flagged_and_leaves_the_parameters_alone():
    """The kernel's own guard (the Python side normally never lets such a batch through)."""
    from deepbind_amd import _lib
    rng = np.random.default_rng(13)
    m = 12
    X, R = _batch(rng, 16, m, 280, 300)
    net, _ = _net(np.random.default_rng(14), 1, 16, m, "max", 8, "nll", rate=0.05)
    before = net.get_params()
    Xd, Rd, Yd = dev(X), dev(R), dev(rng.random((16, 1)).astype(np.float32))
    buf = net._prepare_step(Xd, Rd, Yd)
    need = ctypes.c_size_t(0)
    _lib.call("dbk_train_step_single_workspace", ctypes.addressof(net._step_args), ctypes.addressof(need))
    assert need.value > 0
    buf["work"] = torch.zeros(need.value, dtype=torch.uint8, device="cuda")
    _lib.call("dbk_train_step_single", _lib.stream(), ctypes.addressof(net._step_args), _lib.ptr(buf["work"]), need.value)
    torch.cuda.synchronize()
    assert int(buf["work"][4:8].view(torch.int32).item()) == 2
    with pytest.raises(_lib.DeepbindError, match="256 rows"):
        net.get_params()
    after = net.get_params()
    for pname in before:
        assert np.array_equal(before[pname], after[pname])


def test_abandoned_steps_change_nothing_and_training_resumes_after_the_reset():
    """A launch that the kernel's own guard abandons (a region of more than 256 rows, let through by switching the host's
    check off), and the launch after it on the flagged workspace, leave parameters, momentum and generator position
    alone; the host notices, sets its step counter and generator mirror back, re-arms the workspace, and the next step
    gives the bits of a net that only ever saw the valid steps."""
    from deepbind_amd import _lib, data
    rng = np.random.default_rng(21)
    m, nreg = 12, 16
    letters = lambda n: "".join("ACGT"[c] for c in rng.integers(0, 4, size=n))
    good = [letters(102 + (i & 1)) for i in range(nreg)]                       # 16 regions, 1640 letters
    bad = [letters(290)] + [letters(90) for _ in range(nreg - 1)]              # the same number of regions and letters, one region too long
    Xg, Rg = data.pack_sequences(good, m - 1)
    Xb, Rb = data.pack_sequences(bad, m - 1)
    assert Xg.size == Xb.size and len(Rg) == len(Rb)
    Y = (rng.random((nreg, 1)) < 0.5).astype(np.float32)
    Xgd, Rgd, Xbd, Rbd, Yd = dev(Xg), dev(Rg), dev(Xb), dev(Rb), dev(Y)
    nets = [_net(np.random.default_rng(22), 1, 16, m, "all", 8, "nll", rate=0.05, momentum=0.9, dropout=0.5)[0] for _ in range(2)]
    net, fresh = nets
    for _ in range(2):
        net.train_step(Xgd, Rgd, Yd)
        fresh.train_step(Xgd, Rgd, Yd)
    assert _used_single(net)
    before, count, offset = net.get_params(), net.step_count, net._rng_offset
    momentum = host(net.mP).copy()
    host_check = net._single_work
    net._single_work = lambda buf, R: buf["work"]                               # (the host's look at the region lengths, switched off)
    net.train_step(Xbd, Rbd, Yd)                                                # abandoned by the kernel: status 2
    net.train_step(Xgd, Rgd, Yd)                                                # a valid batch on the flagged workspace: nothing happens
    net._single_work = host_check
    with pytest.raises(_lib.DeepbindError, match="256 rows.*2 step"):
        net.get_params()
    assert net.step_count == count and net._rng_offset == offset == int(net.rng_counter.item())
    after = net.get_params()                                                    # (the status is cleared: no second raise)
    for pname in before:
        assert np.array_equal(before[pname], after[pname]), pname
    assert np.array_equal(momentum, host(net.mP))
    net.train_step(Xgd, Rgd, Yd)
    fresh.train_step(Xgd, Rgd, Yd)
    a, b = net.get_params(), fresh.get_params()
    for pname in a:
        assert np.array_equal(a[pname], b[pname]), "after the reset %s differs from a net that never saw the abandoned steps" % pname
    assert net.step_count == fresh.step_count == 3


def test_region_table_cache_follows_the_tensor_not_its_address():
    """A new region table at the address of an earlier one, with the same version count and row count (what a training
    loop sees when the caching allocator hands a freed block to the next batch's table) is looked at again: its long
    region sends the step to the multi-launch kernels instead of being dropped by the single-launch kernel's guard."""
    from deepbind_amd import data
    rng = np.random.default_rng(23)
    m, nreg = 12, 16
    letters = lambda n: "".join("ACGT"[c] for c in rng.integers(0, 4, size=n))
    Xs, Rs = data.pack_sequences([letters(60) for _ in range(nreg)], m - 1)
    Xl, Rl = data.pack_sequences([letters(300)] + [letters(44) for _ in range(nreg - 1)], m - 1)
    assert Xs.size == Xl.size
    Y = dev((rng.random((nreg, 1)) < 0.5).astype(np.float32))
    net, _ = _net(np.random.default_rng(24), 1, 16, m, "max", 8, "nll", rate=0.05)
    ref, _ = _net(np.random.default_rng(24), 1, 16, m, "max", 8, "nll", rate=0.05, single_launch=False)
    Xd, R1 = dev(Xs), dev(Rs)
    net.train_step(Xd, R1, Y)
    ref.train_step(Xd, dev(Rs), Y)
    assert _used_single(net)
    torch.cuda.synchronize()
    R1.data.copy_(dev(Rl))                   # the next batch's table lands in the same memory ...
    R2 = R1.data                             # ... as a tensor object of its own, version count 0 like the first
    assert R2 is not R1 and R2.data_ptr() == R1.data_ptr() and R2._version == R1._version and R2.shape == R1.shape
    Xd2 = dev(Xl)
    net.train_step(Xd2, R2, Y)
    ref.train_step(Xd2, dev(Rl), Y)
    a, b = net.get_params(), ref.get_params()                                   # (raises if the kernel had to abandon the step)
    assert net.step_count == 2
    for pname in a:
        assert np.abs(a[pname] - b[pname]).max() <= GRAD * np.abs(b[pname]).max(), pname
