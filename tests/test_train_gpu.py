"""GPU parity of whole training steps (forward + backward + Nesterov update) on the benchmark's
training configurations against the float64 CPU oracle, in both execution modes, plus bit-stability."""
import numpy as np
import pytest
import torch

from oracle import deepbind_oracle as orc
from tests.gpu_util import (assert_close, assert_close_per_model, assert_no_further_than_f32_reference as assert_vs_f32, dev, host,
                            model_blocks, record_argmax, record_error)

pytestmark = pytest.mark.gpu

ACT, GRAD = 1e-5, 1e-4


def _f64(d):
    return {k: np.asarray(v, dtype=np.float64).copy() for k, v in d.items()}


def _run_config(cfg, mode, nsteps, dropout_rate=0.0, decay=(0.0, 0.0), weight_decay_start=100, bias_jitter=0.01, name=None):
    from deepbind_amd.model import SequenceNet
    spec = cfg["spec"]
    rng = np.random.default_rng(99)
    params = {k: v.copy() for k, v in cfg["params"].items()}
    for k in params:                                   # non-zero biases so every gradient path is exercised
        if k.startswith("b"):
            params[k] = (rng.standard_normal(params[k].shape) * bias_jitter).astype(np.float32)
    net = SequenceNet(spec.nmodel, spec.nfilter, spec.m, pool=spec.pool[0], hidden=spec.hidden[0], loss=spec.loss,
                      rate=cfg.get("rate", 0.01), momentum=cfg.get("momentum", 0.9), dropout=dropout_rate,
                      decay_conv=decay[0], decay_full=decay[1], weight_decay_start=weight_decay_start, mode=mode)
    net.set_params(params)
    X, R, Y = dev(cfg["X"]), dev(cfg["R"]), dev(cfg["Y"])
    U = cfg.get("U")
    Ud = dev(U) if (U is not None and dropout_rate > 0) else None
    ref_p, ref_m = _f64(params), {k: np.zeros(v.shape) for k, v in params.items()}
    # the same trajectory once more with every array in float32: the reference's own arithmetic, in its own order
    f32_p, f32_m = {k: v.copy() for k, v in params.items()}, {k: np.zeros(v.shape, np.float32) for k, v in params.items()}
    drop = (np.full(spec.nmodel, dropout_rate), U) if dropout_rate > 0 else None
    drop32 = (np.full(spec.nmodel, dropout_rate, np.float32), U) if dropout_rate > 0 else None
    kw = dict(decay_conv=decay[0], decay_full=decay[1], weight_decay_start=weight_decay_start)
    for step in range(nsteps):
        net.train_step(X, R, Y, U=Ud)
        st, g = orc.train_step(ref_p, ref_m, cfg["X"], cfg["R"], cfg["Y"].astype(np.float64), spec.nmodel, spec.pool[0],
                               spec.hidden[0], spec.loss, cfg.get("rate", 0.01), cfg.get("momentum", 0.9), dropout=drop, step=step, **kw)
        _, g32 = orc.train_step(f32_p, f32_m, cfg["X"], cfg["R"], cfg["Y"].astype(np.float32), spec.nmodel, spec.pool[0],
                                spec.hidden[0], spec.loss, cfg.get("rate", 0.01), cfg.get("momentum", 0.9), dropout=drop32, step=step, **kw)
        got_g = net.get_grads()
        for k in g:
            assert_close(got_g[k], g[k], GRAD, "step %d grad %s (%s)" % (step, k, mode))
            if name:
                record_error(name, "gradients", got_g[k], g[k], GRAD)
                assert_vs_f32(name, "gradients", got_g[k], g[k], g32[k], "step %d grad %s (%s)" % (step, k, mode))
    got = net.get_params()
    for k in ref_p:
        assert_close(got[k], ref_p[k], GRAD, "params %s after %d steps (%s)" % (k, nsteps, mode))
        if name:
            record_error(name, "parameters", got[k], ref_p[k], GRAD)
            assert_vs_f32(name, "parameters", got[k], ref_p[k], f32_p[k], "params %s after %d steps (%s)" % (k, nsteps, mode))
    if name:
        # forward pass at the parameters the DEVICE ended with, so that nothing but the forward arithmetic differs
        out = "logistic" if spec.loss == "nll" else "linear"
        st = orc.model_forward(_f64(got), cfg["X"], cfg["R"], spec.nmodel, spec.pool[0], spec.hidden[0], out=out)
        st32 = orc.model_forward(got, cfg["X"], cfg["R"], spec.nmodel, spec.pool[0], spec.hidden[0], out=out)
        net.use_dropout, keep = False, net.use_dropout
        Zd, fw = host(net.predict(X, R)), net.forward(X, R, want_argmax=True)
        for what, a, b, b32 in (("predictions", Zd, st["Zout"], st32["Zout"]), ("pooled", host(fw["pooled"]), st["Pl"], st32["Pl"])):
            assert_close(a, b, ACT, "%s at the final parameters (%s)" % (what, mode))
            record_error(name, "activations", a, b, ACT)
            assert_vs_f32(name, "activations", a, b, b32, "%s at the final parameters (%s)" % (what, mode))
        if fw["argmax"] is not None:
            record_argmax(name, host(fw["argmax"]), st32["I"])
        net.use_dropout = keep
    return net, got


@pytest.mark.parametrize("mode", ["fused", "unfused"])
def test_config2_rna_regression_train_steps(mode):
    from deepbind_amd import synth
    _run_config(synth.config2(), mode, nsteps=3, name="config2 (%s)" % mode)


@pytest.mark.parametrize("mode", ["fused", "unfused"])
def test_config3_classification_train_steps_with_dropout_and_decay(mode):
    from deepbind_amd import synth
    cfg = synth.config3()
    _run_config(cfg, mode, nsteps=3, dropout_rate=0.5, decay=(1e-4, 1e-3), weight_decay_start=1, name="config3 (%s)" % mode)


def test_train_step_is_bit_stable_and_modes_agree():
    from deepbind_amd import synth
    cfg = synth.config3()
    _, a = _run_config(cfg, "fused", nsteps=2, dropout_rate=0.5)
    _, b = _run_config(cfg, "fused", nsteps=2, dropout_rate=0.5)
    for k in a:
        assert np.array_equal(a[k], b[k]), "run-to-run difference in %s" % k
    _, c = _run_config(cfg, "unfused", nsteps=2, dropout_rate=0.5)
    for k in a:
        assert_close(a[k], c[k], GRAD, "fused vs unfused %s" % k)


def test_config1_forward_scores():
    from deepbind_amd import synth
    from deepbind_amd.model import SequenceNet
    cfg = synth.config1()
    spec = cfg["spec"]
    net = SequenceNet(1, spec.nfilter, spec.m, pool="max", hidden=32, loss=None)
    net.set_params(cfg["params"])
    st = orc.model_forward(_f64(cfg["params"]), cfg["X"], cfg["R"], 1, "max", 32)
    st32 = orc.model_forward(cfg["params"], cfg["X"], cfg["R"], 1, "max", 32)
    got = host(net.predict(dev(cfg["X"]), dev(cfg["R"])))
    assert got.shape == (64, 1)
    assert_close(got, st["A"], ACT, "config 1 scores")
    record_error("config1", "activations", got, st["A"], ACT)
    assert_vs_f32("config1", "activations", got, st["A"], st32["A"], "config 1 scores")
    fw = net.forward(dev(cfg["X"]), dev(cfg["R"]), want_argmax=True)
    assert_vs_f32("config1", "activations", host(fw["pooled"]), st["Pl"], st32["Pl"], "config 1 pooled features")
    assert record_argmax("config1", host(fw["argmax"]), st32["I"]) == 0        # taps added in the reference's order: its bits
    assert_close(host(net.forward(dev(cfg["X"]), dev(cfg["R"]))["Z"]), st["A"], ACT, "config 1 scores (layer by layer)")


def test_config4_calibration_batch_mixed_architectures():
    """90 models (30 hyper-parameter draws x 3 folds), pool and hidden size chosen per model, shared batch,
    stepped through the shared launches (one native call for all architecture groups) with every model's own
    drawn dropout rate. The oracle gets the uniforms the library's generator draws at each group's stream
    position. Every model is compared on its OWN block of every array, with that block's own scale: the
    models' initial scales span four orders of magnitude."""
    from deepbind_amd import synth
    from deepbind_amd import deepity_smat as ds
    from deepbind_amd.model import ModelGroup
    cfg = synth.config4()
    spec, hp = cfg["spec"], cfg["hp"]
    assert (hp["dropout"] > 0).sum() >= 20 and (hp["dropout"] == 0).sum() >= 20
    grp = ModelGroup(spec.pool, spec.hidden, spec.nfilter, spec.m, loss="nll", rate=hp["rate"], momentum=hp["momentum"],
                     decay_conv=hp["decay_conv"], decay_full=hp["decay_full"], dropout=hp["dropout"], weight_decay_start=1)
    assert len(grp.groups) <= 4 and sum(len(i) for i, _ in grp.groups) == 90
    init, ref, mom, ref32, mom32 = [], [], [], [], []
    for gi, (idx, net) in enumerate(grp.groups):
        net.rng_seed = 40 + gi
        stacked = {name: np.concatenate([cfg["models"][j][name] for j in idx], axis=axis) for name, _, axis in net.layout}
        net.set_params(stacked)
        init.append(stacked)
        ref.append(_f64(stacked))
        mom.append({k: np.zeros(v.shape) for k, v in stacked.items()})
        ref32.append({k: v.copy() for k, v in stacked.items()})                 # the same trajectory in float32, reference order
        mom32.append({k: np.zeros(v.shape, np.float32) for k, v in stacked.items()})
    CFG = "config4 (shared launches)"
    X, R, Y, M = dev(cfg["X"]), dev(cfg["R"]), dev(cfg["Y"]), dev(cfg["Ymask"])
    nsteps = 3
    for step in range(nsteps):
        # the uniforms each group's head will draw in this step: its generator at (seed, position)
        Us = [host(ds.uniform_like(torch.empty((R.shape[0], net.k * net.ninst), device="cuda"), net.rng_seed, net._rng_offset))
              if net.use_dropout else None for _, net in grp.groups]
        grp.train_step(X, R, Y, M)
        # the oracle steps each architecture group with the same model-axis layout (the reference's scan-filter
        # decay indexing depends on the number of models sharing a graph, so the grouping is part of the semantics)
        for gi, (idx, net) in enumerate(grp.groups):
            drop = (hp["dropout"][idx].astype(np.float64), Us[gi]) if net.use_dropout else None
            drop32 = (hp["dropout"][idx], Us[gi]) if net.use_dropout else None
            kw = dict(Ymask=cfg["Ymask"][:, idx], decay_conv=hp["decay_conv"][idx], decay_full=hp["decay_full"][idx], step=step,
                      weight_decay_start=1)
            _, g = orc.train_step(ref[gi], mom[gi], cfg["X"], cfg["R"], cfg["Y"][:, idx].astype(np.float64), len(idx), net.pool,
                                  net.hidden, "nll", hp["rate"][idx], hp["momentum"][idx], dropout=drop, **kw)
            st32, g32 = orc.train_step(ref32[gi], mom32[gi], cfg["X"], cfg["R"], cfg["Y"][:, idx], len(idx), net.pool,
                                       net.hidden, "nll", hp["rate"][idx], hp["momentum"][idx], dropout=drop32, **kw)
            if step == 0:
                # the pooling winners of the step's own forward launch (at the initial parameters: no momentum yet)
                record_argmax(CFG, host(net._step_buf["argmax"]), st32["I"])
            got_g = net.get_grads()
            for name, _, axis in net.layout:
                what = "step %d %s/%d gradient %s" % (step, net.pool, net.hidden, name)
                assert_close_per_model(got_g[name], g[name], GRAD, len(idx), axis, what)
                for b_, (a, b, b32) in enumerate(zip(model_blocks(got_g[name], len(idx), axis), model_blocks(g[name], len(idx), axis),
                                                     model_blocks(g32[name], len(idx), axis))):
                    record_error(CFG, "gradients", a, b, GRAD)
                    assert_vs_f32(CFG, "gradients", a, b, b32, "%s [model %d]" % (what, b_))
    nmoved = 0
    for gi, (idx, net) in enumerate(grp.groups):
        got = net.get_params()
        for name, _, axis in net.layout:
            assert_close_per_model(got[name], ref[gi][name], GRAD, len(idx), axis, "%s/%d parameters %s" % (net.pool, net.hidden, name))
            for b_, (a, b, b32) in enumerate(zip(model_blocks(got[name], len(idx), axis), model_blocks(ref[gi][name], len(idx), axis),
                                                 model_blocks(ref32[gi][name], len(idx), axis))):
                record_error(CFG, "parameters", a, b, GRAD)
                assert_vs_f32(CFG, "parameters", a, b, b32, "%s/%d parameters %s [model %d]" % (net.pool, net.hidden, name, b_))
        # every model trained: its filters changed by what the reference's update changes them by (compared as
        # CHANGES, so a model whose filters were left alone, or stepped with a neighbour's rate, fails even
        # when the change is far below the weights' own size); float32 storage rounds each of the steps
        for b, (w0, w1, wr) in enumerate(zip(model_blocks(init[gi]["Wc"], len(idx), 1), model_blocks(got["Wc"], len(idx), 1),
                                             model_blocks(ref[gi]["Wc"], len(idx), 1))):
            d_ref, d_got = wr - w0, w1.astype(np.float64) - w0
            slack = (nsteps + 1) * np.spacing(np.abs(w0)).astype(np.float64)
            bad = np.abs(d_got - d_ref) > 2e-2 * np.abs(d_ref).max() + slack
            assert not bad.any(), "model %d of group %d: filter update differs from the reference's" % (b, gi)
            if np.abs(d_ref).max() > 100 * np.spacing(np.float32(np.abs(w0).max())):     # a change float32 can hold
                assert (w1 != w0).mean() > 0.5, "model %d of group %d: filters did not move" % (b, gi)
                nmoved += 1
    assert nmoved >= 80, nmoved
    scores = host(grp.predict(X, R))
    assert scores.shape == (256, 90) and np.isfinite(scores).all() and scores.min() >= 0 and scores.max() <= 1
    col = 0
    for gi, (idx, net) in enumerate(grp.groups):
        st = orc.model_forward(ref[gi], cfg["X"], cfg["R"], len(idx), net.pool, net.hidden, out="logistic",
                               dropout=(hp["dropout"][idx].astype(np.float64), None) if net.use_dropout else None, train=False)
        assert_close(scores[:, idx], st["Zout"], 1e-4, "scores of group %d" % gi)
        record_error(CFG, "activations", scores[:, idx], st["Zout"], ACT)
        # the forward arithmetic alone: float64 and float32 evaluations at the parameters the device ended with
        got = net.get_params()
        dr = lambda t: (hp["dropout"][idx].astype(t), None) if net.use_dropout else None
        s64 = orc.model_forward(_f64(got), cfg["X"], cfg["R"], len(idx), net.pool, net.hidden, out="logistic", dropout=dr(np.float64), train=False)
        s32 = orc.model_forward(got, cfg["X"], cfg["R"], len(idx), net.pool, net.hidden, out="logistic", dropout=dr(np.float32), train=False)
        for b_ in range(len(idx)):
            assert_vs_f32(CFG, "activations", scores[:, idx[b_]], s64["Zout"][:, b_], s32["Zout"][:, b_], "scores of model %d of group %d" % (b_, gi))


def test_reverse_complement_mode_train_and_predict():
    """Interleaved fwd/rev rows: shared dropout draw per pair, only the larger prediction of a pair
    trains, and prediction keeps the pair maximum."""
    from deepbind_amd import data
    from deepbind_amd.model import SequenceNet
    rng = np.random.default_rng(5)
    nm, nf, m, hid, B = 2, 16, 11, 8, 24
    seqs = ["".join(rng.choice(list("ACGTN"), p=[.24, .24, .24, .24, .04], size=int(rng.integers(15, 40)))) for _ in range(B)]
    X, R = data.pack_sequences(seqs, m - 1, reverse_complement=True)
    assert len(R) == 2 * B
    p = {"Wc": rng.standard_normal((4 * m, nf * nm)) * 0.2, "bc": rng.standard_normal((1, nf * nm)) * 0.05,
         "W1": rng.standard_normal((nf * nm, hid)) * 0.3, "b1": rng.standard_normal((1, hid * nm)) * 0.1,
         "W2": rng.standard_normal((hid * nm, 1)) * 0.5, "b2": rng.standard_normal((1, nm)) * 0.1}
    p = {k: v.astype(np.float32) for k, v in p.items()}
    Y = np.repeat((rng.random((B, nm)) < 0.5).astype(np.float32), 2, axis=0)
    U = rng.random((2 * B, nf * nm)).astype(np.float32)
    rate = np.array([0.25, 0.5])
    net = SequenceNet(nm, nf, m, pool="max", hidden=hid, loss="nll", rate=0.05, momentum=0.9, dropout=rate,
                      reverse_complement=True)
    net.set_params(p)
    q = _f64(p); mom = {k: np.zeros(v.shape) for k, v in q.items()}
    Xd, Rd, Yd, Ud = dev(X), dev(R), dev(Y), dev(U)
    for step in range(2):
        net.train_step(Xd, Rd, Yd, U=Ud)
        orc.train_step(q, mom, X, R, Y.astype(np.float64), nm, "max", hid, "nll", 0.05, 0.9, dropout=(rate, U), step=step,
                       reverse_complement=True)
    got = net.get_params()
    for k in q:
        assert_close(got[k], q[k], GRAD, "revcomp params %s" % k)
    st = orc.model_forward(q, X, R, nm, "max", hid, out="logistic", dropout=(rate, None), train=False)
    ref = np.maximum(st["Zout"][0::2], st["Zout"][1::2])
    pred = host(net.predict(Xd, Rd))
    assert pred.shape == (B, nm)
    assert_close(pred, ref, 1e-4, "revcomp predictions")


def test_fused_and_layerwise_steps_draw_the_same_dropout_masks():
    """With no uniforms supplied both modes draw from the library's generator at the same stream
    position, so three steps with dropout end in the same parameters."""
    from deepbind_amd import synth
    from deepbind_amd.model import SequenceNet
    cfg = synth.config3()
    spec = cfg["spec"]
    out = {}
    for mode in ("fused", "unfused"):
        net = SequenceNet(1, spec.nfilter, spec.m, pool="max", hidden=32, loss="nll", rate=0.05, momentum=0.9, dropout=0.5, mode=mode)
        net.rng_seed = 77
        params = {k: v.copy() for k, v in cfg["params"].items()}
        jit = np.random.default_rng(1)
        for k in params:                                 # non-zero biases: a sum that cancels to ~0 has no scale to compare against
            if k.startswith("b"):
                params[k] = (jit.standard_normal(params[k].shape) * 0.01).astype(np.float32)
        net.set_params(params)
        X, R, Y = dev(cfg["X"]), dev(cfg["R"]), dev(cfg["Y"])
        for _ in range(3):
            net.train_step(X, R, Y)
        out[mode] = net.get_params()
        assert int(net.rng_counter.item()) == net._rng_offset == 3 * ((128 * 16 + 3) // 4)
    for k in out["fused"]:
        assert_close(out["fused"][k], out["unfused"][k], GRAD, "fused vs layer-by-layer %s" % k)


def test_head_train_loss_output():
    from deepbind_amd import deepity_smat as ds
    rng = np.random.default_rng(3)
    n, nb, k, h = 300, 5, 16, 32
    Pl = np.abs(rng.standard_normal((n, k * nb))).astype(np.float32)
    W1 = (rng.standard_normal((k * nb, h)) * 0.3).astype(np.float32); b1 = (rng.standard_normal((1, h * nb)) * 0.1).astype(np.float32)
    W2 = (rng.standard_normal((h * nb, 1)) * 0.3).astype(np.float32); b2 = (rng.standard_normal((1, nb)) * 0.1).astype(np.float32)
    Y = (rng.random((n, nb)) < 0.5).astype(np.float32)
    M = rng.random((n, nb)) < 0.8
    g = [torch.empty_like(dev(a)) for a in (W1, b1, W2, b2)]
    Z, dP, L = ds.head_train(dev(Pl), dev(W1), dev(b1), dev(W2), dev(b2), dev(Y), nb, "nll", g[0], g[1], g[2], g[3],
                             Ymask=dev(M), want_loss=True)
    H = orc.relu_fprop(orc.bias_fprop(orc.blockwise_dot(Pl.astype(np.float64), W1.astype(np.float64), nb), b1))
    A = orc.bias_fprop(orc.blockwise_dot(H, W2.astype(np.float64), nb), b2)
    Zr = orc.logistic(A)
    assert_close(host(Z), Zr, ACT, "Z")
    assert_close(host(L), orc.loss_fprop(Zr, Y.astype(np.float64), "nll", nb, Ymask=M), 1e-4, "loss")
    dA = orc.loss_bprop(Zr, Y.astype(np.float64), Ymask=M)
    assert_close(host(g[3]), orc.bias_bprop(dA)[1], GRAD, "db2")
    assert_close(host(g[2]), orc.blockwise_dot_tn(H, dA, nb, W2), GRAD, "dW2")
    dA1 = orc.relu_bprop(orc.blockwise_dot_nt(dA, W2.astype(np.float64), nb), H)
    assert_close(host(g[0]), orc.blockwise_dot_tn(Pl.astype(np.float64), dA1, nb, W1), GRAD, "dW1")
    assert_close(host(dP), orc.blockwise_dot_nt(dA1, W1.astype(np.float64), nb), GRAD, "dpooled")


@pytest.mark.parametrize("k,nfeat,loss,rc", [(16, 0, "nll", False), (32, 0, "nll", True), (16, 16, "mse", False), (32, 0, "hinge", False),
                                             (12, 4, "nll", True)])
def test_head_train_register_body_gives_the_bits_of_the_general_body(k, nfeat, loss, rc):
    """Heads of 32 hidden units on 16 or 32 inputs run with the weights in registers (head_train.hip, head_train_h32);
    with uniforms supplied the call takes the general body. Same uniforms -> every output bit for bit the same:
    the register body forms each sum in the general body's order. 333 rows: the last chunk is ragged."""
    from deepbind_amd import deepity_smat as ds
    rng = np.random.default_rng(k + nfeat)
    n, nb, h = 334 if rc else 333, 6, 32
    kt = k + nfeat
    t = lambda *shape, s=0.3: dev((rng.standard_normal(shape) * s).astype(np.float32))
    Pl = dev(np.abs(rng.standard_normal((n, k * nb))).astype(np.float32))
    W1, b1, W2, b2 = t(kt * nb, h), t(1, h * nb, s=0.1), t(h * nb, 1), t(1, nb, s=0.1)
    F = t(n, nfeat, s=1.0) if nfeat else None
    Y = dev((rng.random((n, nb)) < 0.5).astype(np.float32))
    M = dev(rng.random((n, nb)) < 0.8)
    rate = dev(np.array([0.0, 0.5, 0.25, 0.5, 0.0, 0.9], np.float32))
    seed, offset = 11, 1234
    U = ds.uniform_like(torch.empty((n // 2 if rc else n, k * nb), device="cuda"), seed, offset)
    if rc:
        U = U.repeat_interleave(2, dim=0).contiguous()                # a (fwd, rev) pair shares its draw
    outs = []
    for uniforms in (None, U):
        g = [torch.full_like(w, float("nan")) for w in (W1, b1, W2, b2)]
        Z, dP, L = ds.head_train(Pl, W1, b1, W2, b2, Y, nb, loss, g[0], g[1], g[2], g[3], Ymask=M, rate=rate, U=uniforms, seed=seed,
                                 offset=offset, reverse_complement=rc, want_loss=True, nfeat=nfeat, feats=F)
        outs.append([host(x) for x in (Z, dP, L, *g)])
    for name, a, b in zip(("Z", "dpooled", "loss", "dW1", "db1", "dW2", "db2"), *outs):
        assert np.isfinite(a).all() and np.array_equal(a, b), name
    assert (outs[0][1] == 0).mean() > 0.2                               # dropout did drop inputs


@pytest.mark.parametrize("mode,single", [("fused", True), ("fused", False), ("unfused", False)])
@pytest.mark.parametrize("pool,hidden,nm", [("max", 32, 1), ("all", 0, 3)])
def test_hinge_loss_train_steps(mode, single, pool, hidden, nm):
    """The reference's third loss (linear output, bidirectional hinge: deepity/std/loss.py:157-174) through the
    single-launch step, the multi-launch step and layer by layer, against the oracle's whole step."""
    from deepbind_amd import data
    from deepbind_amd.model import SequenceNet
    rng = np.random.default_rng(41)
    m, nf, B = 12, 16, 96
    seqs = ["".join("ACGT"[c] for c in rng.integers(0, 4, size=int(rng.integers(25, 60)))) for _ in range(B)]
    X, R = data.pack_sequences(seqs, m - 1)
    net = SequenceNet(nm, nf, m, pool=pool, hidden=hidden, loss="hinge", rate=0.05, momentum=0.9, decay_full=1e-3, weight_decay_start=1,
                      mode=mode, single_launch=single)
    params = {name: (rng.standard_normal(shape) * (0.3 if name.startswith("W") else 0.05)).astype(np.float32) for name, shape, _ in net.layout}
    net.set_params(params)
    Y = (rng.random((B, nm)) < 0.5).astype(np.float32)
    Ymask = rng.random((B, nm)) < 0.9
    Xd, Rd, Yd, Md = dev(X), dev(R), dev(Y), dev(Ymask)
    ref_p, ref_m = _f64(params), {k: np.zeros(v.shape) for k, v in params.items()}
    for step in range(3):
        net.train_step(Xd, Rd, Yd, Md)
        st, g = orc.train_step(ref_p, ref_m, X, R, Y.astype(np.float64), nm, pool, hidden, "hinge", 0.05, 0.9, Ymask=Ymask,
                               decay_full=1e-3, step=step, weight_decay_start=1)
        # (a prediction within round-off of a kink would flip a whole row's gradient: none is that close here)
        act = (1 - Y) * st["Zout"] + Y * (1 - st["Zout"])
        assert np.abs(act).min() > 1e-4
        got_g = net.get_grads()
        for name, _, axis in net.layout:
            assert_close_per_model(got_g[name], g[name], GRAD, nm, axis, "step %d gradient %s" % (step, name))
    assert any(buf.get("work") is not None for buf in net._step_bufs.values()) == (single and mode == "fused")
    got = net.get_params()
    for name, _, axis in net.layout:
        assert_close_per_model(got[name], ref_p[name], GRAD, nm, axis, "parameters %s" % name)
    st = net.forward(Xd, Rd)
    want = orc.loss_fprop(orc.model_forward(ref_p, X, R, nm, pool, hidden)["Zout"], Y.astype(np.float64), "hinge", nm, Ymask=Ymask)
    assert_close(net.loss_value(st, Yd, Md), want, 1e-4, "reported hinge loss")


def test_graphed_step_replays_match_eager_steps():
    """A captured step must give the eager result on EVERY replay (fresh dropout masks included), with
    other work and synchronisations between the replays, and across the L1-decay switch-on."""
    from deepbind_amd import synth
    from deepbind_amd.model import SequenceNet
    cfg = synth.config3()
    spec = cfg["spec"]
    jit = np.random.default_rng(2)
    params = {k: (v if not k.startswith("b") else (jit.standard_normal(v.shape) * 0.01).astype(np.float32)) for k, v in cfg["params"].items()}

    def make():
        net = SequenceNet(1, spec.nfilter, spec.m, pool="max", hidden=32, loss="nll", rate=0.05, momentum=0.9, dropout=0.5,
                          decay_conv=1e-4, decay_full=1e-3, weight_decay_start=3)
        net.rng_seed = 5
        net.set_params(params)
        return net

    eager, graphed = make(), make()
    X, R, Y = dev(cfg["X"]), dev(cfg["R"]), dev(cfg["Y"])
    step = graphed.make_graphed_step(X, R, Y, force_graph=True)
    for i in range(6):
        eager.train_step(X, R, Y)
        step()
        junk = torch.rand(1000, device="cuda").sum().item()          # unrelated eager work + a sync between replays
        a, b = eager.get_params(), graphed.get_params()
        for k in a:
            assert np.array_equal(a[k], b[k]), "replay %d differs from the eager step in %s" % (i, k)
    assert graphed.step_count == 6 and graphed._rng_offset == eager._rng_offset
    assert int(graphed.rng_counter.item()) == int(eager.rng_counter.item())


def test_graphed_group_step_matches_eager_group_step():
    """All architecture groups of the calibration batch in one captured graph, dropout on."""
    from deepbind_amd import synth
    from deepbind_amd.model import ModelGroup
    cfg = synth.config4()
    spec, hp = cfg["spec"], cfg["hp"]

    def make():
        grp = ModelGroup(spec.pool, spec.hidden, spec.nfilter, spec.m, loss="nll", rate=hp["rate"], momentum=hp["momentum"],
                         decay_conv=hp["decay_conv"], decay_full=hp["decay_full"], dropout=hp["dropout"], weight_decay_start=2)
        for gi, (idx, net) in enumerate(grp.groups):
            net.rng_seed = 100 + gi
            net.set_params({n: np.concatenate([cfg["models"][j][n] for j in idx], axis=ax) for n, _, ax in net.layout})
        return grp

    eager, graphed = make(), make()
    X, R, Y, M = dev(cfg["X"]), dev(cfg["R"]), dev(cfg["Y"]), dev(cfg["Ymask"])
    step = graphed.make_graphed_step(X, R, Y, M)
    for i in range(7):
        if i == 4:
            # parameters rewritten between two replays: the look-ahead the last step left no longer belongs to them,
            # and the next replay must be the graph that forms its own (replays 1-3 and 5-6 take the one left behind)
            for (_, a), (_, b) in zip(eager.groups, graphed.groups):
                p = a.get_params()
                p["Wc"] = (p["Wc"] * 0.5).astype(np.float32)
                a.set_params(p)
                b.set_params(p)
        eager.train_step(X, R, Y, M)
        step()
        torch.cuda.synchronize()
        for (_, a), (_, b) in zip(eager.groups, graphed.groups):
            pa, pb = a.get_params(), b.get_params()
            for k in pa:
                assert np.array_equal(pa[k], pb[k]), "replay %d, %s/%d group, %s" % (i, a.pool, a.hidden, k)


@pytest.mark.parametrize("mode", ["fused", "unfused"])
@pytest.mark.parametrize("rc", [False, True])
def test_input_dropout_train_steps_and_test_time_rescale(mode, rc):
    """Input-base dropout: training scans the stream with dropped letters (mirrored on the reverse strand),
    prediction scales the scan output by (1 - rate) instead."""
    from deepbind_amd import data
    from deepbind_amd.model import SequenceNet
    rng = np.random.default_rng(31)
    m, F, hid, rate_in = 8, 16, 8, 0.2
    seqs = ["".join("ACGTN"[v] for v in rng.choice(5, int(rng.integers(12, 30)), p=[.24, .24, .24, .24, .04])) for _ in range(20)]
    X, R = data.pack_sequences(seqs, m - 1, reverse_complement=rc)
    n = len(R)
    params = {"Wc": rng.standard_normal((4 * m, F)) * 0.3, "bc": rng.standard_normal((1, F)) * 0.1,
              "W1": rng.standard_normal((F, hid)) * 0.3, "b1": rng.standard_normal((1, hid)) * 0.1,
              "W2": rng.standard_normal((hid, 1)) * 0.3, "b2": rng.standard_normal((1, 1)) * 0.1}
    params = {k: v.astype(np.float32) for k, v in params.items()}
    Y = np.repeat((rng.random((len(seqs), 1)) < 0.5).astype(np.float32), 2 if rc else 1, axis=0)
    net = SequenceNet(1, F, m, pool="max", hidden=hid, loss="nll", rate=0.05, momentum=0.9, mode=mode,
                      reverse_complement=rc, input_dropout=rate_in)
    net.set_params(params)
    ref_p, ref_m = _f64(params), {k: np.zeros(v.shape) for k, v in params.items()}
    Xd, Rd, Yd = dev(X), dev(R), dev(Y)
    for step in range(2):
        U = rng.random(X.shape).astype(np.float32)
        net.train_step(Xd, Rd, Yd, U_input=dev(U))
        Xdrop, _ = orc.dropoutord_fp_train(X, np.float32(rate_in), U, regions=R, reverse_complement=rc)
        assert (Xdrop == 254).sum() > 10
        _, g = orc.train_step(ref_p, ref_m, Xdrop, R, Y.astype(np.float64), 1, "max", hid, "nll", 0.05, 0.9, step=step,
                              reverse_complement=rc)
        got_g = net.get_grads()
        for k in g:
            assert_close(got_g[k], g[k], GRAD, "step %d grad %s" % (step, k))
    # prediction: no letters dropped, scan output scaled
    st = orc.model_forward(ref_p, X, R, 1, "max", hid, out="logistic", input_keep=1.0 - rate_in)
    want = st["Zout"].reshape(-1, 2).max(axis=1, keepdims=True) if rc else st["Zout"]
    assert_close(host(net.predict(Xd, Rd)), want, ACT, "test-time prediction")
    assert_close(host(net.forward(Xd, Rd)["Z"]), st["Zout"], ACT, "test-time forward")


def test_input_dropout_draws_from_the_library_generator_in_both_modes_and_under_a_graph():
    from deepbind_amd import synth
    from deepbind_amd.model import SequenceNet
    cfg = synth.config3()
    spec = cfg["spec"]
    jit = np.random.default_rng(2)
    params = {k: (v if not k.startswith("b") else (jit.standard_normal(v.shape) * 0.01).astype(np.float32)) for k, v in cfg["params"].items()}

    def make(mode):
        net = SequenceNet(1, spec.nfilter, spec.m, pool="max", hidden=32, loss="nll", rate=0.05, momentum=0.9, dropout=0.5,
                          input_dropout=0.1, mode=mode)
        net.rng_seed = 9
        net.set_params(params)
        return net

    fused, layered, graphed = make("fused"), make("unfused"), make("fused")
    X, R, Y = dev(cfg["X"]), dev(cfg["R"]), dev(cfg["Y"])
    step = graphed.make_graphed_step(X, R, Y)
    for i in range(3):
        fused.train_step(X, R, Y)
        layered.train_step(X, R, Y)
        step()
        a, b, c = fused.get_params(), layered.get_params(), graphed.get_params()
        for k in a:
            assert np.array_equal(a[k], c[k]), "graph replay %d differs in %s" % (i, k)
            assert_close(b[k], a[k], GRAD, "layer-by-layer vs fused, step %d, %s" % (i, k))
    assert fused._rng_offset == layered._rng_offset == graphed._rng_offset == int(graphed.rng_counter.item())


def test_slice_model_save_load_and_group_prediction(tmp_path):
    """A model sliced out of a trained batch predicts exactly what its column of the batch predicts,
    before and after a round trip through the .npz export."""
    from deepbind_amd import synth
    from deepbind_amd.model import ModelGroup, SequenceNet
    cfg = synth.config4()
    spec, hp = cfg["spec"], cfg["hp"]
    grp = ModelGroup(spec.pool, spec.hidden, spec.nfilter, spec.m, loss="nll", rate=hp["rate"], momentum=hp["momentum"],
                     decay_conv=hp["decay_conv"], decay_full=hp["decay_full"], dropout=hp["dropout"])
    for idx, net in grp.groups:
        net.set_params({n: np.concatenate([cfg["models"][j][n] for j in idx], axis=ax) for n, _, ax in net.layout})
    X, R, Y, M = dev(cfg["X"]), dev(cfg["R"]), dev(cfg["Y"]), dev(cfg["Ymask"])
    for _ in range(2):
        grp.train_step(X, R, Y, M)
    scores = host(grp.predict(X, R))
    for j in (0, 17, 44, 89):
        one = grp.slice_model(j)
        assert one.ninst == 1 and (one.pool, one.hidden) == (spec.pool[j], spec.hidden[j])
        s1 = host(one.predict(X, R))
        assert_close(s1[:, 0], scores[:, j], ACT, "model %d sliced" % j)
        path = str(tmp_path / ("m%d.npz" % j))
        one.save_npz(path)
        back = SequenceNet.load_npz(path)
        assert np.array_equal(host(back.predict(X, R)), s1)
        for k, v in one.get_params().items():
            assert np.array_equal(back.get_params()[k], v)


def test_training_from_a_sequence_file_reduces_the_loss(tmp_path):
    """Reader -> batcher -> reverse-complement training loop -> export -> prediction, on a planted motif."""
    from deepbind_amd import datasource, predict
    from deepbind_amd.model import SequenceNet
    rng = np.random.default_rng(4)
    lines = ["FoldID\tEventID\tseq\tBound"]
    for i in range(256):
        s = rng.integers(0, 4, 40)
        bound = i % 2
        if bound:
            at = int(rng.integers(0, 32))
            s[at:at + 8] = [2, 0, 3, 3, 0, 1, 0, 2]                      # GATTACAG
            if rng.random() < 0.5:
                s = 3 - s[::-1]                                           # planted on either strand
        lines.append("%s\tseq%d\t%s\t%d" % ("ABC"[i % 3], i, "".join("ACGT"[v] for v in s), bound))
    path = tmp_path / "train.seq"
    path.write_text("\n".join(lines) + "\n")
    d = datasource.SequenceData.fromtxt(str(path))
    train, held = d.extract_fold("A")[:], d.extract_fold("C")
    m = 10
    net = SequenceNet(1, 8, m, pool="max", hidden=0, loss="nll", rate=0.05, momentum=0.9, reverse_complement=True, dropout=0.0)
    init = np.random.default_rng(0)
    net.set_params({"Wc": (init.standard_normal((4 * m, 8)) * 0.1).astype(np.float32), "bc": np.zeros((1, 8), np.float32),
                    "W1": (init.standard_normal((8, 1)) * 0.1).astype(np.float32), "b1": np.zeros((1, 1), np.float32)})
    batches = [{k: dev(v) for k, v in b.items() if k != "rowidx"} for b in d.asbatches(64, padding=m - 1, reverse_complement=True)]

    def mean_loss():
        return float(np.mean([net.loss_value(net.forward(b["X"], b["R"]), b["Y"], b["Ymask"])[0, 0] for b in batches]))

    before = mean_loss()
    for epoch in range(60):
        for b in batches:
            net.train_step(b["X"], b["R"], b["Y"], b["Ymask"])
    after = mean_loss()
    assert after < 0.5 * before, (before, after)
    Z, _ = predict.gen_predictions(net, held.sequences)
    auc_pairs = [(z, y) for z, y in zip(Z.ravel(), held.Y.ravel())]
    pos = [z for z, y in auc_pairs if y == 1]
    neg = [z for z, y in auc_pairs if y == 0]
    auc = np.mean([p > q for p in pos for q in neg])
    assert auc > 0.9, auc


def test_init_params_penalty_and_frozen_filters():
    """Trainer set-up pieces: randn * per-model scale (+ bias shift), the L1 cost added to the reported loss,
    and the scan filters staying frozen while step < start_training."""
    from deepbind_amd import smat, synth
    from deepbind_amd.model import SequenceNet
    Zn = host(smat.randn(1 << 18, 1, seed=3))
    assert abs(Zn.mean()) < 0.01 and abs(Zn.std() - 1.0) < 0.01 and abs((Zn ** 4).mean() - 3.0) < 0.1
    assert np.array_equal(Zn, host(smat.randn(1 << 18, 1, seed=3))) and not np.array_equal(Zn, host(smat.randn(1 << 18, 1, seed=4)))
    assert host(smat.randn(64, 2, dtype=torch.float64, seed=3)).dtype == np.float64

    cfg = synth.config3()
    spec = cfg["spec"]
    ni = 6
    scales = np.array([0.01, 0.02, 0.04, 0.08, 0.16, 0.32])
    net = SequenceNet(ni, spec.nfilter, spec.m, pool="max", hidden=32, loss="nll", rate=0.05, momentum=0.9,
                      decay_conv=np.linspace(1e-4, 6e-4, ni), decay_full=np.linspace(1e-3, 6e-3, ni), weight_decay_start=1,
                      start_training=2)
    net.init_params(init_conv=scales, init_full=2 * scales, init_mu=0.5, seed=11)
    p = net.get_params()
    for b in range(ni):
        assert abs(p["Wc"][:, 16 * b:16 * (b + 1)].std() / scales[b] - 1) < 0.1
        assert abs(p["W1"][16 * b:16 * (b + 1)].std() / (2 * scales[b]) - 1) < 0.15
        assert abs(p["W2"][32 * b:32 * (b + 1)].std() / (2 * scales[b]) - 1) < 0.5
    assert np.all(p["bc"] == 0.5) and np.all(p["b1"] == 0.5) and np.all(p["b2"] == 0.5)
    # cost: zero before weight_decay_start, the per-model L1 sums after
    assert np.all(net.penalty_value() == 0)
    X, R = dev(cfg["X"]), dev(cfg["R"])
    Y = dev(np.repeat(cfg["Y"], ni, axis=1))
    ref_p, ref_m = _f64(p), {k: np.zeros(v.shape) for k, v in p.items()}
    for step in range(3):
        before = net.get_params()["Wc"]
        net.train_step(X, R, Y)
        orc.train_step(ref_p, ref_m, cfg["X"], cfg["R"], np.repeat(cfg["Y"], ni, axis=1).astype(np.float64), ni, "max", 32, "nll",
                       0.05, 0.9, decay_conv=np.linspace(1e-4, 6e-4, ni), decay_full=np.linspace(1e-3, 6e-3, ni), step=step,
                       weight_decay_start=1, start_training=2)
        after = net.get_params()
        assert np.array_equal(before, after["Wc"]) == (step < 2), "filters frozen exactly while step < start_training (step %d)" % step
        for k in ref_p:
            assert_close(after[k], ref_p[k], GRAD, "step %d %s" % (step, k))
    want = orc.weight_cost(_f64(net.get_params()), ni, np.linspace(1e-4, 6e-4, ni), np.linspace(1e-3, 6e-3, ni))
    assert_close(net.penalty_value(), want, ACT, "L1 cost")


@pytest.mark.parametrize("mode", ["unfused", "fused"])
@pytest.mark.parametrize("pool,hidden,loss", [("max", 6, "nll"), ("all", 0, "mse"), ("avg", 4, "nll")])
def test_gradcheck_float64_layer_by_layer(pool, hidden, loss, mode):
    """The trainer's own finite-difference check, on the device in float64: HIP forward against HIP backward,
    no oracle involved; and the checker must notice a wrong gradient. Mode "fused" takes the scan + pool chain through
    the two fused calls, which run the operator kernels in double precision inside the library."""
    from deepbind_amd import data
    from deepbind_amd.gradcheck import gradcheck
    from deepbind_amd.model import SequenceNet
    rng = np.random.default_rng(21)
    m, nf, ni = 5, 3, 2
    seqs = ["".join("ACGTN"[v] for v in rng.choice(5, int(rng.integers(8, 16)), p=[.24, .24, .24, .24, .04])) for _ in range(12)]
    X, R = data.pack_sequences(seqs, m - 1)
    net = SequenceNet(ni, nf, m, pool=pool, hidden=hidden, loss=loss, dtype=torch.float64, dropout=[0.0, 0.3],
                      decay_conv=[1e-3, 1e-3], decay_full=[3e-3, 1e-3], weight_decay_start=0, mode=mode)
    # (equal scan-filter decays: with different ones the reference's gradient uses its rows/ninst block length,
    # kangaroo/_ext/corr1ord.py:126, and is not the derivative of its own cost; that quirk is kept and tested elsewhere)
    net.init_params(init_conv=0.5, init_full=0.5, init_mu=0.1, seed=5)
    Y = dev(rng.random((len(seqs), ni)) if loss == "nll" else rng.standard_normal((len(seqs), ni)))
    Ymask = dev(rng.random((len(seqs), ni)) < 0.8)
    n = gradcheck(net, dev(X), dev(R), Y, Ymask, ncheck=30, rtol=1e-5, atol=1e-6)
    assert n >= 40
    good = net.backward

    def bad(*a, **k):
        good(*a, **k)
        net.g["W1"].mul_(1.01)
    net.backward = bad
    with pytest.raises(AssertionError, match="W1 FAILED"):
        gradcheck(net, dev(X), dev(R), Y, Ymask, ncheck=30, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("pool", ["max", "all"])
def test_bulk_batch_training_step_uses_the_table_kernel_and_matches_layer_by_layer(pool):
    """A batch large enough for the fused forward to pick the table kernel (with argmax for the backward pass):
    one training step must agree with the layer-by-layer drop-in operators, and be bit-stable."""
    from deepbind_amd import data
    from deepbind_amd.model import SequenceNet
    rng = np.random.default_rng(13)
    B, L, m, ni = 12000, 101, 24, 4
    codes = rng.integers(0, 4, (B, L), dtype=np.uint8)
    codes[rng.random((B, L)) < 0.01] = 255
    X, R = data.pack_uniform_ordinals(codes, m - 1)
    Y = (rng.random((B, ni)) < 0.5).astype(np.float32)
    nets = []
    for mode in ("fused", "unfused", "fused"):
        net = SequenceNet(ni, 16, m, pool=pool, hidden=32, loss="nll", rate=0.05, momentum=0.9, mode=mode, dropout=0.0)
        net.init_params(init_conv=0.05, init_full=0.1, init_mu=0.01, seed=3)
        net.train_step(dev(X), dev(R), dev(Y))
        nets.append(net)
    a, b, c = (n.get_grads() for n in nets)
    for k in a:
        assert_close(a[k], b[k], GRAD, "fused vs layer-by-layer gradient %s" % k)
        assert np.array_equal(a[k], c[k]), "run-to-run difference in %s" % k
    assert np.abs(a["Wc"]).max() > 0


@pytest.mark.parametrize("pool,hidden,loss,nesterov,rc", [("max", 0, "nll", True, False), ("all", 8, "mse", False, False),
                                                           ("avg", 4, "nll", True, True), ("all", 0, "nll", True, True)])
def test_natively_issued_step_equals_the_step_issued_call_by_call(pool, hidden, loss, nesterov, rc):
    """dbk_train_step against the same entry points called one by one from the host: every variant of the
    step (pooling, hidden layer, loss, plain momentum, reverse complements with mirrored input dropout,
    frozen filters, the L1-decay switch-on) must leave bit-identical parameters, momenta, gradients and
    generator position."""
    from deepbind_amd import data, deepity_smat as ds
    from deepbind_amd.model import SequenceNet
    rng = np.random.default_rng(17)
    ni, nf, m = 3, 5, 9
    seqs = ["".join(rng.choice(list("ACGTN"), p=[.24, .24, .24, .24, .04], size=rng.integers(12, 40))) for _ in range(24)]
    if rc:
        seqs = orc.insert_reverse_complements(seqs)
    Xh, Rh = data.pack_sequences(seqs, m - 1)
    X, R = dev(Xh), dev(Rh)
    Y = dev(rng.random((len(seqs), ni)).astype(np.float32))
    M = dev(rng.random((len(seqs), ni)) < 0.8)

    def make():
        net = SequenceNet(ni, nf, m, pool=pool, hidden=hidden, loss=loss, rate=[0.05, 0.02, 0.1], momentum=0.8,
                          dropout=[0.0, 0.3, 0.5], decay_conv=1e-3, decay_full=[1e-3, 0.0, 1e-2], weight_decay_start=2,
                          nesterov=nesterov, reverse_complement=rc, input_dropout=0.2 if rc else 0.0, start_training=1,
                          single_launch=False)         # (the one-launch step of small groups has summation orders of its own)
        net.rng_seed = 11
        net.init_params(0.3, 0.3, 0.05, seed=4)
        return net

    native, stepwise = make(), make()
    for i in range(4):
        native.train_step(X, R, Y, M)
        ds.gradstep(stepwise.P, stepwise.dP, stepwise.drate, stepwise.mP, stepwise.mrate,
                    lambda: stepwise._grad_fused(X, R, Y, M, None), nesterov=nesterov)
        stepwise.step_count += 1
        torch.cuda.synchronize()
        for name in ("P", "dP", "mP"):
            a, b = getattr(native, name).cpu().numpy(), getattr(stepwise, name).cpu().numpy()
            assert np.array_equal(a, b), "step %d: %s differs" % (i, name)
        assert int(native.rng_counter.item()) == int(stepwise.rng_counter.item()) == native._rng_offset == stepwise._rng_offset
    assert np.abs(native.mP.cpu().numpy()).max() > 0 and native.step_count == 4
    # the natively issued step keeps the Nesterov look-ahead beside the parameters from one step to the next; whatever
    # changes the parameters, the momentum or the momentum rates in between must make it form the look-ahead afresh
    if nesterov:
        for change in ("params", "rates", "view", "layerwise"):
            for net in (native, stepwise):
                if change == "params":
                    net.set_params({k: v * 0.5 for k, v in net.get_params().items()})
                elif change == "rates":
                    net.set_rates([0.03, 0.01, 0.2], 0.6)
                elif change == "view":
                    net.p["bc"].add_(0.25)
            if change == "layerwise":
                Ux = dev(rng.random((len(seqs), native.k * ni)).astype(np.float32))
                Ui = dev(rng.random(Xh.shape).astype(np.float32)) if native.input_dropout > 0 else None
                native.train_step(X, R, Y, M, U=Ux, U_input=Ui)           # goes through the wrappers, in place
                stepwise.train_step(X, R, Y, M, U=Ux, U_input=Ui)
            for _ in range(2):
                native.train_step(X, R, Y, M)
                ds.gradstep(stepwise.P, stepwise.dP, stepwise.drate, stepwise.mP, stepwise.mrate,
                            lambda: stepwise._grad_fused(X, R, Y, M, None), nesterov=True)
                stepwise.step_count += 1
            torch.cuda.synchronize()
            for name in ("P", "mP"):
                assert np.array_equal(getattr(native, name).cpu().numpy(), getattr(stepwise, name).cpu().numpy()), (change, name)


def test_groups_stepped_in_shared_launches_match_groups_stepped_alone_across_changing_batches():
    """ModelGroup.train_step issues one launch per phase for all its architecture groups (dbk_train_steps);
    every group must end with the bits of its own dbk_train_step, across a change of targets, a smaller batch,
    the L1 term switching on and an accessor in between."""
    from deepbind_amd import synth
    from deepbind_amd.model import ModelGroup
    cfg = synth.config4()
    spec, hp = cfg["spec"], cfg["hp"]

    def make():
        grp = ModelGroup(spec.pool, spec.hidden, spec.nfilter, spec.m, loss="nll", rate=hp["rate"], momentum=hp["momentum"],
                         decay_conv=hp["decay_conv"], decay_full=hp["decay_full"], dropout=hp["dropout"], weight_decay_start=3)
        for gi, (idx, net) in enumerate(grp.groups):
            net.rng_seed = 100 + gi
            net.set_params({n: np.concatenate([cfg["models"][j][n] for j in idx], axis=ax) for n, _, ax in net.layout})
        return grp

    together, alone = make(), make()
    assert len(together.groups) == 4 and {net.pool for _, net in together.groups} == {"max", "all"}
    X, R, Y, M = dev(cfg["X"]), dev(cfg["R"]), dev(cfg["Y"]), dev(cfg["Ymask"])
    rng = np.random.default_rng(3)
    Y2 = dev(rng.random(cfg["Y"].shape).astype(np.float32))
    half = cfg["R"].shape[0] // 2                                    # a second, smaller batch: the first half of the regions
    R3, Y3, M3 = dev(cfg["R"][:half]), dev(cfg["Y"][:half]), dev(cfg["Ymask"][:half])
    batches = [(X, R, Y, M)] * 3 + [(X, R, Y2, M)] * 2 + [(X, R3, Y3, M3)] * 2 + [(X, R, Y, M)]
    for i, (bx, br, by, bm) in enumerate(batches):
        together.train_step(bx, br, by, bm)
        for idx, net in alone.groups:
            ii = torch.as_tensor(idx, device=by.device)
            net.train_step(bx, br, by.index_select(1, ii).contiguous(), bm.index_select(1, ii).contiguous())
        if i == 4:
            assert np.array_equal(host(together.predict(X, R)), host(alone.predict(X, R)))
    assert np.array_equal(host(together.predict(X, R)), host(alone.predict(X, R)))
    for (_, a), (_, b) in zip(together.groups, alone.groups):
        pa, pb = a.get_params(), b.get_params()
        for k in pa:
            assert np.array_equal(pa[k], pb[k]), "%s/%d group, %s" % (a.pool, a.hidden, k)
        assert np.array_equal(host(a.mP), host(b.mP)) and np.array_equal(host(a.dP), host(b.dP))
        assert a.step_count == b.step_count == len(batches) and a._rng_offset == b._rng_offset
        assert host(a.rng_counter) == host(b.rng_counter)


@pytest.mark.parametrize("case", ["mixed_pools_revcomp_input_dropout", "eight_taps", "ten_nets", "different_lengths", "plain_momentum",
                                  "many_regions", "many_regions_16_taps"])
def test_nets_stepped_through_one_call_end_with_the_bits_of_their_own_steps(case):
    """dbk_train_steps either runs each phase of the step as one launch for all the nets (same filter-length tier, a
    look-ahead vector each, at most eight nets) or steps them one after the other; both ways every net must end
    with the bits of its own dbk_train_step. Covers avg / all / max pooling side by side, reverse-complement
    pairs, input dropout (each net scans its own dropped copy), mse and nll, 8-, 16- and 24-tap tiers, more nets
    than one call takes, the two fallbacks (nets of different tiers, a net without Nesterov momentum), and batches
    of enough regions for the many-regions kernel bodies (four filters per lane forward, a wave per region backward)."""
    from deepbind_amd import data
    from deepbind_amd.model import SequenceNet, _native_steps
    rng = np.random.default_rng(11)
    revcomp = case == "mixed_pools_revcomp_input_dropout"
    B = 600 if case.startswith("many_regions") else 40
    seqs = ["".join(rng.choice(list("ACGTN"), p=[.24, .24, .24, .24, .04], size=int(rng.integers(18, 45)))) for _ in range(B)]
    kw = dict(rate=0.05, momentum=0.9, decay_conv=1e-3, decay_full=1e-3, weight_decay_start=1)
    if case == "mixed_pools_revcomp_input_dropout":
        m = 16
        specs = [dict(nmodel=3, pool="avg", hidden=0, loss="mse", reverse_complement=True, dropout=0.25, **kw),
                 dict(nmodel=5, pool="all", hidden=8, loss="nll", reverse_complement=True, input_dropout=0.2, start_training=2, **kw),
                 dict(nmodel=2, pool="max", hidden=0, loss="nll", reverse_complement=True, input_dropout=0.1, dropout=0.5, **kw),
                 dict(nmodel=4, pool="max", hidden=32, loss="mse", reverse_complement=True, **kw)]
        lens = [m] * 4
    elif case == "eight_taps":
        specs = [dict(nmodel=2, pool="all", hidden=0, loss="nll", dropout=0.5, **kw), dict(nmodel=7, pool="max", hidden=4, loss="nll", **kw)]
        lens = [7, 7]
    elif case == "ten_nets":
        specs = [dict(nmodel=1 + i % 3, pool=("max", "all", "avg")[i % 3], hidden=(0, 16)[i % 2], loss="nll", **kw) for i in range(10)]
        lens = [24] * 10
    elif case.startswith("many_regions"):
        specs = [dict(nmodel=3, pool="avg", hidden=0, loss="mse", dropout=0.25, **kw), dict(nmodel=5, pool="all", hidden=8, loss="nll", **kw),
                 dict(nmodel=4, pool="max", hidden=0, loss="nll", input_dropout=0.1, **kw)]
        lens = [24 if case == "many_regions" else 16] * 3
    elif case == "different_lengths":
        specs = [dict(nmodel=2, pool="all", hidden=0, loss="nll", **kw), dict(nmodel=3, pool="max", hidden=8, loss="nll", **kw)]
        lens = [8, 24]
    else:
        specs = [dict(nmodel=2, pool="all", hidden=0, loss="nll", **kw), dict(nmodel=3, pool="max", hidden=8, loss="nll", nesterov=False, **kw)]
        lens = [16, 16]
    X, R = data.pack_sequences(seqs, max(lens) - 1, reverse_complement=revcomp)
    Xd, Rd = dev(X), dev(R)
    rows = len(R)

    def make():
        nets, targets = [], []
        trng = np.random.default_rng(12)
        for i, (spec, m) in enumerate(zip(specs, lens)):
            net = SequenceNet(nfilter=16, m=m, single_launch=False, **spec)   # (compare like with like: the multi-launch step)
            net.init_params(init_conv=0.3, init_full=0.3, init_mu=0.01, seed=40 + i)
            net.rng_seed = 7 + i
            Y = (trng.random((rows // (2 if revcomp else 1), net.ninst)) < 0.5).astype(np.float32)
            Y = np.repeat(Y, 2, axis=0) if revcomp else Y
            M = trng.random((rows, net.ninst)) < 0.8
            nets.append(net)
            targets.append((dev(Y), dev(M)))
        return nets, targets

    (one_call, t1), (by_itself, t2) = make(), make()
    for step in range(4):
        _native_steps([(net, Xd, Rd, Y, M) for net, (Y, M) in zip(one_call, t1)])
        for net, (Y, M) in zip(by_itself, t2):
            net.train_step(Xd, Rd, Y, M)
    torch.cuda.synchronize()
    for i, (a, b) in enumerate(zip(one_call, by_itself)):
        for name in ("P", "mP", "dP"):
            assert np.array_equal(host(getattr(a, name)), host(getattr(b, name))), (case, i, name)
        assert np.abs(host(a.mP)).max() > 0
        assert a.step_count == b.step_count == 4 and a._rng_offset == b._rng_offset
        assert host(a.rng_counter) == host(b.rng_counter)
