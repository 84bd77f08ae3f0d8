"""Benchmark of the motif-scan hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload config5|config5_small]

One step = one pass of the fused forward (scan + bias + ReLU + max pool over every region, then the
dense head) over the whole synthetic batch of the bulk-scoring configuration: 64 models x 16 motif
detectors of width 24 over 100 000 DNA sequences of length 500 (1 % N), producing the 100000 x 64
score matrix. Inputs are resident in HBM before the timed region. Prints ONE JSON line.

Units: a "position" is one row of the (virtual) feature map, sum over sequences of (len + m - 1);
the scan's algorithmic work is positions * filters * m gather-adds (1 FLOP each).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

FP32_VECTOR_PEAK_TFLOPS = 157.3     # MI355X published FP32 vector peak (FMA = 2 FLOP)
FP32_ADD_ISSUE_PEAK_TADDS = 78.6    # the same peak for a stream of plain adds (1 FLOP per lane-operation)
HBM_PEAK_GBS = 8000.0


def _numpy_scanpool(Wc, bc, X, R, m, chunk=4):
    """The NumPy float32 formulation of scan + bias + ReLU + max pool (what the reference's array library falls back
    to on host arrays): m gathers from a per-tap letter table, np.maximum, np.maximum.reduceat over region starts;
    `chunk` sequences at a time so that a chunk's map stays in the host's caches (3x faster than whole-batch maps)."""
    from oracle import deepbind_oracle as orc
    F = Wc.shape[1]
    out = np.empty((len(R), F), np.float32)
    for i in range(0, len(R), chunk):
        Rc = R[i:i + chunk].astype(np.int64)
        a, b = int(Rc[0, 0]), int(Rc[-1, 1])
        Xc = X[a:b + m - 1]
        Z = np.zeros((Xc.size, F), np.float32)
        orc.corr1ord(Wc, Xc, Z)
        A = np.maximum(Z + bc, 0)
        out[i:i + chunk] = np.maximum.reduceat(A[:b - a], Rc[:, 0] - a, axis=0)
    return out


def cpu_baseline(cfg, nseq, budget_s=30.0):
    """Times the reference's CPU path - the NumPy float32 semantics its array library's tests compare against - on a
    bounded subsample of the same workload, after one warm-up: best of up to 5 runs within `budget_s` seconds.
    The checker's plain-C port (OpenMP over all host cores) is timed beside it as a secondary figure."""
    from oracle import oracle_c
    spec, p = cfg["spec"], cfg["params"]
    m = spec.m
    R = np.ascontiguousarray(cfg["R"][:nseq])
    pos = int(R[-1, 1])
    X = np.ascontiguousarray(cfg["X"][:pos + m - 1]).ravel()
    cores = len(os.sched_getaffinity(0))
    _numpy_scanpool(p["Wc"], p["bc"], X, R[:48], m)                    # warm-up
    best, runs, spent = float("inf"), 0, 0.0
    while runs < 5 and (runs == 0 or spent + best <= budget_s):
        t0 = time.perf_counter()
        _numpy_scanpool(p["Wc"], p["bc"], X, R, m)
        dt = time.perf_counter() - t0
        best, runs, spent = min(best, dt), runs + 1, spent + dt
    np_rate = pos / best
    oracle_c.scanpool(p["Wc"], p["bc"], X[:2000 + m], R[:2], 0)       # warm-up (thread pool, page-in)
    cbest = float("inf")
    for _ in range(3):
        t0 = time.perf_counter()
        oracle_c.scanpool(p["Wc"], p["bc"], X, R, 0)
        cbest = min(cbest, time.perf_counter() - t0)
    try:
        from threadpoolctl import threadpool_info
        blas = max([t.get("num_threads", 1) for t in threadpool_info() if t.get("user_api") == "blas"] or [1])
    except Exception:
        blas = None
    return {
        "value": np_rate, "unit": "positions/s", "cores": 1, "kind": "port",
        "sample": "NumPy float32 restatement of the reference's CPU path (per-tap letter-table gathers, np.maximum, np.maximum.reduceat; "
                  "one thread: these NumPy calls do not use BLAS), first %d of the %d sequences x all %d filters = %d positions, "
                  "best of %d runs after a warm-up; scale linearly for the full batch" % (nseq, len(cfg["R"]), spec.F, pos, runs),
        "host": {"os_cpu_count": os.cpu_count(), "sched_affinity": cores, "blas_threads": blas},
        "c_port_positions_per_s": pos / cbest,
        "c_port_sample": "plain-C port of the same chain (OpenMP, %d threads), same sample, best of 3" % cores,
    }


def train_cpu_baseline(cfg, groups, nsteps=2, budget_s=12.0):
    """One optimiser step of the NumPy float32 restatement of the reference's train step on the same batch:
    sequences per second, best of up to `nsteps` timed steps after one warm-up step. groups: list of
    (model indices, pool, hidden, stacked float32 parameter dict) - one entry for a single net, one per
    architecture for the calibration batch (each architecture is one graph in the reference too)."""
    from oracle import deepbind_oracle as orc
    spec = cfg["spec"]
    hp = cfg.get("hp")
    state = []
    for idx, pool, hidden, params in groups:
        p = {k: np.array(v, dtype=np.float32) for k, v in params.items()}
        state.append((idx, pool, hidden, p, {k: np.zeros_like(v) for k, v in p.items()}))
    Y = cfg["Y"].astype(np.float32)
    Ymask = cfg.get("Ymask")
    rng = np.random.default_rng(0)

    def one_step(step):
        for idx, pool, hidden, p, mom in state:
            k = spec.nfilter * (2 if pool == "all" else 1)
            if hp is not None:
                rate, mu = hp["rate"][idx], hp["momentum"][idx]
                drop = (hp["dropout"][idx], rng.random((len(cfg["R"]), k * len(idx)), dtype=np.float32)) if (hp["dropout"][idx] > 0).any() else None
                dc, df = hp["decay_conv"][idx], hp["decay_full"][idx]
            else:
                rate, mu, dc, df = cfg["rate"], cfg["momentum"], 0.0, 0.0
                dr = cfg.get("dropout_rate", 0.0)
                drop = (np.full(1, dr, np.float32), rng.random((len(cfg["R"]), k), dtype=np.float32)) if dr > 0 else None
            orc.train_step(p, mom, cfg["X"], cfg["R"], Y[:, idx], len(idx), pool, hidden, spec.loss, rate, mu,
                           Ymask=None if Ymask is None else Ymask[:, idx], dropout=drop, decay_conv=dc, decay_full=df,
                           step=step, weight_decay_start=0)

    one_step(0)
    best, runs, spent = float("inf"), 0, 0.0
    while runs < nsteps and (runs == 0 or spent + best <= budget_s):
        t0 = time.perf_counter()
        one_step(1 + runs)
        dt = time.perf_counter() - t0
        best, runs, spent = min(best, dt), runs + 1, spent + dt
    nseq = len(cfg["R"])
    return {"value": nseq / best, "unit": "sequences/s", "ms_per_step": best * 1e3, "cores": 1, "kind": "port",
            "model_sequences_per_s": nseq * spec.nmodel / best,
            "sample": "NumPy float32 restatement of the reference's train step (forward, backward, L1 term, Nesterov update) on the "
                      "same batch, all %d models, best of %d steps after a warm-up step; the dense products go through NumPy's BLAS"
                      % (spec.nmodel, runs)}


def measured_traffic(workload):
    """HBM bytes per launch of the dominant kernel as measured offline with rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE (scaled by a copy kernel of known size) for the full-size workload;
    None when no measurement is on file for this workload."""
    if workload != "config5":
        return None
    path = os.path.join(ROOT, "profiles", "scanpool_kmer_config5_counters.md")
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch:"):
                return int(line.split(":")[1])
    except OSError:
        pass
    return None


def profiled_kernels(tag):
    """Dominant kernel of a training configuration and its average duration from the committed rocprofv3 kernel
    trace (profiles/train_step_kernel_trace.md, lines 'dominant[<tag>]: <kernel> <avg_us>'); None when not on file."""
    path = os.path.join(ROOT, "profiles", "train_step_kernel_trace.md")
    try:
        for line in open(path):
            if line.startswith("dominant[%s]:" % tag):
                name, us = line.split(":", 1)[1].rsplit(None, 1)
                return {"kernel": name.strip(), "rocprof_avg_us": float(us)}
    except (OSError, ValueError):
        pass
    return None


def train_throughput(steps=3000, warmup=300, cpu=True):
    """Whole train steps (forward + backward + Nesterov update) per second on the three training configurations,
    fused mode: each step issued natively by one library call (the top-level figures; the calibration batch's
    architecture groups share every launch) and as one captured HIP graph per step ("graphed").
    sequences/s = batch rows * steps / wall time. Roofline: algorithmic adds per step = 2 * positions * filters *
    taps (the scan and the filter gradient cost the same count; bias, ReLU, pooling and the dense head are not
    counted) over the step time, against the FP32 vector peak (FMA-counted) and against the add-issue peak."""
    import torch
    from deepbind_amd import synth
    from deepbind_amd.model import ModelGroup, SequenceNet
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    out = {}

    def timed(fn, nseq, nmodel):
        # Two warm-up bursts: the first pays for scratch buffers and first launches, the second lets the host run as far
        # ahead of the GPU as it does in the timed loop - the first time the launch queue fills up, the HIP runtime
        # stalls one call for tens of milliseconds (measured: 52 ms, once per process), which belongs to neither step.
        # ... and the bursts go on until a quarter of a second of GPU work has passed: after seconds of host-only work
        # (the CPU baselines) the GPU takes a while to return to the clock it holds under load.
        t_warm, bursts = time.perf_counter(), 0
        while bursts < 2 or time.perf_counter() - t_warm < 0.25:
            for _ in range(warmup):
                fn()
            torch.cuda.synchronize()
            bursts += 1
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / steps
        return {"ms_per_step": dt * 1e3, "gpu_ms_per_step": e0.elapsed_time(e1) / steps, "sequences_per_s": nseq / dt,
                "model_sequences_per_s": nseq * nmodel / dt}

    def roofline(tag, cfg, rec):
        spec = cfg["spec"]
        adds = 2.0 * synth.positions(cfg["R"]) * spec.F * spec.m
        rate = adds / (rec["ms_per_step"] * 1e-3) / 1e12
        r = {"bound": "fp32_valu", "algorithmic_adds_per_step": adds, "achieved": rate, "unit": "T adds/s",
             "peak": FP32_VECTOR_PEAK_TFLOPS, "frac": rate / FP32_VECTOR_PEAK_TFLOPS,
             "frac_vs_add_issue_peak": rate / FP32_ADD_ISSUE_PEAK_TADDS}
        dom = profiled_kernels(tag)
        if dom:
            r["dominant_kernel"] = dom
        return r

    cpu_jobs = []                        # the CPU baselines run after every GPU timing: seconds of host-only work in between let the GPU clock down
    for tag, name, cfg, drop in (("config2", "config2_rna_regression", synth.config2(), 0.0),
                                 ("config3", "config3_classification", synth.config3(), 0.5)):
        spec = cfg["spec"]
        net = SequenceNet(1, spec.nfilter, spec.m, pool=spec.pool[0], hidden=spec.hidden[0], loss=spec.loss,
                          rate=cfg["rate"], momentum=cfg["momentum"], dropout=drop)
        net.set_params(cfg["params"])
        X, R, Y = dev(cfg["X"]), dev(cfg["R"]), dev(cfg["Y"])
        out[name] = timed(lambda: net.train_step(X, R, Y), len(cfg["R"]), 1)
        out[name]["graphed"] = timed(net.make_graphed_step(X, R, Y), len(cfg["R"]), 1)
        out[name]["roofline"] = roofline(tag, cfg, out[name])
        if cpu:
            cfg["dropout_rate"] = drop
            cpu_jobs.append((name, cfg, [([0], spec.pool[0], spec.hidden[0], cfg["params"])], 5))
    cfg = synth.config4()
    spec, hp = cfg["spec"], cfg["hp"]
    grp = ModelGroup(spec.pool, spec.hidden, spec.nfilter, spec.m, loss="nll", rate=hp["rate"], momentum=hp["momentum"],
                     decay_conv=hp["decay_conv"], decay_full=hp["decay_full"], dropout=hp["dropout"],
                     weight_decay_start=0)       # the L1 term is on in every timed step (steady state; a captured graph is re-captured when it switches on)
    stacked = []
    for idx, net in grp.groups:
        params = {n: np.concatenate([cfg["models"][j][n] for j in idx], axis=ax) for n, _, ax in net.layout}
        net.set_params(params)
        stacked.append((idx, net.pool, net.hidden, params))
    X, R, Y, M = dev(cfg["X"]), dev(cfg["R"]), dev(cfg["Y"]), dev(cfg["Ymask"])
    name = "config4_calibration_90_models"
    out[name] = timed(lambda: grp.train_step(X, R, Y, M), len(cfg["R"]), spec.nmodel)
    out[name]["graphed"] = timed(grp.make_graphed_step(X, R, Y, M), len(cfg["R"]), spec.nmodel)
    out[name]["roofline"] = roofline("config4", cfg, out[name])
    if cpu:
        cpu_jobs.append((name, cfg, stacked, 2))
    for name, cfg, groups, nsteps in cpu_jobs:
        out[name]["cpu_baseline"] = train_cpu_baseline(cfg, groups, nsteps=nsteps)
    return out


def ops_throughput(reps=5):
    """Per-operator figures for the drop-in operators and the general fused kernels on a mid-size batch
    (8192 sequences x 101 nt, 16 models x 16 motifs x width 24: N = 1.02 M rows, F = 256, map = 1.04 GB).
    bytes = algorithmic HBM bytes (operands read once, results written once); adds = N * F * m."""
    import torch
    from deepbind_amd import data, kangaroo_smat as ks, smat as sm
    rng = np.random.default_rng(7)
    B, L, m, F = 8192, 101, 24, 256
    codes = rng.integers(0, 4, (B, L), dtype=np.uint8)
    codes[rng.random((B, L)) < 0.01] = 255
    Xh, Rh = data.pack_uniform_ordinals(codes, m - 1)
    X, R = torch.from_numpy(Xh).cuda(), torch.from_numpy(Rh).cuda()
    N = X.numel()
    W = torch.randn(4 * m, F, device="cuda") * 0.1
    b = torch.randn(1, F, device="cuda") * 0.1
    Z = sm.zeros((N, F))
    mapbytes, adds = N * F * 4, float(N) * F * m

    def timed(fn):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    out = {"workload": "%d sequences x %d nt, %d filters of width %d: N = %d rows, map %.2f GB" % (B, L, F, m, N, mapbytes / 1e9)}

    def rec(name, ms, nbytes, nadds=None):
        r = {"ms": ms, "GBs": nbytes / ms / 1e6, "hbm_frac": nbytes / ms / 1e6 / HBM_PEAK_GBS}
        if nadds:
            r["Tadds_s"] = nadds / ms / 1e9
            r["fp32_frac"] = nadds / ms / 1e9 / FP32_VECTOR_PEAK_TFLOPS
        out[name] = r

    rec("corr1ord", timed(lambda: ks.corr1ord(W, X, Z, 4)), N + mapbytes, adds)
    A = sm.relu(sm.add_rowvec(Z, b))
    rec("bias+relu (2 launches)", timed(lambda: sm.relu(sm.add_rowvec(Z, b))), 4 * mapbytes)
    for pt in ("max", "all"):
        nout = B * F * 4 * (2 if pt == "all" else 1)
        rec("poolrgn[%s]" % pt, timed(lambda: ks.poolrgn(A, R, pt, want_argmax=True)), mapbytes + nout + B * F * 4)
        P, I = ks.poolrgn(A, R, pt, want_argmax=True)
        dP = torch.randn_like(P)
        dA = sm.zeros_like(A)
        rec("poolrgn_bprop[%s]" % pt, timed(lambda: ks.poolrgn_bprop(dA, R, dP, I, pt)),
            (2 * mapbytes if pt == "all" else 2 * B * F * 4) + nout)
        del dA
    dZ = torch.randn_like(Z)
    dW = torch.zeros_like(W)
    rec("corr1ord_bprop_W", timed(lambda: ks.corr1ord_bprop_W(dW, X, dZ, 4)), N + mapbytes, adds)
    dX = sm.zeros((N, 4))
    rec("corr1ord_bprop_X", timed(lambda: ks.corr1ord_bprop_X(dX, W, dZ, 4)), mapbytes + N * 16, adds)
    del dZ, Z, A
    db = torch.zeros_like(b)
    for pt in ("max", "all"):
        nout = B * F * 4 * (2 if pt == "all" else 1)
        rec("scanpool_fprop general[%s, argmax]" % pt, timed(lambda: ks.scanpool_fprop(W, b, X, R, pt, want_argmax=True, path="general")),
            N + nout + B * F * 4, adds)
        P, I = ks.scanpool_fprop(W, b, X, R, pt, want_argmax=True, path="general")
        dP = torch.randn_like(P)
        rec("scanpool_bprop[%s]" % pt, timed(lambda: ks.scanpool_bprop(W, b, X, R, pt, P, I, dP, dW, db, overwrite=True)),
            N + 2 * nout + B * F * 4, adds if pt == "all" else float(B) * F * m)
        if pt == "all":
            # with the forward pass leaving 1 bit per (row, filter) for the backward pass (N * F / 8 bytes each way)
            act = ks.activity_words(X, W)
            rec("scanpool_fprop general[all, argmax, masks]", timed(lambda: ks.scanpool_fprop(W, b, X, R, pt, want_argmax=True, act=act)),
                N + nout + B * F * 4 + N * F // 8, adds)
            rec("scanpool_bprop[all, masks]", timed(lambda: ks.scanpool_bprop(W, b, X, R, pt, P, I, dP, dW, db, overwrite=True, act=act)),
                N + 2 * nout + B * F * 4 + N * F // 8, adds)
            del act
    rec("scanpool_fprop table[max]", timed(lambda: ks.scanpool_fprop(W, b, X, R, "max", path="kmer")), N + B * F * 4, adds)
    rec("scanpool_fprop table[max, argmax]", timed(lambda: ks.scanpool_fprop(W, b, X, R, "max", want_argmax=True, path="kmer")),
        N + 2 * B * F * 4, adds)
    rec("scanpool_fprop table[all, argmax]", timed(lambda: ks.scanpool_fprop(W, b, X, R, "all", want_argmax=True, path="kmer")),
        N + 3 * B * F * 4, adds)
    del X, R, W, b, dW, db, dX, P, I, dP
    # shorter filters at bulk-scoring size (65 536 sequences x 101 nt): up to 18 taps the table kernel walks through
    # regions that follow each other without a fresh start
    B2 = 65536
    codes = rng.integers(0, 4, (B2, L), dtype=np.uint8)
    codes[rng.random((B2, L)) < 0.01] = 255
    for m2 in (16, 11, 24):
        Xh, Rh = data.pack_uniform_ordinals(codes, m2 - 1)
        X, R = torch.from_numpy(Xh).cuda(), torch.from_numpy(Rh).cuda()
        W = torch.randn(4 * m2, F, device="cuda") * 0.1
        b = torch.randn(1, F, device="cuda") * 0.1
        for path in ("kmer", "mfma"):
            rec("scanpool_fprop %s[max] %d x %d nt, %d taps" % ("table" if path == "kmer" else "matrix cores", B2, L, m2),
                timed(lambda: ks.scanpool_fprop(W, b, X, R, "max", path=path)), X.numel() + B2 * F * 4, float(X.numel()) * F * m2)
        del X, R, W, b
    # per-model dense layer at bulk-scoring size: 100 000 rows, 64 models, 16 -> 32
    from deepbind_amd import deepity_smat as ds
    n, nb, k, h = 100000, 64, 16, 32
    Xp = torch.randn(n, k * nb, device="cuda")
    W1 = torch.randn(k * nb, h, device="cuda") * 0.1
    dH = torch.randn(n, h * nb, device="cuda")
    io = (n * k * nb + n * h * nb + k * nb * h) * 4
    rec("blockwise_dot 100000x(64x16)->(64x32)", timed(lambda: ds.blockwise_dot(Xp, W1, nb)), io)
    rec("blockwise_dot_nt", timed(lambda: ds.blockwise_dot_nt(dH, W1, nb)), io)
    rec("blockwise_dot_tn", timed(lambda: ds.blockwise_dot_tn(Xp, dH, nb, W1)), io)
    rec("sum_axis0 100000x2048", timed(lambda: sm.sum_axis0(dH)), n * h * nb * 4)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="config5", choices=["config5", "config5_small"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-train", action="store_true", help="skip the secondary train-step throughput figures")
    ap.add_argument("--ops", action="store_true", help="only the per-operator figures of the drop-in and general fused kernels")
    ap.add_argument("--train-only", action="store_true", help="only the train-step figures (for profiling the training kernels)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain copy kernel over 1 GiB (reference point for the HBM byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the path shards over models or sequences with no exchange step, "
                 "and this build runs on a single MI355X (got --gpus %d)" % args.gpus)

    import torch
    from deepbind_amd import kangaroo_smat as ks, deepity_smat as ds, synth
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)

    if args.train_only:
        print(json.dumps({"train": train_throughput(steps=args.steps, warmup=args.warmup, cpu=not args.no_cpu_baseline)}))
        return
    if args.ops:
        print(json.dumps({"ops": ops_throughput()}))
        return
    nseq = 100000 if args.workload == "config5" else 5000
    cfg = synth.config5(seed=4, nseq=nseq)
    spec, p = cfg["spec"], cfg["params"]
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    W, b, X, R = dev(p["Wc"]), dev(p["bc"]), dev(cfg["X"]), dev(cfg["R"])
    W1, b1, W2, b2 = dev(p["W1"]), dev(p["b1"]), dev(p["W2"]), dev(p["b2"])
    positions = synth.positions(cfg["R"])
    adds = float(positions) * spec.F * spec.m

    def step():
        pooled, _ = ks.scanpool_fprop(W, b, X, R, "max")
        return ds.head_fprop(pooled, W1, b1, W2, b2, nblock=spec.nmodel)

    if args.calibrate_copy:
        # elementwise kernel that reads 1 GiB and writes 1 GiB (larger than every cache level)
        src = torch.ones(256 << 20, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        torch.mul(src, 2.0, out=dst)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for k in range(args.steps):
        # events bracket the scan+pool launches only (recorded on the stream they run on)
        ev[k][0].record()
        pooled, _ = ks.scanpool_fprop(W, b, X, R, "max")
        ev[k][1].record()
        scores = ds.head_fprop(pooled, W1, b1, W2, b2, nblock=spec.nmodel)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    scan_ms = float(np.mean([a.elapsed_time(c) for a, c in ev]))
    assert tuple(scores.shape) == (nseq, spec.nmodel) and bool(torch.isfinite(scores).all())

    ms_per_step = elapsed / args.steps * 1e3
    adds_per_s = adds / (scan_ms * 1e-3)
    # algorithmic HBM bytes of the scan+pool launch: sequence bytes in, filters in, pooled features out
    hbm_bytes = cfg["X"].size + p["Wc"].nbytes + p["bc"].nbytes + nseq * spec.F * 4
    out = {
        "metric": "seq_positions_per_sec_fwd_scan_pool",
        "value": positions * args.steps / elapsed,
        "unit": "positions/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s: bulk forward scoring, %d models x %d motifs x width %d, %d DNA sequences x %d nt (1%% N), "
                               "fused scan+bias+relu+maxpool then dense 16->32->1; output %d x %d scores"
                               % (args.workload, spec.nmodel, spec.nfilter, spec.m, nseq, 500, nseq, spec.nmodel),
                   "positions_per_step": positions, "filters": spec.F, "motif_width": spec.m},
        "sequences_per_s": nseq * args.steps / elapsed,
        "model_sequences_per_s": nseq * spec.nmodel * args.steps / elapsed,
        "roofline": {
            # compute-bound on the FP32 vector ALUs (a gather-add: no matrix instruction is issued)
            "bound": "fp32_valu", "bound_detail": "FP32 vector ALU gather-add, no MFMA instruction issued; peak = published 157.3 TFLOP/s FP32 vector "
                                                  "(FMA-counted); a stream of plain adds tops out at 78.6 T adds/s",
            "achieved": adds_per_s / 1e12, "peak": FP32_VECTOR_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": adds_per_s / 1e12 / FP32_VECTOR_PEAK_TFLOPS,
            "frac_vs_add_issue_peak": adds_per_s / 1e12 / FP32_ADD_ISSUE_PEAK_TADDS,
            "traffic": measured_traffic(args.workload),
            "traffic_source": "read from the committed counter profile profiles/scanpool_kmer_config5_counters.md (rocprofv3 --pmc FETCH_SIZE / "
                              "WRITE_SIZE runs of this workload, scaled by a copy kernel of known size); not measured in this run",
            "kernel": "fused scan+bias+relu+maxpool (dbk_scanpool_fprop launches)", "kernel_ms": scan_ms,
            "algorithmic_adds_per_launch": adds,
            "hbm": {"algorithmic_bytes_per_launch": hbm_bytes, "achieved_GBs": hbm_bytes / (scan_ms * 1e-3) / 1e9,
                    "peak_GBs": HBM_PEAK_GBS, "frac": hbm_bytes / (scan_ms * 1e-3) / 1e9 / HBM_PEAK_GBS},
        },
    }
    if not args.no_train:
        out["train"] = train_throughput(cpu=not args.no_cpu_baseline)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, nseq=min(nseq, 1000))
    print(json.dumps(out))


if __name__ == "__main__":
    main()
