"""A batch of independent sequence models on the model axis, and one SGD step on all of them.

Host-side mirror of what the reference's node graph and trainer do for this path, built on the
operators of this package:

  layer order   motif scan -> bias -> ReLU -> max / max+avg pool -> dropout -> dense [-> bias -> ReLU -> dense]
                -> bias -> (logistic) -> nll / mse
                (reference: code/libs/kangaroo/kangaroo/model.py:45-132, code/libs/deepity/deepity/_io_/load.py:51-72,
                 code/cfg/classification/M1.cfg, M2.cfg)
  parameters    one flat vector P with its gradient dP, momentum mP and per-element learning / momentum
                rates; every layer's weights are a view into it. Scan filters put the models side by
                side in columns, dense weights stack them in row blocks
                (reference: code/libs/deepity/deepity/sgd.py:287-354, std/full.py:57, kangaroo/_ext/corr1ord.py:57-58)
  step          Nesterov: P += mu*mP; g = grad(P); mP = mu*mP - eta*g; P -= eta*g
                (reference: code/libs/deepity/deepity/_ext/deepity_smat.py:77-117, sgd.py:121-147)
  L1 decay      sign(W)*decay per model added to the weight gradients once step >= weight_decay_start
                (reference: kangaroo/_ext/corr1ord.py:120-127, deepity/std/full.py:111-119)
  loss          dA = (Z - Y)/nrow, masked by Ymask (reference: deepity/std/loss.py:98-112)

Two execution modes give the same numbers: "fused" runs the scan, bias, ReLU and pooling as one kernel
forward and one backward; "unfused" calls the drop-in operators one by one, as the reference's graph does.
All models of one SequenceNet share pool type and hidden size; a calibration batch that mixes
architectures is run as one SequenceNet per architecture (see ModelGroup).
"""
import ctypes
import weakref

import numpy as np
import torch

from . import _lib
from . import deepity_smat as ds
from . import kangaroo_smat as ks
from . import smat as sm


class SequenceNet(object):
    def __init__(self, nmodel, nfilter, m, pool="max", hidden=32, loss="nll", dtype=torch.float32,
                 rate=0.01, momentum=0.9, decay_conv=0.0, decay_full=0.0, dropout=0.0,
                 weight_decay_start=100, nesterov=True, mode="fused", reverse_complement=False, input_dropout=0.0,
                 start_training=0, feature_columns=0, constraint=None, single_launch=True, device="cuda"):
        assert pool in ("max", "avg", "all") and loss in ("nll", "mse", "hinge", None)
        self.ninst, self.nfilter, self.m = int(nmodel), int(nfilter), int(m)
        self.pool, self.hidden, self.loss = pool, int(hidden), loss
        self.dtype, self.device, self.mode, self.nesterov = dtype, device, mode, nesterov
        self.weight_decay_start = weight_decay_start
        # rows interleaved fwd,rev,fwd,rev,...: each pair shares its dropout draw and only the larger
        # prediction of a pair contributes to loss and gradient
        # (reference: kangaroo/kangaroo/data.py:274-306, deepity/std/loss.py:114-119, deepity_smat/dropout.cu:57-77)
        self.reverse_complement = bool(reverse_complement)
        # input-base dropout: while training each letter is replaced by the "contributes nothing" code with
        # this probability; at test time the scan output is scaled by (1 - rate) instead
        # (reference: kangaroo/_ext/dropoutord.py:42-74, kangaroo/_ext/corr1ord.py:104-109)
        self.input_dropout = float(input_dropout)
        # the scan filters' gradient is zeroed while step < start_training (reference: kangaroo/_ext/corr1ord.py:135-136)
        self.start_training = int(start_training)
        # constraint on the scan filters, enforced before the first step and after every update:
        # "pfm", "psam", a (lo, hi) tuple or None (reference: kangaroo/_ext/corr1ord.py:60-77, deepity/sgd.py:103-107,137)
        self.constraint = constraint
        # small groups (1-4 models, at most 64 filters, regions of at most 256 rows) step in ONE launch
        # (dbk_train_step_single) unless this is switched off; same numbers within tolerance, other summation orders
        self.single_launch = bool(single_launch)
        self._single_rows = {}               # longest region of the region tables seen, by tensor identity and version
        self._single_calls = 0               # single-launch steps issued (their status word is looked at now and then)
        self._last_single = False            # the last natively issued step went through the single-launch kernel
        self.step_count = 0
        self._step_args = None               # argument block and work buffers of the natively issued step
        self._step_bufs = {}
        self._step_sig, self._step_buf, self._step_nesterov = None, None, None
        # Nesterov look-ahead kept beside the parameters by the natively issued step (each step's update kernel
        # leaves the next step's look-ahead there); valid while nothing else has touched P, mP or mrate
        self._L, self._L_versions = None, None
        ni, nf = self.ninst, self.nfilter
        self.k = nf * (2 if pool == "all" else 1)          # pooled features per model
        # the reference's first dense layer (its "combiner") has a second input: a feature matrix with
        # feature_columns columns (16 in its models) that all models share. Each model's block of W1 then has
        # k + feature_columns rows, and the L1 cost and decay cover those rows too. The reference's data source
        # fills that matrix with zeros, which is what a batch without `F` means here.
        # (reference: kangaroo/kangaroo/model.py:101-112, data.py:59-69, deepity/std/full.py:137-178)
        self.nfeat = int(feature_columns)
        kw = self.k + self.nfeat                           # rows of one model's block of W1
        h = self.hidden
        # (name, shape, axis along which models are laid out)
        layout = [("Wc", (4 * m, nf * ni), 1), ("bc", (1, nf * ni), 1)]
        if h > 0:
            layout += [("W1", (kw * ni, h), 0), ("b1", (1, h * ni), 1), ("W2", (h * ni, 1), 0), ("b2", (1, ni), 1)]
        else:
            layout += [("W1", (kw * ni, 1), 0), ("b1", (1, ni), 1)]
        self.layout = layout
        sizes = [int(np.prod(shape)) for _, shape, _ in layout]
        self.offsets = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
        n = int(self.offsets[-1])
        z = lambda: torch.zeros((n, 1), dtype=dtype, device=device)
        self.P, self.dP, self.mP, self.drate, self.mrate = z(), z(), z(), z(), z()
        self.p, self.g = {}, {}
        for (name, shape, _), a, b in zip(layout, self.offsets[:-1], self.offsets[1:]):
            self.p[name] = self.P[a:b].view(shape)
            self.g[name] = self.dP[a:b].view(shape)
        self._per_model = {}
        self.set_rates(rate, momentum)
        self.decay_conv = self._vec(decay_conv)
        self.decay_full = self._vec(decay_full)
        self.decay_vec = self._build_decay_vec()
        self.dropout = self._vec(dropout)
        self.use_dropout = bool(np.any(np.asarray(dropout) > 0))
        # position of the dropout generator, kept on the device so that a captured graph advances it
        self.rng_seed = 0
        self.rng_counter = torch.zeros(1, dtype=torch.int64, device=device)
        self._rng_offset = 0                 # host mirror of rng_counter (layer-by-layer mode draws from it)

    # ------------------------------------------------------------------ parameters
    def _vec(self, v):
        v = np.broadcast_to(np.asarray(v, dtype=np.float64), (self.ninst,)).copy()
        return torch.as_tensor(v, dtype=self.dtype, device=self.device)

    def _k_of(self, name):
        """Elements per model along the flat layout, as the reference computes it for madd_bcast
        (reference: code/libs/deepity/deepity/sgd.py:318-323)."""
        _, shape, axis = [l for l in self.layout if l[0] == name][0]
        per_model = (shape[0] // self.ninst, shape[1]) if axis == 0 else (shape[0], shape[1] // self.ninst)
        return per_model[0] * per_model[1] if axis == 0 else per_model[1]

    def set_rates(self, rate, momentum):
        """Per-model learning and momentum rates spread over the flat vectors."""
        self.drate.zero_()
        self.mrate.zero_()
        ones = torch.ones_like(self.P)
        for (name, _, _), a, b in zip(self.layout, self.offsets[:-1], self.offsets[1:]):
            ds.madd_bcast(ones[a:b], self._vec(rate), self._k_of(name), self.drate[a:b])
            ds.madd_bcast(ones[a:b], self._vec(momentum), self._k_of(name), self.mrate[a:b])

    def set_params(self, params):
        """Copies a dict of NumPy arrays shaped like the layout into the flat parameter vector."""
        for name, shape, _ in self.layout:
            src = np.asarray(params[name])
            assert tuple(src.shape) == tuple(shape), "%s: expected %s, got %s" % (name, shape, src.shape)
            self.p[name].copy_(torch.as_tensor(src, dtype=self.dtype))

    def init_params(self, init_conv=0.01, init_full=0.01, init_mu=0.0, seed=0):
        """Random initial parameters the way the reference's trainer sets them up (deepity/deepity/sgd.py:333-352):
        weights = randn * init (one scale per model, spread with madd_bcast), biases = init_mu.
        init_conv / init_full / init_mu: scalar or one value per model. The normal deviates come from
        the library's generator, so equal seeds give equal parameters."""
        self.P.zero_()
        offset = 0
        for name, shape, axis in self.layout:
            view = self.p[name]
            flat = view.view(-1, 1)
            per = view.numel() // self.ninst if axis == 0 else shape[1] // self.ninst      # block length of one model
            if name.startswith("W"):
                scale = self._vec(init_conv if name == "Wc" else init_full)
                ds.madd_bcast(sm.randn(flat.shape[0], 1, dtype=self.dtype, seed=seed, offset=offset, device=self.device), scale, per, flat)
                offset += (flat.shape[0] + 3) // 4
            elif np.any(np.asarray(init_mu) != 0):
                ds.madd_bcast(torch.ones_like(flat), self._vec(init_mu), per, flat)
        self.mP.zero_()

    def penalty_value(self):
        """Per-model L1 weight cost (1 x ninst) that the reference adds to the reported loss once
        step >= weight_decay_start: decay_conv * sum|Wc| + decay_full * (sum|W1| + sum|W2|).
        (reference: kangaroo/_ext/corr1ord.py:111-115, deepity/std/full.py:92-109)"""
        ni = self.ninst
        if self.weight_decay_start > self.step_count:
            return np.zeros((1, ni))
        p = self.p
        self._check_single_status()
        conv = sm.sum_axis0(sm.mul_sign(p["Wc"], p["Wc"]))                     # |W| summed over taps and channels
        torch.cuda.synchronize()
        cost = conv.cpu().numpy().astype(np.float64).reshape(ni, -1).sum(axis=1) * self.decay_conv.cpu().numpy().ravel()
        for name in ("W1", "W2"):
            if name in p:
                absw = sm.mul_sign(p[name], p[name]).view(ni, -1)                # model-major rows: one row per model
                ones = torch.ones((absw.shape[1], 1), dtype=self.dtype, device=self.device)
                rows = sm.dot(absw.contiguous(), ones)
                torch.cuda.synchronize()
                cost = cost + rows.cpu().numpy().astype(np.float64).ravel() * self.decay_full.cpu().numpy().ravel()
        return cost.reshape(1, ni)

    def enforce_constraints(self):
        """Applies the scan filters' constraint to the parameters in place. The trainer calls it once before the
        first step (after the parameters are set) and train_step calls it after every update."""
        if self.constraint is None:
            return
        ks.corr1ord_enforce_constraints(self.p["Wc"], self.constraint)
        self._L_versions = None              # the look-ahead kept beside the parameters no longer matches them

    def _single_work(self, buf, R):
        """Workspace of the single-launch step for this batch shape, or None when the step does not take it."""
        if "work" not in buf:
            need = ctypes.c_size_t(0)
            _lib.call("dbk_train_step_single_workspace", ctypes.addressof(self._step_args), ctypes.addressof(need))
            buf["work"] = torch.zeros(need.value, dtype=torch.uint8, device=self.P.device) if need.value else None
        if buf["work"] is None:
            return None
        # the longest region of this very tensor object in its present state: an address alone says nothing (a new
        # tensor of a later batch can get the address of a freed one), so the entry holds a weak reference to the tensor
        ent = self._single_rows.get(id(R))
        if ent is None or ent[0]() is not R or ent[1] != R._version:
            if len(self._single_rows) >= 256:
                self._single_rows.clear()
            Rl = R.to(torch.int64)           # one read-back per region table: the kernel keeps whole regions in LDS
            rows = int((Rl[:, 1] - Rl[:, 0]).max().item()) if R.shape[0] else 0
            ent = self._single_rows[id(R)] = (weakref.ref(R), R._version, rows)
        return buf["work"] if ent[2] <= 256 else None

    SINGLE_HEADER = 32768                    # bytes of a single-launch workspace before the gradient shares

    def _check_single_status(self):
        """Raises when a single-launch step flagged its workspace. Such a launch, and every launch after it on that
        workspace, changed nothing (parameters, momentum, generator position), so the host's step counter and
        generator mirror are set back to what the device actually did, and the workspace's header is zeroed so that
        the next step runs again."""
        for buf in self._step_bufs.values():
            work = buf.get("work")
            if work is None:
                continue
            torch.cuda.synchronize()
            stepped, status = (int(v) for v in work[0:8].view(torch.int32).tolist())
            if status:
                dropped = max(buf.get("issued", 0) - stepped, 0)
                work[:self.SINGLE_HEADER].zero_()
                buf["issued"] = 0
                self.step_count -= dropped
                self._rng_offset = int(self.rng_counter.item())
                self._L_versions = None
                raise _lib.DeepbindError("RuntimeError: a single-launch training step was abandoned (%s); %d step(s) were not applied" %
                                         ("a workgroup waited too long" if status == 1 else "a region has more than 256 rows", dropped))

    def _count_single_launch(self, buf):
        """Book-keeping after a single-launch step was issued on the workspace in `buf` (or a graph holding one
        replayed): the status word is looked at every 256 launches, so that an abandoned step does not go unnoticed."""
        buf["issued"] = buf.get("issued", 0) + 1
        self._single_calls += 1
        if self._single_calls % 256 == 0:
            self._check_single_status()

    def get_params(self):
        self._check_single_status()
        torch.cuda.synchronize()
        return {name: self.p[name].cpu().numpy().copy() for name, _, _ in self.layout}

    def get_grads(self):
        self._check_single_status()
        torch.cuda.synchronize()
        return {name: self.g[name].cpu().numpy().copy() for name, _, _ in self.layout}

    # ------------------------------------------------------------------ export
    def _config(self):
        return dict(nfilter=self.nfilter, m=self.m, pool=self.pool, hidden=self.hidden, loss=self.loss or "",
                    reverse_complement=self.reverse_complement, input_dropout=self.input_dropout, feature_columns=self.nfeat)

    def slice_model(self, i):
        """A single-model net holding model i's parameters and dropout rate, for export and prediction
        (reference: slice_inst, deepity/deepity/node.py:148-163; hypertrain.py:136-162)."""
        assert 0 <= i < self.ninst
        one = SequenceNet(1, self.nfilter, self.m, pool=self.pool, hidden=self.hidden, loss=self.loss, dtype=self.dtype,
                          dropout=float(self.dropout[i].item()), mode=self.mode, reverse_complement=self.reverse_complement,
                          input_dropout=self.input_dropout, feature_columns=self.nfeat, device=self.device)
        src = self.get_params()
        picked = {}
        for name, shape, axis in self.layout:
            blocks = np.split(src[name], self.ninst, axis=axis)
            picked[name] = blocks[i]
        one.set_params(picked)
        return one

    def save_npz(self, path):
        """Writes the architecture and the parameters of a single-model net to one .npz file."""
        assert self.ninst == 1, "slice one model out first"
        cfg = self._config()
        arrays = {"cfg_" + k: np.asarray(v) for k, v in cfg.items()}
        arrays["cfg_dropout"] = np.asarray(float(self.dropout[0].item()))
        arrays.update({"p_" + k: v for k, v in self.get_params().items()})
        np.savez(path, **arrays)

    @staticmethod
    def load_npz(path, device="cuda", mode="fused"):
        with np.load(path, allow_pickle=False) as f:
            cfg = {k[4:]: f[k].item() for k in f.files if k.startswith("cfg_")}
            params = {k[2:]: f[k] for k in f.files if k.startswith("p_")}
        net = SequenceNet(1, int(cfg["nfilter"]), int(cfg["m"]), pool=str(cfg["pool"]), hidden=int(cfg["hidden"]),
                          loss=(str(cfg["loss"]) or None), dropout=float(cfg["dropout"]), mode=mode,
                          reverse_complement=bool(cfg["reverse_complement"]), input_dropout=float(cfg["input_dropout"]),
                          feature_columns=int(cfg.get("feature_columns", 0)), device=device)
        net.set_params(params)
        return net

    # ------------------------------------------------------------------ forward
    def _drop_inputs(self, X, R, U_input=None):
        """Training-time input dropout; draws come from this net's generator position (device counter in
        fused mode, its host mirror layer by layer) unless uniforms are supplied."""
        if self.input_dropout <= 0:
            return X
        kw = dict(regions=R if self.reverse_complement else None, padding=self.m - 1, seed=self.rng_seed)
        if U_input is not None:
            return ks.dropoutord_fp_train(X, self.input_dropout, U=U_input, **kw)[0]
        draws = (X.numel() + 3) // 4
        if self.mode == "fused":
            Z = ks.dropoutord_fp_train(X, self.input_dropout, counter=self.rng_counter, **kw)[0]
        else:
            Z = ks.dropoutord_fp_train(X, self.input_dropout, offset=self._rng_offset, **kw)[0]
        ds.counter_add(self.rng_counter, draws)
        self._rng_offset += draws
        return Z

    def _conv_forward(self, X, R, want_argmax, train=False):
        p = self.p
        keep = 1.0 if (train or self.input_dropout <= 0) else 1.0 - self.input_dropout
        if self.mode == "fused":
            # test-time rescale folded into the filters (sum of scaled taps instead of scaled sum)
            Wc = p["Wc"] if keep == 1.0 else p["Wc"] * keep
            pooled, amax = ks.scanpool_fprop(Wc, p["bc"], X, R, self.pool, want_argmax=want_argmax)
            return pooled, amax, None
        Z = sm.zeros((X.numel(), p["Wc"].shape[1]), dtype=self.dtype, device=self.device)
        ks.corr1ord(p["Wc"], X, Z, 4)
        if keep != 1.0:
            Z *= keep
        A = sm.relu(sm.add_rowvec(Z, p["bc"]))
        pooled, amax = ks.poolrgn(A, R, self.pool, want_argmax=want_argmax)
        return pooled, amax, A

    def _features(self, F, n):
        """The batch's shared feature matrix (n, feature_columns); None means the reference's all-zero one."""
        if F is None:
            return torch.zeros((n, self.nfeat), dtype=self.dtype, device=self.device)
        _lib.require(F.dtype == self.dtype and tuple(F.shape) == (n, self.nfeat), "ValueError: F must be (rows, feature_columns) of the net's dtype")
        return F

    def _dense1(self, H0, F):
        """First dense layer: the pooled features, or [pooled features | shared feature columns] stacked along
        each model's rows of W1 (reference: deepity/std/full.py:154-160)."""
        if self.nfeat == 0:
            return ds.blockwise_dot(H0, self.p["W1"], self.ninst)
        return ds.blockwise_dot_combined([H0, self._features(F, H0.shape[0])], self.p["W1"], self.ninst, [False, True])

    def _dense1_back(self, H0, F, dA1, want_dW=True):
        """(dW1, dH0) of the first dense layer (reference: deepity/std/full.py:162-178)."""
        W1, ni = self.p["W1"], self.ninst
        if self.nfeat == 0:
            return (ds.blockwise_dot_tn(H0, dA1, ni, W1) if want_dW else None), ds.blockwise_dot_nt(dA1, W1, ni)
        Xs = [H0, self._features(F, H0.shape[0])]
        dW = ds.blockwise_dot_tn_combined(Xs, dA1, W1, ni, [False, True]) if want_dW else None
        return dW, ds.blockwise_dot_nt_combined(Xs, dA1, W1, ni, [False, True])[0]

    def forward(self, X, R, train=False, U=None, want_argmax=False, F=None):
        """Returns the state dict of one forward pass; st["Z"] are the predictions (n x ninst)."""
        p, ni = self.p, self.ninst
        st = {}
        st["pooled"], st["argmax"], st["A0"] = self._conv_forward(X, R, want_argmax, train=train)
        H0 = st["pooled"]
        if self.use_dropout:
            if train:
                if U is None and not self.reverse_complement:
                    # same stream position as the fused head would use
                    U = ds.uniform_like(H0, self.rng_seed, self._rng_offset)
                    self._rng_offset += (H0.numel() + 3) // 4
                    ds.counter_add(self.rng_counter, (H0.numel() + 3) // 4)
                H0, st["M"] = ds.dropout_fp_train(H0, self.dropout, self.reverse_complement, U=U)
            else:
                H0 = ds.dropout_fp_test(H0, self.dropout)
        st["H0"], st["F"] = H0, F
        A1 = sm.add_rowvec(self._dense1(H0, F), p["b1"])
        if self.hidden > 0:
            st["H1"] = sm.relu(A1)
            A2 = sm.add_rowvec(ds.blockwise_dot(st["H1"], p["W2"], ni), p["b2"])
        else:
            A2 = A1
        st["A"] = A2
        st["Z"] = sm.logistic(A2) if self.loss == "nll" else A2
        if self.reverse_complement:
            st["Zmask"] = torch.zeros(st["Z"].shape, dtype=torch.bool, device=self.device)
            ds.calc_Zmask(st["Z"], st["Zmask"])
        return st

    def predict(self, X, R, F=None):
        """Test-mode predictions through the fused scoring head (dropout rescale folded in)."""
        p = self.p
        pooled, _, _ = self._conv_forward(X, R, False)
        if self.dtype != torch.float32:
            Z = self.forward(X, R, F=F)["Z"]
            return ds.pair_max(Z) if self.reverse_complement else Z
        scale = (1.0 - self.dropout) if self.use_dropout else None
        if F is not None:
            self._features(F, pooled.shape[0])
        Z = ds.head_fprop(pooled, p["W1"], p["b1"], p.get("W2"), p.get("b2"), nblock=self.ninst,
                          in_scale=scale, apply_logistic=(self.loss == "nll"), nfeat=self.nfeat, feats=F)
        return ds.pair_max(Z) if self.reverse_complement else Z

    def input_gradients(self, X, R, F=None):
        """Test-mode predictions plus the gradient map used for sequence logos / mutation maps:
        returns (Z (rows, ninst), dX (N, 4)) where dX is the back-propagated gradient w.r.t. the
        one-hot inputs of dA = Z (targets 0, no batch mean, output column 0 only, and with
        reverse complements only each pair's larger prediction). Runs layer by layer because the
        backward pass needs the full (N, F) activation map.
        (reference: deepity/deepity/node.py:298-341, kangaroo/kangaroo/predict.py:168-193,
        kangaroo/_ext/corr1ord.py:129-133, deepity/std/elemwise.py:148-157)"""
        p, ni = self.p, self.ninst
        Z0 = sm.zeros((X.numel(), p["Wc"].shape[1]), dtype=self.dtype, device=self.device)
        ks.corr1ord(p["Wc"], X, Z0, 4)
        if self.input_dropout > 0:
            Z0 *= 1.0 - self.input_dropout           # forward only: the reference's backward pass ignores this factor too
        A0 = sm.relu(sm.add_rowvec(Z0, p["bc"]))
        pooled, amax = ks.poolrgn(A0, R, self.pool, want_argmax=True)
        H0 = ds.dropout_fp_test(pooled, self.dropout) if self.use_dropout else pooled
        A1 = sm.add_rowvec(self._dense1(H0, F), p["b1"])
        if self.hidden > 0:
            H1 = sm.relu(A1)
            A2 = sm.add_rowvec(ds.blockwise_dot(H1, p["W2"], ni), p["b2"])
        else:
            A2 = A1
        Z = sm.logistic(A2) if self.loss == "nll" else A2
        dA = Z.clone()
        if self.reverse_complement:
            Zmask = torch.zeros(Z.shape, dtype=torch.bool, device=self.device)
            ds.calc_Zmask(Z, Zmask)
            ds.maskout(Zmask, dA)
        if dA.shape[1] > 1:
            dA[:, 1:] = 0
        dA1 = sm.mul_sign(ds.blockwise_dot_nt(dA, p["W2"], ni), H1) if self.hidden > 0 else dA
        dH0 = self._dense1_back(H0, F, dA1, want_dW=False)[1]
        if self.use_dropout:
            dH0 = ds.dropout_bp_te(dH0, self.dropout)
        dA0 = sm.zeros_like(A0)
        ks.poolrgn_bprop(dA0, R, dH0, amax, self.pool)
        dZ0 = sm.mul_sign(dA0, A0)
        dX = sm.zeros((X.numel(), 4), dtype=self.dtype, device=self.device)
        ks.corr1ord_bprop_X(dX, p["Wc"], dZ0, 4)
        return Z, dX

    def loss_value(self, st, Y, Ymask=None):
        """Per-model mean loss (1 x ninst), on the host (reference: deepity/std/loss.py:52-82)."""
        L = sm.loss_terms(st["Z"], Y, self.loss)
        if Ymask is not None:
            ds.maskout(Ymask, L)
        if "Zmask" in st:
            ds.maskout(st["Zmask"], L)
        L = sm.sum_axis0(L)
        torch.cuda.synchronize()
        L = L.cpu().numpy() / st["Z"].shape[0]
        return -L if self.loss == "nll" else (L if self.loss == "hinge" else 0.5 * L)

    # ------------------------------------------------------------------ backward
    def backward(self, X, R, st, Y, Ymask=None):
        """Fills dP with the gradient of the summed per-model losses (plus L1 decay when active)."""
        p, g, ni = self.p, self.g, self.ninst
        dA = (sm.hinge_grad if self.loss == "hinge" else sm.sub_scale)(st["Z"], Y, 1.0 / st["Z"].shape[0])
        if Ymask is not None:
            ds.maskout(Ymask, dA)
        if "Zmask" in st:
            ds.maskout(st["Zmask"], dA)
        if self.hidden > 0:
            g["b2"].copy_(sm.sum_axis0(dA))
            g["W2"].copy_(ds.blockwise_dot_tn(st["H1"], dA, ni, p["W2"]))
            dA1 = sm.mul_sign(ds.blockwise_dot_nt(dA, p["W2"], ni), st["H1"])
        else:
            dA1 = dA
        g["b1"].copy_(sm.sum_axis0(dA1))
        dW1, dH0 = self._dense1_back(st["H0"], st.get("F"), dA1)
        g["W1"].copy_(dW1)
        if self.use_dropout:
            dH0 = ds.dropout_bp_tr(dH0, st["M"]) if "M" in st else ds.dropout_bp_te(dH0, self.dropout)
        if self.mode == "fused":
            ks.scanpool_bprop(p["Wc"], p["bc"], X, R, self.pool, st["pooled"], st["argmax"], dH0, g["Wc"], g["bc"], overwrite=True)
        else:
            g["Wc"].zero_()
            dA0 = sm.zeros_like(st["A0"])
            ks.poolrgn_bprop(dA0, R, dH0, st["argmax"], self.pool)
            dZ0 = sm.mul_sign(dA0, st["A0"])
            g["bc"].copy_(sm.sum_axis0(dZ0))
            ks.corr1ord_bprop_W(g["Wc"], X, dZ0, 4)
        if self.weight_decay_start <= self.step_count:
            self._add_decay()
        if self.step_count < self.start_training:
            g["Wc"].zero_()

    def _build_decay_vec(self):
        """One L1 coefficient per element of the flat parameter vector (zero for biases): what
        madd_bcast(sign(W), decay, k, dW) multiplies each sign by (reference: deepity/std/full.py:111-119)."""
        ni = self.ninst
        vec = torch.zeros_like(self.P)
        ones = torch.ones_like(self.P)
        span = {name: (int(a), int(b)) for (name, _, _), a, b in zip(self.layout, self.offsets[:-1], self.offsets[1:])}
        view = lambda name, t: t[span[name][0]:span[name][1]]
        # the reference passes rows/ninst as the block length for the scan filters although their
        # models lie along columns (kangaroo/_ext/corr1ord.py:126); kept as is for step parity
        kq = max(1, self.p["Wc"].shape[0] // ni)
        ds.madd_bcast(view("Wc", ones), self.decay_conv, kq, view("Wc", vec))
        for name in ("W1", "W2"):
            if name in self.p:
                ds.madd_bcast(view(name, ones), self.decay_full, self.p[name].numel() // ni, view(name, vec))
        return vec

    def _add_decay(self):
        ds.l1_decay(self.P, self.decay_vec, self.dP)

    def _grad_fused(self, X, R, Y, Ymask, U, U_input=None, F=None):
        """Gradient of one batch in a handful of launches: fused scan+pool forward, the whole dense head
        forward+backward (+ chunk reduction), fused scan+pool backward (+ slab reduction)."""
        p, g = self.p, self.g
        X = self._drop_inputs(X, R, U_input)
        # average pooling: the forward pass leaves 1 bit per (row, filter), rectifier open or not, for the backward pass
        act = ks.activity_words(X, p["Wc"]) if self.pool != "max" else None
        pooled, amax = ks.scanpool_fprop(p["Wc"], p["bc"], X, R, self.pool, want_argmax=True, act=act)
        rate = self.dropout if self.use_dropout else None
        draws = (pooled.numel() + 3) // 4 if (rate is not None and U is None) else 0
        Z, dpooled, _ = ds.head_train(pooled, p["W1"], p["b1"], p.get("W2"), p.get("b2"), Y, self.ninst, self.loss,
                                      g["W1"], g["b1"], g.get("W2"), g.get("b2"), Ymask=Ymask, rate=rate, U=U,
                                      seed=self.rng_seed, counter=self.rng_counter, counter_advance=draws,
                                      reverse_complement=self.reverse_complement, nfeat=self.nfeat, feats=F)
        self._rng_offset += draws
        ks.scanpool_bprop(p["Wc"], p["bc"], X, R, self.pool, pooled, amax, dpooled, g["Wc"], g["bc"], overwrite=True, act=act)
        if self.weight_decay_start <= self.step_count:
            self._add_decay()
        if self.step_count < self.start_training:
            g["Wc"].zero_()
        return Z

    # ------------------------------------------------------------------ one optimiser step
    def _prepare_step(self, X, R, Y, Ymask=None, F=None):
        """Fills this net's dbk_train_step_args block for one step on the batch and returns the step's work
        buffers (made on the current stream, where the step is issued)."""
        a = self._step_args
        # the same batch tensors as in the previous step (a training loop over resident batches): only the switches move
        sig = (X.data_ptr(), X.numel(), R.data_ptr(), R.shape[0], R._version, Y.data_ptr(), Y.numel(),
               None if Ymask is None else Ymask.data_ptr(), None if F is None else F.data_ptr())
        if a is not None and sig == self._step_sig and not self.nesterov_changed():
            if self.nesterov:
                versions = (self.P._version, self.mP._version, self.mrate._version)
                a.L_ready = int(self._L_versions == versions)
                self._L_versions = versions
            a.decay = self.decay_vec.data_ptr() if self.weight_decay_start <= self.step_count else None
            a.freeze_scan = int(self.step_count < self.start_training)
            return self._step_buf
        ks._u8(X)
        ks._regions(R)
        ni, P = self.ninst, R.shape[0]
        _lib.require(R.shape[1] == 2, "ValueError: the fused path takes 2-column regions")
        _lib.require(Y.dtype == torch.float32 and tuple(Y.shape) == (P, ni), "ValueError: Y must be float32 (rows x models)")
        _lib.require(Ymask is None or (Ymask.dtype == torch.bool and tuple(Ymask.shape) == (P, ni)), "ValueError: Ymask must be bool (rows x models)")
        if a is None:
            a = self._step_args = _lib.TrainStepArgs()
            off = {name: int(o) for (name, _, _), o in zip(self.layout, self.offsets[:-1])}
            a.nmodel, a.nfilter, a.m, a.hidden = ni, self.nfilter, self.m, self.hidden
            a.ptype, a.loss_kind = _lib.str2pooltype[self.pool], _lib.LOSS_KIND[self.loss]
            a.reverse_complement = int(self.reverse_complement)
            a.nparam = self.P.numel()
            a.P, a.dP, a.mP = self.P.data_ptr(), self.dP.data_ptr(), self.mP.data_ptr()
            a.drate, a.mrate = self.drate.data_ptr(), self.mrate.data_ptr()
            a.off_Wc, a.off_bc, a.off_W1, a.off_b1 = off["Wc"], off["bc"], off["W1"], off["b1"]
            a.off_W2, a.off_b2 = off.get("W2", 0), off.get("b2", 0)
            a.rate = self.dropout.data_ptr() if self.use_dropout else None
            a.counter = self.rng_counter.data_ptr()
        key = (X.numel(), P)
        buf = self._step_bufs.get(key)
        if buf is None:
            if len(self._step_bufs) >= 4:
                self._step_bufs.clear()
            dev = self.P.device
            buf = self._step_bufs[key] = dict(
                pooled=torch.empty((P, self.k * ni), dtype=torch.float32, device=dev),
                dpooled=torch.empty((P, self.k * ni), dtype=torch.float32, device=dev),
                argmax=torch.empty((P, self.nfilter * ni), dtype=ks.uindex, device=dev) if self.pool != "avg" else None,
                Z=torch.empty((P, ni), dtype=torch.float32, device=dev),
                act=ks.activity_words(X, self.p["Wc"]) if self.pool != "max" else None,
                Xdrop=torch.empty(X.numel(), dtype=torch.uint8, device=dev) if self.input_dropout > 0 else None,
                Mdrop=torch.empty(X.numel(), dtype=torch.bool, device=dev) if self.input_dropout > 0 else None)
        a.nesterov, a.seed = int(bool(self.nesterov)), int(self.rng_seed)
        if self.nesterov:
            if self._L is None:
                self._L = torch.empty_like(self.P)
            a.L = self._L.data_ptr()
            # in-place changes made through torch (set_params, set_rates, a view written by the caller) move these counters;
            # the wrappers that write through raw pointers (the layer-by-layer and the graphed step) reset _L_versions
            versions = (self.P._version, self.mP._version, self.mrate._version)
            a.L_ready = int(self._L_versions == versions)
            self._L_versions = versions
        else:
            a.L, a.L_ready = None, 0
        pv = lambda t: None if t is None else _lib.ptr(t).value          # checks device + contiguity
        a.X, a.N, a.regions, a.nregion = pv(X), X.numel(), pv(R), P
        a.Y, a.Ymask = pv(Y), pv(Ymask)
        _lib.require(F is None or (F.dtype == torch.float32 and tuple(F.shape) == (P, self.nfeat)), "ValueError: F must be float32 (rows x feature_columns)")
        a.nfeat, a.feats = self.nfeat, pv(F)
        a.input_rate = self.input_dropout
        for name, t in buf.items():
            if name not in ("work", "issued"):
                setattr(a, name, None if t is None else t.data_ptr())
        a.decay = self.decay_vec.data_ptr() if self.weight_decay_start <= self.step_count else None
        a.freeze_scan = int(self.step_count < self.start_training)
        a.loss = None
        self._step_sig, self._step_buf, self._step_nesterov = sig, buf, (bool(self.nesterov), int(self.rng_seed))
        return buf

    def nesterov_changed(self):
        return self._step_nesterov != (bool(self.nesterov), int(self.rng_seed))

    def _finish_step(self, X, R):
        """Host-side mirrors of what a natively issued step moved on the device."""
        if self.input_dropout > 0:
            self._rng_offset += (X.numel() + 3) // 4
        if self.use_dropout:
            self._rng_offset += (R.shape[0] * self.k * self.ninst + 3) // 4
        self.step_count += 1

    def _native_step(self, X, R, Y, Ymask=None, F=None):
        """One fused step through dbk_train_step: one library call issues every launch of the step (the
        scripting host otherwise pays several microseconds per launch, which is what bounds a step on a
        small minibatch). Same kernels in the same order as gradstep(..., _grad_fused), so the same bits."""
        buf = self._prepare_step(X, R, Y, Ymask, F)
        work = self._single_work(buf, R) if self.single_launch else None
        if work is not None:
            _lib.call("dbk_train_step_single", _lib.stream(), ctypes.addressof(self._step_args), _lib.ptr(work), work.numel())
            self._L_versions = None          # (this kernel forms the look-ahead itself and leaves none behind)
        else:
            _lib.call("dbk_train_step", _lib.stream(), ctypes.addressof(self._step_args))
        self._last_single = work is not None
        self._finish_step(X, R)
        if work is not None and not torch.cuda.is_current_stream_capturing():
            self._count_single_launch(buf)   # (may raise: a step that was abandoned must not be trained over in silence)
        self.enforce_constraints()
        return buf["Z"]

    def make_graphed_step(self, X, R, Y, Ymask=None, F=None, force_graph=False):
        """Captures one fused training step on the given (static) batch tensors into a HIP graph and
        returns a function that replays it: for launch-bound batch sizes the step then costs one
        graph launch instead of ~10 kernel launches. Dropout masks stay fresh on every replay because
        the generator position lives in device memory. The graph bakes in whether L1 decay is
        active and whether the scan filters are still frozen, so it is re-captured when the step
        counter crosses weight_decay_start or start_training.
        A step that the single-launch kernel takes is ONE launch already, and replaying a graph of one
        node costs more than issuing that launch (measured 22 against 12 us per step), so for such a
        net the function returned issues the step natively unless force_graph is set."""
        fused = self.mode == "fused" and self.dtype == torch.float32 and self.loss is not None
        if fused and self.single_launch and not force_graph:
            if self._single_work(self._prepare_step(X, R, Y, Ymask, F), R) is not None:
                return lambda: self._native_step(X, R, Y, Ymask, F)
        return _graphed_step([(self, X, R, Y, Ymask, F)])

    def train_step(self, X, R, Y, Ymask=None, U=None, U_input=None, F=None):
        """One optimiser step. U / U_input optionally supply the uniforms of the pooled-feature and the
        input dropout (otherwise the library's generator draws them). F: the batch's shared feature matrix
        (rows x feature_columns), None for all zeros."""
        fused = self.mode == "fused" and self.dtype == torch.float32 and self.loss is not None
        if fused and U is None and U_input is None:
            self._native_step(X, R, Y, Ymask, F)
            return

        self._L_versions = None                 # the step below updates P and mP in place

        def grad():
            if fused:
                self._grad_fused(X, R, Y, Ymask, U, U_input, F)
            else:
                Xd = self._drop_inputs(X, R, U_input)
                st = self.forward(Xd, R, train=True, U=U, want_argmax=True, F=F)
                self.backward(Xd, R, st, Y, Ymask)
        ds.gradstep(self.P, self.dP, self.drate, self.mP, self.mrate, grad, nesterov=self.nesterov)
        self.step_count += 1
        self.enforce_constraints()


def _native_steps(jobs):
    """jobs: list of (net, X, R, Y, Ymask[, F]), nets that step on the same batch. One dbk_train_steps call per eight
    nets on the current stream: every phase of the step is one launch holding all the nets' grids, so nets too
    small to fill the GPU run side by side without extra streams. Each net gets the bits of its own step."""
    if len(jobs) == 1:
        net, X, R, Y, Ymask, *rest = jobs[0]
        net._native_step(X, R, Y, Ymask, rest[0] if rest else None)
        return
    for i in range(0, len(jobs), 8):
        chunk = jobs[i:i + 8]
        blocks = (ctypes.c_void_p * len(chunk))()
        for j, (net, X, R, Y, Ymask, *rest) in enumerate(chunk):
            net._prepare_step(X, R, Y, Ymask, rest[0] if rest else None)
            blocks[j] = ctypes.addressof(net._step_args)
        _lib.call("dbk_train_steps", _lib.stream(), len(chunk), blocks)
        for net, X, R, *_ in chunk:
            net._last_single = False
            net._finish_step(X, R)
            net.enforce_constraints()


def _side_by_side(streams, jobs):
    """Runs job i on streams[i], all forked from the current stream and joined back into it. The nets of
    a group share nothing but read-only inputs, so their small kernels can fill the GPU together.
    (All streams have the default priority; the library keeps its scratch memory per stream.)"""
    cur = torch.cuda.current_stream()
    for s, job in zip(streams, jobs):
        s.wait_stream(cur)
        with torch.cuda.stream(s):
            job()
    for s in streams[:len(jobs)]:
        cur.wait_stream(s)


def _graphed_step(jobs):
    """jobs: list of (net, X, R, Y, Ymask, F) with static device tensors. Returns step(): one replay of a
    HIP graph holding one fused training step of every net (several nets share each launch).
    Two graphs are captured: one whose step forms the look-ahead parameters itself, and one that takes the look-ahead the
    previous step's update left behind (as a natively issued step does). A replay uses the second whenever the step
    before it was such a step and nothing has touched the parameters since (torch's version counters tell)."""
    for net, *_ in jobs:
        assert net.mode == "fused" and net.dtype == torch.float32 and net.loss is not None
    state = {"graphs": None, "decay": None}

    def decay_flags():
        return tuple((net.weight_decay_start <= net.step_count, net.step_count < net.start_training) for net, *_ in jobs)

    def versions(net):
        return (net.P._version, net.mP._version, net.mrate._version)

    def keeps_lookahead(net):
        # (the filters' constraint rewrites the parameters after the update: the look-ahead beside them is stale then)
        return bool(net.nesterov) and net.constraint is None

    def body(ready):
        # the natively issued step on the capturing stream, with or without a look-ahead to start from
        for net, *_ in jobs:
            net._L_versions = versions(net) if (ready and keeps_lookahead(net)) else None
        _native_steps(jobs)

    def capture():
        # The library's scratch buffers belong to a stream and cannot grow under capture: run the step
        # once eagerly on the stream the capture will use (state is restored after it), then capture there.
        if "stream" not in state:
            state["stream"] = torch.cuda.Stream()
        cap = state["stream"]
        live = [t for net, *_ in jobs for t in (net.P, net.mP, net.dP, net.rng_counter)]
        saved = [t.clone() for t in live]
        host_off = [(net._rng_offset, net.step_count) for net, *_ in jobs]
        cap.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(cap):
            body(False)
        torch.cuda.synchronize()
        for t, s_ in zip(live, saved):
            t.copy_(s_)
        for (net, *_), (off, count) in zip(jobs, host_off):
            net._rng_offset, net.step_count = off, count        # the warm-up step must not count (decay / freeze switches are baked in)
        torch.cuda.synchronize()
        graphs = {}
        for ready in (False, True):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=cap):
                body(ready)
            # capturing executes nothing on the device; only the host mirrors of the step moved
            for (net, *_), (off, count) in zip(jobs, host_off):
                net._rng_offset, net.step_count = off, count
            graphs[ready] = g
        for net, *_ in jobs:
            net._L_versions = None              # (the warm-up step's look-ahead belongs to parameters that were put back)
        state["graphs"], state["decay"] = graphs, decay_flags()
        state["single"] = [(net, net._step_buf) for net, *_ in jobs if net._last_single]      # workspaces of single-launch steps in the graph

    def step():
        if state["graphs"] is None or state["decay"] != decay_flags():
            capture()
        ready = all(keeps_lookahead(net) and net._L_versions == versions(net) for net, *_ in jobs)
        state["graphs"][ready].replay()
        for net, X, R, *_ in jobs:
            # the update left the look-ahead of the new parameters (written through raw pointers: the counters stand still)
            net._L_versions = versions(net) if (keeps_lookahead(net) and not net._last_single) else None
            if net.input_dropout > 0:
                net._rng_offset += (X.numel() + 3) // 4
            if net.use_dropout:
                net._rng_offset += (R.shape[0] * net.k * net.ninst + 3) // 4
            net.step_count += 1
        for net, buf in state["single"]:
            net._count_single_launch(buf)

    return step


class ModelGroup(object):
    """A calibration batch whose models differ in pool type / hidden size: one SequenceNet per
    architecture, all stepped on the same shared batch. Column j of the outputs is model j of the
    original ordering."""

    def __init__(self, pools, hiddens, nfilter, m, loss="nll", **per_model):
        self.nmodel = len(pools)
        keys = sorted(set(zip(pools, hiddens)))
        self.groups = []
        for key in keys:
            idx = [j for j in range(self.nmodel) if (pools[j], hiddens[j]) == key]
            kw = {k: (np.asarray(v)[idx] if np.ndim(v) else v) for k, v in per_model.items()}
            self.groups.append((idx, SequenceNet(len(idx), nfilter, m, pool=key[0], hidden=key[1], loss=loss, **kw)))
        self.streams = None
        self._batch_key, self._batch, self._targets = None, None, None

    def _streams(self):
        if self.streams is None:
            self.streams = [torch.cuda.Stream() for _ in self.groups]
        return self.streams

    def train_step(self, X, R, Y, Ymask=None, U=None, F=None):
        """One step of every architecture group on the shared batch: one native call whose every launch
        holds the grids of all the groups (dbk_train_steps), on the current stream. The groups' small
        kernels thereby run side by side without side streams or events; each group gets the bits of a
        step of its own.
        U, when given, is a list with one uniforms tensor per architecture group (see self.groups); that
        path goes through the layer wrappers, one group per side stream."""
        native = U is None and all(net.mode == "fused" and net.dtype == torch.float32 and net.loss is not None
                                   for _, net in self.groups)
        if not native:
            def one(gi, idx, net):
                def run():
                    ii = torch.as_tensor(idx, device=Y.device)
                    Yg = Y.index_select(1, ii).contiguous()
                    Mg = Ymask.index_select(1, ii).contiguous() if Ymask is not None else None
                    net.train_step(X, R, Yg, Mg, U=None if U is None else U[gi], F=F)
                return run
            _side_by_side(self._streams(), [one(gi, idx, net) for gi, (idx, net) in enumerate(self.groups)])
            return
        key = tuple((t.data_ptr(), t._version, tuple(t.shape)) for t in (X, R, Y, Ymask) if t is not None)
        if key != self._batch_key:
            # each group's columns of the targets, kept until the batch changes
            self._targets = []
            for idx, _ in self.groups:
                ii = torch.as_tensor(idx, device=Y.device)
                self._targets.append((Y.index_select(1, ii).contiguous(),
                                      Ymask.index_select(1, ii).contiguous() if Ymask is not None else None))
            self._batch_key, self._batch = key, (X, R, Y, Ymask)
        _native_steps([(net, X, R, Yg, Mg, F) for (_, net), (Yg, Mg) in zip(self.groups, self._targets)])

    def make_graphed_step(self, X, R, Y, Ymask=None, F=None):
        """One HIP graph holding the fused training step of every architecture group on a static batch."""
        jobs = []
        for idx, net in self.groups:
            ii = torch.as_tensor(idx, device=Y.device)
            jobs.append((net, X, R, Y.index_select(1, ii).contiguous(),
                         Ymask.index_select(1, ii).contiguous() if Ymask is not None else None, F))
        return _graphed_step(jobs)

    def slice_model(self, j):
        """Single-model net for model j of the original ordering."""
        for idx, net in self.groups:
            if j in idx:
                return net.slice_model(idx.index(j))
        raise IndexError(j)

    def predict(self, X, R, F=None):
        out = torch.empty((R.shape[0], self.nmodel), dtype=torch.float32, device=X.device)
        for idx, net in self.groups:
            out[:, torch.as_tensor(idx, device=X.device)] = net.predict(X, R, F)
        return out
