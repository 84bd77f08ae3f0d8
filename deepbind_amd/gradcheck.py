"""Numerical check of a SequenceNet's gradient, the reference's opt-in trainer check
(code/libs/deepity/deepity/gradcheck.py:42-130): with dropout in test mode, the back-propagated
gradient of every parameter block is compared with central finite differences of the summed cost
(mean loss per model plus the L1 weight cost once it is active) on the first `ncheck` elements of
the block; step 1e-8 in float64 and 1e-4 in float32, rtol 1e-5, atol 1e-4 as in the reference.
Everything is evaluated by the library's kernels, layer by layer (the path that supports float64).
"""
import numpy as np
import torch


def _cost(net, X, R, Y, Ymask):
    st = net.forward(X, R, train=False)
    return float(np.sum(net.loss_value(st, Y, Ymask)) + np.sum(net.penalty_value()))


def gradcheck(net, X, R, Y, Ymask=None, ncheck=50, rtol=1e-5, atol=1e-4):
    """Raises AssertionError naming the parameter block and the offending elements; returns the number of
    elements checked otherwise."""
    st = net.forward(X, R, train=False, want_argmax=True)
    net.backward(X, R, st, Y, Ymask)
    torch.cuda.synchronize()
    step = 1e-8 if net.dtype == torch.float64 else 1e-4
    failures, checked = {}, 0
    for (name, shape, _), a, b in zip(net.layout, net.offsets[:-1], net.offsets[1:]):
        P = net.P[a:b].view(-1)
        dP = net.dP[a:b].view(-1).cpu().numpy()
        for i in range(min(len(dP), ncheck)):
            x = float(P[i].item())
            P[i] = x - step
            c0 = _cost(net, X, R, Y, Ymask)
            P[i] = x + step
            c1 = _cost(net, X, R, Y, Ymask)
            P[i] = x
            num, sym = (c1 - c0) / (2 * step), float(dP[i])
            checked += 1
            if not np.allclose(num, sym, rtol=rtol, atol=atol) or not np.allclose(sym, num, rtol=rtol, atol=atol):
                failures.setdefault(name, []).append((i, num, sym))
    if failures:
        msg = "gradient check FAILED\n"
        for name, items in failures.items():
            msg += "   %s FAILED at weights:\n" % name
            for i, num, sym in items[:9]:
                msg += "\t\t[%d] num: %.8f sym: %.8f\n" % (i, num, sym)
        raise AssertionError(msg)
    return checked
