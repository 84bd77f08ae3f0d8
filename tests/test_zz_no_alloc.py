"""The allocation-free entry point of the table kernel (scratch built into the library) against the ordinary one."""
import numpy as np
import pytest
import torch

from tests.gpu_util import dev, host, random_codes

pytestmark = pytest.mark.gpu


def _batch(rng, nseq, L, m, pn=0.02, p254=0.0):
    from deepbind_amd import data
    codes = random_codes(rng, nseq * L, pn=pn, p254=p254).reshape(nseq, L)
    return data.pack_uniform_ordinals(codes, m - 1)


def test_static_scratch_entry_point_matches_the_allocating_one_on_consecutive_calls():
    from deepbind_amd import kangaroo_smat as ks, _lib
    rng = np.random.default_rng(8)
    m, F = 24, 96
    W = dev((rng.standard_normal((4 * m, F)) * 0.3).astype(np.float32))
    b = dev((rng.standard_normal((1, F)) * 0.1).astype(np.float32))
    # two calls in a row, the second over a smaller batch (the shared buffer still holds the first call's bytes),
    # then one whose input makes the table kernel stand down (code 254) and one with avg pooling
    cases = [(300, 200, "max", True, 0.0), (40, 57, "max", True, 0.0), (64, 101, "all", True, 0.0), (50, 80, "max", False, 0.01),
             (30, 61, "avg", False, 0.0)]
    for nseq, L, ptype, want_argmax, p254 in cases:
        X, R = _batch(rng, nseq, L, m, p254=p254)
        Xd, Rd = dev(X), dev(R)
        want_p, want_i = ks.scanpool_fprop(W, b, Xd, Rd, ptype, want_argmax=want_argmax, path="kmer")
        out_p = torch.full_like(want_p, float("nan"))
        out_i = torch.zeros_like(want_i) if want_i is not None else None
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats().get("allocation.all.allocated", 0)        # count of allocations torch has made so far
        free_before = torch.cuda.mem_get_info()[0]                                   # free device memory as the driver counts it
        got_p, got_i = ks.scanpool_fprop(W, b, Xd, Rd, ptype, want_argmax=want_argmax, path="kmer_static", out=(out_p, out_i))
        torch.cuda.synchronize()
        assert torch.cuda.memory_stats().get("allocation.all.allocated", 0) == before, "the host wrapper allocated"
        # an allocation made inside the library (hipMalloc, not torch's) shows up here and nowhere else
        assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated or freed during the call"
        assert np.array_equal(host(got_p), host(want_p)), "pooled differs (%d x %d, %s)" % (nseq, L, ptype)
        if want_i is not None:
            assert np.array_equal(host(got_i), host(want_i)), "argmax differs (%d x %d, %s)" % (nseq, L, ptype)


def test_static_scratch_entry_point_rejects_batches_beyond_its_buffer():
    from deepbind_amd import kangaroo_smat as ks, _lib
    m, F = 8, 32
    W = torch.zeros((4 * m, F), dtype=torch.float32, device="cuda")
    b = torch.zeros((1, F), dtype=torch.float32, device="cuda")
    N = (64 << 20) + 1024
    X = torch.zeros(N, dtype=torch.uint8, device="cuda")
    R = dev(np.array([[0, 1000]], dtype=np.uint32))
    with pytest.raises(_lib.DeepbindError, match="built-in buffer"):
        ks.scanpool_fprop(W, b, X, R, "max", path="kmer_static")
