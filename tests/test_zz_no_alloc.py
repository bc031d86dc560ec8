"""dcih_query_noalloc (all scratch from the library's fixed device array, no
allocation) against dcih_query on the same index and queries: identical ids,
distances and counters, on two calls in a row, the second with a smaller input,
plus its size limit, and the one kind of shape where the two agree as sets and to
1e-5 in the distances instead of bit for bit."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _call(dci, fn, Q, k, outer, B, T, blind=0, counters=True):
    from dciknn_cuda_amd import _capi
    nq = Q.shape[0]
    width = min(10 * k, outer) if blind else k
    ids = torch.full((nq, width), -7, dtype=torch.int32, device="cuda")
    dists = torch.full((nq, width), -7.0, dtype=torch.float32, device="cuda")
    ctr = torch.full((nq, 4), -7, dtype=torch.int64, device="cuda") if counters else None
    rc = fn(dci._dci_inst, Q.shape[1], nq, Q.data_ptr(), k, blind, outer, 10 * k, B, T,
            ids.data_ptr(), dists.data_ptr(), ctr.data_ptr() if counters else None,
            torch.cuda.current_stream().cuda_stream)
    _capi.check(rc)
    torch.cuda.synchronize()
    return ids, dists, ctr


@pytest.mark.parametrize("traversal", ["auto", "step"])
def test_noalloc_equals_query_twice_second_smaller(gpu, traversal):
    g = torch.Generator().manual_seed(21)
    dim, M, L, B, T, k, outer = 32, 2, 6, 12, 3, 9, 40
    X = torch.randn(60_000, dim, generator=g).cuda()
    Q1 = torch.randn(300, dim, generator=g).cuda()
    Q2 = torch.randn(41, dim, generator=g).cuda()      # the second call is smaller
    dci = gpu.DCI(dim, M, L, B, T, seed=5, traversal=traversal)
    dci.add(X)
    lib = dci._lib
    for Q in (Q1, Q2):
        want = _call(dci, lib.dcih_query, Q, k, outer, B, T)
        got = _call(dci, lib.dcih_query_noalloc, Q, k, outer, B, T)
        assert torch.equal(got[0], want[0]), "ids differ"
        assert torch.equal(got[1], want[1]), "distances differ"
        assert torch.equal(got[2][:, 1], want[2][:, 1]) and torch.equal(got[2][:, 3], want[2][:, 3])
        assert torch.all(got[0] >= 0)
    # blind, also twice, second smaller
    for Q in (Q1, Q2):
        want = _call(dci, lib.dcih_query, Q, k, outer, B, T, blind=1)
        got = _call(dci, lib.dcih_query_noalloc, Q, k, outer, B, T, blind=1)
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    dci.free()


def test_noalloc_on_a_shape_that_runs_dry(gpu):
    """The reference's example configuration (3000 points in 100 partitions, 5000 iterations):
    the stop rule cannot fire, dcih_query ranks all points directly, dcih_query_noalloc runs the
    traversal.  Same neighbours; the distances are summed in another order and agree to 1e-5."""
    from dciknn_cuda_amd import workloads
    X, Q = workloads.c1()
    dim, M, L, B, T, k, outer = 100, 2, 10, 100, 10, 10, 5000
    dci = gpu.DCI(dim, M, L, B, T, seed=4)
    dci.add(X.cuda())
    for Qd in (Q.cuda(), Q[:77].contiguous().cuda()):
        want = _call(dci, dci._lib.dcih_query, Qd, k, outer, B, T)
        got = _call(dci, dci._lib.dcih_query_noalloc, Qd, k, outer, B, T)
        assert torch.allclose(got[1], want[1], rtol=1e-5, atol=0.0)
        a, b = got[0].cpu().numpy(), want[0].cpu().numpy()
        agree = np.mean([len(set(x.tolist()) & set(y.tolist())) / k for x, y in zip(a, b)])
        assert agree >= 0.999, agree
        assert torch.equal(got[2][:, 1], want[2][:, 1]) and torch.equal(got[2][:, 3], want[2][:, 3])
    dci.free()


def test_noalloc_rejects_what_does_not_fit(gpu):
    from dciknn_cuda_amd import _capi
    g = torch.Generator().manual_seed(22)
    dim, B, T, k = 8, 64, 2, 50
    X = torch.randn(40_000, dim, generator=g).cuda()
    dci = gpu.DCI(dim, 2, 3, B, T, seed=5)
    dci.add(X)
    # 20000 queries * 64 partitions * 50 results * 8 bytes = 512 MB of result lists
    Q = torch.randn(20_000, dim, generator=g).cuda()
    ids = torch.empty((Q.shape[0], k), dtype=torch.int32, device="cuda")
    dists = torch.empty((Q.shape[0], k), dtype=torch.float32, device="cuda")
    rc = dci._lib.dcih_query_noalloc(dci._dci_inst, dim, Q.shape[0], Q.data_ptr(), k, 0, 30, 10 * k, B, T,
                                     ids.data_ptr(), dists.data_ptr(), None, 0)
    assert rc == -1
    msg = dci._lib.dcih_last_error().decode()
    assert "scratch" in msg and str(_capi.NOALLOC_SCRATCH_BYTES) in msg
    # more results per query than the on-chip tables hold
    rc = dci._lib.dcih_query_noalloc(dci._dci_inst, dim, 2, Q.data_ptr(), 9000, 0, 30, 90000, B, T,
                                     ids.data_ptr(), dists.data_ptr(), None, 0)
    assert rc == -4
    # the allocating entry point still takes the large batch, and a small one still works here
    _call(dci, dci._lib.dcih_query, Q, k, 30, B, T, counters=False)
    a = _call(dci, dci._lib.dcih_query, Q[:64].contiguous(), k, 30, B, T)
    b = _call(dci, dci._lib.dcih_query_noalloc, Q[:64].contiguous(), k, 30, B, T)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    dci.free()
