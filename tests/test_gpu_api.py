"""GPU tests of the Python surface kept from dciknn_cuda/core.py:25-169."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _xy(n=2000, nq=20, dim=16, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n + nq, dim, generator=g)
    return x[:n].cuda(), x[n:].cuda()


def test_query_return_contract(gpu):
    X, Q = _xy()
    dci = gpu.DCI(16, 2, 5, 10, 8)
    assert (dci.dim, dci.num_comp_indices, dci.num_simp_indices) == (16, 2, 5)
    dci.add(X)
    assert dci.num_points == 2000
    idx, dist = dci.query(Q, 7, 50)
    assert idx.shape == (20, 7) and dist.shape == (20, 7)
    assert idx.dtype == torch.float32 and dist.dtype == torch.float32   # ids come back as floats
    assert idx.is_cuda and dist.is_cuda
    assert torch.all(dist[:, 1:] >= dist[:, :-1])
    # returned distance belongs to the returned id
    d = (X[idx.long()] - Q[:, None, :]).norm(dim=2)
    assert torch.allclose(d, dist, rtol=1e-5, atol=1e-6)
    # 1-D query is treated as one row
    i1, d1 = dci.query(Q[3], 7, 50)
    assert i1.shape == (1, 7) and torch.equal(i1[0], idx[3]) and torch.equal(d1[0], dist[3])
    dci.free()


def test_second_add_raises_and_clear_allows_again(gpu):
    X, Q = _xy()
    dci = gpu.DCI(16, 2, 5, 10, 8)
    dci.add(X)
    with pytest.raises(RuntimeError):
        dci.add(X)
    a = dci.query(Q, 3, 20)
    dci.clear()
    assert dci.num_points == 0
    with pytest.raises(RuntimeError):
        dci.query(Q, 3, 20)
    dci.add(X)
    b = dci.query(Q, 3, 20)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])   # same directions after clear()


def test_reset_draws_new_seeded_directions(gpu):
    d1 = gpu.DCI(16, 2, 5, 10, 8, seed=5)
    d2 = gpu.DCI(16, 2, 5, 10, 8, seed=5)
    d3 = gpu.DCI(16, 2, 5, 10, 8, seed=6)
    p1 = d1.directions
    assert torch.equal(p1, d2.directions) and not torch.equal(p1, d3.directions)
    assert torch.allclose(p1.double().norm(dim=1), torch.ones(10, dtype=torch.float64), atol=2e-6)
    d1.reset(); d2.reset()
    assert not torch.equal(d1.directions, p1)
    assert torch.equal(d1.directions, d2.directions)    # the sequence itself is seeded


def test_directions_look_isotropic(gpu):
    """Entries of unit Gaussian directions in dim d have mean 0 and variance 1/d."""
    p = gpu.DCI(256, 8, 16, seed=1).directions.double()
    assert abs(p.mean().item()) < 3.0 / np.sqrt(p.numel() * 256)
    assert abs(p.var().item() * 256 - 1.0) < 0.02
    gram = p @ p.T - torch.eye(128, dtype=torch.float64)
    assert gram.abs().max().item() < 0.4                # no two directions nearly parallel


def test_set_directions_round_trip_and_shape_check(gpu):
    dci = gpu.DCI(4, 1, 2, 1, 1)
    dci.directions = torch.tensor([[1., 0, 0, 0], [0, 1., 0, 0]])
    assert torch.equal(dci.directions, torch.tensor([[1., 0, 0, 0], [0, 1., 0, 0]]))
    with pytest.raises(ValueError):
        dci.directions = torch.zeros(3, 4)
    X = torch.tensor([[0., 0, 0, 0], [1, 3, 0, 0], [2, 1, 0, 0], [5, 5, 0, 0]]).cuda()
    dci.add(X)
    with pytest.raises(RuntimeError):
        dci.directions = torch.zeros(2, 4)              # not while points are indexed
    # the hand-derived traversal of tests/golden (k=2): ids [2, 0]
    idx, dist = dci.query(torch.tensor([[1.4, 1.2, 0, 0]]).cuda(), 2, 1, return_int=True)
    assert idx.tolist() == [[2, 0]]
    np.testing.assert_allclose(dist.cpu().numpy(), [[0.6324555, 1.8439089]], rtol=1e-6)


def test_argument_errors(gpu):
    X, Q = _xy()
    dci = gpu.DCI(16, 2, 5, 10, 8)
    with pytest.raises(ValueError):
        dci.add(X[:, :8].contiguous())
    with pytest.raises(TypeError):
        dci.add(X.double())
    with pytest.raises(TypeError):
        dci.add(X.cpu())
    with pytest.raises(ValueError):
        dci.add(X.t().contiguous().t())
    dci.add(X)
    with pytest.raises(TypeError):
        dci.query(Q, 2.5)
    with pytest.raises(ValueError):
        dci.query(Q, 0)
    with pytest.raises(ValueError):
        dci.query(Q, 2001)
    dci._block_size = 11                                # partitioning is part of the index
    with pytest.raises(RuntimeError):
        dci.query(Q, 3)


def test_all_neighbours_default(gpu):
    """num_neighbours=-1 means every indexed point, ranked (core.py:84-85)."""
    X, Q = _xy(n=300, nq=4)
    dci = gpu.DCI(16, 2, 3, 4, 4)
    dci.add(X)
    idx, dist = dci.query(Q, num_outer_iterations=10 ** 6)
    assert idx.shape == (4, 300)
    want = torch.cdist(Q, X).sort(dim=1)
    assert torch.allclose(dist, want.values, rtol=1e-5, atol=1e-6)
    assert torch.equal(idx.long().sort(dim=1).values, torch.arange(300).cuda().expand(4, 300))


def test_mdci_single_device_equals_dci(gpu):
    X, Q = _xy()
    m = gpu.MDCI(16, 2, 5, 10, 8, devices=[0])
    d = gpu.DCI(16, 2, 5, 10, 8, device=0)
    m.add(X.cpu())          # MDCI moves the shard itself (core.py:125)
    d.add(X)
    mi, md = m.query(Q.cpu(), 5, 30)
    di, dd = d.query(Q, 5, 30)
    assert torch.equal(mi, di) and torch.equal(md, dd)
    with pytest.raises(RuntimeError):
        m.query(Q, -1)
    m.clear(); m.reset(); m.free()


def test_non_default_stream(gpu, oracle):
    """Work is enqueued on torch's current stream."""
    X, Q = _xy()
    dci = gpu.DCI(16, 2, 5, 10, 8)
    s = torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(s):
        dci.add(X)
        i1, d1 = dci.query(Q, 5, 30)
    s.synchronize()
    i0, d0 = dci.query(Q, 5, 30)
    assert torch.equal(i0, i1) and torch.equal(d0, d1)


def test_append_equals_one_add_of_the_concatenation(gpu, oracle):
    """Incremental insertion is defined as 'as if built on all rows so far'."""
    g = torch.Generator().manual_seed(3)
    X = torch.randn(9000, 24, generator=g).cuda()
    Q = torch.randn(40, 24, generator=g).cuda()
    whole = gpu.DCI(24, 2, 4, 6, 5, seed=9)
    whole.add(X)
    want = whole.query(Q, 8, 40, return_int=True)
    parts = gpu.DCI(24, 2, 4, 6, 5, seed=9)
    parts.add(X[:2500].contiguous())                  # a borrowed first batch ...
    with pytest.raises(RuntimeError):
        parts.add(X[2500:5000].contiguous())          # ... `add` still works only once
    cuts = [2500, 2501, 6000, 9000]
    for lo, hi in zip(cuts[:-1], cuts[1:]):
        chunk = X[lo:hi].clone()
        parts.append(chunk)
        del chunk                                     # appended rows are copied
        assert parts.num_points == hi
        torch.cuda.synchronize()
        ref = gpu.DCI(24, 2, 4, 6, 5, seed=9)
        ref.add(X[:hi].contiguous())
        a = parts.query(Q, 8, 40, return_int=True)
        b = ref.query(Q, 8, 40, return_int=True)
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
        ref.free()
    got = parts.query(Q, 8, 40, return_int=True)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    # and the oracle on the concatenation agrees
    r = oracle.knn(parts.directions.numpy(), X.cpu().numpy(), Q.cpu().numpy(), 2, 4, 6, 5, 8, 40)
    assert np.array_equal(got[0].cpu().numpy(), r["ids"])
    # append on an empty index, then clear
    fresh = gpu.DCI(24, 2, 4, 6, 5, seed=9)
    fresh.append(X[:100].contiguous())
    fresh.append(X[100:9000].contiguous())
    c = fresh.query(Q, 8, 40, return_int=True)
    assert torch.equal(c[0], want[0]) and torch.equal(c[1], want[1])
    fresh.clear()
    assert fresh.num_points == 0
    fresh.add(X)
    d = fresh.query(Q, 8, 40, return_int=True)
    assert torch.equal(d[0], want[0])


# ------------------------------------------------ num_neighbours beyond the top-k tables
def _full_ranking_case(gpu, oracle, n, nq, dim, M, L, B, T, k, outer=50, seed=8):
    rng = np.random.default_rng(seed)
    X = rng.standard_normal((n, dim)).astype(np.float32)
    Q = rng.standard_normal((nq, dim)).astype(np.float32)
    dci = gpu.DCI(dim, M, L, B, T, seed=seed)
    dci.add(torch.from_numpy(X).cuda())
    ids, dists, ctr = dci.query(torch.from_numpy(Q).cuda(), k, outer, return_int=True, return_counters=True)
    torch.cuda.synchronize()
    from util import engine_index, engine_project
    skeys, sids = engine_index(dci)
    qproj = engine_project(dci.directions.numpy(), Q).T.copy()
    kk = n if k < 0 else k
    ref = oracle.query(skeys, sids, X, Q, qproj, M, L, B, T, kk, outer)
    dci.free()
    return ids.cpu().numpy(), dists.cpu().numpy(), ctr.cpu().numpy(), ref, X, Q


@pytest.mark.parametrize("n,B,T,k", [(20000, 4, 3, -1), (20000, 4, 1, 9000), (9000, 2, 5, -1),
                                     (70000, 16, 8, -1), (40000, 5, 2, 8193)])
def test_full_ranking_beyond_8192(gpu, oracle, n, B, T, k):
    """num_neighbours above the points per partition (core.py:84-85 makes it num_points by
    default): no partition can stop early, so the traversal's answer is the exact ranking
    of all points, which the engine computes directly.  Distances are summed in the
    oracle's order, so ids, distances and all four counters are compared exactly."""
    ids, dists, ctr, ref, X, Q = _full_ranking_case(gpu, oracle, n, 3, 12, 2, 3, B, T, k)
    np.testing.assert_array_equal(ids, ref["ids"])
    np.testing.assert_array_equal(dists, ref["dists"])
    np.testing.assert_array_equal(ctr, ref["counters"].astype(np.int64))
    kk = n if k < 0 else k
    bi, bd = oracle.brute_force(X, Q, kk)
    assert set_agreement_rows(ids, bi) >= 0.999
    np.testing.assert_allclose(dists, bd, rtol=1e-5)


def set_agreement_rows(a, b):
    return float(np.mean([len(set(x.tolist()) & set(y.tolist())) / len(y) for x, y in zip(a, b)]))


@pytest.mark.parametrize("B", [10, 1])
def test_full_ranking_through_the_binding(gpu, B):
    """The reference's route (flat float tensor from _dci_query) with the default
    num_neighbours: every point, ranked."""
    rng = np.random.default_rng(12)
    X = torch.from_numpy(rng.standard_normal((10000, 8)).astype(np.float32)).cuda()
    Q = torch.from_numpy(rng.standard_normal((2, 8)).astype(np.float32)).cuda()
    dci = gpu.DCI(8, 2, 3, B, 4, seed=2)
    dci.add(X)
    ids, dists = dci.query(Q)
    assert ids.shape == (2, 10000) and dists.shape == (2, 10000)
    assert torch.equal(torch.sort(ids.long(), dim=1).values, torch.arange(10000, device="cuda").expand(2, -1))
    assert torch.all(dists[:, 1:] >= dists[:, :-1])
    want = (X[ids.long()] - Q[:, None, :]).norm(dim=2)        # the distance of the id beside it
    assert torch.allclose(dists, want, rtol=1e-5, atol=1e-6)
    dci.free()


@pytest.mark.parametrize("n,B,T,k,outer", [(20000, 2, 1, 9000, 50),     # partitions stop once 9000 of their 10000 points are promoted
                                           (30000, 2, 2, 8200, 100000),  # lane-0 promotions never reach k: runs dry
                                           (9000, 1, 1, -1, 50)])        # k = N = points per partition, with counters
def test_large_k_with_early_stops(gpu, oracle, n, B, T, k, outer):
    """num_neighbours above 8192 but not above the points per partition: the stop rule can
    fire, so the traversal runs (step-by-step kernel, every candidate recorded in a dense
    row per query) and the rows are sorted.  Counters exact, neighbours as in the oracle."""
    ids, dists, ctr, ref, X, Q = _full_ranking_case(gpu, oracle, n, 3, 12, 2, 3, B, T, k, outer=outer)
    np.testing.assert_array_equal(ctr, ref["counters"].astype(np.int64))
    assert set_agreement_rows(ids, ref["ids"]) >= 0.999
    np.testing.assert_array_equal(ids < 0, ref["ids"] < 0)
    np.testing.assert_allclose(dists, ref["dists"], rtol=1e-5)
    if B == 2 and T == 1:
        assert np.all(ctr[:, 1] < n), "the case is meant to stop before everything is promoted"


def test_query_can_be_captured_in_a_graph(gpu):
    """After one warm-up call (workspace sized, hints of this query shape in place) a
    dcih_query enqueues only kernels, so a HIP graph can hold it: every replay, with
    eager calls in between, gives the eager result."""
    from dciknn_cuda_amd import _capi
    X, Q = _xy(n=30000, nq=32, dim=16, seed=5)
    dci = gpu.DCI(16, 2, 5, 8, 4, seed=9)
    dci.add(X)
    nq, k = Q.shape[0], 7
    ids = torch.empty((nq, k), dtype=torch.int32, device="cuda")
    dists = torch.empty((nq, k), dtype=torch.float32, device="cuda")

    def call(stream):
        _capi.check(dci._lib.dcih_query(dci._dci_inst, 16, nq, Q.data_ptr(), k, 0, 60, 10 * k, 8, 4,
                                        ids.data_ptr(), dists.data_ptr(), None, stream))
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        call(s.cuda_stream)
        call(s.cuda_stream)
    s.synchronize()
    want_ids, want_dists = ids.clone(), dists.clone()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        call(torch.cuda.current_stream().cuda_stream)
    for _ in range(4):
        ids.fill_(-5)
        dists.fill_(-5.0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(ids, want_ids) and torch.equal(dists, want_dists)
        call(0)                                # eager work between the replays
        torch.cuda.synchronize()
    del g
    dci.free()
