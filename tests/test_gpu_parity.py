"""GPU parity tests: the HIP engine (through libdci_hip.so) against the CPU oracle.

Two levels.  L1 (traversal parity): the oracle is fed the engine's own sorted
projections and query projections; everything downstream uses exact IEEE
comparisons, so ids, visit counts and candidate counts must match EXACTLY
(distances to 1e-5 relative: the engine sums squares in a different order).
L2 (end to end): only data, queries and directions are shared; tolerance is
>= 99.9 % neighbour-set agreement and 1e-5 relative distance error.
"""
import numpy as np
import pytest
import torch

from util import engine_index, engine_project, engine_segsort, set_agreement

pytestmark = pytest.mark.gpu

DIST_RTOL = 1e-5


def _data(seed, n, nq, dim, kind="normal"):
    rng = np.random.default_rng(seed)
    if kind == "normal":
        x = rng.standard_normal((n + nq, dim))
    elif kind == "lowrank":
        x = rng.random((n + nq, max(2, dim // 3))) @ rng.standard_normal((max(2, dim // 3), dim))
    elif kind == "grid":   # many exactly equal projections and distances
        x = rng.integers(0, 3, (n + nq, dim)).astype(np.float64)
    x = x.astype(np.float32)
    return x[:n], x[n:]


def _run_l1(gpu, oracle, X, Q, M, L, B, T, k, outer, seed=1, max_cand=None, traversal="step"):
    """Engine result + oracle result on the engine's own keys."""
    dci = gpu.DCI(X.shape[1], M, L, B, T, seed=seed, traversal=traversal)
    xd = torch.from_numpy(X).cuda()
    qd = torch.from_numpy(Q).cuda()
    dci.add(xd)
    if max_cand is None:
        ids, dists, ctr = dci.query(qd, k, outer, return_int=True, return_counters=True)
    else:   # max_num_candidates other than 10k: straight through the C-ABI
        from dciknn_cuda_amd import _capi
        nq = Q.shape[0]
        ids = torch.empty((nq, k), dtype=torch.int32, device="cuda")
        dists = torch.empty((nq, k), dtype=torch.float32, device="cuda")
        ctr = torch.empty((nq, 4), dtype=torch.int64, device="cuda")
        _capi.check(dci._lib.dcih_query(dci._dci_inst, X.shape[1], nq, qd.data_ptr(), k, 0, outer,
                                        max_cand, B, T, ids.data_ptr(), dists.data_ptr(),
                                        ctr.data_ptr(), torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    skeys, sids = engine_index(dci)
    P = dci.directions.numpy()
    qproj = engine_project(P, Q).T.copy()
    ref = oracle.query(skeys, sids, X, Q, qproj, M, L, B, T, k, outer, max_cand=max_cand)
    dci.free()
    return ids.cpu().numpy(), dists.cpu().numpy(), ctr.cpu().numpy(), ref


def _assert_l1(ids, dists, ctr, ref, exact_ids=True, visits=True):
    rc = ref["counters"].astype(np.int64)
    if visits:
        np.testing.assert_array_equal(ctr[:, 0], rc[:, 0], err_msg="entries visited")
    # (the other kernels count the index entries they read, which the loop's visits do not bound)
    np.testing.assert_array_equal(ctr[:, 1], rc[:, 1], err_msg="candidates promoted")
    np.testing.assert_array_equal(ctr[:, 3], rc[:, 3], err_msg="outer steps")
    np.testing.assert_allclose(dists, ref["dists"], rtol=DIST_RTOL, atol=1e-6)
    if exact_ids:
        assert set_agreement(ids, ref["ids"]) == 1.0
    assert np.all(np.diff(dists, axis=1) >= 0), "rows must ascend by distance"


# ---------------------------------------------------------------- projection
@pytest.mark.parametrize("n,dim,I", [(1000, 128, 20), (257, 100, 20), (3, 7, 1), (4096, 96, 24),
                                     (513, 33, 37), (70, 960, 24), (5000, 64, 30), (300, 5, 70)])
def test_project_matches_matmul(gpu, oracle, n, dim, I):
    rng = np.random.default_rng(n + dim)
    P = rng.standard_normal((I, dim)).astype(np.float32)
    X = rng.standard_normal((n, dim)).astype(np.float32)
    got = engine_project(P, X)
    want64 = P.astype(np.float64) @ X.astype(np.float64).T
    # fp32 accumulation error bound: dim * eps * sum|p||x|
    bound = dim * 2.0 ** -24 * (np.abs(P).astype(np.float64) @ np.abs(X).astype(np.float64).T)
    assert np.all(np.abs(got - want64) <= bound + 1e-30)
    # same arithmetic as the oracle (one FMA chain over k): bit-identical keys
    np.testing.assert_array_equal(got, oracle.project(P, X))


def test_project_same_vector_same_bits(gpu):
    """A row projects to the same bits whether it sits in a batch of 1 or of many."""
    rng = np.random.default_rng(5)
    P = rng.standard_normal((20, 128)).astype(np.float32)
    X = rng.standard_normal((777, 128)).astype(np.float32)
    full = engine_project(P, X)
    one = engine_project(P, X[500:501])
    np.testing.assert_array_equal(full[:, 500], one[:, 0])


# ------------------------------------------------------------ segmented sort
@pytest.mark.parametrize("n,I,B", [(3000, 20, 100), (1000, 3, 7), (10, 2, 16), (1, 1, 1),
                                   (16384, 2, 1), (16385, 2, 1), (50000, 3, 1), (100000, 2, 3),
                                   (4099, 5, 4), (2049, 2, 1), (4096, 2, 1), (4097, 2, 1), (8200, 3, 2), (10000, 3, 1), (15360, 2, 1), (15361, 2, 1),
                                   (25000, 2, 2), (62500, 3, 2), (32256, 1, 1), (32257, 1, 1),
                                   (70000, 2, 3)])
def test_segsort_matches_oracle(gpu, oracle, n, I, B):
    rng = np.random.default_rng(n * 31 + B)
    keys = rng.standard_normal((I, n)).astype(np.float32)
    keys[:, ::7] = np.round(keys[:, ::7])          # plenty of exact ties
    sk, si = engine_segsort(keys, B)
    rk, ri = oracle.segsort(keys, B)
    np.testing.assert_array_equal(sk, rk)
    np.testing.assert_array_equal(si, ri)


# one slice length inside the range of every instantiation of the LDS radix kernel
@pytest.mark.parametrize("n", [560, 600, 1500, 2000, 2500, 3400, 4200, 5300, 5556, 6000, 8000, 9900, 11000,
                               13000, 14500, 16000, 17858, 19000, 23000, 26000, 29000, 32000])
def test_segsort_every_radix_configuration(gpu, oracle, n):
    rng = np.random.default_rng(n)
    I, B = 6, 3
    keys = (rng.standard_normal((I, n * B - 5)) * 300 + 100).astype(np.float32)
    keys[0, ::5] = np.round(keys[0, ::5])
    keys[1] = np.abs(keys[1])                       # constant sign: a skipped digit
    keys[2, ::3] = -0.0
    keys[2, 1::3] = 0.0
    for rep in range(2):                            # twice: the result must not depend on timing
        sk, si = engine_segsort(keys, B)
        rk, ri = oracle.segsort(keys, B)
        np.testing.assert_array_equal(sk, rk)
        np.testing.assert_array_equal(si, ri)


def test_index_arrays_are_consistent(gpu):
    """sids, the 16-bit partition-relative ids and the inverse permutation describe
    one and the same order (checked through a query that uses all three)."""
    rng = np.random.default_rng(3)
    for n, B in [(40_000, 2), (9_000, 3), (1_000, 5)]:
        X = rng.standard_normal((n, 8)).astype(np.float32)
        dci = gpu.DCI(8, 2, 3, B, 4, seed=3)
        dci.add(torch.from_numpy(X).cuda())
        sk, si = engine_index(dci)
        ppb = -(-n // B)
        for b in range(B):
            lo, hi = b * ppb, min(n, (b + 1) * ppb)
            assert np.all(np.diff(sk[:, lo:hi], axis=1) >= 0)
            assert np.array_equal(np.sort(si[:, lo:hi], axis=1), np.tile(np.arange(lo, hi), (6, 1)))
        dci.free()


@pytest.mark.parametrize("fill_by", ["accessor", "query"])
def test_position_tables(gpu, fill_by):
    """inv is the inverse of every sorted slice; rpos holds the same places in the order of the first
    simple index of each composite (the table the batch traversal scans), whether the inspection call
    or the first batch traversal fills it."""
    from dciknn_cuda_amd import _capi
    rng = np.random.default_rng(11)
    for n, B, M, L in [(40_000, 2, 2, 3), (9_001, 3, 3, 4), (1_000, 5, 1, 2), (777, 4, 2, 1), (4_096, 1, 2, 5)]:
        X = rng.standard_normal((n, 8)).astype(np.float32)
        dci = gpu.DCI(8, M, L, B, 4, seed=3, traversal="batch")
        dci.add(torch.from_numpy(X).cuda())
        if fill_by == "query":
            dci.query(torch.from_numpy(X[:5]).cuda(), 3, 20)
        I = M * L
        d_inv = torch.zeros((I, n), dtype=torch.int16, device="cuda")
        d_rpos = torch.zeros((I, n), dtype=torch.int16, device="cuda")
        _capi.check(dci._lib.dcih_debug_positions(dci._dci_inst, d_inv.data_ptr(), d_rpos.data_ptr(), None))
        inv = d_inv.cpu().numpy().view(np.uint16).astype(np.int64)
        rpos = d_rpos.cpu().numpy().view(np.uint16).astype(np.int64)
        _, si = engine_index(dci)
        ppb = -(-n // B)
        for b in range(B):
            lo, hi = b * ppb, min(n, (b + 1) * ppb)
            if hi <= lo:
                continue
            places = np.arange(hi - lo)
            for i in range(I):
                ids = si[i, lo:hi]
                np.testing.assert_array_equal(inv[i, ids], places, err_msg="inv, index %d partition %d" % (i, b))
                first = (i // L) * L
                if i != first:      # (the first indices' own rows are never written)
                    np.testing.assert_array_equal(rpos[i, lo:hi], inv[i, si[first, lo:hi]],
                                                  err_msg="rpos, index %d partition %d" % (i, b))
        dci.free()


def test_segsort_invariants_large(gpu):
    """Size-independent properties at a partition length beyond one LDS tile."""
    n, I, B = 300_000, 2, 2
    rng = np.random.default_rng(9)
    keys = rng.standard_normal((I, n)).astype(np.float32)
    sk, si = engine_segsort(keys, B)
    ppb = (n + B - 1) // B
    for i in range(I):
        for b in range(B):
            lo, hi = b * ppb, min(n, (b + 1) * ppb)
            assert np.all(np.diff(sk[i, lo:hi]) >= 0)
            assert np.array_equal(np.sort(si[i, lo:hi]), np.arange(lo, hi))
            np.testing.assert_array_equal(keys[i, si[i, lo:hi]], sk[i, lo:hi])


# -------------------------------------------------------- traversal (L1) parity
CASES = [
    # n, nq, dim, M, L, B, T, k, outer, kind
    (3000, 64, 100, 2, 10, 100, 10, 10, 5000, "lowrank"),   # C1 shape: exhaustive
    (3000, 64, 100, 2, 10, 10, 10, 10, 20, "lowrank"),      # early stop by outer*L
    (3000, 64, 100, 2, 10, 3, 4, 10, 5000, "lowrank"),      # stop by c0 >= 10k
    (2000, 32, 16, 2, 5, 1, 1, 5, 50, "normal"),            # textbook regime T=1, B=1
    (2000, 32, 16, 3, 4, 7, 64, 20, 3, "normal"),           # full-wave windows
    (2000, 16, 16, 2, 3, 5, 100, 8, 2, "normal"),           # T > 64
    (500, 16, 8, 1, 1, 4, 3, 3, 10, "normal"),              # single simple index
    (100, 16, 8, 2, 3, 200, 2, 5, 10, "normal"),            # B > n: empty partitions
    (257, 16, 12, 2, 20, 3, 5, 257, 10, "normal"),          # k = n, 8-bit counters
    (4000, 16, 24, 2, 10, 2, 16, 100, 30, "grid"),          # ties everywhere
    (1500, 8, 10, 70, 1, 6, 8, 4, 15, "normal"),            # more than 64 simple indices
    (40000, 16, 24, 2, 12, 2, 16, 10, 200, "normal"),       # step limit ends it: hundreds of promotions, large tables
    (30000, 16, 16, 2, 15, 2, 4, 50, 300, "normal"),        # L = 15: 4-bit counters with the promoted bitmap
    (30000, 16, 16, 2, 14, 3, 8, 40, 100, "normal"),        # L = 14: promoted points marked in the counters
    (40000, 16, 24, 2, 12, 8, 16, 10, 200, "normal"),       # the step limit ends it after most of the index (dense regime)
    (30000, 16, 16, 2, 15, 16, 4, 50, 300, "normal"),       # L = 15, several hundred promotions per partition
    (20000, 16, 16, 3, 8, 4, 16, 100, 40, "normal"),        # three composites, k = 100
    (6000, 16, 12, 2, 6, 3, 2, 5, 10_000, "normal"),        # narrow windows, stop by c0 >= 10k
    (9000, 16, 16, 2, 4, 2, 300, 10, 3, "normal"),          # T > 256
    (40000, 16, 24, 2, 12, 4, 12, 10, 200, "normal"),       # 10032 windows per composite: the largest dense tables
    (3000, 8, 512, 2, 4, 3, 16, 10, 5, "normal"),           # long rows: two 1 KiB pieces
    (3000, 8, 1100, 2, 4, 3, 16, 10, 5, "normal"),          # long rows: five pieces, the last one short
    (120000, 8, 16, 3, 16, 2, 8, 10, 30, "normal"),         # 60000-point partitions, 48 indices: the step kernel's counters leave LDS, the batch kernel's flags do not
    (60000, 48, 16, 2, 10, 3, 2, 10, 100, "normal"),        # the batch kernel's compact tables, two-stage scan; one wavefront per item
    (60000, 48, 16, 2, 10, 3, 4, 15, 100, "normal"),        # ... with items that outgrow them and go to its second pass
    (64000, 16, 8, 26, 1, 1, 2, 10, 5, "normal"),           # compact tables, 26 composites: the full tables would not fit LDS (no second pass)
]


def _dense_fits(n, M, L, B, T, k):
    ppb = -(-n // B)
    return (M <= 64 and L <= 64 and ppb <= 32766 and min(k, ppb) <= 512 and
            L * (ppb // T + 3) <= 41 * 256)


@pytest.mark.parametrize("traversal", ["step", "batch", "dense", "auto"])
@pytest.mark.parametrize("case", CASES, ids=[str(c[:9]) for c in CASES])
def test_traversal_parity(gpu, oracle, case, traversal):
    n, nq, dim, M, L, B, T, k, outer, kind = case
    if traversal == "batch" and (2 * M * L > 256 or M > 64 or min(k, -(-n // B)) > 512):
        pytest.skip("shape outside the batch kernel's tables (it refuses; auto mode falls back)")
    if traversal == "dense" and not _dense_fits(n, M, L, B, T, k):
        pytest.skip("shape outside the dense kernel's tables (it refuses; auto mode does not route there)")
    X, Q = _data(n * 7 + T, n, nq, dim, kind)
    ids, dists, ctr, ref = _run_l1(gpu, oracle, X, Q, M, L, B, T, k, outer, traversal=traversal)
    _assert_l1(ids, dists, ctr, ref, exact_ids=(kind != "grid"), visits=(traversal == "step"))
    if kind == "grid":    # equal distances may swap ids: compare as distance multisets
        assert set_agreement(ids, ref["ids"]) >= 0.9


def test_traversal_parity_small_max_candidates(gpu, oracle):
    X, Q = _data(77, 5000, 32, 20, "normal")
    ids, dists, ctr, ref = _run_l1(gpu, oracle, X, Q, 2, 6, 4, 8, 5, 10_000, max_cand=7)
    _assert_l1(ids, dists, ctr, ref)


def test_queries_equal_to_data_points(gpu, oracle):
    """Query projections equal to stored keys exercise the strict '<' of the search."""
    X, _ = _data(3, 1000, 0, 32, "normal")
    Q = X[::50].copy()
    ids, dists, ctr, ref = _run_l1(gpu, oracle, X, Q, 2, 4, 4, 4, 3, 2000)
    _assert_l1(ids, dists, ctr, ref)
    assert np.array_equal(ids[:, 0], np.arange(0, 1000, 50)) and np.all(dists[:, 0] == 0)


def test_global_counter_fallback(gpu, oracle):
    """A partition too large for LDS counters takes the global-scratch path."""
    X, Q = _data(11, 400_000, 8, 8, "normal")
    ids, dists, ctr, ref = _run_l1(gpu, oracle, X, Q, 2, 3, 1, 32, 10, 40)
    _assert_l1(ids, dists, ctr, ref)


# ------------------------------------------------------ known answer: C1 regime
def test_c1_exhaustive_equals_brute_force(gpu, oracle):
    """n_b*T < outer and n_b < 10k: no partition can stop early, every point is
    promoted, so the answer is the exact k-NN whatever the directions are."""
    from dciknn_cuda_amd import workloads
    X, Q = workloads.c1()
    dci = gpu.DCI(100, 2, 10, 100, 10, seed=4)
    dci.add(X.cuda())
    ids, dists, ctr = dci.query(Q.cuda(), 10, 5000, return_int=True, return_counters=True)
    bi, bd = oracle.brute_force(X.numpy(), Q.numpy(), 10)
    assert set_agreement(ids.cpu().numpy(), bi) >= 0.999
    np.testing.assert_allclose(dists.cpu().numpy(), bd, rtol=DIST_RTOL)
    assert np.all(ctr[:, 1].cpu().numpy() == 3000)      # every point promoted
    assert np.all(ctr[:, 0].cpu().numpy() == 3000 * 20)  # every entry visited


# ------------------------------------------------------------ end to end (L2)
@pytest.mark.parametrize("B,T,outer", [(10, 10, 40), (4, 32, 10)])
def test_end_to_end_parity(gpu, oracle, B, T, outer):
    from dciknn_cuda_amd import workloads
    X, Q = workloads.c2(n=50_000, nq=200)
    M, L, k = 2, 10, 10
    dci = gpu.DCI(128, M, L, B, T, seed=21)
    dci.add(X.cuda())
    ids, dists = dci.query(Q.cuda(), k, outer, return_int=True)
    ref = oracle.knn(dci.directions.numpy(), X.numpy(), Q.numpy(), M, L, B, T, k, outer)
    assert set_agreement(ids.cpu().numpy(), ref["ids"]) >= 0.999
    np.testing.assert_allclose(np.sort(dists.cpu().numpy(), 1), np.sort(ref["dists"], 1),
                               rtol=DIST_RTOL)


def test_monotone_in_outer_iterations(gpu):
    """More outer iterations never lose a neighbour that was already found."""
    X, Q = _data(5, 20_000, 32, 32, "normal")
    dci = gpu.DCI(32, 2, 5, 4, 16, seed=2)
    dci.add(torch.from_numpy(X).cuda())
    qd = torch.from_numpy(Q).cuda()
    prev = None
    for outer in (5, 20, 80, 320):
        _, d = dci.query(qd, 5, outer)
        d = d.cpu().numpy()
        if prev is not None:
            assert np.all(d <= prev * (1 + 1e-6))
        prev = d
