"""Pins for the CPU oracle (no GPU needed).

The reference ships no golden vectors, so the oracle is pinned by
  * hand-derived traces (tests/golden/hand_traces.json),
  * library routines: numpy.searchsorted, numpy stable sort, float64 matmul,
  * the exhaustive regime, where the answer must equal exact brute force,
  * an independent heap-based Prioritized DCI written from the paper
    (arXiv 1703.00440, Algorithm 2) for T=1, B=1,
  * an independent "sort every window" model for general (B, T) that never
    simulates the loop: it ranks windows globally and derives promotion times,
  * invariants (monotonicity in the iteration budget, no duplicates, bounds).
None of them re-types the oracle's loop.
"""
import heapq
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "hand_traces.json")) as f:
    GOLD = json.load(f)

f32 = np.float32


# ----------------------------------------------------------------- hand traces
@pytest.mark.parametrize("case", GOLD["window_sequences"], ids=lambda c: c["name"][:40])
def test_window_sequence_hand_traces(oracle, case):
    cur, prio = oracle.window_sequence(np.array(case["keys"], f32), case["T"], case["q"])
    assert cur.tolist() == case["cur"]
    assert prio.tolist() == [float(p) for p in case["prio"]]


@pytest.mark.parametrize("case", GOLD["searches"], ids=lambda c: "%s-%s" % (c["keys"], c["q"]))
def test_search_hand_cases(oracle, case):
    assert oracle.search(np.array(case["keys"], f32), case["q"]) == case["pos"]


@pytest.mark.parametrize("case", GOLD["traversals"], ids=lambda c: c["name"][:40])
def test_traversal_hand_traces(oracle, case):
    P = np.array(case["directions"], f32)
    X = np.array(case["data"], f32)
    Q = np.array(case["query"], f32)
    r = oracle.knn(P, X, Q, case["M"], case["L"], case["B"], case["T"], case["k"],
                   case["outer"], max_cand=case["max_cand"])
    assert r["ids"].tolist() == case["ids"]
    np.testing.assert_allclose(r["dists"], np.array(case["dists"], f32), rtol=1e-6)
    assert r["counters"][:, 0].tolist() == case["visited"]
    assert r["counters"][:, 1].tolist() == case["candidates"]
    assert r["counters"][:, 3].tolist() == case["steps"]


@pytest.mark.parametrize("case", GOLD["blind_traversals"], ids=lambda c: c["name"][:40])
def test_blind_traversal_hand_traces(oracle, case):
    P = np.array(case["directions"], f32)
    X = np.array(case["data"], f32)
    Q = np.array(case["query"], f32)
    sk, si = oracle.build_index(P, X, case["B"])
    r = oracle.query_blind(sk, si, oracle.project(Q, P), case["M"], case["L"], case["B"],
                           case["T"], case["k"], case["outer"], max_cand=case["max_cand"])
    assert r["ids"].tolist() == case["ids"]
    assert r["steps"].astype(np.int64).tolist() == [[s if s >= 0 else 0xffffffff for s in row]
                                                    for row in case["steps"]]
    assert r["counters"][:, 0].tolist() == case["visited"]
    assert r["counters"][:, 1].tolist() == case["candidates"]
    assert r["counters"][:, 3].tolist() == case["num_steps"]


# ------------------------------------------------------------ library routines
def test_search_is_searchsorted_left_minus_one(oracle):
    rng = np.random.default_rng(0)
    for n in (1, 2, 3, 17, 1000):
        key = np.sort(rng.integers(-20, 20, n).astype(f32))   # many duplicates
        for q in np.concatenate([key[:20], rng.uniform(-25, 25, 40).astype(f32)]):
            assert oracle.search(key, q) == int(np.searchsorted(key, q, "left")) - 1


def test_normalize_gives_unit_rows(oracle):
    rng = np.random.default_rng(1)
    P = oracle.normalize(rng.standard_normal((24, 960)).astype(f32) * 37.0)
    np.testing.assert_allclose(np.linalg.norm(P.astype(np.float64), axis=1), 1.0, atol=2e-6)
    # direction preserved
    P2 = oracle.normalize(P * 5.0)
    np.testing.assert_allclose(P2, P, atol=1e-6)


def test_project_is_matmul_nt(oracle):
    rng = np.random.default_rng(2)
    A = rng.standard_normal((7, 33)).astype(f32)
    B = rng.standard_normal((50, 33)).astype(f32)
    got = oracle.project(A, B)
    assert got.shape == (7, 50)        # [rows of A][rows of B]: keys are [index][point]
    np.testing.assert_allclose(got, A.astype(np.float64) @ B.astype(np.float64).T,
                               rtol=1e-5, atol=1e-5)
    # a transposed operand or swapped roles would fail this asymmetric check
    assert abs(got[3, 41] - float(A[3].astype(np.float64) @ B[41].astype(np.float64))) < 1e-4


@pytest.mark.parametrize("n,B", [(10, 3), (100, 7), (64, 64), (5, 9), (1000, 1)])
def test_segsort_is_stable_sort_per_partition(oracle, n, B):
    rng = np.random.default_rng(n + B)
    keys = np.round(rng.standard_normal((3, n)) * 3).astype(f32)     # ties
    sk, si = oracle.segsort(keys, B)
    ppb = -(-n // B)
    for i in range(3):
        for b in range(B):
            lo, hi = b * ppb, min(n, (b + 1) * ppb)
            if lo >= hi:
                continue
            order = np.argsort(keys[i, lo:hi], kind="stable")
            np.testing.assert_array_equal(si[i, lo:hi], lo + order)
            np.testing.assert_array_equal(sk[i, lo:hi], keys[i, lo:hi][order])


# ------------------------------------------------- exhaustive regime = brute force
def test_exhaustive_regime_equals_brute_force(oracle):
    """C1: n_b*T = 300 < outer and n_b = 30 < 10k, so no partition may stop
    early; every point is promoted and the result is the exact k-NN."""
    from dciknn_cuda_amd import workloads
    X, Q = workloads.c1()
    X, Q = X.numpy(), Q.numpy()[:100]
    P = oracle.normalize(workloads.directions(1, 20, 100).numpy())
    r = oracle.knn(P, X, Q, 2, 10, 100, 10, 10, 5000)
    bi, bd = oracle.brute_force(X, Q, 10)
    np.testing.assert_array_equal(r["ids"], bi)
    np.testing.assert_allclose(r["dists"], bd, rtol=2e-6)
    assert np.all(r["counters"][:, 1] == 3000) and np.all(r["counters"][:, 0] == 60000)


# ------------------------------------- textbook Prioritized DCI (T = 1, B = 1)
def _textbook(keys, ids, qp, M, L, k, k1, k0):
    """Prioritized DCI query as in the paper: one priority queue per composite
    index holding, for each simple index, its closest not yet visited point;
    each iteration pops the nearest, counts it, and pushes the next closest of
    that simple index.  Stops after k1 iterations or k0 candidates (once k
    candidates exist, as the CUDA code adds).  keys/ids: [I][n] sorted; qp: [I].
    Returns the candidates in the order they are found."""
    I, n = keys.shape
    lo, hi = np.zeros(I, int), np.zeros(I, int)   # next unvisited on the left / right
    heaps = [[] for _ in range(M)]

    def push(i):
        m, h = divmod(i, L)
        l, r = lo[i], hi[i]
        cand = []
        if l >= 0:
            cand.append((f32(qp[i]) - keys[i, l], 0, l))
        if r < n:
            cand.append((keys[i, r] - f32(qp[i]), 1, r))
        if not cand:
            return
        # nearer side first; on a tie the left one (strict '<' in the CUDA code)
        if len(cand) == 2 and cand[1][0] < cand[0][0]:
            d, side, pos = cand[1]
        else:
            d, side, pos = cand[0]
        if side == 0:
            lo[i] -= 1
        else:
            hi[i] += 1
        heapq.heappush(heaps[m], (abs(f32(d)), h, pos))

    for i in range(I):
        p = int(np.searchsorted(keys[i], qp[i], "left")) - 1
        lo[i], hi[i] = p, p + 1
        push(i)
    counts = np.zeros((M, n), int)
    seen = set()
    out = []
    it = 0
    while any(heaps):
        for m in range(M):
            if not heaps[m]:
                continue
            _, h, pos = heapq.heappop(heaps[m])
            i = m * L + h
            pt = ids[i, pos]
            counts[m, pt] += 1
            if counts[m, pt] == L and pt not in seen:
                seen.add(pt)
                out.append(pt)
            push(i)
        if len(out) >= k and (it + 1 >= k1 or len(out) >= k0):
            break
        it += 1
    return out


@pytest.mark.parametrize("seed,n,dim,M,L,k,outer", [(0, 200, 8, 2, 3, 5, 4), (1, 500, 16, 3, 4, 3, 30),
                                                    (2, 64, 4, 1, 5, 10, 2), (3, 300, 6, 2, 2, 300, 7)])
def test_textbook_prioritized_dci(oracle, seed, n, dim, M, L, k, outer):
    rng = np.random.default_rng(seed)
    X = rng.standard_normal((n, dim)).astype(f32)
    Q = rng.standard_normal((6, dim)).astype(f32)
    P = oracle.normalize(rng.standard_normal((M * L, dim)).astype(f32))
    sk, si = oracle.build_index(P, X, 1)
    qp = oracle.project(Q, P)
    r = oracle.query(sk, si, X, Q, qp, M, L, 1, 1, k, outer, cand_cap=n)
    for j in range(Q.shape[0]):
        want = _textbook(sk, si, qp[j], M, L, k, outer * L, 10 * k)
        got = r["cand_ids"][j, :r["cand_cnt"][j]].tolist()
        assert got == want


# ---------------------------- independent model for general (B, T): rank, don't loop
def _index_windows(key, T, q):
    """Windows of one simple index in the order the code consumes them, as
    (priority, start).  Two sorted streams (left / right window starts) merged
    with the code's comparison; the ghost rule is the reference's bounds."""
    n = len(key)
    p = int(np.searchsorted(key, q, "left")) - 1
    rights, s = [], p + 1
    while s < n + T - 1:
        rights.append(s); s += T
    lefts, s = [], p - T + 1
    while s > -T:
        lefts.append(s); s -= T
    dR = [f32(key[min(s, n - 1)]) - f32(q) for s in rights]
    dL = [f32(q) - f32(key[max(s, 0)]) for s in lefts]
    out, a, b = [], 0, 0
    while a < len(lefts) or b < len(rights):
        take_right = a >= len(lefts) or (b < len(rights) and dR[b] < dL[a])
        if take_right:
            out.append((abs(dR[b]), rights[b])); b += 1
        else:
            out.append((abs(dL[a]), lefts[a])); a += 1
    return out


def _rank_model(sk, si, qp, n_off, n, M, L, T, k, outer, max_cand, with_times=False):
    """Promotion events of one partition without running the step loop.
    Composite m consumes its windows in ascending (priority, simple index,
    own order); a point's promotion time under m is the largest rank among the
    L windows that hold it; it is a candidate at the earliest (time, m)."""
    first = {}       # pt -> (time, m, lane0)
    nwin = []
    visited_at = []  # per composite: in-range entries per rank
    for m in range(M):
        wins = []
        for h in range(L):
            i = m * L + h
            for seq, (pr, start) in enumerate(_index_windows(sk[i, n_off:n_off + n], T, qp[i])):
                wins.append((pr, h, seq, start))
        wins.sort(key=lambda w: (w[0], w[1], w[2]))
        nwin.append(len(wins))
        last = {}    # pt -> (rank, lane)
        cnt = {}
        vis = []
        for rank, (pr, h, seq, start) in enumerate(wins):
            i = m * L + h
            inr = 0
            for t in range(T):
                pos = start + t
                if 0 <= pos < n:
                    inr += 1
                    pt = int(si[i, n_off + pos])
                    cnt[pt] = cnt.get(pt, 0) + 1
                    last[pt] = (rank, t)        # ranks ascend, so this ends as the max
            vis.append(inr)
        visited_at.append(vis)
        for pt, c in cnt.items():
            if c == L:
                rank, lane = last[pt]
                ev = (rank, m, lane == 0)
                if pt not in first or ev[:2] < first[pt][:2]:
                    first[pt] = ev
    events = sorted((t, m, pt, l0) for pt, (t, m, l0) in first.items())
    stop_at = outer * L
    bound = n * L * T
    maxw = max(nwin)
    # c0 after each step; find the stop step
    c0 = 0
    stop = None
    e = 0
    last_step = min(bound, maxw + 1) - 1     # loop ends by exhaustion (one idle pass) or bound
    for kk in range(last_step + 1):
        while e < len(events) and events[e][0] == kk:
            c0 += 1 if events[e][3] else 0
            e += 1
        if c0 >= k and (kk + 1 >= stop_at or c0 >= max_cand):
            stop = kk
            break
    end = stop if stop is not None else last_step
    cands = [pt for (t, m, pt, l0) in events if t <= end]
    visited = sum(sum(v[:end + 1]) for v in visited_at)
    if with_times:
        return [(t, pt) for (t, m, pt, l0) in events if t <= end]
    return cands, visited, end + 1


MODEL_CASES = [
    # seed, n, dim, M, L, B, T, k, outer
    (0, 120, 6, 2, 3, 1, 4, 3, 2),
    (1, 300, 8, 2, 4, 3, 5, 4, 3),
    (2, 90, 4, 3, 2, 4, 7, 2, 1),
    (3, 200, 5, 1, 3, 2, 1, 5, 50),
    (4, 64, 3, 2, 2, 1, 70, 2, 1),      # T > n
    (5, 150, 6, 2, 5, 7, 2, 10, 1000),  # runs to exhaustion
    (6, 400, 10, 2, 6, 2, 16, 3, 1),    # stops by c0 >= k right after outer*L
]


@pytest.mark.parametrize("case", MODEL_CASES, ids=[str(c) for c in MODEL_CASES])
def test_rank_model_agrees_with_oracle(oracle, case):
    seed, n, dim, M, L, B, T, k, outer = case
    rng = np.random.default_rng(seed)
    X = rng.standard_normal((n, dim)).astype(f32)
    Q = rng.standard_normal((5, dim)).astype(f32)
    P = oracle.normalize(rng.standard_normal((M * L, dim)).astype(f32))
    sk, si = oracle.build_index(P, X, B)
    qp = oracle.project(Q, P)
    r = oracle.query(sk, si, X, Q, qp, M, L, B, T, k, outer, cand_cap=n)
    ppb = -(-n // B)
    for j in range(Q.shape[0]):
        cands, visited, steps = [], 0, 0
        for b in range(B):
            off = b * ppb
            nb = min(n - off, ppb)
            if nb <= 0:
                continue
            c, v, s = _rank_model(sk, si, qp[j], off, nb, M, L, T, k, outer, 10 * k)
            cands += c; visited += v; steps += s
        got = r["cand_ids"][j, :r["cand_cnt"][j]].tolist()
        assert sorted(got) == sorted(cands)
        assert int(r["counters"][j, 0]) == visited
        assert int(r["counters"][j, 3]) == steps
        # the reported neighbours are the k best of exactly those candidates
        d = np.sqrt(((X[cands].astype(np.float64) - Q[j].astype(np.float64)) ** 2).sum(1))
        best = [cands[t] for t in np.argsort(d, kind="stable")[:k]]
        assert set(r["ids"][j].tolist()) - {-1} == set(best)


@pytest.mark.parametrize("case", MODEL_CASES, ids=[str(c) for c in MODEL_CASES])
@pytest.mark.parametrize("max_cand", [None, 3])
def test_rank_model_agrees_with_blind_oracle(oracle, case, max_cand):
    """Blind result = the model's promotion events of all partitions sorted by
    (time, id), cut to min(max_cand, outer) slots."""
    seed, n, dim, M, L, B, T, k, outer = case
    if max_cand is None:
        max_cand = 10 * k
    rng = np.random.default_rng(seed)
    X = rng.standard_normal((n, dim)).astype(f32)
    Q = rng.standard_normal((5, dim)).astype(f32)
    P = oracle.normalize(rng.standard_normal((M * L, dim)).astype(f32))
    sk, si = oracle.build_index(P, X, B)
    qp = oracle.project(Q, P)
    r = oracle.query_blind(sk, si, qp, M, L, B, T, k, outer, max_cand=max_cand)
    R = min(max_cand, outer)
    assert r["ids"].shape == (5, R)
    ppb = -(-n // B)
    for j in range(5):
        ev = []
        for b in range(B):
            off = b * ppb
            nb = min(n - off, ppb)
            if nb > 0:
                ev += _rank_model(sk, si, qp[j], off, nb, M, L, T, k, outer, max_cand, with_times=True)
        ev.sort()
        assert int(r["counters"][j, 1]) == len(ev)
        want_ids = [pt for _, pt in ev][:R] + [-1] * max(0, R - len(ev))
        want_steps = [t for t, _ in ev][:R] + [0xffffffff] * max(0, R - len(ev))
        assert r["ids"][j].tolist() == want_ids
        assert r["steps"][j].astype(np.int64).tolist() == want_steps


def test_blind_candidates_are_the_query_candidates(oracle):
    """The blind ids are points whose distances the ordinary query computes (all of
    them when they fit the slots), in step order, and the counters coincide."""
    rng = np.random.default_rng(21)
    n, dim, M, L = 1500, 10, 2, 3
    X = rng.standard_normal((n, dim)).astype(f32)
    Q = rng.standard_normal((6, dim)).astype(f32)
    P = oracle.normalize(rng.standard_normal((M * L, dim)).astype(f32))
    fitted = 0
    for B, T, k, outer, max_cand in [(1, 1, 6, 100000, 60), (4, 5, 6, 40, 100000), (3, 2, 4, 2000, 25)]:
        sk, si = oracle.build_index(P, X, B)
        qp = oracle.project(Q, P)
        full = oracle.query(sk, si, X, Q, qp, M, L, B, T, k, outer, max_cand=max_cand, cand_cap=n)
        blind = oracle.query_blind(sk, si, qp, M, L, B, T, k, outer, max_cand=max_cand)
        np.testing.assert_array_equal(full["counters"], blind["counters"])
        R = min(max_cand, outer)
        for j in range(6):
            nc = int(full["cand_cnt"][j])
            cands = set(full["cand_ids"][j, :nc].tolist())
            got = blind["ids"][j]
            m = min(nc, R)
            assert set(got[:m].tolist()) <= cands and len(set(got[:m].tolist())) == m
            assert np.all(got[m:] == -1)
            if nc <= R:
                fitted += 1
                assert set(got[:m].tolist()) == cands
            st = blind["steps"][j, :m].astype(np.int64)
            assert np.all(np.diff(st) >= 0)
            same = np.diff(st) == 0
            assert np.all(np.diff(got[:m])[same] > 0), "equal steps rank by id"
    assert fitted > 0


# ------------------------------------------------------------------ invariants
def test_invariants(oracle):
    rng = np.random.default_rng(10)
    n, dim, M, L, B, T, k = 2000, 12, 2, 4, 5, 6, 7
    X = rng.standard_normal((n, dim)).astype(f32)
    Q = rng.standard_normal((8, dim)).astype(f32)
    P = oracle.normalize(rng.standard_normal((M * L, dim)).astype(f32))
    sk, si = oracle.build_index(P, X, B)
    qp = oracle.project(Q, P)
    prev = None
    for outer in (1, 4, 16, 64, 100000):
        r = oracle.query(sk, si, X, Q, qp, M, L, B, T, k, outer, cand_cap=n)
        sets = []
        for j in range(8):
            c = r["cand_ids"][j, :r["cand_cnt"][j]].tolist()
            assert len(c) == len(set(c)), "a point was emitted twice"
            sets.append(set(c))
            assert r["counters"][j, 0] <= M * L * n
            assert np.all(np.diff(r["dists"][j]) >= 0)
            assert len(set(r["ids"][j].tolist())) == k
            # reported distance is the exact distance of the reported id
            d = np.sqrt(((X[r["ids"][j]].astype(np.float64) - Q[j]) ** 2).sum(1))
            np.testing.assert_allclose(r["dists"][j], d, rtol=1e-5)
        if prev is not None:
            for a, b in zip(prev, sets):
                assert a <= b, "candidate set must grow with the iteration budget"
        prev = sets
    # with an unbounded budget and max_cand out of reach everything is promoted
    r = oracle.query(sk, si, X, Q, qp, M, L, B, T, k, 10 ** 9, max_cand=10 ** 9)
    assert np.all(r["counters"][:, 1] == n)
    bi, _ = oracle.brute_force(X, Q, k)
    np.testing.assert_array_equal(r["ids"], bi)


def test_rejects_bad_arguments(oracle):
    X = np.zeros((4, 2), f32)
    P = np.eye(2, dtype=f32)
    sk, si = oracle.build_index(P, X, 1)
    qp = oracle.project(X[:1], P)
    with pytest.raises(ValueError):
        oracle.query(sk, si, X, X[:1], qp, 1, 2, 1, 1, 5, 1)     # k > N
    with pytest.raises(ValueError):
        oracle.query(sk, si, X, X[:1], qp, 1, 2, 1, 1, 0, 1)     # k = 0
