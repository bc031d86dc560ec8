"""The three large benchmark configurations beside the headline one:

  C3  10M x 96, unit-norm Gaussian rows, m=3 L=8 k=100, recall@100 >= 0.9
  C4  1M x 960 on a 32-dimensional manifold, m=2 L=12 k=10
  C5  20 batches of 1M x 64 N(0,1) rows added one after the other, m=2 L=15 k=50

Each is checked twice.  At reduced N, with the configuration's own generator, shape
parameters (m, L, k, dim) and per-partition regime, the engine is compared with the
CPU oracle: traversal parity on the engine's own keys (ids, distances, candidate and
step counters; visits for the step kernel) for every traversal kernel, and end to end
from shared directions.  At full size, where the oracle would take minutes, the checks
are properties that do not depend on the size: recall against exact k-NN, every
returned distance being the distance of the id beside it, the traversal kernels
agreeing with each other bit for bit on a query sample, and for C5 the index grown by
twenty appends answering exactly like one built by a single add of all rows.
"""
import sys
import time

import numpy as np
import pytest
import torch

import bench
from util import batch_fits, dense_fits, engine_index, engine_project, set_agreement

pytestmark = pytest.mark.gpu

DIST_RTOL = 1e-5

# the settings bench.py runs these configurations at (block_size, thread_size, outer)
C3_SETTING, C4_SETTING, C5_SETTING = ((bench.TUNED[c]["bs"], bench.TUNED[c]["ts"], bench.TUNED[c]["outer"])
                                      for c in ("c3", "c4", "c5"))


def _say(*a):
    print(*a, flush=True, file=sys.stderr)


def _l1(gpu, oracle, dci, X, Q, M, L, B, T, k, outer, modes):
    """Every traversal kernel in `modes` against the oracle walking the engine's own keys."""
    skeys, sids = engine_index(dci)
    qproj = engine_project(dci.directions.numpy(), Q).T.copy()
    ref = oracle.query(skeys, sids, X, Q, qproj, M, L, B, T, k, outer, max_cand=10 * k)
    rc = ref["counters"].astype(np.int64)
    qd = torch.from_numpy(Q).cuda()
    first = None
    n = X.shape[0]
    for mode in modes:
        if (mode == "dense" and not dense_fits(n, M, L, B, T, k)) or (mode == "batch" and not batch_fits(n, M, L, B, k)):
            continue    # these kernels refuse shapes beyond their tables
        dci.set_traversal(mode)
        ids, dists, ctr = dci.query(qd, k, outer, return_int=True, return_counters=True)
        torch.cuda.synchronize()
        ids, dists, ctr = ids.cpu().numpy(), dists.cpu().numpy(), ctr.cpu().numpy()
        if mode == "step":
            np.testing.assert_array_equal(ctr[:, 0], rc[:, 0], err_msg="entries visited (%s)" % mode)
        np.testing.assert_array_equal(ctr[:, 1], rc[:, 1], err_msg="candidates promoted (%s)" % mode)
        np.testing.assert_array_equal(ctr[:, 3], rc[:, 3], err_msg="outer steps (%s)" % mode)
        np.testing.assert_allclose(dists, ref["dists"], rtol=DIST_RTOL, atol=1e-6)
        assert set_agreement(ids, ref["ids"]) >= 0.999, mode
        if first is None:
            first = (ids, dists)
        else:   # the kernels agree with each other bit for bit
            np.testing.assert_array_equal(ids, first[0], err_msg=mode)
            np.testing.assert_array_equal(dists, first[1], err_msg=mode)
    dci.set_traversal("auto")
    return ref


def _l2(oracle, dci, X, Q, M, L, B, T, k, outer):
    """End to end: only rows, queries and directions are shared with the oracle."""
    ids, dists = dci.query(torch.from_numpy(Q).cuda(), k, outer, return_int=True)
    ref = oracle.knn(dci.directions.numpy(), X, Q, M, L, B, T, k, outer)
    assert set_agreement(ids.cpu().numpy(), ref["ids"]) >= 0.999
    np.testing.assert_allclose(np.sort(dists.cpu().numpy(), 1), np.sort(ref["dists"], 1), rtol=DIST_RTOL)


def _properties(dci, Xd, Qd, k, outer, want_recall):
    """Size-independent checks of one query batch; returns the recall."""
    from dciknn_cuda_amd import workloads
    ids, dists = dci.query(Qd, k, outer, return_int=True)
    truth = workloads.exact_knn(Xd, Qd, k)
    recall = workloads.recall_at_k(ids, truth)
    assert recall >= want_recall, recall
    assert torch.all(dists[:, 1:] >= dists[:, :-1])
    assert torch.all(ids >= 0) and torch.all(ids < Xd.shape[0])
    for s in range(0, Qd.shape[0], 64):      # a returned distance is the distance of its id
        d = (Xd[ids[s:s + 64].long()] - Qd[s:s + 64, None, :]).norm(dim=2)
        assert torch.allclose(d, dists[s:s + 64], rtol=1e-5, atol=1e-4)
    srt = ids.sort(dim=1).values
    assert torch.all(srt[:, 1:] != srt[:, :-1])    # no id twice
    return recall


def _kernels_agree(dci, Qd, k, outer, modes):
    out = {}
    for mode in modes:
        dci.set_traversal(mode)
        out[mode] = dci.query(Qd, k, outer, return_int=True, return_counters=True)
        torch.cuda.synchronize()
    dci.set_traversal("auto")
    a = out[modes[0]]
    for mode in modes[1:]:
        b = out[mode]
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1]), mode
        assert torch.equal(a[2][:, 1], b[2][:, 1]) and torch.equal(a[2][:, 3], b[2][:, 3]), mode


# ------------------------------------------------------------------ reduced N, oracle
@pytest.mark.parametrize("n,B,T,outer,modes", [
    # slices of 65000 points: the build sorts them as tiles + merge passes; near the batch kernel's limit
    (130_000, 2, 32, 1700, ["step", "batch", "auto"]),
    # the full-size setting's partition length (25000) and windows: stops by c0 >= 100, ~12800 promotions
    (75_000, 3, 128, 100, ["step", "dense", "auto"]),
    # an earlier full-size setting: 20000-point partitions, stops by the step limit
    (60_000, 3, 32, 530, ["step", "batch", "dense", "auto"]),
    # narrow windows: stops by c0 >= k well before the step limit
    (60_000, 6, 1, 60, ["step", "batch", "dense", "auto"]),
])
def test_c3_reduced_against_oracle(gpu, oracle, n, B, T, outer, modes):
    from dciknn_cuda_amd import workloads
    M, L, k, dim, nq = 3, 8, 100, 96, 32
    _say("c3 reduced", n, B, T, outer)
    X, Q = workloads.c3(n=n, nq=nq)
    X, Q = X.numpy(), Q.numpy()
    dci = gpu.DCI(dim, M, L, B, T, seed=33)
    dci.add(torch.from_numpy(X).cuda())
    _l1(gpu, oracle, dci, X, Q, M, L, B, T, k, outer, modes)
    _l2(oracle, dci, X, Q, M, L, B, T, k, outer)
    dci.free()


@pytest.mark.parametrize("n,B,T,outer,modes", [
    (30_000, 3, 64, 126, ["step", "dense", "auto"]),              # the full-size setting: step limit, ~1300 promotions per partition
    (30_000, 3, 16, 500, ["step", "batch", "dense", "auto"]),     # the same regime with narrower windows
    (30_000, 3, 10, 500, ["step", "batch", "dense", "auto"]),     # the reference example's thread_size
    (70_000, 2, 4, 2000, ["step", "batch", "auto"]),              # 35000-point slices
])
def test_c4_reduced_against_oracle(gpu, oracle, n, B, T, outer, modes):
    from dciknn_cuda_amd import workloads
    M, L, k, dim, nq = 2, 12, 10, 960, 32
    _say("c4 reduced", n, B, T, outer)
    X, Q = workloads.c4(n=n, nq=nq)
    X, Q = X.numpy(), Q.numpy()
    dci = gpu.DCI(dim, M, L, B, T, seed=44)
    dci.add(torch.from_numpy(X).cuda())
    _l1(gpu, oracle, dci, X, Q, M, L, B, T, k, outer, modes)
    _l2(oracle, dci, X, Q, M, L, B, T, k, outer)
    dci.free()


@pytest.mark.parametrize("batch_rows,B,T,outer", [(20_000, 4, 8, 500), (7_001, 5, 2, 100)])
def test_c5_reduced_appends_against_oracle(gpu, oracle, batch_rows, B, T, outer):
    """L = 15 built by successive appends; after every append the index answers like the
    oracle's index over all rows so far."""
    from dciknn_cuda_amd import workloads
    M, L, k, dim, nq = 2, 15, 50, 64, 24
    Q = workloads.c5_queries(nq=nq).numpy()
    dci = gpu.DCI(dim, M, L, B, T, seed=55)
    rows = []
    for batch in range(4):
        _say("c5 reduced", batch_rows, B, T, "append", batch)
        xb = workloads.c5_batch(batch, n=batch_rows)
        rows.append(xb.numpy())
        dci.append(xb.cuda())
        X = np.concatenate(rows)
        modes = ["step", "batch", "dense", "auto"] if batch in (0, 3) else ["auto"]
        _l1(gpu, oracle, dci, X, Q, M, L, B, T, k, outer, modes)
    _l2(oracle, dci, X, Q, M, L, B, T, k, outer)
    # and exactly the index a single add builds
    one = gpu.DCI(dim, M, L, B, T, directions=dci.directions)
    one.add(torch.from_numpy(X).cuda())
    ka, ia = engine_index(dci)
    kb, ib = engine_index(one)
    np.testing.assert_array_equal(ka, kb)
    np.testing.assert_array_equal(ia, ib)
    one.free()
    dci.free()


def test_c5_reduced_at_the_full_size_operating_point(gpu, oracle):
    """The regime the benchmark runs C5 in at 20M points: 22223 points per partition, windows of
    128, 10 outer iterations, L = 15, k = 50 (the stop is set by c0 >= 50: thousands of promotions
    per partition).  Three such partitions against the oracle."""
    from dciknn_cuda_amd import workloads
    B20, T, outer = C5_SETTING
    ppb = -(-20_000_000 // B20)
    M, L, k, dim, nq, B = 2, 15, 50, 64, 24, 3
    n = B * ppb
    Q = workloads.c5_queries(nq=nq).numpy()
    X = workloads.c5_batch(0, n=n).numpy()
    dci = gpu.DCI(dim, M, L, B, T, seed=56)
    dci.add(torch.from_numpy(X).cuda())
    assert -(-n // B) == ppb
    _l1(gpu, oracle, dci, X, Q, M, L, B, T, k, outer, ["step", "batch", "dense", "auto"])
    _l2(oracle, dci, X, Q, M, L, B, T, k, outer)
    dci.free()


# ------------------------------------------------------------------ full size, properties
def test_c3_full_size(gpu):
    from dciknn_cuda_amd import workloads
    B, T, outer = C3_SETTING
    t = time.time()
    X, Q = workloads.c3()
    _say("c3 full: generated in %.1f s" % (time.time() - t))
    Xd, Qd = X.cuda(), Q[:192].contiguous().cuda()
    del X
    dci = gpu.DCI(96, 3, 8, B, T, seed=4)
    dci.add(Xd)
    recall = _properties(dci, Xd, Qd, 100, outer, 0.9)
    _say("c3 full: recall@100 %.4f" % recall)
    _kernels_agree(dci, Qd[:6].contiguous(), 100, outer, ["step", "batch", "dense", "auto"])
    # the sorted slices are sorted, and hold every id of their partition once (one simple index)
    n, ppb = Xd.shape[0], -(-Xd.shape[0] // B)
    keys, ids = engine_index(dci)
    for i in (0, 11, 23):
        kk, ii = torch.from_numpy(keys[i]).cuda().view(B, ppb), torch.from_numpy(ids[i]).cuda().view(B, ppb)
        assert torch.all(kk[:, 1:] >= kk[:, :-1])
        assert torch.equal(ii.sort(dim=1).values, torch.arange(n, device="cuda", dtype=torch.int32).view(B, ppb))
        proj = Xd @ dci.directions[i].cuda()
        assert torch.allclose(proj[ii.flatten().long()], kk.flatten(), rtol=1e-4, atol=1e-5)
    dci.free()


def test_c4_full_size(gpu):
    from dciknn_cuda_amd import workloads
    B, T, outer = C4_SETTING
    t = time.time()
    X, Q = workloads.c4()
    _say("c4 full: generated in %.1f s" % (time.time() - t))
    Xd, Qd = X.cuda(), Q[:512].contiguous().cuda()
    del X
    dci = gpu.DCI(960, 2, 12, B, T, seed=4)
    dci.add(Xd)
    recall = _properties(dci, Xd, Qd, 10, outer, 0.95)
    _say("c4 full: recall@10 %.4f" % recall)
    _kernels_agree(dci, Qd[:48].contiguous(), 10, outer, ["step", "batch", "dense", "auto"])
    dci.free()


def test_c5_full_size_appends_equal_one_add(gpu):
    from dciknn_cuda_amd import workloads
    B, T, outer = C5_SETTING
    k, dim = 50, 64
    Qd = workloads.c5_queries(nq=128).cuda()
    grown = gpu.DCI(dim, 2, 15, B, T, seed=4)
    Xd = torch.empty((20_000_000, dim), dtype=torch.float32, device="cuda")
    recalls = []
    t = time.time()
    for batch in range(20):
        xb = workloads.c5_batch(batch).cuda()
        Xd[batch * 1_000_000:(batch + 1) * 1_000_000] = xb
        grown.append(xb)
        if batch in (0, 9):
            recalls.append(_properties(grown, Xd[:(batch + 1) * 1_000_000], Qd[:64].contiguous(), k, outer, 0.0))
    _say("c5 full: 20 appends (with generation) in %.1f s" % (time.time() - t))
    recalls.append(_properties(grown, Xd, Qd, k, outer, 0.9))
    _say("c5 full: recall@50 after 1, 10, 20 batches", recalls)
    _kernels_agree(grown, Qd[:6].contiguous(), k, outer, ["step", "dense", "auto"])
    one = gpu.DCI(dim, 2, 15, B, T, directions=grown.directions)
    one.add(Xd)
    for mode in ("auto", "step"):
        grown.set_traversal(mode)
        one.set_traversal(mode)
        q = Qd if mode == "auto" else Qd[:4].contiguous()
        a = grown.query(q, k, outer, return_int=True, return_counters=True)
        b = one.query(q, k, outer, return_int=True, return_counters=True)
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
        assert torch.equal(a[2][:, 1], b[2][:, 1]) and torch.equal(a[2][:, 3], b[2][:, 3])
        if mode == "step":
            assert torch.equal(a[2], b[2])
    one.free()
    grown.free()
