"""The hand-over from the batch traversal kernel to the dense one under automatic kernel
choice: an item whose traversal turns out to need many promotions is abandoned half-way by
the batch kernel, entered in a per-die list and computed from scratch by the dense kernel;
from the second call on, partitions whose earlier stops needed that many are handed over
before any work is done on them.  Which kernel finishes an item must not show in ids,
distances or counters.  The shapes stop on the step limit after 50 to 300 promotions per
partition (found with the CPU oracle), so with the threshold just above what routes a
whole call to the dense kernel some items cross twice the threshold and others do not."""
import numpy as np
import pytest
import torch

from util import engine_index, engine_project, set_agreement

pytestmark = pytest.mark.gpu

# n, dim, M, L, B, T, k, outer
SHAPES = [(24_000, 12, 2, 4, 3, 4, 8, 700), (16_000, 8, 2, 3, 2, 4, 10, 400)]


def _threshold(n, L, B, T, k, outer):
    """Smallest DCIH_OPT_DENSE_MIN_PROMOTIONS that leaves the call with the batch kernel: above
    k * T and above the promotions the step limit is estimated to need (query.hip's rule)."""
    ppb = -(-n // B)
    f = min(1.0, outer * T / ppb)
    return int(max(k * T, min(ppb * f ** L, 10 * k * T))) + 1


@pytest.mark.parametrize("shape", SHAPES, ids=[str(s) for s in SHAPES])
def test_items_handed_to_the_dense_kernel_answer_alike(gpu, oracle, shape):
    from dciknn_cuda_amd import _capi
    n, dim, M, L, B, T, k, outer = shape
    rng = np.random.default_rng(n + dim)
    X = rng.standard_normal((n, dim)).astype(np.float32)
    Q = rng.standard_normal((96, dim)).astype(np.float32)
    dci = gpu.DCI(dim, M, L, B, T, seed=9)
    lib, h = dci._lib, dci._dci_inst
    dci.add(torch.from_numpy(X).cuda())
    skeys, sids = engine_index(dci)
    qproj = engine_project(dci.directions.numpy(), Q).T.copy()
    ref = oracle.query(skeys, sids, X, Q, qproj, M, L, B, T, k, outer, max_cand=10 * k)
    rc = ref["counters"].astype(np.int64)
    dmp = _threshold(n, L, B, T, k, outer)
    # the premise: partitions on both sides of the hand-over point (twice the threshold)
    per_item = rc[:, 1] / B
    assert per_item.max() > 2 * dmp > per_item.min(), (per_item.min(), per_item.max(), dmp)
    qd = torch.from_numpy(Q).cuda()
    dci.set_traversal("step")
    want = dci.query(qd, k, outer, return_int=True, return_counters=True)
    dci.set_traversal("auto")
    _capi.check(lib.dcih_profile(h, 1))
    tms = (_capi.ctypes.c_float * _capi.NUM_TIMERS)()

    def run(value):
        _capi.check(lib.dcih_set_option(h, _capi.OPT_DENSE_MIN_PROMOTIONS, value))
        out = dci.query(qd, k, outer, return_int=True, return_counters=True)
        torch.cuda.synchronize()
        _capi.check(lib.dcih_last_timings(h, tms))
        return out, float(tms[_capi.T_BATCH]), float(tms[_capi.T_DENSE])

    # first call: items cross the hand-over point in mid-traversal; second call: the hints
    # learnt by the first send whole partitions over at the start
    for call in range(2):
        got, t_batch, t_dense = run(dmp)
        assert t_batch >= 0.0 and t_dense >= 0.0, "call %d: both kernels must have run" % call
        ids, dists, ctr = (v.cpu().numpy() for v in got)
        np.testing.assert_array_equal(ctr[:, 1], rc[:, 1], err_msg="candidates promoted, call %d" % call)
        np.testing.assert_array_equal(ctr[:, 3], rc[:, 3], err_msg="outer steps, call %d" % call)
        assert set_agreement(ids, ref["ids"]) == 1.0
        np.testing.assert_allclose(dists, ref["dists"], rtol=1e-5, atol=1e-6)
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]), "differs from the step kernel"
    # 0 = the dense kernel is never used
    got, t_batch, t_dense = run(0)
    assert t_batch >= 0.0 and t_dense < 0.0
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    assert torch.equal(got[2][:, [1, 3]], want[2][:, [1, 3]])
    # a threshold nobody reaches: the lists exist and stay empty
    got, t_batch, t_dense = run(100_000)
    assert t_batch >= 0.0
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    dci.free()


def test_items_that_outgrow_the_compact_tables_answer_alike(gpu, oracle):
    """The batch kernel's one-wavefront variants keep an item's flags in a small hashed set; an
    item that promotes more points than the set takes is listed and computed again by the
    variant with the full tables.  The phase profile counts the items handed back: some must
    be (the premise), and ids, distances and counters must not show it."""
    from dciknn_cuda_amd import _capi
    n, dim, M, L, B, T, k, outer, nq = 60_000, 16, 2, 10, 3, 4, 15, 100, 96
    rng = np.random.default_rng(5)
    X = rng.standard_normal((n, dim)).astype(np.float32)
    Q = rng.standard_normal((nq, dim)).astype(np.float32)
    dci = gpu.DCI(dim, M, L, B, T, seed=9, traversal="batch")
    lib, h = dci._lib, dci._dci_inst
    dci.add(torch.from_numpy(X).cuda())
    skeys, sids = engine_index(dci)
    qproj = engine_project(dci.directions.numpy(), Q).T.copy()
    ref = oracle.query(skeys, sids, X, Q, qproj, M, L, B, T, k, outer, max_cand=10 * k)
    rc = ref["counters"].astype(np.int64)
    qd = torch.from_numpy(Q).cuda()
    ticks = torch.zeros(16, dtype=torch.int64, device="cuda")
    _capi.check(lib.dcih_phase_profile(h, ticks.data_ptr()))
    for call in range(2):       # the second call routes by the recorded stops as well
        ids, dists, ctr = dci.query(qd, k, outer, return_int=True, return_counters=True)
        torch.cuda.synchronize()
        ids, dists, ctr = ids.cpu().numpy(), dists.cpu().numpy(), ctr.cpu().numpy().astype(np.int64)
        np.testing.assert_array_equal(ids, ref["ids"])
        np.testing.assert_allclose(dists, ref["dists"], rtol=1e-5, atol=1e-6)
        np.testing.assert_array_equal(ctr[:, 1], rc[:, 1])
        np.testing.assert_array_equal(ctr[:, 3], rc[:, 3])
    _capi.check(lib.dcih_phase_profile(h, None))
    t = ticks.cpu().numpy()
    assert t[10] > 0, "no item was handed from the compact tables to the second pass"
    assert t[9] == 2 * nq * B, (t[9], "every item finished in the batch kernel, first or second pass")
    dci.free()
