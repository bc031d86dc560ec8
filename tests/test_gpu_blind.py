"""GPU parity of blind querying (query_config.blind, src/dci_cuda_kernel.cu:498-505,
:754-773, :859-864): the HIP engine through libdci_hip.so against the CPU oracle.

Blind querying computes no distance, so everything is integer work and must
match the oracle EXACTLY: candidate ids in (promoting step, id) order, the
steps themselves, and the traversal counters.  The oracle is fed the engine's
own sorted projections and query projections, as in the traversal parity tests.
"""
import numpy as np
import pytest
import torch

from util import engine_index, engine_project

pytestmark = pytest.mark.gpu


def _data(seed, n, nq, dim, kind="normal"):
    rng = np.random.default_rng(seed)
    if kind == "grid":   # many exactly equal projections
        x = rng.integers(0, 3, (n + nq, dim)).astype(np.float64)
    else:
        x = rng.standard_normal((n + nq, dim))
    x = x.astype(np.float32)
    return x[:n], x[n:]


def _engine_blind(dci, qd, k, outer, max_cand, B, T, want_steps=True):
    """Straight through the C-ABI: ids [nq][R], steps [nq][R] or None, counters."""
    from dciknn_cuda_amd import _capi
    nq, dim = qd.shape
    R = min(max_cand, outer)
    ids = torch.full((nq, R), -7, dtype=torch.int32, device="cuda")
    steps = torch.full((nq, R), -7.0, dtype=torch.float32, device="cuda") if want_steps else None
    ctr = torch.empty((nq, 4), dtype=torch.int64, device="cuda")
    _capi.check(dci._lib.dcih_query(dci._dci_inst, dim, nq, qd.data_ptr(), k, 1, outer, max_cand,
                                    B, T, ids.data_ptr(), steps.data_ptr() if want_steps else None,
                                    ctr.data_ptr(), torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return ids.cpu().numpy(), steps.cpu().numpy() if want_steps else None, ctr.cpu().numpy()


def _check(ids, steps, ctr, ref, visits):
    np.testing.assert_array_equal(ids, ref["ids"])
    if steps is not None:
        want = ref["steps"].astype(np.float64)
        want[ref["ids"] < 0] = np.inf
        np.testing.assert_array_equal(steps.astype(np.float64), want)
    rc = ref["counters"].astype(np.int64)
    if visits:
        np.testing.assert_array_equal(ctr[:, 0], rc[:, 0])
    np.testing.assert_array_equal(ctr[:, 1], rc[:, 1])
    np.testing.assert_array_equal(ctr[:, 3], rc[:, 3])


CASES = [
    # n, nq, dim, M, L, B, T, k, outer, max_cand, kind
    (3000, 32, 100, 2, 10, 100, 10, 10, 5000, 100, "normal"),   # exhaustive: every point is a candidate, 100 slots
    (3000, 32, 100, 2, 10, 10, 10, 10, 20, 100, "normal"),      # 20 slots, stop by outer*L
    (3000, 32, 40, 2, 10, 3, 4, 10, 5000, 100, "normal"),       # stop by c0 >= max_cand
    (2000, 32, 16, 2, 5, 1, 1, 5, 50, 50, "normal"),            # T=1, B=1
    (2000, 16, 16, 3, 4, 7, 64, 20, 3, 200, "normal"),          # 3 slots only
    (500, 16, 8, 1, 1, 4, 3, 3, 10, 30, "normal"),              # single simple index
    (100, 16, 8, 2, 3, 200, 2, 5, 300, 50, "normal"),           # B > n: empty partitions, more slots than candidates
    (4000, 16, 24, 2, 10, 2, 16, 100, 30, 1000, "grid"),        # ties everywhere
    (40000, 16, 24, 2, 12, 2, 16, 10, 200, 100, "normal"),      # hundreds of promotions per partition
    (30000, 16, 16, 2, 15, 2, 4, 50, 300, 500, "normal"),       # L = 15
    (20000, 8, 16, 2, 6, 4, 8, 100, 3000, 1000, "normal"),      # 1000 slots: beyond the batch kernel's tables
]


@pytest.mark.parametrize("traversal", ["step", "batch", "auto"])
@pytest.mark.parametrize("case", CASES, ids=[str(c[:10]) for c in CASES])
def test_blind_parity(gpu, oracle, case, traversal):
    n, nq, dim, M, L, B, T, k, outer, max_cand, kind = case
    R = min(max_cand, outer)
    if traversal == "batch" and min(R, -(-n // B)) > 512:
        pytest.skip("more slots per partition than the batch kernel's tables hold (auto mode falls back)")
    X, Q = _data(n * 3 + T, n, nq, dim, kind)
    dci = gpu.DCI(dim, M, L, B, T, seed=5, traversal=traversal)
    dci.add(torch.from_numpy(X).cuda())
    qd = torch.from_numpy(Q).cuda()
    ids, steps, ctr = _engine_blind(dci, qd, k, outer, max_cand, B, T)
    skeys, sids = engine_index(dci)
    qproj = engine_project(dci.directions.numpy(), Q).T.copy()
    ref = oracle.query_blind(skeys, sids, qproj, M, L, B, T, k, outer, max_cand=max_cand)
    dci.free()
    _check(ids, steps, ctr, ref, visits=(traversal == "step"))


def test_blind_without_step_output(gpu, oracle):
    """d_dists may be NULL in blind mode (src/dci_cuda_kernel.cu:776)."""
    X, Q = _data(9, 5000, 16, 12)
    dci = gpu.DCI(12, 2, 4, 5, 6, seed=1)
    dci.add(torch.from_numpy(X).cuda())
    qd = torch.from_numpy(Q).cuda()
    ids, _, ctr = _engine_blind(dci, qd, 4, 25, 40, 5, 6, want_steps=False)
    skeys, sids = engine_index(dci)
    qproj = engine_project(dci.directions.numpy(), Q).T.copy()
    ref = oracle.query_blind(skeys, sids, qproj, 2, 4, 5, 6, 4, 25, max_cand=40)
    dci.free()
    _check(ids, None, ctr, ref, visits=False)


def test_blind_python_surface(gpu, oracle):
    """DCI.query(blind=True) and MDCI.query(blind=True): ids as floats like every
    result of the reference's binding (src/dci_cuda.cpp:106-115), min(10k, outer)
    columns, second tensor = promoting steps; candidates are exactly those whose
    distances the ordinary query computes."""
    X, Q = _data(4, 8000, 8, 16)
    k, outer = 5, 40
    xd, qd = torch.from_numpy(X).cuda(), torch.from_numpy(Q).cuda()
    dci = gpu.DCI(16, 2, 5, 4, 8, seed=3)
    dci.add(xd)
    ids, steps = dci.query(qd, k, outer, blind=True)
    assert ids.shape == (8, 40) and steps.shape == (8, 40) and ids.dtype == torch.float32
    ids2, steps2, ctr = dci.query(qd, k, outer, blind=True, return_int=True, return_counters=True)
    assert ids2.dtype == torch.int32
    assert torch.equal(ids, ids2.to(torch.float32)) and torch.equal(steps, steps2)
    skeys, sids = engine_index(dci)
    qproj = engine_project(dci.directions.numpy(), Q).T.copy()
    ref = oracle.query_blind(skeys, sids, qproj, 2, 5, 4, 8, k, outer)
    np.testing.assert_array_equal(ids2.cpu().numpy(), ref["ids"])
    # the ordinary query of the same shape stops at the same place
    _, _, ctr_plain = dci.query(qd, k, outer, return_int=True, return_counters=True)
    assert torch.equal(ctr[:, 1], ctr_plain[:, 1]) and torch.equal(ctr[:, 3], ctr_plain[:, 3])
    dci.free()
    mdci = gpu.MDCI(16, 2, 5, 4, 8, devices=[0], seed=3)
    mdci.add(xd)
    mids, msteps = mdci.query(qd, k, outer, blind=True)
    assert torch.equal(mids, ids) and torch.equal(msteps, steps)
    mdci.free()


def test_blind_more_than_8192_slots(gpu, oracle):
    """min(10k, outer) above the top-k tables: candidates are recorded in a dense row
    per query and sorted from there; same ids, steps and counters as the oracle."""
    n, dim, M, L, B, T, k, outer = 30000, 8, 2, 3, 2, 4, 1000, 9000      # 9000 slots
    X, Q = _data(2, n, 3, dim)
    dci = gpu.DCI(dim, M, L, B, T, seed=1)
    dci.add(torch.from_numpy(X).cuda())
    ids, steps, ctr = _engine_blind(dci, torch.from_numpy(Q).cuda(), k, outer, 10 * k, B, T)
    skeys, sids = engine_index(dci)
    qproj = engine_project(dci.directions.numpy(), Q).T.copy()
    ref = oracle.query_blind(skeys, sids, qproj, M, L, B, T, k, outer, max_cand=10 * k)
    dci.free()
    assert ids.shape == (3, 9000)
    _check(ids, steps, ctr, ref, visits=True)
