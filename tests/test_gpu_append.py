"""dcih_append by merging (old slices split into runs of the new ones, new points sorted,
runs merged) against a single add of all rows: the sorted keys and ids must be bit-equal,
and queries through every traversal kernel (which also read the 16-bit local ids and the
inverse permutation the merge writes) must answer alike.  Shapes cover partitions that grow a
little, double, grow many-fold (several merge passes), stay the same length, block sizes above
the number of points and a single partition."""
import numpy as np
import pytest
import torch

from util import batch_fits, dense_fits, engine_index

pytestmark = pytest.mark.gpu

SHAPES = [
    # dim, M, L, B, batch sizes
    (16, 2, 3, 4, [1000, 1000, 1000, 1000]),          # 250 -> 500 -> 750 -> 1000 per partition
    (8, 1, 2, 7, [5000, 300, 7, 1, 20000]),           # small growth, same partition length, then five-fold
    (8, 2, 2, 3, [100, 5000]),                        # fifty-fold: many runs per new slice, several passes
    (12, 2, 4, 1, [3000, 2000, 9000]),                # one partition
    (8, 1, 3, 50, [20, 40, 3000]),                    # more partitions than points at first
    (32, 2, 5, 16, [40000, 40000, 40000, 100000]),    # slices of 2500 .. 13750
    (8, 1, 2, 2, [30000, 30000]),                     # slices of 30000: the longest the merge takes
    (64, 2, 15, 6, [9000, 9000, 9000]),               # the incremental workload's index shape
]


@pytest.mark.parametrize("shape", SHAPES, ids=[str(s[:4]) + "x%d" % len(s[4]) for s in SHAPES])
def test_append_by_merge_equals_one_add(gpu, shape):
    from dciknn_cuda_amd import _capi
    dim, M, L, B, batches = shape
    rng = np.random.default_rng(sum(batches) + B)
    grown = gpu.DCI(dim, M, L, B, 4, seed=7)
    _capi.check(grown._lib.dcih_set_option(grown._dci_inst, _capi.OPT_APPEND, _capi.APPEND_MERGE))
    resorted = gpu.DCI(dim, M, L, B, 4, directions=grown.directions)
    _capi.check(resorted._lib.dcih_set_option(resorted._dci_inst, _capi.OPT_APPEND, _capi.APPEND_SORT))
    rows = []
    for nb in batches:
        x = rng.standard_normal((nb, dim)).astype(np.float32)
        x[::5] = np.round(x[::5])                      # equal keys across old and new points
        rows.append(x)
        xd = torch.from_numpy(x).cuda()
        grown.append(xd)
        resorted.append(xd)
        ka, ia = engine_index(grown)
        kb, ib = engine_index(resorted)
        np.testing.assert_array_equal(ka, kb)
        np.testing.assert_array_equal(ia, ib)
    X = np.concatenate(rows)
    one = gpu.DCI(dim, M, L, B, 4, directions=grown.directions)
    one.add(torch.from_numpy(X).cuda())
    kc, ic = engine_index(one)
    np.testing.assert_array_equal(ka, kc)
    np.testing.assert_array_equal(ia, ic)
    n = X.shape[0]
    k = min(10, -(-n // B))
    Q = torch.from_numpy(rng.standard_normal((8, dim)).astype(np.float32)).cuda()
    for mode in ("step", "batch", "dense", "auto"):
        if (mode == "dense" and not dense_fits(n, M, L, B, 4, k)) or (mode == "batch" and not batch_fits(n, M, L, B, k)):
            continue
        grown.set_traversal(mode)
        one.set_traversal(mode)
        a = grown.query(Q, k, 30, return_int=True, return_counters=True)
        b = one.query(Q, k, 30, return_int=True, return_counters=True)
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1]), mode
        # candidates and steps always; entries visited and probes are exact for the step kernel
        # only (the other kernels' own counts depend on what earlier queries taught the handle)
        cols = [0, 1, 2, 3] if mode == "step" else [1, 3]
        assert torch.equal(a[2][:, cols], b[2][:, cols]), mode
    for d in (grown, resorted, one):
        d.free()


def test_merge_refuses_long_partitions(gpu):
    from dciknn_cuda_amd import _capi
    d = gpu.DCI(8, 1, 2, 1, 4, seed=1)
    _capi.check(d._lib.dcih_set_option(d._dci_inst, _capi.OPT_APPEND, _capi.APPEND_MERGE))
    x = torch.randn(20000, 8, device="cuda")
    d.append(x)                                        # the first append has nothing to merge with
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        with pytest.raises(_capi.DCIError):
            d.append(x)                                # one partition of 40000 points
    torch.cuda.synchronize()
    # a refused append allocates nothing it keeps (the buffers for 40000 rows would be 1.9 MB a call)
    assert torch.cuda.mem_get_info()[0] >= free_before - (1 << 20)
    assert d.num_points == 20000
    _capi.check(d._lib.dcih_set_option(d._dci_inst, _capi.OPT_APPEND, _capi.APPEND_AUTO))
    d.append(x)                                        # left to choose, it sorts
    assert d.num_points == 40000
    d.free()
