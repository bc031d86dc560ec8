"""Host-side checks that need no GPU: the C-ABI library loads and exports what
include/*.h declare, argument errors come back as status codes, and the
Python front end validates its inputs like dciknn_cuda/core.py:53-92 does."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    names = set()
    for header in ("dci_hip.h", "dci_hip_debug.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(dcih_[a-z_]+)\s*\(", text))
    return sorted(names)


def test_library_exports_every_declared_symbol():
    from dciknn_cuda_amd import _capi
    lib = ctypes.CDLL(_capi.LIB_PATH)
    names = _declared()
    assert len(names) >= 15
    for name in names:
        assert hasattr(lib, name), "libdci_hip.so lacks %s" % name
        assert name in _capi.SIGNATURES, "no ctypes signature for %s" % name
    assert set(_capi.SIGNATURES) == set(names)
    assert _capi.lib().dcih_abi_version() == 2


def test_null_and_bad_arguments_return_status_codes():
    """No compute: only paths that fail before any HIP call."""
    from dciknn_cuda_amd import _capi
    lib = _capi.lib()
    assert lib.dcih_add(None, 4, 10, None, 1, 1, None) == -1
    assert b"null handle" in lib.dcih_last_error()
    assert lib.dcih_query(None, 4, 1, None, 1, 0, 1, 10, 1, 1, None, None, None, None) == -1
    assert lib.dcih_query_noalloc(None, 4, 1, None, 1, 0, 1, 10, 1, 1, None, None, None, None) == -1
    assert lib.dcih_create(0, 1, 1, 0, 0, ctypes.byref(ctypes.c_void_p())) == -1
    assert lib.dcih_create(4, 1, 1, 0, 0, None) == -1
    assert lib.dcih_project(None, 1, None, 1, 1, None, None) == -1
    assert lib.dcih_segsort(None, 1, 1, 1, None, None, None) == -1
    assert lib.dcih_free(None) == 0
    assert lib.dcih_num_points(None) == 0
    with pytest.raises(_capi.DCIError):
        _capi.check(lib.dcih_clear(None))


@pytest.mark.parametrize("xcds,B,nq", [(8, 56, 10), (8, 100, 7), (8, 3, 5), (8, 1, 1), (8, 9, 16),
                                       (4, 10, 3), (1, 5, 4), (8, 13, 1), (8, 8, 3)])
def test_batch_kernel_launch_map_covers_every_item_once(xcds, B, nq):
    """Every (partition, query) pair belongs to exactly one workgroup, workgroup w runs on
    die w mod xcds, a die works through one partition's queries before the next partition's,
    and the dies' shares differ by at most one run of the leftover partitions."""
    from dciknn_cuda_amd import _capi
    lib = _capi.lib()
    b, q, per = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    items = lib.dcih_debug_launch_map(xcds, B, nq, -1, None, None, ctypes.byref(per))
    assert per.value == nq and items >= B * nq and items * 256 < 2 ** 32
    seen = {}
    load = [0] * xcds
    order = [[] for _ in range(xcds)]
    for w in range(items):
        assert lib.dcih_debug_launch_map(xcds, B, nq, w, ctypes.byref(b), ctypes.byref(q), None) == items
        if b.value < 0:
            assert q.value < 0
            continue
        assert 0 <= b.value < B and 0 <= q.value < nq
        assert (b.value, q.value) not in seen
        seen[(b.value, q.value)] = w
        load[w % xcds] += 1
        order[w % xcds].append(b.value)
    assert len(seen) == B * nq
    assert max(load) - min(load) <= -(-((B % xcds) * nq) // xcds)
    for o in order:      # partitions appear in runs: never back to an earlier one
        assert o == sorted(o)


def test_batch_kernel_launch_is_chunked_below_the_thread_limit():
    from dciknn_cuda_amd import _capi
    lib = _capi.lib()
    per = ctypes.c_int()
    # 10000 queries x 4000 partitions would be 40 M workgroups of 256 threads: over 2^32 threads
    items = lib.dcih_debug_launch_map(8, 4000, 10000, -1, None, None, ctypes.byref(per))
    assert 0 < per.value < 10000
    assert items * 256 < 2 ** 32
    assert lib.dcih_debug_launch_map(8, 2 ** 30, 10, -1, None, None, ctypes.byref(per)) == -1


def test_extension_module_exports_the_reference_names():
    """The seven functions dciknn_cuda/core.py:19 imports, plus the handle accessor."""
    from dciknn_cuda_amd import _dci_cuda
    for name in ("_dci_new", "_dci_add", "_dci_query", "_dci_clear", "_dci_reset", "_dci_free",
                 "_dci_multi_query", "_dci_handle"):
        assert callable(getattr(_dci_cuda, name))


def test_constructor_needs_a_gpu():
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from dciknn_cuda_amd import DCI
    with pytest.raises(RuntimeError):
        DCI(8)


def _bare(dim=4):
    """A DCI object without a device handle, for the pure-Python validation."""
    from dciknn_cuda_amd import DCI
    d = DCI.__new__(DCI)
    d._dim, d._num_comp_indices, d._num_simp_indices = dim, 2, 3
    d._dci_inst, d._capsule, d._array, d.num_points = None, None, None, 0
    return d


def test_check_data_exception_types():
    d = _bare(4)

    class FakeCuda(torch.Tensor):
        @property
        def is_cuda(self):
            return True

    ok = torch.zeros(3, 4).as_subclass(FakeCuda)
    d._check_data(ok)
    with pytest.raises(ValueError):
        d._check_data(torch.zeros(3, 5).as_subclass(FakeCuda))            # wrong dim
    with pytest.raises(TypeError):
        d._check_data(torch.zeros(3, 4, dtype=torch.float64).as_subclass(FakeCuda))
    with pytest.raises(ValueError):
        d._check_data(torch.zeros(4, 3).t().as_subclass(FakeCuda))         # not C-contiguous
    with pytest.raises(TypeError):
        d._check_data(torch.zeros(3, 4))                                   # not on the GPU


def test_positive_integer_rule():
    d = _bare()
    d._ensure_positive_integer(3)
    with pytest.raises(TypeError):
        d._ensure_positive_integer(3.0)
    with pytest.raises(ValueError):
        d._ensure_positive_integer(0)


def test_freed_instance_raises():
    d = _bare()
    with pytest.raises(RuntimeError):
        d.add(torch.zeros(2, 4))
    with pytest.raises(RuntimeError):
        d.query(torch.zeros(2, 4), 1)


def test_float_ids_are_refused_where_they_would_be_rounded():
    """float32 cannot hold ids above 2**24: the default (float) result is refused there,
    before any device work, and return_int=True is the way through."""
    from dciknn_cuda_amd import core

    class FakeCuda(torch.Tensor):
        @property
        def is_cuda(self):
            return True

    d = _bare(4)
    d._dci_inst = object()
    q = torch.zeros(2, 4).as_subclass(FakeCuda)
    d.num_points = (1 << 24) + 2
    with pytest.raises(ValueError, match="return_int=True"):
        d.query(q, 3)
    core._refuse_rounded_ids((1 << 24) + 1)      # ids 0 .. 2**24 are all exact
    with pytest.raises(ValueError):
        core._refuse_rounded_ids(20_000_000)


def test_mdci_accepts_one_device_only():
    from dciknn_cuda_amd import MDCI
    with pytest.raises(NotImplementedError):
        MDCI(8, devices=[0, 1])
    with pytest.raises(NotImplementedError):
        MDCI(8, devices=[])


def test_import_name_of_the_reference_package():
    import dciknn_cuda
    import dciknn_cuda_amd
    assert dciknn_cuda.DCI is dciknn_cuda_amd.DCI and dciknn_cuda.MDCI is dciknn_cuda_amd.MDCI


def test_workload_generators_are_seeded():
    from dciknn_cuda_amd import workloads
    a, qa = workloads.c2(n=2000, nq=10)
    b, qb = workloads.c2(n=2000, nq=10)
    assert torch.equal(a, b) and torch.equal(qa, qb)
    assert a.shape == (2000, 128) and a.min() >= 0 and torch.equal(a, a.round())
    x, q = workloads.c1(n=300, nq=20)
    assert x.shape == (300, 100) and q.shape == (20, 100)
    x3, _ = workloads.c3(n=1000, nq=10)
    assert torch.allclose(x3.norm(dim=1), torch.ones(1000), atol=1e-5)
    x4, _ = workloads.c4(n=500, nq=5)
    assert x4.shape == (500, 960)
    assert workloads.c5_batch(0, n=100).shape == (100, 64)


def test_bench_refuses_more_than_one_gpu():
    """bench.py is a one-GPU benchmark: --gpus N > 1 exits with a message, before any GPU work."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr and r.stdout.strip() == ""


def test_traffic_table_names_commits_of_this_history():
    """Every row of profiles/hbm_traffic.json (the counter runs bench.py's `traffic` comes from) names
    the setting it was taken at and a commit that exists in this repository's history."""
    import json
    import subprocess
    runs = json.load(open(os.path.join(ROOT, "profiles", "hbm_traffic.json")))["runs"]
    assert runs
    have_git = os.path.isdir(os.path.join(ROOT, ".git"))
    for r in runs:
        assert {"config", "bs", "ts", "outer", "queries", "kernel", "commit"} <= set(r), r
        assert re.fullmatch(r"[0-9a-f]{7,40}", r["commit"]), r["commit"]
        if have_git:
            kind = subprocess.run(["git", "-C", ROOT, "cat-file", "-t", r["commit"]], capture_output=True, text=True)
            assert kind.stdout.strip() == "commit", r["commit"]
