"""Python interface of the MI355X Prioritized DCI engine.

`DCI` and `MDCI` keep the public behaviour of the reference's
dciknn_cuda/core.py:25-169 (argument names, defaults, exception types, return
shapes and dtypes).  Like there, the seven `_dci_*` functions come from the
compiled torch extension `_dci_cuda` (csrc/_dci_cuda.cpp), which calls the
C-ABI of libdci_hip.so; what the reference has no function for (directions,
counters, kernel choice) goes to the C-ABI directly.  Additions, all keyword-only and
optional: `seed` / `directions` at construction and the `directions` property
(the reference can neither seed, inject nor read its directions), and
`return_int` / `return_counters` on `query`, and `traversal` / `set_traversal`
to pick the query kernel.  One deliberate difference: an index of more than
2**24 + 1 points refuses to return ids as float32 (they would be rounded) and
asks for `return_int=True`.
"""
import torch

from . import _capi
from . import _dci_cuda as _ext   # built by `python -m dciknn_cuda_amd.build`; no fallback


def _stream_ptr(device):
    return torch.cuda.current_stream(device).cuda_stream


# float32 holds every integer up to 2**24 exactly and none of the odd ones above
_MAX_FLOAT_ID = 1 << 24


def _refuse_rounded_ids(num_points):
    """The reference returns ids as float32 (src/dci_cuda.cpp:111), which rounds ids
    above 2**24 to a neighbouring point's.  An index that large answers only with
    integer ids."""
    if num_points > _MAX_FLOAT_ID + 1:
        raise ValueError(
            "this index holds %d points and float32 ids are exact only up to %d: "
            "pass return_int=True to query() to get int32 ids" % (num_points, _MAX_FLOAT_ID))


class DCI(object):

    def __init__(self, dim, num_comp_indices=2, num_simp_indices=7, bs=100, ts=10, device=0,
                 *, seed=0, directions=None, traversal="auto"):
        if not torch.cuda.is_available():
            raise RuntimeError("DCI requires GPU access, please check the ROCm driver.")
        self._dim = dim
        self._num_comp_indices = num_comp_indices
        self._num_simp_indices = num_simp_indices
        self._device = torch.device("cuda", device if isinstance(device, int) else
                                    torch.device(device).index or 0)
        self._lib = _capi.lib()
        self._capsule = _ext._dci_new(dim, num_comp_indices, num_simp_indices,
                                      self._device.index, seed)
        # the same handle as a plain pointer, for direct C-ABI calls
        self._dci_inst = _capi.ctypes.c_void_p(_ext._dci_handle(self._capsule))
        self._array = None
        self._block_size = bs
        self._thread_size = ts
        self.num_points = 0
        if directions is not None:
            self.directions = directions
        if traversal != "auto":
            self.set_traversal(traversal)

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass

    @property
    def dim(self):
        return self._dim

    @property
    def num_comp_indices(self):
        return self._num_comp_indices

    @property
    def num_simp_indices(self):
        return self._num_simp_indices

    @property
    def directions(self):
        """The unit projection directions, a CPU float32 tensor [m*L, dim]."""
        self._require_handle()
        out = torch.empty(self._num_comp_indices * self._num_simp_indices, self._dim,
                          dtype=torch.float32)
        _capi.check(self._lib.dcih_get_directions(self._dci_inst, out.data_ptr()))
        return out

    @directions.setter
    def directions(self, value):
        self._require_handle()
        value = torch.as_tensor(value, dtype=torch.float32).cpu().contiguous()
        want = (self._num_comp_indices * self._num_simp_indices, self._dim)
        if tuple(value.shape) != want:
            raise ValueError("directions must have shape %s" % (want,))
        _capi.check(self._lib.dcih_set_directions(self._dci_inst, value.data_ptr()))

    def set_traversal(self, mode):
        """Pick the query kernel: "auto", "step" (one wavefront per partition,
        one window per step), "batch" (one workgroup per partition, whole index
        ranges per epoch) or "dense" (one workgroup per partition, the promoting
        step of every point at once).  All return the same neighbours."""
        self._require_handle()
        value = {"auto": _capi.TRAVERSAL_AUTO, "step": _capi.TRAVERSAL_STEP,
                 "batch": _capi.TRAVERSAL_BATCH, "dense": _capi.TRAVERSAL_DENSE}[mode]
        _capi.check(self._lib.dcih_set_option(self._dci_inst, _capi.OPT_TRAVERSAL, value))

    def _require_handle(self):
        if self._dci_inst is None:
            raise RuntimeError("this DCI instance has been freed")

    def _ensure_positive_integer(self, x):
        if not isinstance(x, int):
            raise TypeError("number must be an integer")
        elif x <= 0:
            raise ValueError("number must be positive")

    def _check_data(self, arr):
        if arr.shape[1] != self.dim:
            raise ValueError("mismatch between tensor dimension (%d) and the declared dimension of this DCI instance (%d)" % (arr.shape[1], self.dim))
        if arr.dtype != torch.float:
            raise TypeError("tensor must consist of single-precision floats")
        if not arr.is_contiguous():
            raise ValueError("the memory layout of tensor must be in row-major (C-order)")
        if not arr.is_cuda:
            raise TypeError("tensor must be a cuda tensor")

    def add(self, data):
        self._require_handle()
        if self.num_points > 0:
            raise RuntimeError("DCI class does not support insertion of more than one tensor. Must combine all tensors into one tensor before inserting")
        self._check_data(data)
        if data.device != self._device:
            raise ValueError("tensor is on %s but this DCI instance lives on %s" % (data.device, self._device))
        _ext._dci_add(self._capsule, self._dim, data.shape[0], data.flatten(),
                      self._block_size, self._thread_size)
        self.num_points = data.shape[0]
        self._array = data   # the index borrows this memory

    def append(self, data):
        """Insert more rows (not in the reference, whose `add` works once): the
        index becomes what `add` would build over all rows given so far; ids
        continue after the existing ones.  The rows are copied."""
        self._require_handle()
        self._check_data(data)
        if data.device != self._device:
            raise ValueError("tensor is on %s but this DCI instance lives on %s" % (data.device, self._device))
        _capi.check(self._lib.dcih_append(self._dci_inst, self._dim, data.shape[0], data.data_ptr(),
                                          self._block_size, self._thread_size,
                                          _stream_ptr(self._device)))
        self.num_points += data.shape[0]
        self._array = None    # the index owns its rows now

    # query is num_queries x dim, returns num_queries x num_neighbours
    def query(self, query, num_neighbours=-1, num_outer_iterations=5000, blind=False,
              *, return_int=False, return_counters=False):
        self._require_handle()
        if len(query.shape) < 2:
            _query = query.unsqueeze(0)
        else:
            _query = query
        self._check_data(_query)
        if num_neighbours < 0:
            num_neighbours = self.num_points
        self._ensure_positive_integer(num_neighbours)
        if self.num_points == 0:
            raise RuntimeError("query on an empty DCI instance; call add() first")
        if num_neighbours > self.num_points:
            raise ValueError("num_neighbours exceeds the number of indexed points")
        max_num_candidates = 10 * num_neighbours
        nq = _query.shape[0]
        if not return_int:
            _refuse_rounded_ids(self.num_points)
        if not return_int and not return_counters:
            # the reference's own route: one flat float tensor, ids first (core.py:90-92)
            _query_result = _ext._dci_query(self._capsule, self._dim, nq, _query.flatten(),
                                            num_neighbours, blind, num_outer_iterations,
                                            max_num_candidates, self._block_size, self._thread_size)
            half = _query_result.shape[0] // 2
            return _query_result[:half].reshape(nq, -1), _query_result[half:].reshape(nq, -1)
        # blind: candidate ids in the order they were promoted and the steps that promoted
        # them, as many as the reference's result buffer holds (src/dci_cuda_kernel.cu:782-783)
        width = min(max_num_candidates, num_outer_iterations) if blind else num_neighbours
        ids = torch.empty((nq, width), dtype=torch.int32, device=self._device)
        dists = torch.empty((nq, width), dtype=torch.float32, device=self._device)
        counters = None
        if return_counters:
            counters = torch.empty((nq, _capi.NUM_COUNTERS), dtype=torch.int64, device=self._device)
        _capi.check(self._lib.dcih_query(
            self._dci_inst, self._dim, nq, _query.data_ptr(), num_neighbours, 1 if blind else 0,
            num_outer_iterations, max_num_candidates, self._block_size, self._thread_size,
            ids.data_ptr(), dists.data_ptr(),
            counters.data_ptr() if counters is not None else None,
            _stream_ptr(self._device)))
        if not return_int:
            ids = ids.to(torch.float32)   # the reference returns ids as floats
        if return_counters:
            return ids, dists, counters
        return ids, dists

    def clear(self):
        self._require_handle()
        _ext._dci_clear(self._capsule)
        self.num_points = 0
        self._array = None

    def reset(self):
        self._require_handle()
        _ext._dci_reset(self._capsule)
        self.num_points = 0
        self._array = None

    def free(self):
        if getattr(self, "_dci_inst", None) is not None:
            _ext._dci_free(self._capsule)
            self._dci_inst = None
        self.num_points = 0
        self._array = None


class MDCI(object):
    """Multi-device front end of the reference, accepted with one device only."""

    def __init__(self, dim, num_comp_indices=2, num_simp_indices=7, bs=100, ts=10, devices=[0],
                 **kwargs):
        devices = list(devices)
        if len(devices) != 1:
            raise NotImplementedError(
                "this build runs on one GPU: pass devices=[<one device id>]")
        self.devices = devices
        self.num_devices = 1
        self.dcis = [DCI(dim, num_comp_indices, num_simp_indices, bs, ts, dev, **kwargs)
                     for dev in devices]
        self.data_per_device = 0

    def add(self, data):
        self.data_per_device = data.shape[0] // self.num_devices + 1
        cur_data = data[0:self.data_per_device].to(self.dcis[0]._device)
        self.dcis[0].add(cur_data)

    def query(self, query, num_neighbours=-1, num_outer_iterations=5000, blind=False):
        if num_neighbours <= 0:
            raise RuntimeError('num_neighbours must be positive')
        if len(query.shape) < 2:
            _query = query.unsqueeze(0)
        else:
            _query = query
        _query = _query.detach().clone().to(self.dcis[0]._device)
        d0 = self.dcis[0]
        d0._check_data(_query)
        _refuse_rounded_ids(d0.num_points)
        max_num_candidates = 10 * num_neighbours
        res = _ext._dci_multi_query([dc._capsule for dc in self.dcis], d0._dim, _query.shape[0],
                                    [_query.flatten()], num_neighbours, blind, num_outer_iterations,
                                    max_num_candidates, d0._block_size, d0._thread_size)
        half = res[0].shape[0] // 2
        nns = res[0][:half].reshape(_query.shape[0], -1)
        dists = res[0][half:].reshape(_query.shape[0], -1)
        if blind:     # already ordered by promoting step; nothing to merge with one device
            return nns, dists
        _, sort_indices = torch.sort(dists, dim=1, stable=True)
        sort_indices = sort_indices[:, :num_neighbours]
        return torch.gather(nns, 1, sort_indices), torch.gather(dists, 1, sort_indices)

    def clear(self):
        for dci in self.dcis:
            dci.clear()

    def reset(self):
        for dci in self.dcis:
            dci.reset()

    def free(self):
        for dci in self.dcis:
            dci.free()
