"""Helpers shared by the parity tests."""
import numpy as np
import torch


def set_agreement(ids_a, ids_b):
    """Mean fraction of each row of ids_a found in the same row of ids_b."""
    ids_a, ids_b = np.asarray(ids_a), np.asarray(ids_b)
    hit = 0
    for a, b in zip(ids_a, ids_b):
        hit += len(set(a.tolist()) & set(b.tolist()))
    return hit / ids_a.size


def assert_ids_agree_up_to_rounding(ids, ref_ids, X, Q, rtol, tag=""):
    """Rows of ids and ref_ids hold the same points, except where the points that
    differ lie within rtol (relative) of one another: two candidates that close
    at the k-th place swap with the summation order of a float32 distance."""
    for q, (a, b) in enumerate(zip(np.asarray(ids), np.asarray(ref_ids))):
        sa, sb = set(a.tolist()), set(b.tolist())
        if sa == sb:
            continue
        assert len(sa) == len(sb) and -1 not in (sa ^ sb), "%s query %d: %s" % (tag, q, sorted(sa ^ sb))
        q64 = Q[q].astype(np.float64)
        d = {i: np.sqrt(((X[i].astype(np.float64) - q64) ** 2).sum()) for i in sa ^ sb}
        lo, hi = min(d.values()), max(d.values())
        assert hi - lo <= rtol * hi, "%s query %d: the rows differ in %s" % (tag, q, d)


def engine_index(dci):
    """(skeys, sids) of a built DCI instance as numpy arrays [I][N]."""
    from dciknn_cuda_amd import _capi
    I = dci.num_comp_indices * dci.num_simp_indices
    keys = np.empty((I, dci.num_points), np.float32)
    ids = np.empty((I, dci.num_points), np.int32)
    _capi.check(dci._lib.dcih_get_index(dci._dci_inst, keys.ctypes.data, ids.ctypes.data))
    return keys, ids


def engine_project(dirs, rows):
    """dcih_project on cuda:0: numpy [I][dim], [n][dim] -> numpy [I][n]."""
    from dciknn_cuda_amd import _capi
    d = torch.as_tensor(dirs, dtype=torch.float32).cuda().contiguous()
    r = torch.as_tensor(rows, dtype=torch.float32).cuda().contiguous()
    out = torch.empty((d.shape[0], r.shape[0]), dtype=torch.float32, device="cuda")
    _capi.check(_capi.lib().dcih_project(d.data_ptr(), d.shape[0], r.data_ptr(), r.shape[0],
                                         d.shape[1], out.data_ptr(),
                                         torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return out.cpu().numpy()


def engine_segsort(keys, block_size):
    """dcih_segsort on cuda:0: numpy [I][n] -> (skeys, sids) numpy."""
    from dciknn_cuda_amd import _capi
    k = torch.as_tensor(keys, dtype=torch.float32).cuda().contiguous()
    sk = torch.empty_like(k)
    si = torch.empty(k.shape, dtype=torch.int32, device="cuda")
    _capi.check(_capi.lib().dcih_segsort(k.data_ptr(), k.shape[0], k.shape[1], block_size,
                                         sk.data_ptr(), si.data_ptr(),
                                         torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return sk.cpu().numpy(), si.cpu().numpy()


def dense_fits(n, M, L, B, T, k):
    """Shapes the dense traversal kernel's tables take (it refuses the others)."""
    ppb = -(-n // B)
    return (M <= 64 and L <= 64 and ppb <= 32766 and min(k, ppb) <= 512 and
            L * (ppb // T + 3) <= 41 * 256)


def batch_fits(n, M, L, B, k):
    """Shapes the batch traversal kernel's tables take (it refuses the others)."""
    return 2 * M * L <= 256 and M <= 64 and min(k, -(-n // B)) <= 512 and -(-n // B) <= 65536
