"""Benchmark of the Prioritized DCI hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2]
                    [--bs B --ts T --outer O] [--nq NQ] [--no-cpu] [--no-extras]

A step is one pass of the query path (query projection, traversal, exact
distances, top-k) over the whole seeded query batch of the workload, with the
index built and all inputs resident in HBM.  The build (projection + segmented
sort) is timed separately and reported as build_points_per_s; for the
incremental workload (c5) the index is grown by appends, each timed, and the
steps run on the final index.  Prints ONE JSON line:

  value          queries/s over the timed steps
  recall_at_k    against exact k-NN, recall_ok = the workload's target is met
  per_query      exact traversal counters of the reference algorithm (step-by-step
                 kernel = oracle counts) on a query sample, and what the timed
                 kernels themselves streamed
  kernel_ms      HIP-event times of the query kernels inside the library
  build          HIP-event times of projection and sort, their HBM fractions
  roofline       the kernel that took most of the step, against the limit that binds
                 it: `frac` is always achieved / peak of that limit (<= 1).  For the
                 batch traversal kernel the limit is vector-ALU issue (lane
                 instructions; its L2-side figure is given beside it), for the dense
                 traversal kernel HBM bytes (candidate rows + index slices); the figure by the reference's 8-byte index
                 entries is kept as contract_bytes_* and is not a bound.  `traffic`
                 = HBM bytes per launch from profiles/hbm_traffic.json (rocprofv3
                 counter runs of this file), null when that file has no entry for
                 the configuration and setting being run
  cpu_baseline   the CPU restatement of the reference algorithm on this box's host
                 cores on a bounded sample of the same workload
  first_call, outer_sweep, blind   extra measurements outside the timed steps
  other_configs  (default run only) compact legs of the other workloads and of this one at
                 the reference's constructor defaults, each from a run of this file in a
                 process of its own: value, recall, setting, kernel times, roofline fraction
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0   # MI355X HBM3E
# vector-ALU issue peak: 256 CUs x 4 SIMDs x 16 lanes x 2.4 GHz lane instructions per second
VALU_PEAK_GOPS = 256 * 4 * 16 * 2.4
# lane instructions the batch kernel cannot do without per index entry it scans: three packed
# 16-bit instructions per PAIR of entries (position - run start, minus run length with
# saturation, running maximum)
MIN_INSTR_PER_ENTRY = 1.5
# L2 -> CU read peak: 8 XCDs x 16 channels x 128 B per clock x 2.4 GHz
L2_PEAK_GBS = 8 * 16 * 128 * 2.4
# compact legs of the other workloads (and of this one at the reference's own defaults) that the
# default run adds to its line: (name, extra arguments)
OTHER_LEGS = [
    ("c1", ["--config", "c1"]),
    ("c2_reference_defaults_outer500", ["--config", "c2", "--bs", "100", "--ts", "10", "--outer", "500"]),
    ("c2_reference_defaults_outer5000", ["--config", "c2", "--bs", "100", "--ts", "10", "--outer", "5000"]),
    ("c4", ["--config", "c4"]),
    ("c3", ["--config", "c3"]),
    ("c5", ["--config", "c5"]),
]

# (block_size, thread_size, num_outer_iterations) used when none are given: the fastest
# setting found that meets the workload's recall target (RECALL_TARGET; c5 has none and runs
# at the fastest setting found with recall@50 above 0.9 at 20M points: wide windows, stop as
# soon as 50 windows' first points are promoted).
TUNED = {
    "c1": dict(bs=100, ts=10, outer=5000),
    "c2": dict(bs=58, ts=2, outer=500),
    "c3": dict(bs=400, ts=128, outer=100),
    "c4": dict(bs=100, ts=64, outer=126),
    "c5": dict(bs=900, ts=128, outer=10),
}
RECALL_TARGET = {"c1": 0.95, "c2": 0.95, "c3": 0.9, "c4": 0.95, "c5": None}
# queries per leg that would otherwise take minutes on the large workloads
LEG_QUERIES = {
    "c1": dict(recall=500, counters=500, cpu=500, blind=500),
    "c2": dict(recall=10_000, counters=512, cpu=2048, blind=10_000),
    "c3": dict(recall=1024, counters=32, cpu=768, blind=64),
    "c4": dict(recall=5000, counters=256, cpu=512, blind=1000),
    "c5": dict(recall=1024, counters=32, cpu=512, blind=256, growth=1024),
}
# the CPU baseline of the two 10M+ workloads runs on the first CPU_SAMPLE_POINTS points
# with block_size scaled to keep the points per partition; its rate is scaled to full size
CPU_SAMPLE_POINTS = 1_000_000


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=3)
    p.add_argument("--warmup", type=int, default=1)
    p.add_argument("--config", default="c2", choices=sorted(TUNED))
    p.add_argument("--bs", type=int)
    p.add_argument("--ts", type=int)
    p.add_argument("--outer", type=int)
    p.add_argument("--nq", type=int, help="use only the first NQ queries")
    p.add_argument("--n", type=int, help="override the number of data points (c5: per batch)")
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    p.add_argument("--no-extras", action="store_true",
                   help="skip first_call, outer_sweep and blind (profiling runs)")
    p.add_argument("--no-others", action="store_true",
                   help="skip the compact legs of the other workloads that the default run (c2 at its "
                        "tuned setting, extras on) appends as other_configs")
    p.add_argument("--build-reps", type=int, default=3)
    p.add_argument("--traversal", default="auto", choices=["auto", "step", "batch", "dense"])
    p.add_argument("--c5-batches", type=int, default=20, help="batches of the incremental workload")
    p.add_argument("--append", default="auto", choices=["auto", "sort", "merge"],
                   help="c5: how an append forms the new index (merge old slices with the sorted new "
                        "points, or sort everything again)")
    p.add_argument("--copy-calibration", action="store_true",
                   help="also run a plain 1 GiB device copy (known HBM traffic) so that "
                        "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings can be scaled")
    return p.parse_args()


def load_traffic(config, cfg, traversal, n, nq):
    """HBM bytes per launch of the dominant kernel from the committed counter summary."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    try:
        with open(path) as f:
            table = json.load(f)
    except (OSError, ValueError):
        return None
    for row in table.get("runs", []):
        if (row.get("config") == config and row.get("bs") == cfg["bs"] and row.get("ts") == cfg["ts"]
                and row.get("outer") == cfg["outer"] and row.get("traversal", "auto") == traversal
                and row.get("points") == n and row.get("queries") == nq):
            return row
    return None


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported "
              "(every box in this pipeline has one GPU)" % a.gpus, file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    from dciknn_cuda_amd import build as engine_build
    engine_build.ensure_built()      # loads what is built; compiles only in a tree without libraries
    import dciknn_cuda_amd as D
    from dciknn_cuda_amd import _capi, workloads

    def say(*msg):
        print("[bench]", *msg, file=sys.stderr, flush=True)

    config = a.config
    cfg = dict(TUNED[config])
    for key in ("bs", "ts", "outer"):
        if getattr(a, key) is not None:
            cfg[key] = getattr(a, key)
    shape = dict(workloads.SHAPES[int(config[1])])
    legs = LEG_QUERIES[config]
    M, L, k, dim = shape["m"], shape["l"], shape["k"], shape["dim"]
    I = M * L
    outer = cfg["outer"]

    dci = D.DCI(dim, M, L, cfg["bs"], cfg["ts"], seed=4, traversal=a.traversal)
    lib = dci._lib
    _capi.check(lib.dcih_profile(dci._dci_inst, 1))
    tms = (_capi.ctypes.c_float * _capi.NUM_TIMERS)()

    def timers():
        _capi.check(lib.dcih_last_timings(dci._dci_inst, tms))   # waits for the call's events
        return [float(v) for v in tms]

    if a.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)      # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    # ---- data and build ---------------------------------------------------------
    per_size = None
    if config == "c5":
        _capi.check(lib.dcih_set_option(dci._dci_inst, _capi.OPT_APPEND,
                                        {"auto": _capi.APPEND_AUTO, "sort": _capi.APPEND_SORT,
                                         "merge": _capi.APPEND_MERGE}[a.append]))
        n_batch = a.n or shape["n"]
        Q = workloads.c5_queries(shape["nq"])
        if a.nq:
            Q = Q[:a.nq].contiguous()
        Qd = Q.cuda()
        nq = Q.shape[0]
        Xd = torch.empty((a.c5_batches * n_batch, dim), dtype=torch.float32, device="cuda")
        X_cpu_sample = None
        per_size = []
        Qg = Qd[:min(nq, legs["growth"])].contiguous()     # the queries run after every append
        for b in range(a.c5_batches):
            xb_host = workloads.c5_batch(b, n=n_batch)
            if b == 0:
                X_cpu_sample = xb_host
            xb = xb_host.cuda()
            Xd[b * n_batch:(b + 1) * n_batch] = xb
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            dci.append(xb)
            torch.cuda.synchronize()
            t_add = time.perf_counter() - t0
            tt = timers()
            dci.query(Qg, k, outer, return_int=True)          # warm-up (hints, workspace)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            ids, _ = dci.query(Qg, k, outer, return_int=True)
            torch.cuda.synchronize()
            t_q = time.perf_counter() - t0
            nrec = min(Qg.shape[0], 256)
            truth = workloads.exact_knn(Xd[:(b + 1) * n_batch], Qg[:nrec], k)
            per_size.append(dict(points=dci.num_points, append_ms=t_add * 1e3,
                                 project_ms=tt[_capi.T_PROJECT], segsort_ms=tt[_capi.T_SEGSORT],
                                 new_points_per_s=n_batch / t_add,
                                 total_points_per_s=dci.num_points / t_add,
                                 queries_per_s=Qg.shape[0] / t_q, queries=Qg.shape[0],
                                 recall_at_k=workloads.recall_at_k(ids[:nrec], truth)))
            say("c5 batch", b, "append %.2f ms, %.0f queries/s" % (t_add * 1e3, Qg.shape[0] / t_q))
        N = dci.num_points
        Xd = Xd[:N]
        appends = [r["append_ms"] for r in per_size]
        build_wall = appends[-1] * 1e-3
        build_cold = appends[0] * 1e-3
        proj_t, sort_t = per_size[-1]["project_ms"], per_size[-1]["segsort_ms"]
        new_rows = n_batch
        workload_text = "C5: %d appends of %d x %d fp32 N(0,1), %d queries, m=%d L=%d k=%d" % (
            a.c5_batches, n_batch, dim, nq, M, L, k)
    else:
        if a.n:
            shape["n"] = a.n
        X, Q = getattr(workloads, config)(n=shape["n"], nq=shape["nq"])
        if a.nq:
            Q = Q[:a.nq].contiguous()
        N, nq = X.shape[0], Q.shape[0]
        Xd, Qd = X.cuda(), Q.cuda()
        X_cpu_sample = X[:CPU_SAMPLE_POINTS] if N > 2 * CPU_SAMPLE_POINTS else X
        del X
        torch.cuda.synchronize()
        build_s, proj_ms, sort_ms = [], [], []
        for rep in range(a.build_reps + 1):
            dci.clear() if dci.num_points else None
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            dci.add(Xd)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            tt = timers()
            if rep == 0:   # first add of the handle: allocates its arrays, loads code objects
                build_cold = t1 - t0
            else:          # clear + add on the same handle: steady-state rebuild
                build_s.append(t1 - t0)
                proj_ms.append(tt[_capi.T_PROJECT])
                sort_ms.append(tt[_capi.T_SEGSORT])
        build_wall = float(np.median(build_s))
        proj_t, sort_t = float(np.median(proj_ms)), float(np.median(sort_ms))
        new_rows = N
        workload_text = "%s: %d pts x %d fp32, %d queries, m=%d L=%d k=%d" % (
            config.upper(), N, dim, nq, M, L, k)
    say("built", N, "points; build %.3f ms" % (build_wall * 1e3))

    # ---- first call of this query shape: nothing learnt about where traversals stop ----
    first_call = None
    if not a.no_extras:
        say("first call of the query shape")
        dci.query(Qd, k, outer, return_int=True)                  # workspace and kernel attributes in place
        _capi.check(lib.dcih_set_option(dci._dci_inst, _capi.OPT_FORGET_HINTS, 0))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        dci.query(Qd, k, outer, return_int=True)
        torch.cuda.synchronize()
        t_first = time.perf_counter() - t0
        first_call = dict(queries_per_s=nq / t_first, ms=t_first * 1e3,
                          note="same batch with the stop-step hints forgotten (they size the batch "
                               "kernel's epochs and are learnt from earlier queries; results do not depend on them)")
        _capi.check(lib.dcih_set_option(dci._dci_inst, _capi.OPT_FORGET_HINTS, 0))

    # ---- query: warmup, then K timed steps ----------------------------------------
    say("warm-up and timed steps")
    for _ in range(a.warmup):
        dci.query(Qd, k, outer, return_int=True)
    tsum = np.zeros(_capi.NUM_TIMERS)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        ids, dists = dci.query(Qd, k, outer, return_int=True)
        tsum += np.maximum(np.array(timers()), 0.0)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / a.steps
    qps = nq / (ms_per_step * 1e-3)
    tavg = tsum / a.steps
    trav_ms, batch_ms, dense_ms = tavg[_capi.T_TRAVERSE], tavg[_capi.T_BATCH], tavg[_capi.T_DENSE]
    say("%.0f queries/s, traverse %.2f ms (batch %.2f, dense %.2f)" % (qps, trav_ms, batch_ms, dense_ms))

    # ---- outside the timed region: recall and traversal counters ---------------------
    nrec = min(nq, legs["recall"])
    truth = workloads.exact_knn(Xd, Qd[:nrec].contiguous(), k)
    recall = workloads.recall_at_k(ids[:nrec], truth)
    target = RECALL_TARGET[config]
    say("recall@%d %.4f on %d queries" % (k, recall, nrec))
    # what the kernels that were timed streamed / probed themselves
    say("counters of the timed kernels")
    _, _, ctr = dci.query(Qd, k, outer, return_int=True, return_counters=True)
    torch.cuda.synchronize()
    own = ctr.double().mean(0).cpu().numpy()
    # exact counters of the reference algorithm (identical to the oracle's: the parity
    # tests check that) from the step-by-step kernel on a sample of the queries
    nqc = min(nq, legs["counters"])
    say("exact counters from the step-by-step kernel on", nqc, "queries")
    dci.set_traversal("step")
    _, _, ctr = dci.query(Qd[:nqc].contiguous(), k, outer, return_int=True, return_counters=True)
    torch.cuda.synchronize()
    dci.set_traversal(a.traversal)
    V, C, S, steps_q = (float(v) for v in ctr.double().mean(0).cpu().numpy())

    # ---- roofline of the kernel that took most of the step ----------------------------
    # By the reference's layout a query moves: its row, 8 bytes (key, id) per search probe and
    # per visited entry, one data row per promoted point, k results.  That figure is kept for
    # comparison only: this engine stores ids apart from keys, 2 bytes each, and an XCD works
    # on one partition at a time so most entries come from its L2.
    contract_bytes = 4 * dim + 8 * S + 8 * V + 4 * dim * C + 8 * k
    ppb = -(-N // cfg["bs"])
    if a.traversal == "step":
        kernel, launch_ms = "traverse_kernel", trav_ms
    elif dense_ms > batch_ms:
        kernel, launch_ms = "traverse_dense_kernel", dense_ms
    elif batch_ms > 0:
        kernel, launch_ms = "traverse_block_kernel", batch_ms
    else:   # neither traversal kernel ran: the traversal provably runs dry and the ranking is computed directly
        kernel, launch_ms = "exact_dists_kernel + segmented sort", trav_ms
    # bytes the launch has to bring from HBM in this layout: the index slices once (keys,
    # 16-bit ids, 16-bit inverse positions), per query its row, the rows of its candidates and
    # its per-partition result lists
    hbm_bytes = 8.0 * I * N + nq * (4.0 * dim + 4.0 * dim * C + 8.0 * min(k, ppb) * cfg["bs"])
    hbm_model = ("index slices once (8 B per entry) + per query its row, %.0f candidate rows of %d B and "
                 "its per-partition result lists" % (C, 4 * dim))
    if kernel.startswith("exact_dists"):
        # direct ranking: the rows once, per (query, point) a distance written, sorted and read back
        hbm_bytes = 4.0 * N * dim + nq * (4.0 * dim + 12.0 * N + 8.0 * k)
        hbm_model = "rows once + per (query, point) a 4-byte distance out and 8 bytes through the sort"
    hbm_gbs = hbm_bytes / (launch_ms * 1e-3) / 1e9
    valu_ops = MIN_INSTR_PER_ENTRY * float(own[0]) * nq
    valu_gops = valu_ops / (launch_ms * 1e-3) / 1e9
    if kernel == "traverse_block_kernel":
        roofline = dict(bound="valu", kernel=kernel, achieved=valu_gops, peak=VALU_PEAK_GOPS,
                        unit="G lane-instr/s", frac=valu_gops / VALU_PEAK_GOPS,
                        model="%.1f lane instructions per index entry scanned (3 packed 16-bit instructions per "
                              "pair) x %.4g entries per launch" % (MIN_INSTR_PER_ENTRY, float(own[0]) * nq))
        # memory side of the same kernel: what it reads through L2 in this layout -- 2 bytes per
        # entry scanned (16-bit position), 4 per key read, the candidates' rows
        l2_bytes = nq * (2.0 * float(own[0]) + 4.0 * float(own[2]) + 4.0 * dim * C)
        roofline.update(l2_model_bytes_per_launch=l2_bytes,
                        l2_model_gbs=l2_bytes / (launch_ms * 1e-3) / 1e9,
                        l2_frac=l2_bytes / (launch_ms * 1e-3) / 1e9 / L2_PEAK_GBS,
                        l2_model="2 B per index entry scanned + 4 B per key read + candidate rows, against "
                                 "%.0f GB/s (8 XCDs x 16 channels x 128 B/clk x 2.4 GHz)" % L2_PEAK_GBS)
    else:
        roofline = dict(bound="hbm", kernel=kernel, achieved=hbm_gbs, peak=HBM_PEAK_GBS,
                        unit="GB/s", frac=hbm_gbs / HBM_PEAK_GBS,
                        model=hbm_model)
    roofline.update(avg_launch_ms=launch_ms, hbm_bytes_per_launch=hbm_bytes, hbm_gbs=hbm_gbs,
                    hbm_frac=hbm_gbs / HBM_PEAK_GBS, valu_min_lane_instr_per_launch=valu_ops,
                    valu_frac=valu_gops / VALU_PEAK_GOPS,
                    contract_bytes_per_launch=contract_bytes * nq,
                    contract_bytes_gbs=contract_bytes * nq / (launch_ms * 1e-3) / 1e9,
                    contract_note="contract_bytes_* prices every visit at the reference's 8 bytes per "
                                  "(key, id) entry; it is not a bound for this layout and may exceed the HBM peak")
    prof = load_traffic(config, cfg, a.traversal, N, nq)
    roofline["traffic"] = prof["fetch_bytes"] + prof["write_bytes"] if prof else None
    if prof:
        roofline["traffic_source"] = {key: prof[key] for key in prof if key not in ("fetch_bytes", "write_bytes")}
        roofline["traffic_fetch_bytes"], roofline["traffic_write_bytes"] = prof["fetch_bytes"], prof["write_bytes"]
        if "valu_issue_frac" in prof:
            roofline["valu_issue_frac_profiled"] = prof["valu_issue_frac"]
        if "l2_read_bytes" in prof:     # TCP_TCC_READ_REQ_sum x 128 B in the counter run
            roofline["l2_read_bytes_profiled"] = prof["l2_read_bytes"]
            roofline["l2_frac_profiled"] = prof["l2_frac"]

    build_bytes_proj = 4.0 * new_rows * (dim + I)
    build_bytes_sort = 12.0 * N * I
    build = dict(points_per_s=new_rows / build_wall, wall_ms=build_wall * 1e3,
                 first_add_wall_ms=build_cold * 1e3,
                 project_ms=proj_t, segsort_ms=sort_t,
                 project_gbs=build_bytes_proj / (proj_t * 1e-3) / 1e9,
                 segsort_gbs=build_bytes_sort / (sort_t * 1e-3) / 1e9,
                 project_frac=build_bytes_proj / (proj_t * 1e-3) / 1e9 / HBM_PEAK_GBS,
                 segsort_frac=build_bytes_sort / (sort_t * 1e-3) / 1e9 / HBM_PEAK_GBS)
    if per_size is not None:
        build["note"] = ("last append (mode %s): %d new rows projected, the index over all %d rows formed; "
                         "points_per_s counts the new rows" % (a.append, new_rows, N))
        build["append_mode"] = a.append
        build["total_points_per_s"] = N / build_wall

    # ---- extras: sweep of num_outer_iterations, blind querying ------------------------
    outer_sweep = None
    blind = None
    if not a.no_extras:
        if config == "c2":
            outer_sweep = []
            say("sweep of num_outer_iterations")
            for o in (500, 1000, 2000, 5000, 10000, 20000):
                say("  num_outer_iterations", o)
                dci.query(Qd, k, o, return_int=True)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(2):
                    oi, _ = dci.query(Qd, k, o, return_int=True)
                torch.cuda.synchronize()
                dt = (time.perf_counter() - t0) / 2
                outer_sweep.append(dict(num_outer_iterations=o, queries_per_s=nq / dt,
                                        recall_at_k=workloads.recall_at_k(oi[:nrec], truth)))
            dci.query(Qd, k, outer, return_int=True)
        if min(10 * k, outer) <= 8192:
            # no distances: per query the first min(10k, outer) promoted candidates by promoting step
            nqb = min(nq, legs["blind"])
            say("blind querying of", nqb, "queries")
            Qb = Qd[:nqb].contiguous()
            bids, _ = dci.query(Qb, k, outer, blind=True, return_int=True)
            torch.cuda.synchronize()
            reps = min(a.steps, 3)
            t0 = time.perf_counter()
            for _ in range(reps):
                bids, _ = dci.query(Qb, k, outer, blind=True, return_int=True)
            torch.cuda.synchronize()
            blind_ms = (time.perf_counter() - t0) * 1e3 / reps
            nb = min(nqb, nrec)
            hit = (truth[:nb].unsqueeze(2) == bids[:nb].long().unsqueeze(1)).any(2).float().mean().item()
            blind = dict(queries_per_s=nqb / (blind_ms * 1e-3), ms_per_step=blind_ms, queries=nqb,
                         slots_per_query=int(bids.shape[1]), true_neighbours_among_slots=hit)

    # ---- CPU baseline: the oracle on this box's host cores, bounded sample ----------
    cpu = None
    if not a.no_cpu:
        from oracle import dci_oracle as O
        say("CPU baseline")
        P = dci.directions.numpy()
        Xn = X_cpu_sample.numpy()
        n_cpu = Xn.shape[0]
        scale = n_cpu / float(N)          # the sample keeps the points per partition
        bs_cpu = max(1, int(round(cfg["bs"] * scale)))
        nqb = min(nq, legs["cpu"])
        Qn = Q[:nqb].numpy()
        t0 = time.perf_counter()
        skeys, sids = O.build_index(P, Xn, bs_cpu)
        t_build = time.perf_counter() - t0
        qproj = O.project(Qn, P)
        say("CPU index built in %.1f s; querying" % t_build)
        t0 = time.perf_counter()
        ref = O.query(skeys, sids, Xn, Qn, qproj, M, L, bs_cpu, cfg["ts"], k, outer)
        t_query = time.perf_counter() - t0
        agree = None
        if n_cpu == N:
            agree = float(np.mean([len(set(x.tolist()) & set(y.tolist())) / k
                                   for x, y in zip(ids[:nqb].cpu().numpy(), ref["ids"])]))
        nex = min(nqb, 128)
        t0 = time.perf_counter()
        torch.cdist(torch.from_numpy(Qn[:nex]), torch.from_numpy(Xn)).topk(k, largest=False)
        t_exact = time.perf_counter() - t0
        if n_cpu == N:
            sample = ("oracle (CPU restatement of the reference algorithm) on the first %d queries of the "
                      "same workload, same (bs, ts, outer); build timed on all %d points" % (nqb, N))
        else:
            sample = ("oracle (CPU restatement of the reference algorithm) on the first %d points and %d "
                      "queries of the same workload with block_size %d (the same %d points per partition), "
                      "same (ts, outer); a query's work is proportional to the number of partitions, so "
                      "value = the measured %.1f queries/s x %d / %d" %
                      (n_cpu, nqb, bs_cpu, ppb, nqb / t_query, n_cpu, N))
        cpu = dict(value=nqb / t_query * scale, unit="queries/s", cores=O.max_threads(), kind="port",
                   sample=sample, measured_queries_per_s_on_sample=nqb / t_query,
                   sample_points=n_cpu, sample_queries=nqb, seconds=t_query + t_build,
                   build_points_per_s=n_cpu / t_build, set_agreement_with_gpu=agree,
                   exact_cdist_topk_queries_per_s=nex / t_exact * scale,
                   host_cpus=os.cpu_count(), torch_threads=torch.get_num_threads())

    # ---- the other workloads, compactly (default run only) -----------------------------
    others = None
    default_run = (config == "c2" and not a.no_extras and not a.no_others and a.traversal == "auto"
                   and all(getattr(a, key) is None for key in ("bs", "ts", "outer", "nq", "n")))
    if default_run:
        import subprocess
        dci.free()
        del Xd, Qd
        torch.cuda.empty_cache()
        others = {}
        for name, extra in OTHER_LEGS:
            say("other configuration:", name)
            t0 = time.perf_counter()
            try:
                r = subprocess.run([sys.executable, os.path.abspath(__file__), "--steps", "2", "--warmup", "1",
                                    "--no-cpu", "--no-extras", "--build-reps", "1"] + extra,
                                   capture_output=True, text=True, timeout=280)
                if r.returncode != 0 or not r.stdout.strip():
                    raise RuntimeError("exit code %d: %s" % (r.returncode, r.stderr.strip()[-300:]))
                line = json.loads(r.stdout.strip().splitlines()[-1])
                others[name] = dict(
                    value=line["value"], unit=line["unit"], workload=line["config"]["workload"],
                    block_size=line["config"]["block_size"], thread_size=line["config"]["thread_size"],
                    num_outer_iterations=line["config"]["num_outer_iterations"],
                    recall_at_k=line["recall_at_k"], recall_target=line["recall_target"],
                    ms_per_step=line["ms_per_step"], kernel_ms=line["kernel_ms"],
                    build_points_per_s=line["build_points_per_s"],
                    roofline={key: line["roofline"][key] for key in ("bound", "kernel", "frac", "achieved", "peak", "unit")},
                    seconds=time.perf_counter() - t0)
            except Exception as exc:       # a leg that fails or runs out of time is reported as such
                others[name] = dict(error="%s: %s" % (type(exc).__name__, str(exc)[:200]))

    out = {
        "metric": "queries/sec at recall@10>=0.95, 1Mx128 fp32 k=10; index build points/sec"
                  if config == "c2" else "queries/sec; index build points/sec",
        "value": qps, "unit": "queries/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": workload_text,
                   "block_size": cfg["bs"], "thread_size": cfg["ts"],
                   "num_outer_iterations": outer},
        "recall_at_k": recall, "recall_queries": nrec, "recall_target": target,
        "recall_ok": None if target is None else recall >= target,
        "build_points_per_s": new_rows / build_wall,
        "per_query": {"visited": V, "candidates": C, "probes": S, "outer_steps": steps_q,
                      "contract_bytes": contract_bytes, "counter_sample_queries": nqc,
                      "entries_streamed_by_timed_kernels": float(own[0]),
                      "key_reads_by_timed_kernels": float(own[2])},
        "kernel_ms": {"traverse": trav_ms, "batch_kernel": batch_ms, "dense_kernel": dense_ms,
                      "merge": tavg[_capi.T_MERGE], "query_project": tavg[_capi.T_QPROJECT]},
        "build": build,
        "first_call": first_call,
        "outer_sweep": outer_sweep,
        "blind": blind,
        "per_size": per_size,
        "other_configs": others,
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
