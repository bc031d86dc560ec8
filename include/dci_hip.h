/*
 * C-ABI of the MI355X (gfx950) Prioritized DCI engine: libdci_hip.so.
 *
 * Plain C types only: pointers, sizes, an opaque handle and a stream passed as
 * void* (a hipStream_t; NULL = the default stream).  Every entry point returns
 * 0 on success or a negative DCIH_E* code; dcih_last_error() then holds a
 * message for the calling thread.  Device pointers are marked d_, host
 * pointers h_.  Unless stated otherwise a call only enqueues work on `stream`;
 * outputs are valid once the stream has been synchronised.
 *
 * Each entry point names the interface of the CUDA reference
 * (niopeng/dciknn_cuda, paths relative to its root) that it stands in for.
 */
#ifndef DCI_HIP_H
#define DCI_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct dcih_index dcih_index;

enum {
    DCIH_OK = 0,
    DCIH_EINVAL = -1,      /* bad argument (the reference would assert) */
    DCIH_ESTATE = -2,      /* call not valid in this state, e.g. add() twice */
    DCIH_EHIP = -3,        /* a HIP runtime call failed */
    DCIH_EUNSUPPORTED = -4 /* valid in the reference, not built here yet */
};

/* Per-query traversal counters written by dcih_query when asked for. */
enum {
    DCIH_CTR_VISITED = 0,   /* in-range index entries visited (step-by-step kernel: the reference loop's
                               count exactly; the other kernels: the index entries they read)  */
    DCIH_CTR_CANDIDATES = 1,/* points promoted = exact distances computed */
    DCIH_CTR_PROBES = 2,    /* key reads made by the positioning search   */
    DCIH_CTR_STEPS = 3,     /* outer steps executed, summed over partitions */
    DCIH_NUM_COUNTERS = 4
};

/* Kernels timed by dcih_profile / dcih_last_timings. */
enum {
    DCIH_T_PROJECT = 0,   /* build: projection of the data            */
    DCIH_T_SEGSORT = 1,   /* build: segmented sort                    */
    DCIH_T_QPROJECT = 2,  /* query: projection of the queries         */
    DCIH_T_TRAVERSE = 3,  /* query: traversal + distances + top-k, all kernels of it */
    DCIH_T_MERGE = 4,     /* query: merge of the per-partition top-k  */
    DCIH_T_BATCH = 5,     /* query: the batch kernel's share of DCIH_T_TRAVERSE (all its launches) */
    DCIH_T_DENSE = 6,     /* query: the dense kernel's share of DCIH_T_TRAVERSE */
    DCIH_NUM_TIMERS = 7
};

/*
 * Options of dcih_set_option.  DCIH_OPT_TRAVERSAL picks the query kernel:
 * 0 = automatic (the batch kernel when the shape fits its tables, else the
 * step-by-step kernel; items whose traversal needs many promotions are finished
 * by the dense kernel), 1 = step-by-step kernel (one wavefront per partition,
 * one window per step), 2 = batch kernel (one workgroup per partition, whole
 * index ranges per epoch; errors out if the shape does not fit), 3 = dense kernel
 * (one workgroup per partition computes the promoting step of every point;
 * errors out if the shape does not fit).  All give the same neighbours; with the
 * batch and dense kernels DCIH_CTR_VISITED counts the entries they processed (a
 * superset of the reference's visits: the batch kernel overshoots the stop step
 * inside its last epoch, the dense kernel looks at every entry) and
 * DCIH_CTR_PROBES their own key reads.  DCIH_OPT_DENSE_MIN_PROMOTIONS: under
 * automatic choice, the number of promotions per (query, partition) from which
 * the dense kernel is used (default 160; 0 = never): a call whose stop rule needs
 * that many (num_neighbours * thread_size) goes there as a whole, and the batch
 * kernel hands over single items that reach twice that many.
 * DCIH_OPT_FORGET_HINTS (value ignored): drops what earlier queries taught the
 * handle about where traversals stop (used only to size the batch kernel's
 * epochs, never visible in results), so that the next call runs like a first one.
 * DCIH_OPT_APPEND: how dcih_append forms the new index: 0 = automatic (today: sorts,
 * the faster of the two wherever it was measured), 1 = sort all projections again
 * (only the new rows are projected), 2 = merge: the old slices are split into sorted
 * runs of the new ones, the new points sorted, the runs merged (error where the shape
 * does not allow it: partitions of more than 32256 points).  All give the same index.
 */
enum { DCIH_OPT_TRAVERSAL = 0, DCIH_OPT_DENSE_MIN_PROMOTIONS = 1, DCIH_OPT_FORGET_HINTS = 2, DCIH_OPT_APPEND = 3 };

/* Message for the last failing call on this thread ("" if none). */
const char* dcih_last_error(void);

/*
 * Library/ABI version, bumped on any change a caller built against an older header
 * could trip over.  2: dcih_last_timings writes DCIH_NUM_TIMERS = 7 values (5 in
 * version 1), DCIH_OPT_TRAVERSAL accepts 3, DCIH_OPT_APPEND and dcih_query_noalloc
 * exist, and the two inspection entry points moved to dci_hip_debug.h.
 */
int dcih_abi_version(void);

/*
 * Replaces dci_init (include/dci.h:61, src/dci_cuda_kernel.cu:93-110) and the
 * handle allocation in py_dci_new (src/dci_cuda.cpp:54-66).  Draws
 * num_comp_indices*num_simp_indices N(0,1) directions of length dim on the
 * HOST from `seed` (the reference draws them on device from an unseeded libc
 * rand(), src/util_kernel.cu:119-137) and scales each row to unit L2 norm the
 * way normalize_proj_vecs does (src/dci_cuda_kernel.cu:52-73).  Synchronous.
 */
int dcih_create(int dim, int num_comp_indices, int num_simp_indices, int device,
                uint64_t seed, dcih_index** out);

/*
 * No counterpart in the reference (its directions can be neither read nor
 * injected); needed so two implementations can be compared on identical
 * directions.  h_dirs is row-major [num_comp*num_simp][dim].  `set` stores the
 * values as given (no normalisation) and is only legal while the index is
 * empty.  Both synchronous.
 */
int dcih_get_directions(const dcih_index* h, float* h_dirs);
int dcih_set_directions(dcih_index* h, const float* h_dirs);

/*
 * Replaces dci_add (include/dci.h:68, src/dci_cuda_kernel.cu:149-187): projects
 * num_points rows of d_data (row-major [num_points][dim], fp32) on every
 * direction and sorts each (simple index, partition) slice, with
 * ceil(num_points/block_size) points per partition.  Like the reference the
 * index BORROWS d_data: it must stay valid and unchanged until dcih_clear /
 * dcih_reset / dcih_free.  A second add on a non-empty index returns
 * DCIH_ESTATE (the reference asserts, :157).  thread_size does not influence
 * the result of the build and is accepted for signature parity.
 */
int dcih_add(dcih_index* h, int dim, int64_t num_points, const float* d_data,
             int block_size, int thread_size, void* stream);

/*
 * Incremental insertion; no counterpart in the reference, which refuses a second
 * add (dciknn_cuda/core.py:70-71, src/dci_cuda_kernel.cu:157).  The result is
 * exactly the index dcih_add would build over all rows given so far, in the order
 * given (ids continue where the previous call stopped).  Unlike dcih_add the rows
 * are COPIED into a buffer the index owns, so d_data may be released after the
 * call; rows of an earlier dcih_add are copied as well.  The index also keeps the
 * unsorted projections of its rows, so only the new rows are projected; the
 * partition boundaries depend on the total, so every slice is formed again.  The
 * next index is built beside the current one (twice the index's memory while the
 * call runs): if the call fails, for lack of memory or otherwise, the index is
 * what it was before.  Synchronises the stream.
 */
int dcih_append(dcih_index* h, int dim, int64_t num_points, const float* d_data,
                int block_size, int thread_size, void* stream);

/*
 * Replaces dci_query (include/dci.h:71, src/dci_cuda_kernel.cu:777-875).
 * d_query is [num_queries][dim]; with blind == 0, for each query
 * d_nn / d_dists [num_queries][num_neighbours] receive the ids and Euclidean
 * distances of the num_neighbours best promoted candidates, ascending by
 * (distance, id); slots beyond the number of candidates get id -1 and +inf.
 * block_size must equal the value given to dcih_add (the partitioning is part
 * of the built index); thread_size is the window width.  d_counters is NULL or
 * [num_queries][DCIH_NUM_COUNTERS].
 *
 * num_neighbours may be as large as the number of indexed points (what
 * dciknn_cuda/core.py:84-85 passes when the caller gives none).  Up to 8192 the
 * traversal keeps its best candidates in on-chip tables.  Above 8192 and above the
 * points per partition, ceil(num_points / block_size), the stop rule (:598-607),
 * which counts promotions of one partition, can never fire: every point is
 * promoted, and the result, the num_neighbours closest of all points by (distance,
 * id), is computed directly (all distances, summed in index order like
 * compute_dist_device, :36-44; one sort per query; the counters from their closed
 * forms).  The same direct computation is used for any num_neighbours when the stop
 * rule provably cannot fire (a partition holds fewer points than max_num_candidates
 * and fewer windows per simple index than num_outer_iterations) and the kernel
 * choice is left automatic.  Above 8192 otherwise, the traversal records every candidate's distance
 * in a row of num_points cells per query and the rows are sorted; both paths work
 * through the queries in chunks and use up to 2 GB of workspace.
 *
 * blind != 0 (query_config.blind, :498-505, :754-773, :859-864): the same
 * traversal under the same stop rule, but no distance is computed.  d_nn is
 * [num_queries][R] with R = min(max_num_candidates, num_outer_iterations), the
 * size the reference asks of its caller (:775-776, :782-783), and receives the
 * ids of the first R promoted candidates of the query, ascending by (outer step
 * of its partition's traversal at which the point was promoted, id), then -1.
 * d_dists may be NULL (:776); if not, it is [num_queries][R] and receives those
 * step numbers as floats (+inf beside -1).  The reference ranks blind
 * candidates by a count that is 1 for every one of them and collects them
 * through per-thread cursors that overwrite each other, so it defines no order;
 * this one does.  R above 8192 takes the row-per-query path described above and
 * needs step numbers below 2^24 (else DCIH_EUNSUPPORTED).
 */
int dcih_query(dcih_index* h, int dim, int num_queries, const float* d_query,
               int num_neighbours, int blind, int num_outer_iterations,
               int max_num_candidates, int block_size, int thread_size,
               int32_t* d_nn, float* d_dists, uint64_t* d_counters, void* stream);

/*
 * dcih_query for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference.  Same arguments and same traversal kernels as
 * dcih_query, and the same results bit for bit, with one exception: where
 * dcih_query computes the answer directly because the stop rule provably cannot
 * fire (see there; the reference's own example configuration is such a shape), this
 * entry point still runs the traversal, whose distances are summed in a different
 * order: the neighbour sets are then the same and the distances agree to 1e-5
 * relative, not in every bit (and neighbours at tied distances may swap places).
 * Every byte of scratch (query projections, per-partition result
 * lists, hand-over lists between the traversal kernels and between the batch
 * kernel's two passes, global visit counters of partitions too large for on-chip
 * memory) comes from one array of
 * DCIH_NOALLOC_SCRATCH_BYTES that is part of the library's code object, so each
 * GPU the library runs on holds one such array until the process ends.  The call
 * makes no hipMalloc / hipFree and uses no allocating library routine.  A call
 * that needs more scratch than the array holds returns DCIH_EINVAL and says how
 * much it needs (the need grows with num_queries * block_size *
 * min(num_neighbours, points per partition): pass fewer queries per call); more
 * than 8192 results per query return DCIH_EUNSUPPORTED.  All calls on one GPU
 * share that GPU's array: calls that overlap in time on the same GPU (different
 * streams or threads) race and must be serialised by the caller; a call that
 * follows another on the same stream is safe, it overwrites what it uses.
 */
#define DCIH_NOALLOC_SCRATCH_BYTES (32u << 20)
int dcih_query_noalloc(dcih_index* h, int dim, int num_queries, const float* d_query,
                       int num_neighbours, int blind, int num_outer_iterations,
                       int max_num_candidates, int block_size, int thread_size,
                       int32_t* d_nn, float* d_dists, uint64_t* d_counters, void* stream);

/*
 * Inspection of the built index (no counterpart in the reference besides the
 * debug printer dci_dump, src/dci_cuda_kernel.cu:901-912).  Copies the sorted
 * projections and point ids, both [num_indices][num_points], to host buffers;
 * either pointer may be NULL.  Synchronous.
 */
int dcih_get_index(const dcih_index* h, float* h_keys, int32_t* h_ids);

/* Tuning knobs (no counterpart in the reference); see the DCIH_OPT_* list. */
int dcih_set_option(dcih_index* h, int option, int value);

/*
 * Per-kernel timing with HIP events on the caller's stream (no counterpart in
 * the reference).  After dcih_profile(h, 1) every dcih_add / dcih_query
 * brackets its kernels with events; dcih_last_timings waits for them and
 * writes DCIH_NUM_TIMERS durations in milliseconds (-1 for a kernel that has
 * not run since profiling was switched on).
 */
int dcih_profile(dcih_index* h, int enable);
int dcih_last_timings(dcih_index* h, float* h_ms);

/* Number of points currently indexed (0 when empty). */
int64_t dcih_num_points(const dcih_index* h);

/*
 * Replaces dci_clear (include/dci.h:77, src/dci_cuda_kernel.cu:878-885).  The
 * index becomes empty; the device memory its arrays occupied stays with the
 * handle, so that the next dcih_add allocates nothing, and is returned by
 * dcih_free.
 */
int dcih_clear(dcih_index* h);

/*
 * Replaces dci_reset (include/dci.h:80, src/dci_cuda_kernel.cu:887-891): clear,
 * then draw fresh directions (the next draw of the handle's seeded sequence).
 */
int dcih_reset(dcih_index* h);

/*
 * Replaces dci_free (include/dci.h:82, src/dci_cuda_kernel.cu:893-899) plus the
 * handle release in py_dci_free (src/dci_cuda.cpp:162-173).  NULL is a no-op.
 */
int dcih_free(dcih_index* h);

/*
 * Stand-alone pieces of the build, exposed so each kernel can be checked and
 * timed on its own.  d_keys is [num_indices][num_points].
 *   dcih_project : out[r][c] = sum_k d_rows[c][k] * d_dirs[r][k]  (the SGEMM at
 *                  src/util_kernel.cu:76 as used at src/dci_cuda_kernel.cu:167-169)
 *   dcih_segsort : copy_to_indices + sort_indices
 *                  (src/dci_cuda_kernel.cu:113-146), ties by id; -0.0 compares
 *                  equal to +0.0 (so they tie on the id) and is stored as +0.0
 */
int dcih_project(const float* d_dirs, int num_indices, const float* d_rows,
                 int64_t num_rows, int dim, float* d_out, void* stream);
int dcih_segsort(const float* d_keys, int num_indices, int64_t num_points,
                 int block_size, float* d_skeys, int32_t* d_sids, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DCI_HIP_H */
