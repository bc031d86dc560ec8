/*
 * Inspection entry points of libdci_hip.so that are not part of the product
 * surface in dci_hip.h: they mirror nothing in the CUDA reference
 * (niopeng/dciknn_cuda) and exist for tests and for profiling the traversal
 * kernels.  Same conventions as dci_hip.h (status codes, dcih_last_error()).
 */
#ifndef DCI_HIP_DEBUG_H
#define DCI_HIP_DEBUG_H

#include "dci_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Phase profile of the batch traversal kernel (no counterpart in the
 * reference).  d_ticks is NULL (off) or a zeroed device array of 16 uint64 that
 * later dcih_query calls add to: [0..7] = 100 MHz ticks one thread of every
 * workgroup spent in set-up, bound selection, range search, streaming, undo,
 * promotion ranking, replay, distances/top-k; [8] = epochs, [9] = items finished by
 * the batch kernel (either pass), [10] = items it handed back (to its second pass with
 * the full tables, or to the step-by-step kernel), [11..14] = those by reason.
 */
int dcih_phase_profile(dcih_index* h, uint64_t* d_ticks);

/*
 * Launch geometry of the batch traversal kernel (no counterpart in the reference;
 * pure host arithmetic, no GPU needed): with `xcds` dies, block_size partitions and
 * num_queries queries, returns the number of workgroups one launch starts, or -1
 * if the shape cannot be launched; if b and q are not NULL and 0 <= block < that
 * number, *b / *q receive the partition and query workgroup `block` works on, or
 * -1 / -1 if it has nothing to do.  *queries_per_launch (if not NULL) receives how
 * many queries one launch may cover (a launch is limited to 2^32 - 1 threads).
 */
int64_t dcih_debug_launch_map(int xcds, int block_size, int num_queries, int64_t block,
                              int* b, int* q, int* queries_per_launch);

/*
 * The two position tables of the index (no counterpart in the reference, which keeps only
 * (key, id) pairs): d_inv and d_rpos each receive [num_indices][num_points] uint16 values, or
 * may be NULL.  inv[i][p] = place of point p in the sorted slice of simple index i that holds
 * it; rpos[i][e] = inv[i][id at element e of the FIRST simple index of i's composite], i.e.
 * the same places in that index's order (the rows of the first simple indices themselves are
 * never written and come back as zeros).  The second table is filled here if no query has
 * needed it yet.  DCIH_EUNSUPPORTED for an index whose partitions exceed 65536 points (it
 * keeps neither table).  Synchronises the stream.
 */
int dcih_debug_positions(dcih_index* h, uint16_t* d_inv, uint16_t* d_rpos, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DCI_HIP_DEBUG_H */
