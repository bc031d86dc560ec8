// Internal launch interface between the kernel translation units and api.hip.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dcih {

// out[r][c] = sum_k rows[c][k] * dirs[r][k]; row r of out starts at d_out + r * out_stride
// (out_stride >= num_rows).
int project(const float* d_dirs, int num_dirs, const float* d_rows, int64_t num_rows,
            int dim, float* d_out, int64_t out_stride, hipStream_t s);

// Sorts every (simple index, partition) slice of the keys by (key, id); the keys of
// index i start at d_keys + i * key_stride (key_stride >= n), the outputs are
// [num_indices][n].  d_tmp is scratch of segsort_tmp_bytes() bytes (may be null when
// that is 0).
size_t segsort_tmp_bytes(int num_indices, int64_t n, int block_size);
// d_inv: null, or [num_indices][n] receiving each point's position inside its
// sorted slice (the inverse of d_sids) as a 16-bit value (only meaningful when a partition
// holds at most 65536 points).  d_lids: null, or [num_indices][n] receiving the ids relative
// to their partition's first point as 16-bit values (no kernel reads them any more; the
// index does not keep them).
int segsort(const float* d_keys, int64_t key_stride, int num_indices, int64_t n, int block_size,
            float* d_skeys, int32_t* d_sids, uint16_t* d_inv, uint16_t* d_lids, void* d_tmp,
            hipStream_t s);

// Appending: the index over n1 points from the sorted arrays of the index over their first
// n0 points (same block_size) and the unsorted keys of the others (index i's key of point id
// at d_keys + i * key_stride + id): old slices are split into runs of the new ones, the new
// points sorted, the runs merged; nothing of the old part is sorted again.  Outputs as
// segsort's; d_tmp = segsort_append_tmp_bytes() bytes.
bool segsort_append_supported(int64_t n0, int64_t n1, int block_size);
size_t segsort_append_tmp_bytes(int num_indices, int64_t n1);
int segsort_append(const float* d_old_skeys, const int32_t* d_old_sids, int64_t n0,
                   const float* d_keys, int64_t key_stride, int num_indices, int64_t n1, int block_size,
                   float* d_skeys, int32_t* d_sids, uint16_t* d_inv, uint16_t* d_lids, void* d_tmp,
                   hipStream_t s);

// rpos (above inv's layout, [I][n] 16-bit values): rpos[i][e] = inv[i][sids[first(i)][e]], first(i) = the first simple
// index of i's composite; the rows of the first simple indices themselves are left alone (the identity).
int fill_positions_by_first(const int32_t* d_sids, const uint16_t* d_inv, uint16_t* d_rpos, int64_t n, int M, int L,
                            hipStream_t s);

struct QueryArgs {
    const float* skeys;      // [I][N] sorted projections
    const int32_t* sids;     // [I][N] point ids in the same order
    const uint16_t* inv;     // [I][N] position of every point inside its sorted slice (null if ppb > 65536)
    const uint16_t* rpos;    // [I][N] the same positions in the order of the composite's FIRST simple index: entry s of a
                             // slice is the position, in this simple index, of the point that stands at place s of the
                             // first one's slice (null if ppb > 65536; filled on the first use, see fill_positions_by_first)
    int* rpos_ready;         // host flag of the index: rpos has been filled
    const float* data;       // [N][dim]
    const float* query;      // [nq][dim]
    const float* qproj;      // [I][nq]
    int64_t N;
    int64_t ppb;             // points per partition = ceil(N / B)
    int dim, M, L, B, T, nq;
    int k;                   // results per query
    int k_stop;              // promotions by a window's first lane that arm the stop rule (num_neighbours)
    int blind;               // 1: a candidate is scored by the step that promoted it, no distance is computed
    unsigned T_magic;        // ceil(2^32 / T) for T > 1: d / T == mulhi(d, T_magic) for 0 <= d < 65536
    int kcap;                // min(k, ppb): results kept per (query, partition)
    int64_t stop_at;         // num_outer_iterations * L
    int64_t max_cand;
    unsigned long long* part;      // [nq][B][kcap] packed (dist bits << 32 | id); blind: (step << 32 | id)
    unsigned long long* counters;  // null or [nq][4]
    uint32_t* gscratch;      // global visit counters when they do not fit LDS
    int32_t* redo_items;     // [nq*B] (query, partition) pairs the batch kernel hands back
    uint32_t* redo_count;    // their number
    const int32_t* item_list;    // step-by-step kernel: null = all nq*B items, else this list
    const uint32_t* item_count;  // ... of this length
    float* stop_hint;        // null, or [3][B] per partition: running averages of the stop step and of the promotions at the stop, stops seen
    int hints_cold;          // the table was cleared for this call: nothing is known yet about where traversals stop
    unsigned long long* phase_ticks;  // null, or 16 accumulators for the batch kernel's phases
    int mode;                // 0 = pick, 1 = step-by-step kernel, 2 = batch kernel, 3 = dense kernel
    // hand-over from the batch kernel to the dense kernel: one list of items per die
    int32_t* dense_items;    // null, or [xcds][dense_cap]
    uint32_t* dense_count;   // [xcds]
    int64_t dense_cap;
    int dense_min_promos;    // promotions per (query, partition) from which the dense kernel is the cheaper one
    // second pass of the batch kernel: items that outgrow its compact per-item tables are listed and
    // taken up again by the variant with the full tables
    int32_t* wide_items;     // null, or [wide_cap]
    uint32_t* wide_count;
    int64_t wide_cap;
    const int32_t* block_list;        // null = the launch covers queries q_first .. q_first + q_count; else workgroup w takes block_list[w]
    const uint32_t* block_list_count; // ... for w below this number
    int full_tables;         // 1: the batch kernel keeps its per-point flags as bits whatever the shape
    int xcds;                // accelerator dies of the device (each has an L2 of its own)
    int q_first, q_count;    // batch kernel: the queries one launch covers
    int32_t* out_ids;        // [nq][k]
    float* out_dists;        // [nq][k]; blind: null, or the promoting steps as floats
    float* dense;            // null, or [nq][N]: the step-by-step kernel stores every candidate's score here instead of keeping a top-k
};
// The query scratch keeps its list lengths in 64 consecutive words that one kernel clears: the
// step-by-step kernel's redo list, one hand-over list per die (up to 32), and in the last word
// the batch kernel's second-pass list.
constexpr int kListCountWords = 64;

// Work order of the batch kernel.  Workgroups go to the XCDs round-robin by their
// number and every XCD has an L2 of its own, so XCD x is given the partitions x,
// x + X, ... and works through them one after the other, all queries of a
// partition before the next: the workgroups an XCD runs at any moment share one
// partition's slices.  The B mod X partitions that do not fill a round are spread
// over all X dies as equal runs of the (partition, query) list, so no die idles.
// block_items = workgroups one launch over nq queries needs; block_item maps a
// workgroup to its partition b and query q (false: nothing to do).
__host__ __device__ inline int64_t block_items(int X, int B, int nq) {
    const int full = B / X, rest = B - full * X;
    return (int64_t)X * ((int64_t)full * nq + ((int64_t)rest * nq + X - 1) / X);
}
__host__ __device__ inline bool block_item(int64_t block, int X, int B, int nq, int& b, int& q) {
    const int xcd = (int)(block % X);
    const int64_t seq = block / X;
    const int full = B / X, rest = B - full * X;
    const int64_t full_items = (int64_t)full * nq;
    if (seq < full_items) {
        b = xcd + X * (int)(seq / nq);
        q = (int)(seq % nq);
        return true;
    }
    const int64_t run = ((int64_t)rest * nq + X - 1) / X;
    const int64_t e = (seq - full_items) + (int64_t)xcd * run;
    if (seq - full_items >= run || e >= (int64_t)rest * nq) return false;
    b = X * full + (int)(e / nq);
    q = (int)(e % nq);
    return true;
}
// Queries one launch of the batch kernel may cover: a launch is limited to 2^32 - 1
// threads in all (256 per workgroup).
__host__ __device__ inline int block_queries_per_launch(int X, int B, int nq) {
    const int64_t max_items = 0xffffffffLL / 256;
    const int64_t per_query = (int64_t)B + X;          // upper bound of block_items / nq
    const int64_t fit = max_items / per_query;
    return (int)(fit < 1 ? 0 : (fit < nq ? fit : nq));
}
// Workgroups of the step-by-step kernel: it strides over its items, and a launch is
// limited to 2^32 - 1 threads in all (64 per workgroup).
__host__ __device__ inline int64_t step_grid_cap() { return (int64_t)1 << 20; }

size_t query_part_bytes(const QueryArgs& a);
// Clears n 64-bit words with a kernel (a memset node is not safe in a captured graph).
int zero_words64(void* d_p, int64_t n, hipStream_t s);
// Bytes of global counter scratch the traversal needs (0 when LDS suffices).
size_t query_gscratch_bytes(const QueryArgs& a);
// Batch traversal (traverse_block.hip): whether the shape fits its fixed LDS
// tables, and the launch itself.
bool block_traversal_supported(const QueryArgs& a, size_t* lds_bytes);
int query_block(const QueryArgs& a, hipStream_t s);
// Dense traversal (traverse_dense.hip): every point's promoting step at once.  Works
// through the lists the batch kernel filled (a.dense_items) or, with a.mode == 3,
// through all items.
bool dense_traversal_supported(const QueryArgs& a, size_t* lds_bytes);
int query_dense_items(const QueryArgs& a, hipStream_t s);

// Full ranking (exhaustive.hip) for num_neighbours above the points per partition,
// where the traversal provably visits everything: queries are processed `chunk` at
// a time in `ws` (exhaustive_ws_bytes(N, chunk) bytes); a.qproj is needed only when
// a.counters is set.
int exhaustive_chunk(int64_t N, int nq);
size_t exhaustive_ws_bytes(int64_t N, int chunk);
int query_exhaustive(const QueryArgs& a, void* ws, int chunk, hipStream_t s);
// The pieces of it that the dense-row traversal (query_dense) shares: rows of N values
// at rank_rows_input(ws), `rows` <= chunk of them; rank_rows sorts every row by (value,
// column) and writes the first k columns (id = column, or -1 for +inf when asked).
float* rank_rows_input(void* ws);
int fill_rows(float* d_rows, int64_t cells, float value, hipStream_t s);
int rank_rows(void* ws, int chunk, int rows, int64_t N, int k, bool inf_is_empty,
              int32_t* out_ids, float* out_vals, hipStream_t s);
// More results per query than the top-k tables hold, early stops possible: the
// step-by-step kernel writes every candidate's score into a dense row of its query
// (+inf = not a candidate), rank_rows does the rest.  Projects the queries itself
// (d_dirs), chunk by chunk; ws = I*chunk floats + exhaustive_ws_bytes(N, chunk) bytes.
int query_dense(const QueryArgs& a, const float* d_dirs, void* ws, int chunk, hipStream_t s);

// ev: null, or five events recorded before the traversal, after the batch kernel (if it
// ran: ran[0]), after the dense kernel (if it ran: ran[1]), between traversal and merge,
// and after the merge.
int query(const QueryArgs& a, hipStream_t s, hipEvent_t* ev, bool* ran);

}  // namespace dcih
