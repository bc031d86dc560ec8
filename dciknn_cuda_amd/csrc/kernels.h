// Internal launch interface between the kernel translation units and api.hip.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dcih {

// out[r][c] = sum_k rows[c][k] * dirs[r][k]; out is [num_dirs][num_rows].
int project(const float* d_dirs, int num_dirs, const float* d_rows, int64_t num_rows,
            int dim, float* d_out, hipStream_t s);

// Sorts every (simple index, partition) slice of keys [num_indices][n] by
// (key, id).  d_tmp is scratch of segsort_tmp_bytes() bytes (may be null when
// that is 0).
size_t segsort_tmp_bytes(int num_indices, int64_t n, int block_size);
int segsort(const float* d_keys, int num_indices, int64_t n, int block_size,
            float* d_skeys, int32_t* d_sids, void* d_tmp, hipStream_t s);

struct QueryArgs {
    const float* skeys;      // [I][N] sorted projections
    const int32_t* sids;     // [I][N] point ids in the same order
    const float* data;       // [N][dim]
    const float* query;      // [nq][dim]
    const float* qproj;      // [I][nq]
    int64_t N;
    int64_t ppb;             // points per partition = ceil(N / B)
    int dim, M, L, B, T, nq, k;
    int kcap;                // min(k, ppb): results kept per (query, partition)
    int64_t stop_at;         // num_outer_iterations * L
    int64_t max_cand;
    unsigned long long* part;      // [nq][B][kcap] packed (dist bits << 32 | id)
    unsigned long long* counters;  // null or [nq][4]
    uint32_t* gscratch;      // global visit counters when they do not fit LDS
    int32_t* out_ids;        // [nq][k]
    float* out_dists;        // [nq][k]
};
size_t query_part_bytes(const QueryArgs& a);
// Bytes of global counter scratch the traversal needs (0 when LDS suffices).
size_t query_gscratch_bytes(const QueryArgs& a);
// ev: null, or three events recorded before the traversal, between traversal
// and merge, and after the merge.
int query(const QueryArgs& a, hipStream_t s, hipEvent_t* ev);

}  // namespace dcih
