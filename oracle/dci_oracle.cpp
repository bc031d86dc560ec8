/*
 * CPU oracle for Prioritized DCI (build + query).
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It is a from-scratch CPU
 * restatement of the semantics of niopeng/dciknn_cuda's data-parallel hot path,
 * written from reading that code as text.  Only tests, the smoke check and the
 * benchmark's CPU-baseline leg may load it; the shipped GPU path never does.
 *
 * Every function cites the reference lines (relative to the reference root)
 * whose behaviour it restates.  Deliberate, documented deviations:
 *   - directions are supplied by the caller (the reference draws them with
 *     cuRAND on device, src/util_kernel.cu:119-137);
 *   - ties in the per-segment sort are ordered (key asc, id asc); the
 *     reference's quicksort (src/dci_cuda_kernel.cu:205-235) leaves them
 *     unspecified;
 *   - the result is the k best of the UNION of all emitted candidates, the
 *     evident intent of src/dci_cuda_kernel.cu:691-701; the reference's scratch
 *     indexing at :514-534 makes (block, thread) pairs with equal sums share
 *     slots, which is a data race and not a semantics anyone can restate;
 *   - once every simple index of every composite index is exhausted the
 *     traversal stops; the reference spins to the loop bound at :458 without
 *     touching any state, so results are identical;
 *   - loop bounds use 64-bit arithmetic where the reference multiplies ints.
 *
 * Pinning status (what checks this file besides itself): the reference ships no
 * tests, golden vectors or fixtures for this path, so nothing of the
 * reference's own pins it.  It is pinned by tests/test_oracle_*.py against:
 * exact brute force in the exhaustive regime, numpy.searchsorted, torch/numpy
 * matmul and stable sort, an independent heap-based textbook Prioritized DCI
 * (T=1, B=1), an independent sort-all-windows model for general (B, T), and
 * hand-derived traces on tiny inputs.  Parts no check can reach without
 * running the CUDA reference ("parity unpinned"): the cuRAND direction stream,
 * the unstable-sort tie order, cuBLAS's summation order.
 */
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <numeric>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

const float kInf = std::numeric_limits<float>::infinity();

/* src/dci_cuda_kernel.cu:46-49 (abs_d) */
inline float abs_d(float x) { return x > 0 ? x : -x; }

/* src/dci_cuda_kernel.cu:35-44 (compute_dist_device): sequential fp32 sum of
 * squared differences, then sqrt. */
inline float euclid(const float* a, const float* b, int dim) {
    float sq = 0.0f;
    for (int i = 0; i < dim; i++) {
        float diff = a[i] - b[i];
        sq += diff * diff;
    }
    return std::sqrt(sq);
}

/* src/dci_cuda_kernel.cu:279-297 (dci_search_index): largest j with
 * key[j] < q, or -1. */
inline int search_index(const float* key, float q, int n, uint64_t* probes) {
    int start_pos = -1, end_pos = n - 1;
    int cur_pos = (start_pos + end_pos + 2) / 2;
    while (start_pos < end_pos) {
        if (probes) ++*probes;
        if (key[cur_pos] < q) start_pos = cur_pos;
        else end_pos = cur_pos - 1;
        cur_pos = (start_pos + end_pos + 2) / 2;
    }
    return start_pos;
}

/* src/dci_cuda_kernel.cu:250-273 (dci_next_closest_proj); T = blockDim.x. */
inline int next_window(const float* key, int n, int T, int* left, int* right,
                       float q) {
    int cur;
    const int lower = -T;
    const int upper = n + T - 1;
    if (*left <= lower && *right >= upper) {
        cur = lower;
    } else if (*left <= lower) {
        cur = *right; *right += T;
    } else if (*right >= upper) {
        cur = *left; *left -= T;
    } else if (key[std::min(*right, n - 1)] - q < q - key[std::max(*left, 0)]) {
        cur = *right; *right += T;
    } else {
        cur = *left; *left -= T;
    }
    return cur;
}

/* src/dci_cuda_kernel.cu:572-590 (and :339-352 for the initial fill): clamp
 * the window start into range and take |key - q| there; an out-of-range start
 * means the simple index is exhausted. */
inline float window_priority(const float* key, int n, int T, int* cur, float q) {
    int position;
    if (*cur < 0 && *cur > -T) position = 0;
    else if (*cur < n + T - 1 && *cur >= n) position = n - 1;
    else position = *cur;
    if (position >= 0 && position < n) return abs_d(key[position] - q);
    *cur = -T;
    return kInf;
}

/* A candidate and what ranks it: its distance, or, in blind querying, the
 * outer step of its partition's traversal that promoted it. */
template <class Score> struct Cand { Score score; int id; };
template <class Score>
inline bool cand_less(const Cand<Score>& a, const Cand<Score>& b) {
    return a.score < b.score || (a.score == b.score && a.id < b.id);
}

struct Scratch {
    std::vector<uint16_t> counts;   /* [M][n_b] */
    std::vector<uint8_t> seen;      /* [n_b]    */
    std::vector<int> left, right, cur;
    std::vector<float> prio;
};

struct Stats { uint64_t visited = 0, cands = 0, probes = 0, steps = 0; };

/* One partition of one query: src/dci_cuda_kernel.cu:401-626 with
 * blockIdx.x = b, blockDim.x = T.  Emits (id, outer step) for every promoted
 * point; the caller computes the distance (:506-511) or, blind, records the
 * point (:498-505). */
template <class Emit>
void traverse_partition(const float* skeys, const int* sids,
                        const float* qp, int64_t N,
                        int M, int L, int T, int64_t seg_off, int n, int k,
                        int64_t outer, int64_t max_cand, Scratch& s, Stats& st,
                        Emit emit) {
    const int I = M * L;
    s.counts.assign((size_t)M * n, 0);
    s.seen.assign((size_t)n, 0);
    s.left.resize(I); s.right.resize(I); s.cur.resize(I); s.prio.resize(I);

    /* :300-318 search_index, :320-355 init_index_priority */
    for (int i = 0; i < I; i++) {
        const float* key = skeys + (int64_t)i * N + seg_off;
        int p = search_index(key, qp[i], n, &st.probes);
        s.left[i] = p - T + 1;
        s.right[i] = s.left[i] + T;
    }
    for (int i = 0; i < I; i++) {
        const float* key = skeys + (int64_t)i * N + seg_off;
        s.cur[i] = next_window(key, n, T, &s.left[i], &s.right[i], qp[i]);
        s.prio[i] = window_priority(key, n, T, &s.cur[i], qp[i]);
    }

    const int64_t bound = (int64_t)n * L * T;       /* :458 */
    const int64_t stop_at = outer * (int64_t)L;     /* :600-602 */
    int64_t kk = 0;
    int64_t c0 = 0;  /* promotions made by lane 0 only (:413, :598-599) */
    while (kk < bound) {
        bool any = false;
        for (int m = 0; m < M; m++) {
            /* :466-478 first strict minimum against +inf */
            float top = kInf; int top_h = -1;
            for (int h = 0; h < L; h++) {
                if (s.prio[m * L + h] < top) { top = s.prio[m * L + h]; top_h = h; }
            }
            if (top_h < 0) continue;
            any = true;
            const int i = m * L + top_h;
            const float* key = skeys + (int64_t)i * N + seg_off;
            const int* ids = sids + (int64_t)i * N + seg_off;
            const int position = s.cur[i];
            uint16_t* cnt = s.counts.data() + (size_t)m * n;
            for (int t = 0; t < T; t++) {                       /* :487-562 */
                const int cur_index = position + t;
                if (cur_index < 0 || cur_index >= n) continue;
                const int pt = ids[cur_index];
                const int local = (int)(pt - seg_off);
                st.visited++;
                if (++cnt[local] == L && !s.seen[local]) {
                    s.seen[local] = 1;
                    st.cands++;
                    emit(pt, kk);
                    if (t == 0) c0++;
                }
            }
            s.cur[i] = next_window(key, n, T, &s.left[i], &s.right[i], qp[i]); /* :567-571 */
            s.prio[i] = window_priority(key, n, T, &s.cur[i], qp[i]);          /* :572-590 */
        }
        st.steps++;
        if (c0 >= k && (kk + 1 >= stop_at || c0 >= max_cand)) break;  /* :598-607 */
        if (!any) break;  /* everything exhausted: the reference would idle to `bound` */
        kk++;
    }
}

}  // namespace

extern "C" {

/* src/dci_cuda_kernel.cu:52-73 (normalize_proj_vecs): per row, sequential fp32
 * sum of squares, sqrtf, divide each entry. */
void dci_oracle_normalize(float* P, int I, int dim) {
    for (int r = 0; r < I; r++) {
        float sq = 0.0f;
        for (int k = 0; k < dim; k++) sq += P[(int64_t)r * dim + k] * P[(int64_t)r * dim + k];
        float norm = sqrtf(sq);
        for (int k = 0; k < dim; k++) P[(int64_t)r * dim + k] /= norm;
    }
}

/* src/util_kernel.cu:45-80 with the call at src/dci_cuda_kernel.cu:167-169:
 * row-major out[R][C] = A[R][dim] . B[C][dim]^T in fp32.  cuBLAS's summation
 * order is unspecified; this restatement fixes it as ONE fused multiply-add
 * chain over k = 0..dim-1 starting from +0 (what a compiled CUDA loop with the
 * default -fmad=true does), which any IEEE-754 machine reproduces bit for bit.
 * Build: A = directions, B = data -> [I][N].  Query (:802-803): A = queries,
 * B = directions -> [nq][I]. */
void dci_oracle_matmul_nt(const float* A, const float* B, float* out, int64_t R,
                          int64_t C, int dim) {
#pragma omp parallel for schedule(static)
    for (int64_t c = 0; c < C; c++) {
        for (int64_t r = 0; r < R; r++) {
            float acc = 0.0f;
            const float* a = A + r * dim;
            const float* b = B + c * dim;
            for (int k = 0; k < dim; k++) acc = std::fmaf(a[k], b[k], acc);
            out[r * C + c] = acc + 0.0f;   /* -0 -> +0, so equal keys always tie on the id */
        }
    }
}

/* src/dci_cuda_kernel.cu:132-146 (copy_to_indices: value = e % N) and :113-129
 * (sort_indices) with points_per_block = ceil(N/B) (:178): every (simple index,
 * partition) slice is sorted ascending by key on its own; ties by id. */
void dci_oracle_segsort(const float* keys, int64_t N, int I, int B,
                        float* skeys, int* sids) {
    const int64_t ppb = (N + B - 1) / B;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int i = 0; i < I; i++) {
        for (int b = 0; b < B; b++) {
            const int64_t off = (int64_t)b * ppb;
            const int64_t n = std::min(N - off, ppb);
            if (n <= 0) continue;
            std::vector<int> perm((size_t)n);
            std::iota(perm.begin(), perm.end(), 0);
            const float* kseg = keys + (int64_t)i * N + off;
            std::stable_sort(perm.begin(), perm.end(),
                             [kseg](int a, int c) { return kseg[a] < kseg[c]; });
            for (int64_t j = 0; j < n; j++) {
                skeys[(int64_t)i * N + off + j] = kseg[perm[j]];
                sids[(int64_t)i * N + off + j] = (int)(off + perm[j]);
            }
        }
    }
}

/* src/dci_cuda_kernel.cu:279-297, exposed for unit tests. */
int dci_oracle_search(const float* key, float q, int n) {
    return search_index(key, q, n, nullptr);
}

/* The window sequence of ONE simple index, for hand traces: positions the
 * query as :309-315 does, then repeats next/priority (:250-273, :572-590)
 * until exhaustion.  Writes window starts and priorities; returns the count. */
int dci_oracle_window_sequence(const float* key, int n, int T, float q,
                               int* out_cur, float* out_prio, int cap) {
    int p = search_index(key, q, n, nullptr);
    int left = p - T + 1, right = left + T;
    int cnt = 0;
    while (cnt < cap) {
        int cur = next_window(key, n, T, &left, &right, q);
        float pr = window_priority(key, n, T, &cur, q);
        if (!(pr < kInf)) break;
        out_cur[cnt] = cur; out_prio[cnt] = pr; cnt++;
    }
    return cnt;
}

}  // extern "C"

namespace {

/* Shared body of the two query entry points below.  BLIND == false: the k_out
 * best of all promoted candidates by (distance, id), src/dci_cuda_kernel.cu
 * :506-554 and :691-701.  BLIND == true: the first k_out of them by (promoting
 * step, id), see dci_oracle_query_blind. */
template <bool BLIND, class Score>
int query_impl(const float* skeys, const int* sids, const float* data,
               const float* query, const float* qproj, int64_t N, int dim,
               int M, int L, int B, int T, int nq, int k, int64_t k_out,
               int64_t outer, int64_t max_cand, int* out_ids, Score* out_scores,
               Score empty_score, uint64_t* counters, int* cand_ids,
               int64_t cand_cap, int64_t* cand_cnt, int num_threads) {
    if (k <= 0 || k > N || k_out <= 0 || B <= 0 || T <= 0 || M <= 0 || L <= 0 || L > 65535) return -1;
    const int I = M * L;
    const int64_t ppb = (N + B - 1) / B;   /* :424 */
#ifdef _OPENMP
    if (num_threads > 0) omp_set_num_threads(num_threads);
#endif
#pragma omp parallel
    {
        Scratch s;
        std::vector<Cand<Score>> heap;  /* max-heap of the k_out best so far */
#pragma omp for schedule(dynamic, 1)
        for (int j = 0; j < nq; j++) {
            heap.clear();
            Stats st;
            int64_t ncand = 0;
            const float* q = query + (int64_t)j * dim;
            const float* qp = qproj + (int64_t)j * I;
            for (int b = 0; b < B; b++) {
                const int64_t off = (int64_t)b * ppb;
                const int64_t n = std::min(N - off, ppb);   /* :425-427 */
                if (n <= 0) continue;                       /* :429 */
                traverse_partition(
                    skeys, sids, qp, N, M, L, T, off, (int)n, k,
                    outer, max_cand, s, st, [&](int id, int64_t step) {
                        if (cand_ids && ncand < cand_cap)
                            cand_ids[(int64_t)j * cand_cap + ncand] = id;
                        ncand++;
                        Cand<Score> c;
                        if constexpr (BLIND) c.score = (Score)step;
                        else c.score = euclid(data + (int64_t)id * dim, q, dim);
                        c.id = id;
                        if ((int64_t)heap.size() < k_out) {
                            heap.push_back(c);
                            std::push_heap(heap.begin(), heap.end(), cand_less<Score>);
                        } else if (cand_less(c, heap.front())) {
                            std::pop_heap(heap.begin(), heap.end(), cand_less<Score>);
                            heap.back() = c;
                            std::push_heap(heap.begin(), heap.end(), cand_less<Score>);
                        }
                    });
            }
            std::sort_heap(heap.begin(), heap.end(), cand_less<Score>);
            for (int64_t r = 0; r < k_out; r++) {
                const bool have = r < (int64_t)heap.size();
                out_ids[(int64_t)j * k_out + r] = have ? heap[r].id : -1;
                if (out_scores) out_scores[(int64_t)j * k_out + r] = have ? heap[r].score : empty_score;
            }
            if (counters) {
                counters[(int64_t)j * 4 + 0] = st.visited;
                counters[(int64_t)j * 4 + 1] = st.cands;
                counters[(int64_t)j * 4 + 2] = st.probes;
                counters[(int64_t)j * 4 + 3] = st.steps;
            }
            if (cand_cnt) cand_cnt[j] = ncand;
        }
    }
    return 0;
}

}  // namespace

extern "C" {

/* src/dci_cuda_kernel.cu:777-865 (dci_query) over src/dci_cuda_kernel.cu:401-626
 * per (query, partition), then the k best of the union (:691-701).
 *
 *   skeys, sids : [I][N] segment-sorted keys / point ids (dci_oracle_segsort)
 *   data [N][dim], query [nq][dim], qproj [nq][I]
 *   out_ids, out_dists : [nq][k], ascending (dist, id); unfilled slots (fewer
 *                        than k candidates) get id -1, dist +inf
 *   counters : nullable [nq][4] = entries visited, candidates, search probes,
 *              outer steps executed (summed over partitions)
 *   cand_ids / cand_cnt : nullable dump of every emitted candidate id per query
 *              in emission order, up to cand_cap each; cand_cnt gets the true
 *              count even when it exceeds cand_cap.
 * Returns 0, or -1 on invalid arguments (the reference asserts, :787-789).
 */
int dci_oracle_query(const float* skeys, const int* sids, const float* data,
                     const float* query, const float* qproj, int64_t N, int dim,
                     int M, int L, int B, int T, int nq, int k, int64_t outer,
                     int64_t max_cand, int* out_ids, float* out_dists,
                     uint64_t* counters, int* cand_ids, int64_t cand_cap,
                     int64_t* cand_cnt, int num_threads) {
    return query_impl<false, float>(skeys, sids, data, query, qproj, N, dim, M, L, B, T, nq, k, k,
                                    outer, max_cand, out_ids, out_dists, kInf, counters,
                                    cand_ids, cand_cap, cand_cnt, num_threads);
}

/*
 * Blind querying: dci_query with query_config.blind == true
 * (src/dci_cuda_kernel.cu:498-505 records a promoted point instead of computing
 * its distance; :754-773 and :859-864 return max_possible_num_candidates =
 * min(max_num_candidates, num_outer_iterations) ids per query, :782-783).  The
 * traversal and its stop rule (:598-607, armed by k = num_neighbours) are those
 * of dci_oracle_query.  The reference ranks the recorded points by how often
 * they were recorded, which is once each (a point belongs to one partition and
 * :497 admits it once), and records them through per-thread cursors that
 * overwrite each other (:500-504), so it fixes no order among them.  This
 * restatement fixes one: ascending by (outer step kk of the partition's
 * traversal at which the point was promoted, id).
 *
 *   out_ids   : [nq][R], R = min(max_cand, outer); -1 beyond the candidates
 *   out_steps : nullable [nq][R]; 0xffffffff beside -1
 * Returns 0, or -1 on invalid arguments.
 */
int dci_oracle_query_blind(const float* skeys, const int* sids,
                           const float* qproj, int64_t N,
                           int M, int L, int B, int T, int nq, int k, int64_t outer,
                           int64_t max_cand, int* out_ids, uint32_t* out_steps,
                           uint64_t* counters, int num_threads) {
    const int64_t R = std::min(max_cand, outer);
    return query_impl<true, uint32_t>(skeys, sids, nullptr, nullptr, qproj, N, 0, M, L, B, T, nq,
                                      k, R, outer, max_cand, out_ids, out_steps, 0xffffffffu,
                                      counters, nullptr, 0, nullptr, num_threads);
}

int dci_oracle_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

}  // extern "C"
