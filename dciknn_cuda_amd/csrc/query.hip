// Query path: prioritized traversal of one partition per wavefront, exact
// distances of the promoted points, k best per partition, then a per-query
// merge over partitions.
//
// Stands in for dci_query (src/dci_cuda_kernel.cu:777-875) and the kernels it
// launches once per query: init_dist / init_counts / init_candidate_dists
// (:703-716, :357-382), dci_query_single_point_by_block (:401-626) with
// search_index / init_index_priority / dci_next_closest_proj (:250-355), and
// get_top_candidates (:691-701).
//
// All queries run in one launch: workgroup = one 64-lane wavefront = one
// (query, partition) pair.  The visit counters the reference keeps in global
// memory and re-initialises for every query (4*M*N + 4*N bytes per query) live
// in LDS as packed bit fields, sized by the partition, plus one "seen" bit per
// point; when a partition is too large for LDS they fall back to a per-
// workgroup slice of global scratch.  A window of T sorted entries is visited
// by T lanes at once (in 64-lane slabs when T > 64); promoted points are found
// with a ballot and their rows are read by the whole wavefront.
#include <math.h>

#include "common.h"
#include "kernels.h"

namespace dcih {

namespace {

constexpr int kMaxLds = 160 * 1024;       // LDS per workgroup on gfx950
constexpr int kLdsMargin = 1024;
constexpr int kTopkLdsMax = 2048;         // k up to which the per-partition top-k stays in LDS
constexpr int kMaxSlots = 4096;           // resident workgroups in the global-counter fallback
constexpr int kMergeThreads = 256;

__host__ __device__ inline int counter_bits(int L) {
    return L <= 15 ? 4 : (L <= 255 ? 8 : (L <= 65535 ? 16 : 32));
}

struct Layout {
    int cbits;          // bits per visit counter
    int wpc;            // 32-bit words per composite index counter array
    int seen_words;
    int counter_words;  // M * wpc + seen_words
    int state_bytes;    // left/right/cur/prio/qp + query row
    int topk_bytes;     // 0 when the top-k lives in global memory
    bool lds_counters;
    size_t lds_bytes;
};

Layout make_layout(const QueryArgs& a) {
    Layout y;
    y.cbits = counter_bits(a.L);
    const int64_t fpw = 32 / y.cbits;
    y.wpc = (int)((a.ppb + fpw - 1) / fpw);
    y.seen_words = (int)((a.ppb + 31) / 32);
    const int64_t cw = (int64_t)a.M * y.wpc + y.seen_words;
    y.counter_words = (int)cw;
    const int I = a.M * a.L;
    y.state_bytes = 5 * I * 4 + ((a.dim + 3) & ~3) * 4;
    y.topk_bytes = a.kcap <= kTopkLdsMax ? a.kcap * 8 : 0;
    const int64_t fixed = y.state_bytes + y.topk_bytes + 64;
    y.lds_counters = fixed + cw * 4 <= kMaxLds - kLdsMargin;
    y.lds_bytes = (size_t)(fixed + (y.lds_counters ? cw * 4 : 0));
    return y;
}

// dci_next_closest_proj (src/dci_cuda_kernel.cu:250-273)
__device__ inline int next_window(const float* __restrict__ key, int n, int T, int& left,
                                  int& right, float q) {
    const int lower = -T, upper = n + T - 1;
    int cur;
    if (left <= lower && right >= upper) {
        cur = lower;
    } else if (left <= lower) {
        cur = right; right += T;
    } else if (right >= upper) {
        cur = left; left -= T;
    } else if (key[min(right, n - 1)] - q < q - key[max(left, 0)]) {
        cur = right; right += T;
    } else {
        cur = left; left -= T;
    }
    return cur;
}

// Priority of the window starting at cur (src/dci_cuda_kernel.cu:572-590).
__device__ inline float window_priority(const float* __restrict__ key, int n, int T, int& cur,
                                        float q) {
    int position;
    if (cur < 0 && cur > -T) position = 0;
    else if (cur < n + T - 1 && cur >= n) position = n - 1;
    else position = cur;
    if (position >= 0 && position < n) return fabsf(key[position] - q);
    cur = -T;
    return __builtin_inff();
}

template <bool LDS_COUNTERS>
__global__ __launch_bounds__(kWave) void traverse_kernel(QueryArgs a, Layout y) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int I = a.M * a.L;
    const int lane = threadIdx.x;
    int* s_left = reinterpret_cast<int*>(smem);
    int* s_right = s_left + I;
    int* s_cur = s_right + I;
    float* s_prio = reinterpret_cast<float*>(s_cur + I);
    float* s_qp = s_prio + I;
    float* s_q = s_qp + I;
    unsigned long long* s_top =
        reinterpret_cast<unsigned long long*>(smem + ((y.state_bytes + 15) & ~15));
    uint32_t* s_cnt = reinterpret_cast<uint32_t*>(smem + ((y.state_bytes + 15) & ~15) + y.topk_bytes);

    const int64_t items = a.item_list ? (int64_t)*a.item_count : (int64_t)a.nq * a.B;
    const uint32_t cmask = y.cbits == 32 ? 0xffffffffu : ((1u << y.cbits) - 1u);
    const int fshift = y.cbits == 4 ? 3 : (y.cbits == 8 ? 2 : (y.cbits == 16 ? 1 : 0));  // log2(fields/word)

    for (int64_t slot = blockIdx.x; slot < items; slot += gridDim.x) {
        const int64_t item = a.item_list ? (int64_t)a.item_list[slot] : slot;
        const int b = (int)(item % a.B);
        const int qi = (int)(item / a.B);
        const int64_t off = (int64_t)b * a.ppb;
        const int n = (int)min(a.N - off, a.ppb);
        unsigned long long* top = y.topk_bytes ? s_top : a.part + item * a.kcap;
        unsigned long long* part_out = a.part + item * a.kcap;
        if (n <= 0) {   // empty partition (src/dci_cuda_kernel.cu:429)
            if (!a.dense)
                for (int j = lane; j < a.kcap; j += kWave) part_out[j] = ~0ull;
            continue;
        }
        uint32_t* cnt = LDS_COUNTERS ? s_cnt
                                     : a.gscratch + (size_t)blockIdx.x * (size_t)y.counter_words;
        uint32_t* seen = cnt + (size_t)a.M * y.wpc;

        __syncthreads();
        for (int w = lane; w < y.counter_words; w += kWave) cnt[w] = 0;
        for (int j = lane; j < a.dim; j += kWave) s_q[j] = a.query[(int64_t)qi * a.dim + j];
        if (!LDS_COUNTERS) __threadfence();

        // positioning search (:279-318) and first window of every simple index (:320-355)
        unsigned long long probes = 0;
        for (int i = lane; i < I; i += kWave) {
            const float* key = a.skeys + (int64_t)i * a.N + off;
            const float qp = a.qproj[(int64_t)i * a.nq + qi];
            int start_pos = -1, end_pos = n - 1;
            int cur_pos = (start_pos + end_pos + 2) / 2;
            while (start_pos < end_pos) {
                probes++;
                if (key[cur_pos] < qp) start_pos = cur_pos; else end_pos = cur_pos - 1;
                cur_pos = (start_pos + end_pos + 2) / 2;
            }
            int left = start_pos - a.T + 1;
            int right = left + a.T;
            int cur = next_window(key, n, a.T, left, right, qp);
            const float pr = window_priority(key, n, a.T, cur, qp);
            s_left[i] = left; s_right[i] = right; s_cur[i] = cur; s_prio[i] = pr; s_qp[i] = qp;
        }
        __syncthreads();

        const int64_t bound = (int64_t)n * a.L * a.T;     // :458
        int64_t kk = 0, c0 = 0;
        unsigned long long visited = 0, ncand = 0, steps = 0;
        int tk_count = 0;                 // entries in `top`
        unsigned long long tk_max = 0;    // largest packed entry once full
        int tk_maxslot = 0;

        while (kk < bound) {
            bool any = false;
            for (int m = 0; m < a.M; m++) {
                // first strict minimum of the L priorities (:466-478)
                uint32_t best = 0x7f800000u;   // +inf: an exhausted simple index never wins
                int best_h = 0x7fffffff;
                for (int h = lane; h < a.L; h += kWave) {
                    const uint32_t p = __builtin_bit_cast(uint32_t, s_prio[m * a.L + h]);
                    if (p < best) { best = p; best_h = h; }
                }
                const uint32_t wbest = wave_min_u32(best);
                if (wbest >= 0x7f800000u) continue;
                const int top_h = (int)wave_min_u32(best == wbest ? (uint32_t)best_h : 0x7fffffffu);
                any = true;
                const int i = m * a.L + top_h;
                const int position = s_cur[i];
                const int32_t* ids = a.sids + (int64_t)i * a.N + off;
                uint32_t* mcnt = cnt + (size_t)m * y.wpc;

                for (int t0 = 0; t0 < a.T; t0 += kWave) {     // :487-562
                    const int t = t0 + lane;
                    const int cur_index = position + t;
                    const bool valid = t < a.T && cur_index >= 0 && cur_index < n;
                    int pt = -1;
                    bool promoted = false;
                    if (valid) {
                        pt = ids[cur_index];
                        const uint32_t local = (uint32_t)(pt - off);
                        const uint32_t sh = (local & ((1u << fshift) - 1u)) * y.cbits;
                        const uint32_t old = atomicAdd(&mcnt[local >> fshift], 1u << sh);
                        if (((old >> sh) & cmask) + 1u == (uint32_t)a.L) {
                            const uint32_t bit = 1u << (local & 31);
                            promoted = (atomicOr(&seen[local >> 5], bit) & bit) == 0;
                        }
                    }
                    visited += __popcll(__ballot(valid));
                    unsigned long long pm = __ballot(promoted);
                    while (pm) {
                        const int src = __ffsll((long long)pm) - 1;
                        pm &= pm - 1;
                        const int cpt = __shfl(pt, src, kWave);
                        uint32_t score;
                        if (a.blind) {
                            score = (uint32_t)kk;     // (:498-505: recorded, no distance)
                        } else {
                            // exact distance (:36-44), row read by the whole wavefront
                            const float* const rows1[1] = {a.data + (int64_t)cpt * a.dim};
                            float dist1[1];
                            wave_row_dists<1>(rows1, s_q, a.dim, rows_vec4(a.data, a.dim), dist1);
                            score = __builtin_bit_cast(uint32_t, dist1[0]);
                        }
                        const unsigned long long e = ((unsigned long long)score << 32) | (uint32_t)cpt;
                        ncand++;
                        if (t0 + src == 0) c0++;          // only lane 0's promotions count (:413, :598)
                        if (a.dense) {
                            // every candidate is kept: its score goes to its own cell of the query's row
                            if (lane == 0)
                                a.dense[(int64_t)qi * a.N + cpt] =
                                    a.blind ? (float)score : __builtin_bit_cast(float, score);
                        } else if (tk_count < a.kcap) {
                            if (lane == 0) top[tk_count] = e;
                            if (tk_count == 0 || e > tk_max) { tk_max = e; tk_maxslot = tk_count; }
                            tk_count++;
                        } else if (e < tk_max) {
                            if (lane == 0) top[tk_maxslot] = e;
                            __syncthreads();
                            if (!y.topk_bytes) __threadfence();
                            unsigned long long mx = 0;
                            for (int j = lane; j < a.kcap; j += kWave) {
                                const unsigned long long v = top[j];
                                if (v > mx) mx = v;
                            }
                            mx = wave_max_u64(mx);
                            int slot = 0x7fffffff;
                            for (int j = lane; j < a.kcap; j += kWave)
                                if (top[j] == mx) slot = min(slot, j);
                            tk_max = mx;
                            tk_maxslot = (int)wave_min_u32((uint32_t)slot);
                        }
                    }
                }
                __syncthreads();
                if (lane == 0) {        // :566-591
                    const float* key = a.skeys + (int64_t)i * a.N + off;
                    int left = s_left[i], right = s_right[i];
                    const float qp = s_qp[i];
                    int cur = next_window(key, n, a.T, left, right, qp);
                    const float pr = window_priority(key, n, a.T, cur, qp);
                    s_left[i] = left; s_right[i] = right; s_cur[i] = cur; s_prio[i] = pr;
                }
                __syncthreads();
            }
            steps++;
            if (c0 >= a.k_stop && (kk + 1 >= a.stop_at || c0 >= a.max_cand)) break;   // :598-607
            if (!any) break;   // every simple index exhausted: nothing can change any more
            kk++;
        }

        __syncthreads();
        if (!y.topk_bytes) __threadfence();
        for (int j = lane; j < (a.dense ? 0 : a.kcap); j += kWave) {
            const unsigned long long v = j < tk_count ? top[j] : ~0ull;
            part_out[j] = v;
        }
        if (a.counters) {
            for (int o = 32; o > 0; o >>= 1) probes += __shfl_xor(probes, o, kWave);
            if (lane == 0) {
                atomicAdd(&a.counters[(int64_t)qi * 4 + 0], visited);
                atomicAdd(&a.counters[(int64_t)qi * 4 + 1], ncand);
                atomicAdd(&a.counters[(int64_t)qi * 4 + 2], probes);
                atomicAdd(&a.counters[(int64_t)qi * 4 + 3], steps);
            }
        }
    }
}

// k best of the B*kcap per-partition results of one query (get_top_candidates,
// src/dci_cuda_kernel.cu:691-701): repeated LDS bitonic sorts of the running
// best k plus as many new entries as fit.
__global__ __launch_bounds__(kMergeThreads) void merge_topk_kernel(QueryArgs a, int cap) {
    extern __shared__ unsigned long long buf[];
    const int qi = blockIdx.x;
    const unsigned long long* src = a.part + (int64_t)qi * a.B * a.kcap;
    const int64_t total = (int64_t)a.B * a.kcap;
    const int keep = a.k < cap ? a.k : cap;   // host guarantees k <= cap / 2
    const int room = cap - keep;
    for (int j = threadIdx.x; j < keep; j += blockDim.x) buf[j] = ~0ull;
    for (int64_t p = 0; p < total; p += room) {
        const int m = (int)min((int64_t)room, total - p);
        __syncthreads();
        for (int j = threadIdx.x; j < room; j += blockDim.x)
            buf[keep + j] = j < m ? src[p + j] : ~0ull;
        bitonic_sort_u64(buf, cap);
    }
    __syncthreads();
    for (int j = threadIdx.x; j < a.k; j += blockDim.x) {
        const unsigned long long v = buf[j];
        const bool empty = v == ~0ull;
        a.out_ids[(int64_t)qi * a.k + j] = empty ? -1 : (int32_t)(uint32_t)v;
        if (a.out_dists)
            a.out_dists[(int64_t)qi * a.k + j] =
                empty ? __builtin_inff()
                      : (a.blind ? (float)(uint32_t)(v >> 32) : __builtin_bit_cast(float, (uint32_t)(v >> 32)));
    }
}

// Clears n 64-bit words at p and also_n 32-bit words at `also` (either may be null / 0).
__global__ void zero_u64_kernel(unsigned long long* p, int64_t n, uint32_t* also, int also_n) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += stride) p[e] = 0;
    if (also && blockIdx.x == 0 && (int)threadIdx.x < also_n) also[threadIdx.x] = 0;
}

// Words of the merge's sort buffer: room for the k best plus at least as many new entries, and
// no more than the per-partition lists hold in all (a sort of 2048 words for 590 entries would
// spend most of its stages on padding).
int merge_cap(int k, int64_t total) {
    int cap = 2048;
    while (cap < 2 * k) cap <<= 1;
    int need = 64;
    while ((int64_t)need < (int64_t)k + total && need < cap) need <<= 1;
    return need < cap ? need : cap;
}

}  // namespace

// The traversal and merge kernels may use all of a CU's LDS.
static int allow_full_lds() {
    static DeviceOnce once;
    return once.run([]() -> int {
        DCIH_HIP(hipFuncSetAttribute((const void*)traverse_kernel<true>,
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds));
        DCIH_HIP(hipFuncSetAttribute((const void*)traverse_kernel<false>,
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds));
        DCIH_HIP(hipFuncSetAttribute((const void*)merge_topk_kernel,
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds));
        return 0;
    });
}

int zero_words64(void* d_p, int64_t n, hipStream_t s) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(zero_u64_kernel, dim3((unsigned)max((int64_t)1, min((int64_t)1024, (n + 255) / 256))),
                       dim3(256), 0, s, (unsigned long long*)d_p, n, (uint32_t*)nullptr, 0);
    DCIH_HIP(hipGetLastError());
    return 0;
}

size_t query_part_bytes(const QueryArgs& a) {
    return (size_t)a.nq * a.B * a.kcap * sizeof(unsigned long long);
}

static int64_t traverse_grid(const QueryArgs& a, const Layout& y) {
    const int64_t items = (int64_t)a.nq * a.B;
    if (y.lds_counters) return min(items, step_grid_cap());   // the kernel strides over its items
    return min(items, (int64_t)kMaxSlots);
}

size_t query_gscratch_bytes(const QueryArgs& a) {
    const Layout y = make_layout(a);
    if (y.lds_counters) return 0;
    return (size_t)traverse_grid(a, y) * (size_t)y.counter_words * 4;
}

int query(const QueryArgs& a_in, hipStream_t s, hipEvent_t* ev, bool* ran) {
    QueryArgs a = a_in;
    if (a.nq <= 0) return 0;
    if (a.k > 8192)
        return fail(-4, a.blind ? "query: more than 8192 blind candidates per query are not supported"
                                : "query: num_neighbours above 8192 is not supported");
    if (a.blind && (int64_t)a.L * (a.ppb + 2 * (int64_t)a.T) >= 0x7fffffffLL)
        return fail(-4, "query: blind querying needs step numbers that fit 31 bits");
    if ((int64_t)a.M * a.ppb * 8 > 0x7fffffffLL)
        return fail(-4, "query: partition too large for the visit counters; use a larger block_size");
    const Layout y = make_layout(a);
    if (y.lds_bytes > (size_t)kMaxLds)
        return fail(-4, "query: dim / num_indices / num_neighbours too large for LDS state");
    const bool can_block = block_traversal_supported(a, nullptr);
    const bool can_dense = dense_traversal_supported(a, nullptr);
    if (a.mode == 2 && !can_block)
        return fail(-4, "query: this shape does not fit the batch traversal kernel");
    if (a.mode == 3 && !can_dense)
        return fail(-4, "query: this shape does not fit the dense traversal kernel");
    // Left to choose: the stop rule needs k promotions by a window's first lane, which takes
    // about k * T promotions in all; from the number at which the dense kernel is the cheaper
    // one, every item goes straight to it (no hints needed: also a first call is routed right).
    // The step limit can ask for more: a traversal that must consume the fraction f of a
    // composite's windows before it may stop has by then promoted about f^L of the partition
    // (a point needs all L of its windows; nearby windows come first, so this is on the low
    // side), unless max_candidates first-lane promotions end it earlier.
    if (a.mode == 0 && can_dense && !a.blind && a.dense_min_promos > 0) {
        const double windows = (double)a.L * ((double)a.ppb / (double)a.T);
        const double f = fmin(1.0, (double)a.stop_at / fmax(1.0, windows));
        const double by_steps = fmin((double)a.ppb * pow(f, (double)a.L), (double)a.max_cand * (double)a.T);
        if (fmax((double)a.k_stop * (double)a.T, by_steps) >= (double)a.dense_min_promos) a.mode = 3;
    }
    const bool use_block = a.mode != 1 && a.mode != 3 && can_block;
    // the batch kernel hands items that need many promotions to the dense kernel
    if (!(use_block && a.mode == 0 && can_dense && a.dense_items && a.dense_min_promos > 0)) {
        if (a.mode != 3) a.dense_items = nullptr;
    }
    {
        const int rc = allow_full_lds();
        if (rc) return rc;
    }
    {   // zero the counters and the list lengths with a kernel (safe under graph capture);
        // the dense lists' lengths follow the hand-over list's
        const int64_t cells = a.counters ? (int64_t)a.nq * 4 : 0;
        hipLaunchKernelGGL(zero_u64_kernel, dim3((unsigned)max((int64_t)1, min((int64_t)1024, (cells + 255) / 256))),
                           dim3(256), 0, s, a.counters, cells, a.redo_count, kListCountWords);
    }
    if (ev) (void)hipEventRecord(ev[0], s);
    a.item_list = nullptr;
    a.item_count = nullptr;
    if (use_block || a.mode == 3) {
        if (use_block) {
            if (a.rpos_ready && !*a.rpos_ready) {      // the first batch traversal over this index
                const int rc = fill_positions_by_first(a.sids, a.inv, const_cast<uint16_t*>(a.rpos), a.N, a.M, a.L, s);
                if (rc) return rc;
                *a.rpos_ready = 1;
            }
            const int rc = query_block(a, s);
            if (rc) return rc;
            if (ev) (void)hipEventRecord(ev[1], s);
            if (ran) ran[0] = true;
        }
        if (a.mode == 3 || a.dense_items) {
            const int rc = query_dense_items(a, s);
            if (rc) return rc;
            if (ev) (void)hipEventRecord(ev[2], s);
            if (ran) ran[1] = true;
        }
        // whatever those kernels handed back goes through the step-by-step kernel
        a.item_list = a.redo_items;
        a.item_count = a.redo_count;
        if (y.lds_counters) {
            const int64_t grid = min((int64_t)a.nq * a.B, (int64_t)1024);
            hipLaunchKernelGGL(traverse_kernel<true>, dim3((unsigned)grid), dim3(kWave), y.lds_bytes, s, a, y);
        } else {      // partitions whose visit counters do not fit LDS: a slice of global scratch per workgroup
            if (!a.gscratch) return fail(-1, "query: counter scratch missing");
            const int64_t grid = min(traverse_grid(a, y), (int64_t)1024);
            hipLaunchKernelGGL(traverse_kernel<false>, dim3((unsigned)grid), dim3(kWave), y.lds_bytes, s, a, y);
        }
    } else {
        const int64_t grid = traverse_grid(a, y);
        if (y.lds_counters) {
            hipLaunchKernelGGL(traverse_kernel<true>, dim3((unsigned)grid), dim3(kWave), y.lds_bytes, s, a, y);
        } else {
            if (!a.gscratch) return fail(-1, "query: counter scratch missing");
            hipLaunchKernelGGL(traverse_kernel<false>, dim3((unsigned)grid), dim3(kWave), y.lds_bytes, s, a, y);
        }
    }
    DCIH_HIP(hipGetLastError());
    if (ev) (void)hipEventRecord(ev[3], s);
    const int cap = merge_cap(a.k, (int64_t)a.B * a.kcap);
    hipLaunchKernelGGL(merge_topk_kernel, dim3((unsigned)a.nq), dim3(kMergeThreads),
                       (size_t)cap * sizeof(unsigned long long), s, a, cap);
    if (ev) (void)hipEventRecord(ev[4], s);
    DCIH_HIP(hipGetLastError());
    return 0;
}

int query_dense(const QueryArgs& a_in, const float* d_dirs, void* ws, int chunk, hipStream_t s) {
    if (a_in.nq <= 0) return 0;
    const int I = a_in.M * a_in.L;
    if ((int64_t)a_in.M * a_in.ppb * 8 > 0x7fffffffLL)
        return fail(-4, "query: partition too large for the visit counters; use a larger block_size");
    // blind scores are step numbers stored as floats: they must stay exact
    if (a_in.blind && (int64_t)a_in.L * (a_in.ppb + 2 * (int64_t)a_in.T) >= (1 << 24))
        return fail(-4, "query: this many blind results need step numbers below 2^24; use a larger block_size");
    {
        const int rc = allow_full_lds();
        if (rc) return rc;
    }
    const size_t qp_bytes = ((size_t)I * chunk * sizeof(float) + 255) & ~(size_t)255;
    float* d_qproj = (float*)ws;
    void* ws_rank = (char*)ws + qp_bytes;
    for (int q0 = 0; q0 < a_in.nq; q0 += chunk) {
        QueryArgs a = a_in;             // this chunk's queries as a query batch of their own
        a.nq = min(chunk, a_in.nq - q0);
        a.query = a_in.query + (int64_t)q0 * a.dim;
        a.qproj = d_qproj;
        a.counters = a_in.counters ? a_in.counters + (int64_t)q0 * 4 : nullptr;
        a.kcap = 1;                     // no per-partition lists
        a.part = nullptr;
        a.item_list = nullptr;
        a.item_count = nullptr;
        a.dense = rank_rows_input(ws_rank);
        int rc = project(d_dirs, I, a.query, a.nq, a.dim, d_qproj, a.nq, s);
        if (rc) return rc;
        rc = fill_rows(a.dense, (int64_t)a.nq * a.N, __builtin_inff(), s);
        if (rc) return rc;
        const Layout y = make_layout(a);
        if (y.lds_bytes > (size_t)kMaxLds)
            return fail(-4, "query: dim / num_indices too large for LDS state");
        const int64_t cells = a.counters ? (int64_t)a.nq * 4 : 0;
        hipLaunchKernelGGL(zero_u64_kernel, dim3((unsigned)max((int64_t)1, min((int64_t)1024, (cells + 255) / 256))),
                           dim3(256), 0, s, a.counters, cells, (uint32_t*)nullptr, 0);
        const int64_t grid = traverse_grid(a, y);
        if (y.lds_counters) {
            hipLaunchKernelGGL(traverse_kernel<true>, dim3((unsigned)grid), dim3(kWave), y.lds_bytes, s, a, y);
        } else {
            if (!a.gscratch) return fail(-1, "query: counter scratch missing");
            hipLaunchKernelGGL(traverse_kernel<false>, dim3((unsigned)grid), dim3(kWave), y.lds_bytes, s, a, y);
        }
        DCIH_HIP(hipGetLastError());
        rc = rank_rows(ws_rank, chunk, a.nq, a.N, a_in.k, true, a_in.out_ids + (int64_t)q0 * a_in.k,
                       a_in.out_dists ? a_in.out_dists + (int64_t)q0 * a_in.k : nullptr, s);
        if (rc) return rc;
    }
    return 0;
}

}  // namespace dcih
