// Full ranking: num_neighbours beyond what the traversal's top-k tables hold.
//
// dci_query (src/dci_cuda_kernel.cu:777-875) with num_neighbours up to the
// number of indexed points, which is what dciknn_cuda/core.py:84-85 asks for
// when the caller leaves num_neighbours at -1.  The stop rule (:598-607) needs
// c0 >= num_neighbours, and c0 counts promotions inside ONE partition, so with
// num_neighbours above the points per partition no partition ever stops early:
// every window of every simple index is consumed (the loop bound of :458 is
// never below the number of windows), every point is promoted, and the result
// is the num_neighbours closest of ALL points by (distance, id).  That closed
// form is computed here directly: exact distances of every (query, point) pair,
// one sort per query with the build's segmented sort, first num_neighbours
// columns copied out.  The traversal counters have closed forms too: every
// index entry is visited once, every point is a candidate, and the outer steps
// follow from the window counts on either side of the positioning search.
#include "common.h"
#include "kernels.h"

namespace dcih {

namespace {

typedef const __attribute__((address_space(4))) float cfloat;

constexpr int kExThreads = 256;
constexpr int kExQueries = 8;     // queries a thread carries for its point

// out[q][row] = || data[row] - query[q] ||, the squares summed one after the
// other in index order like compute_dist_device (src/dci_cuda_kernel.cu:36-44);
// multiply and add rounded separately, as a CPU build of that loop does.
__global__ __launch_bounds__(kExThreads) void exact_dists_kernel(
    const float* __restrict__ data, int64_t N, int dim, const float* __restrict__ query, int nq,
    float* __restrict__ out) {
#pragma clang fp contract(off)     // no fused multiply-add: product and sum are rounded separately
    const int64_t row = (int64_t)blockIdx.x * kExThreads + threadIdx.x;
    if (row >= N) return;
    const int q0 = blockIdx.y * kExQueries;
    float acc[kExQueries];
    const cfloat* qv[kExQueries];     // wave-uniform: read through the scalar cache
#pragma unroll
    for (int j = 0; j < kExQueries; j++) {
        acc[j] = 0.0f;
        qv[j] = (const cfloat*)(uintptr_t)(query + (int64_t)min(q0 + j, nq - 1) * dim);
    }
    const float* x = data + row * dim;
#pragma unroll 1
    for (int k = 0; k < dim; k++) {
        const float v = x[k];
#pragma unroll
        for (int j = 0; j < kExQueries; j++) {
            const float d = v - qv[j][k];
            acc[j] = acc[j] + d * d;
        }
    }
#pragma unroll
    for (int j = 0; j < kExQueries; j++)
        // (the square root taken in double and rounded once more is the correctly rounded
        //  single-precision root: 53 bits are more than twice 24 plus two)
        if (q0 + j < nq) out[(int64_t)(q0 + j) * N + row] = (float)sqrt((double)acc[j]);
}

// The first k columns of every sorted row.  Columns past the end of a row and, when
// asked, entries whose value is +inf (points that never became candidates) read as
// "no result": id -1, +inf.
__global__ __launch_bounds__(256) void take_columns_kernel(
    const float* __restrict__ skeys, const int32_t* __restrict__ sids, int64_t N, int k,
    int inf_is_empty, int32_t* __restrict__ out_ids, float* __restrict__ out_vals) {
    const int q = blockIdx.y;
    for (int j = blockIdx.x * 256 + threadIdx.x; j < k; j += gridDim.x * 256) {
        const float v = j < N ? skeys[(int64_t)q * N + j] : __builtin_inff();
        const bool empty = j >= N || (inf_is_empty && v == __builtin_inff());
        out_ids[(int64_t)q * k + j] = empty ? -1 : sids[(int64_t)q * N + j];
        if (out_vals) out_vals[(int64_t)q * k + j] = v;
    }
}

__global__ void fill_f32_kernel(float* p, int64_t n, float v) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += stride) p[e] = v;
}

// Counters of a traversal that runs every partition dry, one wavefront per
// (query, partition): the positioning search (:279-318) gives p, the largest
// position with key < projection; the left stream then has ceil((p+1)/T)
// windows and the right one ceil((n+T-1 - (p+1))/T) (starts below n+T-1, :250-273);
// a composite needs as many steps as its L indices have windows, and the loop
// runs one idle step more unless its bound n*L*T (:458) ends it first.
__global__ __launch_bounds__(kWave) void exhaustive_counters_kernel(QueryArgs a) {
    const int lane = threadIdx.x;
    const int b = (int)(blockIdx.x % a.B);
    const int qi = (int)(blockIdx.x / a.B);
    const int64_t off = (int64_t)b * a.ppb;
    const int n = (int)min(a.N - off, a.ppb);
    if (n <= 0) return;
    unsigned long long probes = 0, maxw = 0;
    for (int m = 0; m < a.M; m++) {
        unsigned long long w = 0;
        for (int h = lane; h < a.L; h += kWave) {
            const int i = m * a.L + h;
            const float* key = a.skeys + (int64_t)i * a.N + off;
            const float qp = a.qproj[(int64_t)i * a.nq + qi];
            int start_pos = -1, end_pos = n - 1;
            int cur_pos = (start_pos + end_pos + 2) / 2;
            while (start_pos < end_pos) {
                probes++;
                if (key[cur_pos] < qp) start_pos = cur_pos; else end_pos = cur_pos - 1;
                cur_pos = (start_pos + end_pos + 2) / 2;
            }
            const int64_t p1 = (int64_t)start_pos + 1;
            const int64_t rem = (int64_t)n + a.T - 1 - p1;
            w += (unsigned long long)((p1 + a.T - 1) / a.T) +
                 (unsigned long long)(rem > 0 ? (rem + a.T - 1) / a.T : 0);
        }
        for (int o = kWave / 2; o > 0; o >>= 1) w += __shfl_xor(w, o, kWave);
        maxw = max(maxw, w);
    }
    for (int o = kWave / 2; o > 0; o >>= 1) probes += __shfl_xor(probes, o, kWave);
    if (lane == 0) {
        const unsigned long long bound = (unsigned long long)n * a.L * a.T;
        atomicAdd(&a.counters[(int64_t)qi * 4 + 0], (unsigned long long)n * a.M * a.L);
        atomicAdd(&a.counters[(int64_t)qi * 4 + 1], (unsigned long long)n);
        atomicAdd(&a.counters[(int64_t)qi * 4 + 2], probes);
        atomicAdd(&a.counters[(int64_t)qi * 4 + 3], min(bound, maxw + 1));
    }
}

__global__ void zero_counters_kernel(unsigned long long* p, int64_t n) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e < n) p[e] = 0;
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

}  // namespace

int exhaustive_chunk(int64_t N, int nq) {
    // 64 M (query, point) pairs at a time: 1.8 GB of scratch
    return (int)max((int64_t)1, min(min((int64_t)nq, (int64_t)32768), ((int64_t)1 << 26) / N));
}

size_t exhaustive_ws_bytes(int64_t N, int chunk) {
    const size_t cells = (size_t)chunk * (size_t)N;
    return 3 * align256(cells * 4) + align256(segsort_tmp_bytes(chunk, N, 1));
}

float* rank_rows_input(void* ws) { return (float*)ws; }

int fill_rows(float* d_rows, int64_t cells, float value, hipStream_t s) {
    hipLaunchKernelGGL(fill_f32_kernel, dim3((unsigned)min((int64_t)8192, (cells + 255) / 256)), dim3(256), 0, s,
                       d_rows, cells, value);
    DCIH_HIP(hipGetLastError());
    return 0;
}

int rank_rows(void* ws, int chunk, int rows, int64_t N, int k, bool inf_is_empty,
              int32_t* out_ids, float* out_vals, hipStream_t s) {
    const size_t cells = (size_t)chunk * (size_t)N;
    char* base = (char*)ws;
    float* d_in = (float*)base;
    float* d_sorted = (float*)(base + align256(cells * 4));
    int32_t* d_sids = (int32_t*)(base + 2 * align256(cells * 4));
    void* d_tmp = segsort_tmp_bytes(chunk, N, 1) ? (void*)(base + 3 * align256(cells * 4)) : nullptr;
    const int rc = segsort(d_in, N, rows, N, 1, d_sorted, d_sids, nullptr, nullptr, d_tmp, s);
    if (rc) return rc;
    hipLaunchKernelGGL(take_columns_kernel, dim3((unsigned)min(1024, (k + 255) / 256), (unsigned)rows),
                       dim3(256), 0, s, d_sorted, d_sids, N, k, inf_is_empty ? 1 : 0, out_ids, out_vals);
    DCIH_HIP(hipGetLastError());
    return 0;
}

int query_exhaustive(const QueryArgs& a, void* ws, int chunk, hipStream_t s) {
    if (a.nq <= 0) return 0;
    if ((a.N + kExThreads - 1) / kExThreads > 0x7fffffffLL || (int64_t)a.nq * a.B > 0x7fffffffLL)
        return fail(-4, "query: too many points for the full-ranking path");
    float* d_dist = rank_rows_input(ws);
    for (int q0 = 0; q0 < a.nq; q0 += chunk) {
        const int nqc = min(chunk, a.nq - q0);
        hipLaunchKernelGGL(exact_dists_kernel,
                           dim3((unsigned)((a.N + kExThreads - 1) / kExThreads),
                                (unsigned)((nqc + kExQueries - 1) / kExQueries)),
                           dim3(kExThreads), 0, s, a.data, a.N, a.dim,
                           a.query + (int64_t)q0 * a.dim, nqc, d_dist);
        DCIH_HIP(hipGetLastError());
        const int rc = rank_rows(ws, chunk, nqc, a.N, a.k, false, a.out_ids + (int64_t)q0 * a.k,
                                 a.out_dists + (int64_t)q0 * a.k, s);
        if (rc) return rc;
    }
    if (a.counters) {
        const int64_t cellsc = (int64_t)a.nq * 4;
        hipLaunchKernelGGL(zero_counters_kernel, dim3((unsigned)((cellsc + 255) / 256)), dim3(256), 0, s,
                           a.counters, cellsc);
        hipLaunchKernelGGL(exhaustive_counters_kernel, dim3((unsigned)((int64_t)a.nq * a.B)), dim3(kWave),
                           0, s, a);
        DCIH_HIP(hipGetLastError());
    }
    return 0;
}

}  // namespace dcih
