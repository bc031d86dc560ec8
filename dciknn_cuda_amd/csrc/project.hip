// Projection of rows onto directions: out[r][c] = sum_k rows[c][k] * dirs[r][k].
//
// Stands in for the cuBLAS SGEMM the reference issues from matmul_device
// (src/util_kernel.cu:45-80) for the build (src/dci_cuda_kernel.cu:167-169,
// result [num_indices][num_points]) and for the queries (:802-803).
//
// The contraction is thin (a few tens of directions), so every row is read
// from HBM exactly once, a 128-byte line at a time, staged through a
// wavefront-private LDS tile with coalesced 16-byte loads, and each lane keeps
// one row's dot products with up to 32 directions in registers.  Direction
// values are wave-uniform and are fetched through the scalar cache.  Output stores are coalesced along the row index.
// Each dot product is one sequential fp32 FMA chain over k = 0..dim-1, so a
// vector gives bit-identical projections whether it is indexed or queried.
#include "common.h"
#include "kernels.h"

namespace dcih {

// Direction values are read through the constant address space: the address is
// wave-uniform and the memory does not change while the kernel runs, so every
// read becomes a scalar-cache load and the FMAs take their operand from SGPRs.
typedef const __attribute__((address_space(4))) float cfloat;
typedef float v4f __attribute__((ext_vector_type(4)));   // plain vector: stays in registers

constexpr int kProjRows = 64;     // rows per workgroup = one wavefront, so no workgroup barrier is ever waited on
constexpr int kProjChunk = 32;    // columns staged per LDS tile: one 128-byte line of every row
constexpr int kProjStride = 36;   // LDS row pitch in floats (16 B aligned, conflict-free b128 reads)
constexpr int kProjTpr = kProjChunk / 4;          // lanes that cover one row's chunk with 16-byte loads
constexpr int kProjRpp = kProjRows / kProjTpr;    // rows covered per load instruction of the wavefront
constexpr int kProjLoads = kProjRows / kProjRpp;  // 16-byte loads per lane and chunk

// Fast path: dim % 4 == 0, 16-byte aligned rows, at least kProjRows rows.  The
// workgroup is a single wavefront: the tile is private to it, __syncthreads()
// only orders its own LDS traffic and costs no barrier wait.  The last
// workgroup is shifted back to end on the last row; the rows it shares with its
// neighbour are computed twice and stored twice with identical bits.
template <int RT>
__global__ __launch_bounds__(kProjRows) void project_kernel(
    const float* __restrict__ dirs, int r0, const float* __restrict__ rows,
    int64_t num_rows, int dim, float* __restrict__ out, int64_t out_stride) {
    __shared__ float tile[kProjRows * kProjStride];
    const int tid = threadIdx.x;
    const int64_t row0 = min((int64_t)blockIdx.x * kProjRows, num_rows - kProjRows);

    float acc[RT];
#pragma unroll
    for (int r = 0; r < RT; r++) acc[r] = 0.0f;

    // Eight lanes read one row's 128-byte line, so a line is fetched from HBM
    // once, and the whole next chunk is in flight in registers while the current
    // one is consumed.  Rows are read exactly once, hence the streaming
    // (nontemporal) loads.  Columns past the end repeat the last valid 16 bytes;
    // the tile columns they fill are never read.
    const int kq = (tid % kProjTpr) * 4;
    const float* lane_rows = rows + (row0 + tid / kProjTpr) * dim;
    const int64_t pass_pitch = (int64_t)kProjRpp * dim;
    float* lane_tile = &tile[(tid / kProjTpr) * kProjStride + kq];
    v4f pre[kProjLoads];
    auto prefetch = [&](int k0) {
        const float* p = lane_rows + min(k0 + kq, dim - 4);
#pragma unroll
        for (int j = 0; j < kProjLoads; j++)
            pre[j] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(p + j * pass_pitch));
    };
    prefetch(0);
#pragma unroll 1
    for (int k0 = 0; k0 < dim; k0 += kProjChunk) {
        const int kc = min(kProjChunk, dim - k0);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < kProjLoads; j++)
            *reinterpret_cast<v4f*>(lane_tile + j * kProjRpp * kProjStride) = pre[j];
        if (k0 + kProjChunk < dim) prefetch(k0 + kProjChunk);
        __syncthreads();
        const cfloat* dk = (const cfloat*)(uintptr_t)(dirs + (int64_t)r0 * dim + k0);
        if (kc == kProjChunk) {
            // The chunk is consumed in steps of 16 columns x 2 directions: one
            // 64-byte scalar load per direction feeds 16 FMAs of that direction's
            // chain, k ascending.  Scalar loads return out of order, so a wait
            // drains all of them; each step therefore waits for its own operands,
            // issues the next step's loads and then computes, which gives those
            // loads the step's 32 FMAs to land.
            constexpr int NB = (RT + 1) / 2;              // direction pairs
            constexpr int NS = NB * (kProjChunk / 16);    // steps per chunk
            float x[16], dcur[2][16];
            auto load_x = [&](float (&v)[16], int kh) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const v4f t = *reinterpret_cast<const v4f*>(&tile[tid * kProjStride + kh + 4 * q]);
                    v[4 * q] = t.x; v[4 * q + 1] = t.y; v[4 * q + 2] = t.z; v[4 * q + 3] = t.w;
                }
            };
            auto load_d = [&](float (&d)[2][16], int step) {
                const int kh = (step / NB) * 16, rb = (step % NB) * 2;
#pragma unroll
                for (int i = 0; i < 2; i++)
                    if (rb + i < RT) {
                        const cfloat* p = dk + (int64_t)(rb + i) * dim + kh;
#pragma unroll
                        for (int q = 0; q < 16; q++) d[i][q] = p[q];
                    }
            };
            load_x(x, 0);
            load_d(dcur, 0);
#pragma unroll
            for (int step = 0; step < NS; step++) {
                const int rb = (step % NB) * 2;
                float dnext[2][16], xnext[16];
                // the first FMA makes the wait for this step's operands land here,
                // ahead of the loads issued for the next step
                acc[rb] = __builtin_fmaf(x[0], dcur[0][0], acc[rb]);
                __builtin_amdgcn_sched_barrier(0);
                if (step + 1 < NS) {
                    load_d(dnext, step + 1);
                    if ((step + 1) % NB == 0) load_x(xnext, ((step + 1) / NB) * 16);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < 2; i++)
                    if (rb + i < RT) {
#pragma unroll
                        for (int q = (i == 0 ? 1 : 0); q < 16; q++)
                            acc[rb + i] = __builtin_fmaf(x[q], dcur[i][q], acc[rb + i]);
                    }
                __builtin_amdgcn_sched_barrier(0);
                if (step + 1 < NS) {
#pragma unroll
                    for (int i = 0; i < 2; i++)
#pragma unroll
                        for (int q = 0; q < 16; q++) dcur[i][q] = dnext[i][q];
                    if ((step + 1) % NB == 0) {
#pragma unroll
                        for (int q = 0; q < 16; q++) x[q] = xnext[q];
                    }
                }
            }
        } else {
#pragma unroll 1
            for (int kk = 0; kk < kc; kk++) {
                const float x = tile[tid * kProjStride + kk];
#pragma unroll
                for (int r = 0; r < RT; r++)
                    acc[r] = __builtin_fmaf(x, dk[(int64_t)r * dim + kk], acc[r]);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < RT; r++)
        out[(int64_t)(r0 + r) * out_stride + row0 + tid] = acc[r] + 0.0f;  // -0.0 -> +0.0
}

// Any shape: one row per thread straight from global memory, same FMA order.
template <int RT>
__global__ __launch_bounds__(256) void project_generic_kernel(
    const float* __restrict__ dirs, int r0, const float* __restrict__ rows,
    int64_t num_rows, int dim, float* __restrict__ out, int64_t out_stride) {
    const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (row >= num_rows) return;
    float acc[RT];
#pragma unroll
    for (int r = 0; r < RT; r++) acc[r] = 0.0f;
    const float* x = rows + row * dim;
    const cfloat* dk = (const cfloat*)(uintptr_t)(dirs + (int64_t)r0 * dim);
#pragma unroll 1
    for (int k = 0; k < dim; k++) {
        const float v = x[k];
#pragma unroll
        for (int r = 0; r < RT; r++) acc[r] = __builtin_fmaf(v, dk[(int64_t)r * dim + k], acc[r]);
    }
#pragma unroll
    for (int r = 0; r < RT; r++) out[(int64_t)(r0 + r) * out_stride + row] = acc[r] + 0.0f;
}

template <int RT>
static void launch_project(const float* dirs, int r0, const float* rows,
                           int64_t num_rows, int dim, float* out, int64_t out_stride, hipStream_t s) {
    // float4 loads need 16-byte aligned row starts
    const bool fast = (dim & 3) == 0 && (reinterpret_cast<uintptr_t>(rows) & 15) == 0 &&
                      num_rows >= kProjRows;
    if (fast) {
        const int64_t blocks = (num_rows + kProjRows - 1) / kProjRows;
        hipLaunchKernelGGL(project_kernel<RT>, dim3((unsigned)blocks), dim3(kProjRows), 0, s,
                           dirs, r0, rows, num_rows, dim, out, out_stride);
    } else {
        const int64_t blocks = (num_rows + 255) / 256;
        hipLaunchKernelGGL(project_generic_kernel<RT>, dim3((unsigned)blocks), dim3(256), 0, s,
                           dirs, r0, rows, num_rows, dim, out, out_stride);
    }
}

template <int RT>
static void dispatch_tail(int rt, const float* dirs, int r0, const float* rows,
                          int64_t num_rows, int dim, float* out, int64_t out_stride, hipStream_t s) {
    if constexpr (RT >= 1) {
        if (rt == RT) launch_project<RT>(dirs, r0, rows, num_rows, dim, out, out_stride, s);
        else dispatch_tail<RT - 1>(rt, dirs, r0, rows, num_rows, dim, out, out_stride, s);
    }
}

int project(const float* d_dirs, int num_dirs, const float* d_rows, int64_t num_rows,
            int dim, float* d_out, int64_t out_stride, hipStream_t s) {
    if (num_rows <= 0 || num_dirs <= 0) return 0;
    if (out_stride < num_rows) return fail(-1, "project: output rows overlap");
    if ((num_rows + kProjRows - 1) / kProjRows > 0x7fffffffLL)
        return fail(-1, "project: too many rows for one launch");
    int r0 = 0;
    while (num_dirs - r0 > 0) {
        const int rt = min(32, num_dirs - r0);
        dispatch_tail<32>(rt, d_dirs, r0, d_rows, num_rows, dim, d_out, out_stride, s);
        r0 += rt;
    }
    DCIH_HIP(hipGetLastError());
    return 0;
}

}  // namespace dcih
