// Projection of rows onto directions: out[r][c] = sum_k rows[c][k] * dirs[r][k].
//
// Stands in for the cuBLAS SGEMM the reference issues from matmul_device
// (src/util_kernel.cu:45-80) for the build (src/dci_cuda_kernel.cu:167-169,
// result [num_indices][num_points]) and for the queries (:802-803).
//
// The contraction is thin (a few tens of directions), so every row is read
// from HBM exactly once, staged through LDS in 16-column chunks with coalesced
// 16-byte loads, and each thread keeps one row's dot products with up to 32
// directions in registers.  Direction values are wave-uniform and are fetched
// through the scalar cache.  Output stores are coalesced along the row index.
// Each dot product is one sequential fp32 FMA chain over k = 0..dim-1, so a
// vector gives bit-identical projections whether it is indexed or queried.
#include "common.h"
#include "kernels.h"

namespace dcih {

constexpr int kProjRows = 256;    // rows per workgroup = threads per workgroup
constexpr int kProjChunk = 16;    // columns staged per LDS tile
constexpr int kProjStride = 20;   // LDS row pitch in floats (16 B aligned, conflict-free b128 reads)
constexpr int kProjTpr = kProjChunk / 4;          // threads that cover one row's chunk with float4 loads
constexpr int kProjRpp = kProjRows / kProjTpr;    // rows covered per pass of the workgroup

template <int RT>
__global__ __launch_bounds__(kProjRows) void project_kernel(
    const float* __restrict__ dirs, int r0, const float* __restrict__ rows,
    int64_t num_rows, int dim, int vec4_ok, float* __restrict__ out) {
    __shared__ float tile[kProjRows * kProjStride];
    const int tid = threadIdx.x;
    const int64_t row0 = (int64_t)blockIdx.x * kProjRows;
    const int rows_here = (int)min((int64_t)kProjRows, num_rows - row0);
    const bool vec4 = vec4_ok != 0;

    float acc[RT];
#pragma unroll
    for (int r = 0; r < RT; r++) acc[r] = 0.0f;

    // The next chunk's global reads are issued into registers before the current
    // chunk is consumed, so their latency hides behind the FMAs of this workgroup
    // instead of leaving its waves parked at the barrier.
    const int kq = (tid % kProjTpr) * 4;      // float4 path: kProjTpr threads cover one row's chunk
    float4 pre[kProjRows / kProjRpp];
    auto prefetch = [&](int k0) {
        const int kc = min(kProjChunk, dim - k0);
#pragma unroll
        for (int j = 0; j < kProjRows / kProjRpp; j++) {
            const int row = tid / kProjTpr + kProjRpp * j;
            pre[j] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (row < rows_here && kq < kc)
                pre[j] = *reinterpret_cast<const float4*>(rows + (row0 + row) * dim + k0 + kq);
        }
    };
    if (vec4) prefetch(0);
    for (int k0 = 0; k0 < dim; k0 += kProjChunk) {
        const int kc = min(kProjChunk, dim - k0);
        __syncthreads();
        if (vec4) {
#pragma unroll
            for (int j = 0; j < kProjRows / kProjRpp; j++)
                *reinterpret_cast<float4*>(&tile[(tid / kProjTpr + kProjRpp * j) * kProjStride + kq]) = pre[j];
            if (k0 + kProjChunk < dim) prefetch(k0 + kProjChunk);
        } else {
            for (int e = tid; e < kProjRows * kProjChunk; e += kProjRows) {
                const int row = e / kProjChunk, kk = e % kProjChunk;
                float v = 0.f;
                if (row < rows_here && kk < kc) v = rows[(row0 + row) * dim + k0 + kk];
                tile[row * kProjStride + kk] = v;
            }
        }
        __syncthreads();
        const float* dk = dirs + (int64_t)r0 * dim + k0;
        if (kc == kProjChunk) {
#pragma unroll
            for (int kk = 0; kk < kProjChunk; kk += 4) {
                const float4 x = *reinterpret_cast<const float4*>(&tile[tid * kProjStride + kk]);
#pragma unroll
                for (int r = 0; r < RT; r++) {
                    const float* d = dk + (int64_t)r * dim + kk;
                    acc[r] = __builtin_fmaf(x.x, d[0], acc[r]);
                    acc[r] = __builtin_fmaf(x.y, d[1], acc[r]);
                    acc[r] = __builtin_fmaf(x.z, d[2], acc[r]);
                    acc[r] = __builtin_fmaf(x.w, d[3], acc[r]);
                }
            }
        } else {
            for (int kk = 0; kk < kc; kk++) {
                const float x = tile[tid * kProjStride + kk];
#pragma unroll
                for (int r = 0; r < RT; r++)
                    acc[r] = __builtin_fmaf(x, dk[(int64_t)r * dim + kk], acc[r]);
            }
        }
    }
    if (tid < rows_here) {
#pragma unroll
        for (int r = 0; r < RT; r++)
            out[(int64_t)(r0 + r) * num_rows + row0 + tid] = acc[r] + 0.0f;  // -0.0 -> +0.0
    }
}

template <int RT>
static void launch_project(const float* dirs, int r0, const float* rows,
                           int64_t num_rows, int dim, float* out, hipStream_t s) {
    const int64_t blocks = (num_rows + kProjRows - 1) / kProjRows;
    // float4 loads need 16-byte aligned row starts
    const int vec4_ok = (dim & 3) == 0 && (reinterpret_cast<uintptr_t>(rows) & 15) == 0;
    hipLaunchKernelGGL(project_kernel<RT>, dim3((unsigned)blocks), dim3(kProjRows), 0, s,
                       dirs, r0, rows, num_rows, dim, vec4_ok, out);
}

template <int RT>
static void dispatch_tail(int rt, const float* dirs, int r0, const float* rows,
                          int64_t num_rows, int dim, float* out, hipStream_t s) {
    if constexpr (RT >= 1) {
        if (rt == RT) launch_project<RT>(dirs, r0, rows, num_rows, dim, out, s);
        else dispatch_tail<RT - 1>(rt, dirs, r0, rows, num_rows, dim, out, s);
    }
}

int project(const float* d_dirs, int num_dirs, const float* d_rows, int64_t num_rows,
            int dim, float* d_out, hipStream_t s) {
    if (num_rows <= 0 || num_dirs <= 0) return 0;
    if ((num_rows + kProjRows - 1) / kProjRows > 0x7fffffffLL)
        return fail(-1, "project: too many rows for one launch");
    int r0 = 0;
    while (num_dirs - r0 > 0) {
        const int rt = min(32, num_dirs - r0);
        dispatch_tail<32>(rt, d_dirs, r0, d_rows, num_rows, dim, d_out, s);
        r0 += rt;
    }
    DCIH_HIP(hipGetLastError());
    return 0;
}

}  // namespace dcih
