// Segmented sort of the projections: every (simple index, partition) slice of
// keys[num_indices][n] becomes (key, id) pairs ascending by key, ties by id.
//
// Stands in for copy_to_indices + sort_indices + mix_sort/quick_sort/
// insertion_sort (src/dci_cuda_kernel.cu:113-146,190-247), where each of
// block_size*thread_size threads quicksorts whole slices serially.
//
// Here a (key, position-in-slice) pair is one 64-bit word whose unsigned order
// is the wanted order, so a slice of up to kTileCap points is sorted by one
// workgroup entirely in LDS: one coalesced read of the keys, one coalesced
// write of the sorted keys and ids.  Longer slices are sorted tile by tile and
// the tiles are then merged pairwise in global memory (merge path), each pass
// doubling the run length.
#include "common.h"
#include "kernels.h"

namespace dcih {

constexpr int kTileCap = 16384;       // elements one workgroup sorts in LDS (128 KB)
constexpr int kMergeThreads = 256;
constexpr int kMergeItems = 8;
constexpr int kMergeChunk = kMergeThreads * kMergeItems;  // divides kTileCap

struct SegGeom {
    int64_t n;        // points
    int64_t ppb;      // points per partition
    int B;            // partitions
    int tiles;        // tiles per partition (by the longest partition)
};

__device__ inline unsigned long long pack_key(float key, uint32_t pos) {
    // key + 0.0f folds -0.0 into +0.0 so equal floats always tie on the id
    return ((unsigned long long)f2ord(key + 0.0f) << 32) | pos;
}

// One workgroup sorts one tile of one slice.  FINAL: the tile is the whole
// slice and the result goes straight to skeys/sids; otherwise the packed words
// go to `packed` for the merge passes.
template <bool FINAL>
__global__ void segsort_tile_kernel(const float* __restrict__ keys, SegGeom g,
                                    float* __restrict__ skeys, int32_t* __restrict__ sids,
                                    uint32_t* __restrict__ inv, uint16_t* __restrict__ lids,
                                    unsigned long long* __restrict__ packed, int np2) {
    extern __shared__ unsigned long long s[];
    const int64_t flat = blockIdx.x;
    const int tile = (int)(flat % g.tiles);
    const int b = (int)((flat / g.tiles) % g.B);
    const int64_t i = flat / ((int64_t)g.tiles * g.B);
    const int64_t off = (int64_t)b * g.ppb;
    const int64_t nseg = min(g.n - off, g.ppb);
    const int64_t t0 = (int64_t)tile * kTileCap;
    if (nseg <= 0 || t0 >= nseg) return;
    const int m = (int)min((int64_t)kTileCap, nseg - t0);
    const int64_t base = i * g.n + off + t0;

    for (int j = threadIdx.x; j < np2; j += blockDim.x)
        s[j] = j < m ? pack_key(keys[base + j], (uint32_t)(t0 + j)) : ~0ull;
    bitonic_sort_u64(s, np2);
    for (int j = threadIdx.x; j < m; j += blockDim.x) {
        const unsigned long long w = s[j];
        if (FINAL) {
            skeys[base + j] = ord2f((uint32_t)(w >> 32));
            sids[base + j] = (int32_t)(off + (uint32_t)w);
            if (lids) lids[base + j] = (uint16_t)(uint32_t)w;
        } else {
            packed[base + j] = w;
        }
    }
    if (FINAL && inv) {
        // inverse permutation inv[point] = position of the point inside its
        // sorted slice, transposed through LDS so the global write is coalesced.
        // The position table overlays the sorted words, so each thread first
        // pulls its words' low halves into registers.
        uint32_t local[kTileCap / 1024];
#pragma unroll
        for (int r = 0; r < kTileCap / 1024; r++) {
            const int j = threadIdx.x + r * blockDim.x;
            local[r] = j < m ? (uint32_t)s[j] - (uint32_t)t0 : 0u;
        }
        __syncthreads();
        uint32_t* pos_of = reinterpret_cast<uint32_t*>(s);
#pragma unroll
        for (int r = 0; r < kTileCap / 1024; r++) {
            const int j = threadIdx.x + r * blockDim.x;
            if (j < m) pos_of[local[r]] = (uint32_t)j;
        }
        __syncthreads();
        for (int j = threadIdx.x; j < m; j += blockDim.x) inv[base + j] = pos_of[j];
    }
}

// One merge pass: within every slice, neighbouring sorted runs of length `run`
// are merged into runs of 2*run.  A workgroup produces kMergeChunk outputs.
__global__ __launch_bounds__(kMergeThreads) void segsort_merge_kernel(
    const unsigned long long* __restrict__ src, unsigned long long* __restrict__ dst,
    SegGeom g, int chunks, int64_t run) {
    const int64_t flat = blockIdx.x;
    const int chunk = (int)(flat % chunks);
    const int b = (int)((flat / chunks) % g.B);
    const int64_t i = flat / ((int64_t)chunks * g.B);
    const int64_t off = (int64_t)b * g.ppb;
    const int64_t nseg = min(g.n - off, g.ppb);
    const int64_t o0 = (int64_t)chunk * kMergeChunk;
    if (nseg <= 0 || o0 >= nseg) return;
    const int64_t base = i * g.n + off;

    const int64_t ps = (o0 / (2 * run)) * (2 * run);        // start of this pair of runs
    const int64_t a0 = ps, a1 = min(ps + run, nseg);
    const int64_t b0 = a1, b1 = min(ps + 2 * run, nseg);
    const int64_t la = a1 - a0, lb = b1 - b0;
    const unsigned long long* A = src + base + a0;
    const unsigned long long* Bv = src + base + b0;

    int64_t d = o0 - ps + (int64_t)threadIdx.x * kMergeItems;   // first output of this thread
    if (d >= la + lb) return;
    // merge path: number of A elements among the first d outputs
    int64_t lo = max((int64_t)0, d - lb), hi = min(d, la);
    while (lo < hi) {
        const int64_t a = (lo + hi) >> 1;
        if (A[a] < Bv[d - 1 - a]) lo = a + 1; else hi = a;
    }
    int64_t ia = lo, ib = d - lo;
    unsigned long long* out = dst + base + ps + d;
    const int cnt = (int)min((int64_t)kMergeItems, la + lb - d);
    unsigned long long va = ia < la ? A[ia] : ~0ull;
    unsigned long long vb = ib < lb ? Bv[ib] : ~0ull;
    for (int t = 0; t < cnt; t++) {
        const bool takeA = ib >= lb || (ia < la && va < vb);
        if (takeA) { out[t] = va; ia++; va = ia < la ? A[ia] : ~0ull; }
        else       { out[t] = vb; ib++; vb = ib < lb ? Bv[ib] : ~0ull; }
    }
}

__global__ void segsort_unpack_kernel(const unsigned long long* __restrict__ packed,
                                      int64_t total, int64_t n, int64_t ppb,
                                      float* __restrict__ skeys, int32_t* __restrict__ sids,
                                      uint32_t* __restrict__ inv, uint16_t* __restrict__ lids) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += stride) {
        const unsigned long long w = packed[e];
        const int64_t col = e % n;
        const int64_t off = (col / ppb) * ppb;
        skeys[e] = ord2f((uint32_t)(w >> 32));
        sids[e] = (int32_t)(off + (uint32_t)w);
        if (inv) inv[e - col + off + (uint32_t)w] = (uint32_t)(col - off);
        if (lids) lids[e] = (uint16_t)(uint32_t)w;
    }
}

size_t segsort_tmp_bytes(int num_indices, int64_t n, int block_size) {
    const int64_t ppb = (n + block_size - 1) / block_size;
    if (ppb <= kTileCap) return 0;
    return (size_t)2 * num_indices * n * sizeof(unsigned long long);
}

static int next_pow2(int v) {
    int p = 2;
    while (p < v) p <<= 1;
    return p;
}

int segsort(const float* d_keys, int num_indices, int64_t n, int block_size,
            float* d_skeys, int32_t* d_sids, uint32_t* d_inv, uint16_t* d_lids, void* d_tmp,
            hipStream_t s) {
    if (n <= 0) return 0;
    SegGeom g;
    g.n = n;
    g.B = block_size;
    g.ppb = (n + block_size - 1) / block_size;
    g.tiles = (int)((g.ppb + kTileCap - 1) / kTileCap);
    const int np2 = next_pow2((int)min((int64_t)kTileCap, g.ppb));
    // at most kTileCap / 1024 elements per thread (the inverse-permutation pass relies on it)
    const int threads = max(64, min(1024, np2 / 2));
    const size_t lds = (size_t)np2 * sizeof(unsigned long long);
    const int64_t blocks = (int64_t)num_indices * g.B * g.tiles;
    if (blocks > 0x7fffffffLL) return fail(-1, "segsort: too many slices for one launch");

    static bool attr_done[2] = {false, false};
    if (!attr_done[0]) {
        DCIH_HIP(hipFuncSetAttribute((const void*)segsort_tile_kernel<true>,
                                     hipFuncAttributeMaxDynamicSharedMemorySize,
                                     kTileCap * (int)sizeof(unsigned long long)));
        DCIH_HIP(hipFuncSetAttribute((const void*)segsort_tile_kernel<false>,
                                     hipFuncAttributeMaxDynamicSharedMemorySize,
                                     kTileCap * (int)sizeof(unsigned long long)));
        attr_done[0] = true;
    }

    if (g.tiles == 1) {
        hipLaunchKernelGGL(segsort_tile_kernel<true>, dim3((unsigned)blocks), dim3(threads), lds, s,
                           d_keys, g, d_skeys, d_sids, d_inv, d_lids, (unsigned long long*)nullptr, np2);
        DCIH_HIP(hipGetLastError());
        return 0;
    }
    if (!d_tmp) return fail(-1, "segsort: scratch buffer missing");
    unsigned long long* bufA = (unsigned long long*)d_tmp;
    unsigned long long* bufB = bufA + (size_t)num_indices * n;
    hipLaunchKernelGGL(segsort_tile_kernel<false>, dim3((unsigned)blocks), dim3(threads), lds, s,
                       d_keys, g, (float*)nullptr, (int32_t*)nullptr, (uint32_t*)nullptr, (uint16_t*)nullptr, bufA, np2);
    const int chunks = (int)((g.ppb + kMergeChunk - 1) / kMergeChunk);
    const int64_t mblocks = (int64_t)num_indices * g.B * chunks;
    if (mblocks > 0x7fffffffLL) return fail(-1, "segsort: too many merge chunks for one launch");
    for (int64_t run = kTileCap; run < g.ppb; run *= 2) {
        hipLaunchKernelGGL(segsort_merge_kernel, dim3((unsigned)mblocks), dim3(kMergeThreads), 0, s,
                           bufA, bufB, g, chunks, run);
        unsigned long long* t = bufA; bufA = bufB; bufB = t;
    }
    const int64_t total = (int64_t)num_indices * n;
    const int ublocks = (int)min((int64_t)65536, (total + 255) / 256);
    hipLaunchKernelGGL(segsort_unpack_kernel, dim3(ublocks), dim3(256), 0, s,
                       bufA, total, n, g.ppb, d_skeys, d_sids, d_inv, d_lids);
    DCIH_HIP(hipGetLastError());
    return 0;
}

}  // namespace dcih
