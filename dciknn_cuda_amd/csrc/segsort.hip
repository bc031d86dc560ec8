// Segmented sort of the projections: every (simple index, partition) slice of
// keys[num_indices][n] becomes (key, id) pairs ascending by key, ties by id.
//
// Stands in for copy_to_indices + sort_indices + mix_sort/quick_sort/
// insertion_sort (src/dci_cuda_kernel.cu:113-146,190-247), where each of
// block_size*thread_size threads quicksorts whole slices serially.
//
// Here a (key, position-in-slice) pair is one 64-bit word whose unsigned order
// is the wanted order.  A slice of up to 32256 points is sorted by one
// workgroup entirely in LDS: one coalesced read of the keys, one coalesced
// write of the sorted keys and ids.  Longer slices are sorted tile by tile and
// the tiles are then merged pairwise (merge path, staged through LDS), each
// pass doubling the run length, the last one writing the final arrays.
#include "common.h"
#include "kernels.h"
#include "radix_core.h"

namespace dcih {

constexpr int kTileCap = 16384;       // elements one workgroup sorts in LDS (128 KB)
constexpr int kMergeThreads = 256;
constexpr int kMergeItems = 8;
constexpr int kMergeChunk = kMergeThreads * kMergeItems;  // divides kTileCap

struct SegGeom {
    int64_t kstride;  // distance between the unsorted key rows of two indices (>= n)
    int64_t n;        // points
    int64_t ppb;      // points per partition
    int B;            // partitions
    int tiles;        // tiles per partition (by the longest partition)
    int tile_size;    // points per tile
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
                                    uint16_t* __restrict__ inv, uint16_t* __restrict__ lids,
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
    const int64_t kbase = i * g.kstride + off + t0;

    for (int j = threadIdx.x; j < np2; j += blockDim.x)
        s[j] = j < m ? pack_key(keys[kbase + j], (uint32_t)(t0 + j)) : ~0ull;
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
        for (int j = threadIdx.x; j < m; j += blockDim.x) inv[base + j] = (uint16_t)pos_of[j];
    }
}

// ---------------------------------------------------------------------------
// LDS radix sort of one whole slice (512 < points <= 32256) by one workgroup:
// least-significant-digit passes of 4 bits over the order-preserving 32-bit
// image of the key.  Every thread owns IPT consecutive items in registers (key
// + packed id/rank); a pass counts digits in per-thread private 16-bit LDS
// counters laid out digit-major (with returning atomics, so that a thread's
// updates pipeline), scans the 16 * threads counters, and moves keys, then ids,
// through one LDS staging buffer.  Thread-private counters plus the digit-major
// scan make every pass stable, so equal keys keep ascending ids.  Nibbles that
// are constant over the slice (typically the exponent's) are skipped.  The
// per-pass cost that does not depend on the slice (scan, barriers) grows with
// the thread count, so the workgroup is the smallest of 64 / 128 / 256 / 512
// threads that covers the slice with at most ~45 (512 threads: 63) items per
// thread; a single wavefront needs no barrier at all.  Global traffic: keys
// read once (all reads of a thread in flight together), sorted keys / ids /
// inverse written once, all coalesced.
constexpr int kRadixMax = 63 * 512;
constexpr int kRadixMin = 512;        // up to this the bitonic tile kernel is faster
constexpr int kRadixTile = 30 * 1024; // longest tile of a slice that needs merge passes

constexpr int radix_lds_bytes(int threads, int ipt) { return (ipt * threads + 8 * threads + 64) * 4; }

template <int kRadixThreads, int IPT>
__global__ __launch_bounds__(kRadixThreads, (kRadixThreads == 256 && IPT > 45) ? 2 : 1) void segsort_radix_kernel(
    const float* __restrict__ keys, SegGeom g, float* __restrict__ skeys,
    int32_t* __restrict__ sids, uint16_t* __restrict__ inv, uint16_t* __restrict__ lids,
    unsigned long long* __restrict__ packed) {
    extern __shared__ uint32_t rs[];
    uint32_t* stage = rs;                                         // IPT*1024 words
    uint16_t* stage16 = reinterpret_cast<uint16_t*>(rs);
    uint32_t* cnt32 = rs + IPT * kRadixThreads;                      // digit counters, [16][threads] 16-bit
    uint32_t* misc = rs + IPT * kRadixThreads + 8 * kRadixThreads;   // 64 words

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    // packed == null: the workgroup sorts a whole slice and writes the final arrays;
    // else it sorts one tile of a slice into packed (key, position in slice) words
    // for the merge passes
    const int tiles = packed ? g.tiles : 1;
    const int tile = (int)(blockIdx.x % tiles);
    const int b = (int)((blockIdx.x / tiles) % g.B);
    const int64_t i = blockIdx.x / ((int64_t)tiles * g.B);
    const int64_t off = (int64_t)b * g.ppb;
    const int64_t t0 = packed ? (int64_t)tile * g.tile_size : 0;
    const int64_t nseg = min(g.n - off, g.ppb) - t0;
    const int n = (int)(packed ? min(nseg, (int64_t)g.tile_size) : nseg);
    if (n <= 0) return;
    const int64_t base = i * g.n + off + t0;
    const int64_t kbase = i * g.kstride + off + t0;

    if (tid < 2) misc[32 + tid] = tid ? 0xffffffffu : 0u;        // OR / AND of all keys
    uint32_t k[IPT], rp[IPT];      // rp: id in the low half, rank / position in the high half
    // coalesced reads, all in flight at once (the slice is read with one round trip),
    // then through LDS into the blocked arrangement
#pragma unroll
    for (int r = 0; r < IPT; r++) {
        const int j = min(r * kRadixThreads + tid, n - 1);       // unconditional: no branch per load
        k[r] = __builtin_bit_cast(uint32_t, keys[kbase + j]);
    }
#pragma unroll
    for (int r = 0; r < IPT; r++) {
        const int j = r * kRadixThreads + tid;                    // pads sort last and stay last
        stage[j] = j < n ? f2ord(__builtin_bit_cast(float, k[r]) + 0.0f) : 0xffffffffu;
    }
    __syncthreads();
    uint32_t vor = 0, vand = 0xffffffffu;
#pragma unroll
    for (int r = 0; r < IPT; r++) {
        k[r] = stage[tid * IPT + r];
        rp[r] = (uint32_t)(tid * IPT + r);
        const bool real = tid * IPT + r < n;
        vor |= real ? k[r] : 0u;
        vand &= real ? k[r] : 0xffffffffu;
    }
    for (int o = 32; o > 0; o >>= 1) {
        vor |= (uint32_t)__shfl_xor((int)vor, o, 64);
        vand &= (uint32_t)__shfl_xor((int)vand, o, 64);
    }
    if (lane == 0) { atomicOr(&misc[32], vor); atomicAnd(&misc[33], vand); }
    __syncthreads();
    const uint32_t varying = misc[32] ^ misc[33];

    lds_radix_passes<kRadixThreads, IPT>(k, rp, stage, cnt32, misc, varying);

    if (packed) {      // (same on every thread) keys, then ids, through LDS into coalesced order
        __syncthreads();
#pragma unroll
        for (int r = 0; r < IPT; r++) stage[tid * IPT + r] = k[r];
        __syncthreads();
#pragma unroll
        for (int r = 0; r < IPT; r++) k[r] = stage[r * kRadixThreads + tid];
        __syncthreads();
#pragma unroll
        for (int r = 0; r < IPT; r++) stage[tid * IPT + r] = rp[r] & 0xffffu;
        __syncthreads();
#pragma unroll
        for (int r = 0; r < IPT; r++) {
            const int j = r * kRadixThreads + tid;
            if (j < n)
                packed[base + j] = ((unsigned long long)k[r] << 32) | (uint32_t)(t0 + stage[j]);
        }
        return;
    }

    // results, through LDS so that every global write is coalesced
    __syncthreads();
#pragma unroll
    for (int r = 0; r < IPT; r++) stage[tid * IPT + r] = k[r];
    __syncthreads();
    for (int j = tid; j < n; j += kRadixThreads) skeys[base + j] = ord2f(stage[j]);
    __syncthreads();
    uint16_t* pos_of = stage16 + IPT * kRadixThreads;            // second half of the staging buffer
#pragma unroll
    for (int r = 0; r < IPT; r++) {
        const int pos = tid * IPT + r;
        const uint32_t id = rp[r] & 0xffffu;
        stage16[pos] = (uint16_t)id;
        if (pos < n) pos_of[id] = (uint16_t)pos;                 // the first n sorted items are the real ones
    }
    __syncthreads();
    for (int j = tid; j < n; j += kRadixThreads) {
        const uint32_t id = stage16[j];
        sids[base + j] = (int32_t)(off + id);
        if (lids) lids[base + j] = (uint16_t)id;
        if (inv) inv[base + j] = pos_of[j];
    }
}

template <int NT, int IPT>
static int launch_radix(const float* d_keys, const SegGeom& g, int num_indices, float* d_skeys,
                        int32_t* d_sids, uint16_t* d_inv, uint16_t* d_lids,
                        unsigned long long* d_packed, hipStream_t s) {
    const size_t lds = (size_t)radix_lds_bytes(NT, IPT);
    static DeviceOnce once;
    {
        const int rc = once.run([lds]() -> int {
            DCIH_HIP(hipFuncSetAttribute((const void*)segsort_radix_kernel<NT, IPT>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            return 0;
        });
        if (rc) return rc;
    }
    const int64_t blocks = (int64_t)num_indices * g.B * (d_packed ? g.tiles : 1);
    if (blocks > 0x7fffffffLL) return fail(-1, "segsort: too many slices for one launch");
    hipLaunchKernelGGL((segsort_radix_kernel<NT, IPT>), dim3((unsigned)blocks), dim3(NT), lds, s,
                       d_keys, g, d_skeys, d_sids, d_inv, d_lids, d_packed);
    DCIH_HIP(hipGetLastError());
    return 0;
}

// Merge path: how many elements of A are among the first d outputs of merging A
// (la elements) with B (lb elements), A winning ties (its positions are smaller).
// One wavefront searches 64 split points per round.
__device__ inline int64_t merge_split_wave(const unsigned long long* __restrict__ A, int64_t la,
                                           const unsigned long long* __restrict__ Bv, int64_t lb,
                                           int64_t d, int lane) {
    int64_t lo = max((int64_t)0, d - lb), hi = min(d, la);
    while (lo < hi) {       // smallest a in [lo, hi] with !(A[a] < B[d-1-a]); wave-uniform
        const int64_t step = (hi - lo + kWave - 1) / kWave;
        const int64_t a = lo + (int64_t)lane * step;
        const bool valid = a < hi;
        const bool below = valid && A[a] < Bv[d - 1 - a];
        const int t = __popcll(__ballot(below));      // the predicate is monotone: a prefix of lanes
        if (t == 0) { hi = lo; break; }
        const int64_t new_lo = lo + (int64_t)(t - 1) * step + 1;
        hi = min(hi, lo + (int64_t)t * step);
        lo = new_lo;
    }
    return lo;
}

// One merge pass: within every slice, neighbouring sorted runs of length `run`
// (a multiple of kMergeChunk / 2) are merged into runs of 2*run.  A workgroup
// produces kMergeChunk outputs: two wavefronts find where its piece starts and
// ends in either run, the two pieces are read into LDS with coalesced loads,
// every thread merges kMergeItems outputs there, and the outputs leave in
// coalesced stores.  The last pass (skeys != null) writes the final arrays
// instead of packed words.
__global__ __launch_bounds__(kMergeThreads) void segsort_merge_kernel(
    const unsigned long long* __restrict__ src, unsigned long long* __restrict__ dst,
    SegGeom g, int chunks, int64_t run, float* __restrict__ skeys, int32_t* __restrict__ sids,
    uint16_t* __restrict__ inv, uint16_t* __restrict__ lids) {
    __shared__ unsigned long long s_in[kMergeChunk];
    __shared__ unsigned long long s_out[kMergeChunk];
    __shared__ int64_t s_split[2];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
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
    const int64_t d0 = o0 - ps;                               // first output of this workgroup
    const int64_t d1 = min(d0 + kMergeChunk, la + lb);
    const int cnt = (int)(d1 - d0);
    if (wave < 2) {
        const int64_t sp = merge_split_wave(A, la, Bv, lb, wave ? d1 : d0, lane);
        if (lane == 0) s_split[wave] = sp;
    }
    __syncthreads();
    const int64_t ia0 = s_split[0], ia1 = s_split[1];
    const int64_t ib0 = d0 - ia0;
    const int na = (int)(ia1 - ia0), nb = cnt - na;
    for (int j = tid; j < cnt; j += kMergeThreads)
        s_in[j] = j < na ? A[ia0 + j] : Bv[ib0 + (j - na)];
    __syncthreads();
    {
        const unsigned long long* LA = s_in;
        const unsigned long long* LB = s_in + na;
        const int d = tid * kMergeItems;
        if (d < cnt) {
            int lo = max(0, d - nb), hi = min(d, na);
            while (lo < hi) {
                const int a = (lo + hi) >> 1;
                if (LA[a] < LB[d - 1 - a]) lo = a + 1; else hi = a;
            }
            int ia = lo, ib = d - lo;
            const int m = min(kMergeItems, cnt - d);
            unsigned long long va = ia < na ? LA[ia] : ~0ull;
            unsigned long long vb = ib < nb ? LB[ib] : ~0ull;
            for (int t = 0; t < m; t++) {
                const bool takeA = ib >= nb || (ia < na && va < vb);
                if (takeA) { s_out[d + t] = va; ia++; va = ia < na ? LA[ia] : ~0ull; }
                else       { s_out[d + t] = vb; ib++; vb = ib < nb ? LB[ib] : ~0ull; }
            }
        }
    }
    __syncthreads();
    const int64_t out0 = base + ps + d0;
    if (!skeys) {
        for (int j = tid; j < cnt; j += kMergeThreads) dst[out0 + j] = s_out[j];
    } else {
        for (int j = tid; j < cnt; j += kMergeThreads) {
            const unsigned long long w = s_out[j];
            const int64_t e = out0 + j;
            skeys[e] = ord2f((uint32_t)(w >> 32));
            sids[e] = (int32_t)(off + (uint32_t)w);
            if (inv) inv[base + (uint32_t)w] = (uint16_t)(ps + d0 + j);
            if (lids) lids[e] = (uint16_t)(uint32_t)w;
        }
    }
}

size_t segsort_tmp_bytes(int num_indices, int64_t n, int block_size) {
    const int64_t ppb = (n + block_size - 1) / block_size;
    if (ppb <= 63 * 512) return 0;       // one LDS pass (bitonic tile or radix kernel)
    return (size_t)2 * num_indices * n * sizeof(unsigned long long);
}

static int next_pow2(int v) {
    int p = 2;
    while (p < v) p <<= 1;
    return p;
}

int segsort(const float* d_keys, int64_t key_stride, int num_indices, int64_t n, int block_size,
            float* d_skeys, int32_t* d_sids, uint16_t* d_inv, uint16_t* d_lids, void* d_tmp,
            hipStream_t s) {
    if (n <= 0) return 0;
    if (key_stride < n) return fail(-1, "segsort: key rows overlap");
    SegGeom g;
    g.kstride = key_stride;
    g.n = n;
    g.B = block_size;
    g.ppb = (n + block_size - 1) / block_size;
    g.tiles = (int)((g.ppb + kTileCap - 1) / kTileCap);
    g.tile_size = kTileCap;
    const int np2 = next_pow2((int)min((int64_t)kTileCap, g.ppb));
    // at most kTileCap / 1024 elements per thread (the inverse-permutation pass relies on it)
    const int threads = max(64, min(1024, np2 / 2));
    const size_t lds = (size_t)np2 * sizeof(unsigned long long);
    const int64_t blocks = (int64_t)num_indices * g.B * g.tiles;
    if (blocks > 0x7fffffffLL) return fail(-1, "segsort: too many slices for one launch");

    static DeviceOnce once;
    {
        const int rc = once.run([]() -> int {
            DCIH_HIP(hipFuncSetAttribute((const void*)segsort_tile_kernel<true>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize,
                                         kTileCap * (int)sizeof(unsigned long long)));
            return 0;
        });
        if (rc) return rc;
    }

    if (g.ppb > kRadixMin && g.ppb <= kRadixMax) {
        // odd items-per-thread keep the blocked LDS accesses free of bank conflicts
#define DCIH_RADIX(NT, IPT) \
    if (g.ppb <= (int64_t)(NT) * (IPT))  \
        return launch_radix<NT, IPT>(d_keys, g, num_indices, d_skeys, d_sids, d_inv, d_lids, nullptr, s)
        DCIH_RADIX(64, 9); DCIH_RADIX(64, 17); DCIH_RADIX(64, 25); DCIH_RADIX(64, 33);
        DCIH_RADIX(128, 21); DCIH_RADIX(128, 27); DCIH_RADIX(128, 33);
        DCIH_RADIX(256, 21); DCIH_RADIX(256, 27); DCIH_RADIX(256, 33); DCIH_RADIX(256, 39); DCIH_RADIX(256, 45);
        DCIH_RADIX(256, 51); DCIH_RADIX(256, 57);      // two workgroups share a CU: one's passes cover the other's loads and stores
        DCIH_RADIX(512, 33); DCIH_RADIX(512, 39); DCIH_RADIX(512, 45);
        DCIH_RADIX(512, 51); DCIH_RADIX(512, 57); DCIH_RADIX(512, 63);
#undef DCIH_RADIX
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
    // Slices beyond one LDS pass: as few radix-sorted tiles as cover the slice (runs of a
    // multiple of 1024 points, so that a merge chunk never straddles two pairs of runs),
    // then merge passes.
    g.tiles = (int)((g.ppb + kRadixTile - 1) / kRadixTile);
    g.tile_size = (int)((((g.ppb + g.tiles - 1) / g.tiles) + 1023) / 1024 * 1024);
    {
        int rc = -1;
#define DCIH_RADIX_TILE(NT, IPT) \
    if (rc < 0 && g.tile_size <= (NT) * (IPT))  \
        rc = launch_radix<NT, IPT>(d_keys, g, num_indices, nullptr, nullptr, nullptr, nullptr, bufA, s)
        DCIH_RADIX_TILE(512, 33); DCIH_RADIX_TILE(512, 39); DCIH_RADIX_TILE(512, 45);
        DCIH_RADIX_TILE(512, 51); DCIH_RADIX_TILE(512, 57); DCIH_RADIX_TILE(512, 63);
#undef DCIH_RADIX_TILE
        if (rc) return rc < 0 ? fail(-1, "segsort: no radix configuration for the tile size") : rc;
    }
    const int chunks = (int)((g.ppb + kMergeChunk - 1) / kMergeChunk);
    const int64_t mblocks = (int64_t)num_indices * g.B * chunks;
    if (mblocks > 0x7fffffffLL) return fail(-1, "segsort: too many merge chunks for one launch");
    for (int64_t run = g.tile_size; run < g.ppb; run *= 2) {
        const bool last = run * 2 >= g.ppb;       // the last pass writes the final arrays
        hipLaunchKernelGGL(segsort_merge_kernel, dim3((unsigned)mblocks), dim3(kMergeThreads), 0, s,
                           bufA, bufB, g, chunks, run, last ? d_skeys : (float*)nullptr, d_sids, d_inv, d_lids);
        unsigned long long* t = bufA; bufA = bufB; bufB = t;
    }
    DCIH_HIP(hipGetLastError());
    return 0;
}

}  // namespace dcih
