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
#include <algorithm>

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
    // appending (radix kernel, packed output): only the points with ids from tail_from on are
    // sorted, one run per partition from partition b_first on; -1 = everything
    int64_t tail_from;
    int b_first;
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
    const int lane = tid & 63;
    // packed == null: the workgroup sorts a whole slice and writes the final arrays;
    // else it sorts one tile of a slice into packed (key, position in slice) words
    // for the merge passes
    const bool tail = g.tail_from >= 0;
    const int tiles = packed && !tail ? g.tiles : 1;
    const int parts = tail ? g.B - g.b_first : g.B;
    const int tile = (int)(blockIdx.x % tiles);
    const int b = (int)((blockIdx.x / tiles) % parts) + (tail ? g.b_first : 0);
    const int64_t i = blockIdx.x / ((int64_t)tiles * parts);
    const int64_t off = (int64_t)b * g.ppb;
    const int64_t t0 = tail ? max((int64_t)0, g.tail_from - off) : (packed ? (int64_t)tile * g.tile_size : 0);
    const int64_t nseg = min(g.n - off, g.ppb) - t0;
    const int n = (int)(packed && !tail ? min(nseg, (int64_t)g.tile_size) : nseg);
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
    const int64_t blocks = g.tail_from >= 0 ? (int64_t)num_indices * (g.B - g.b_first)
                                            : (int64_t)num_indices * g.B * (d_packed ? g.tiles : 1);
    if (blocks > 0x7fffffffLL) return fail(-1, "segsort: too many slices for one launch");
    hipLaunchKernelGGL((segsort_radix_kernel<NT, IPT>), dim3((unsigned)blocks), dim3(NT), lds, s,
                       d_keys, g, d_skeys, d_sids, d_inv, d_lids, d_packed);
    DCIH_HIP(hipGetLastError());
    return 0;
}


// ---------------------------------------------------------------------------
// The same sort moving ONE word per item: (16 key bits << 16 | id).  Four passes order the
// items by the low half of their keys, then every item fetches the high half of its key by id
// (the slice was read a moment ago and sits in L2) and four more passes order by that; LSD
// passes are stable, so the result is ordered by (key, id).  Half the scatters and reads of the
// two-word kernel, half the registers, and with the digit counters inside the staging buffer a
// slice takes 4 bytes of LDS per point: two workgroups share a CU up to 20 k points, and one's
// barrier-separated phases overlap the other's.  Destinations come from a second round of
// returning atomics on the scanned counters (no separate rank table), held two to a register
// until every thread has its own (the scatter overwrites the counters).
template <int NT, int IPT>
__device__ inline void lds_radix_half(uint32_t (&w)[IPT], uint32_t* stage, uint32_t* misc, uint32_t varying16) {
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    uint32_t* cnt32 = stage;                                   // [16][NT] 16-bit counters, digit-major
    const uint32_t half = (uint32_t)(tid & 1) * 16u;
    for (int shift = 16; shift < 32; shift += 4) {
        if (((varying16 >> (shift - 16)) & 15u) == 0u) continue;     // same nibble everywhere
        __syncthreads();
#pragma unroll
        for (int q = 0; q < 8; q++) cnt32[tid + q * NT] = 0;
        __syncthreads();
#pragma unroll
        for (int r = 0; r < IPT; r++) {
            const uint32_t a = ((w[r] >> shift) & 15u) * NT + tid;
            atomicAdd(&cnt32[a >> 1], 1u << half);
        }
        __syncthreads();
        {   // exclusive scan of the 16 * NT counters in memory order
            uint32_t v[8];
            uint32_t sum = 0;
#pragma unroll
            for (int q = 0; q < 8; q++) { v[q] = cnt32[tid * 8 + q]; sum += (v[q] & 0xffffu) + (v[q] >> 16); }
            uint32_t incl = sum;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const uint32_t t = (uint32_t)__shfl_up((int)incl, o, 64);
                if (lane >= o) incl += t;
            }
            if (lane == 63) misc[wave] = incl;
            __syncthreads();
            uint32_t run = incl - sum;
            for (int w2 = 0; w2 < wave; w2++) run += misc[w2];
#pragma unroll
            for (int q = 0; q < 8; q++) {
                const uint32_t lo = v[q] & 0xffffu, hi = v[q] >> 16;
                cnt32[tid * 8 + q] = run | ((run + lo) << 16);
                run += lo + hi;
            }
        }
        __syncthreads();
        uint32_t dst[(IPT + 1) / 2];                           // destinations, two to a register
        {
            int shift2 = shift;
            asm volatile("" : "+s"(shift2));
#pragma unroll
            for (int r = 0; r < IPT; r++) {
                const uint32_t a = ((w[r] >> shift2) & 15u) * NT + tid;
                const uint32_t d = (atomicAdd(&cnt32[a >> 1], 1u << half) >> half) & 0xffffu;
                if (r & 1) dst[r >> 1] |= d << 16; else dst[r >> 1] = d;
                if ((r & 7) == 7) __builtin_amdgcn_sched_barrier(0);
            }
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < IPT; r++) {
            stage[(r & 1) ? (dst[r >> 1] >> 16) : (dst[r >> 1] & 0xffffu)] = w[r];
            if ((r & 7) == 7) __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < IPT; r++) {
            w[r] = stage[tid * IPT + r];
            if ((r & 7) == 7) __builtin_amdgcn_sched_barrier(0);
        }
    }
}

template <int NT, int IPT, int WPS>
__global__ __launch_bounds__(NT, WPS) void segsort_radix1w_kernel(
    const float* __restrict__ keys, SegGeom g, float* __restrict__ skeys,
    int32_t* __restrict__ sids, uint16_t* __restrict__ inv, uint16_t* __restrict__ lids) {
    extern __shared__ uint32_t rs[];
    uint32_t* stage = rs;                                         // IPT * NT words (>= 8 * NT)
    uint16_t* stage16 = reinterpret_cast<uint16_t*>(rs);
    uint32_t* misc = rs + IPT * NT;                               // 64 words
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int b = (int)(blockIdx.x % g.B);
    const int64_t i = blockIdx.x / g.B;
    const int64_t off = (int64_t)b * g.ppb;
    const int n = (int)min(g.n - off, g.ppb);
    if (n <= 0) return;
    const int64_t base = i * g.n + off;
    const float* kin = keys + i * g.kstride + off;

    if (tid < 2) misc[32 + tid] = tid ? 0xffffffffu : 0u;        // OR / AND of all keys
    uint32_t w[IPT];
    {   // coalesced reads, all in flight at once; (low key half, position) words through LDS into
        // the blocked arrangement; pads sort last and stay last
        uint32_t vor = 0, vand = 0xffffffffu;
#pragma unroll
        for (int r = 0; r < IPT; r++) w[r] = __builtin_bit_cast(uint32_t, kin[min(r * NT + tid, n - 1)]);
#pragma unroll
        for (int r = 0; r < IPT; r++) {
            const int j = r * NT + tid;
            const uint32_t o = f2ord(__builtin_bit_cast(float, w[r]) + 0.0f);
            vor |= j < n ? o : 0u;
            vand &= j < n ? o : 0xffffffffu;
            stage[j] = j < n ? ((o << 16) | (uint32_t)j) : (0xffff0000u | (uint32_t)(j & 0xffff));
        }
        for (int o = 32; o > 0; o >>= 1) {
            vor |= (uint32_t)__shfl_xor((int)vor, o, 64);
            vand &= (uint32_t)__shfl_xor((int)vand, o, 64);
        }
        if (lane == 0) { atomicOr(&misc[32], vor); atomicAnd(&misc[33], vand); }
    }
    __syncthreads();
    const uint32_t varying = misc[32] ^ misc[33];
#pragma unroll
    for (int r = 0; r < IPT; r++) w[r] = stage[tid * IPT + r];

    lds_radix_half<NT, IPT>(w, stage, misc, varying & 0xffffu);
    // the other half of every key, by id (the first n sorted items are the real ones); the
    // slice was read a moment ago and sits in L2
#pragma unroll
    for (int r = 0; r < IPT; r++) {
        const uint32_t id = w[r] & 0xffffu;
        const bool real = tid * IPT + r < n;
        const float kv = kin[real ? id : 0];
        const uint32_t o = f2ord(kv + 0.0f);
        w[r] = real ? ((o & 0xffff0000u) | id) : (0xffff0000u | id);
    }
    lds_radix_half<NT, IPT>(w, stage, misc, varying >> 16);

    // results, through LDS so that every global write is coalesced: keys (fetched whole by id), ids
    uint32_t full[IPT];
#pragma unroll
    for (int r = 0; r < IPT; r++) {
        const bool real = tid * IPT + r < n;
        full[r] = f2ord(kin[real ? (w[r] & 0xffffu) : 0] + 0.0f);
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < IPT; r++) stage[tid * IPT + r] = full[r];
    __syncthreads();
    for (int j = tid; j < n; j += NT) skeys[base + j] = ord2f(stage[j]);
    __syncthreads();
    uint16_t* pos_of = stage16 + IPT * NT;                        // second half of the staging buffer
#pragma unroll
    for (int r = 0; r < IPT; r++) {
        const int pos = tid * IPT + r;
        const uint32_t id = w[r] & 0xffffu;
        stage16[pos] = (uint16_t)id;
        if (pos < n) pos_of[id] = (uint16_t)pos;
    }
    __syncthreads();
    for (int j = tid; j < n; j += NT) {
        const uint32_t id = stage16[j];
        sids[base + j] = (int32_t)(off + id);
        if (lids) lids[base + j] = (uint16_t)id;
        if (inv) inv[base + j] = pos_of[j];
    }
}

template <int NT, int IPT, int WPS>
static int launch_radix1w(const float* d_keys, const SegGeom& g, int num_indices, float* d_skeys,
                          int32_t* d_sids, uint16_t* d_inv, uint16_t* d_lids, hipStream_t s) {
    const size_t lds = (size_t)(IPT * NT + 64) * 4;
    static DeviceOnce once;
    {
        const int rc = once.run([lds]() -> int {
            DCIH_HIP(hipFuncSetAttribute((const void*)segsort_radix1w_kernel<NT, IPT, WPS>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            return 0;
        });
        if (rc) return rc;
    }
    const int64_t blocks = (int64_t)num_indices * g.B;
    if (blocks > 0x7fffffffLL) return fail(-1, "segsort: too many slices for one launch");
    hipLaunchKernelGGL((segsort_radix1w_kernel<NT, IPT, WPS>), dim3((unsigned)blocks), dim3(NT), lds, s,
                       d_keys, g, d_skeys, d_sids, d_inv, d_lids);
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

// Outputs [d0, d1) (at most kMergeChunk of them) of the merge of the sorted runs A (la words)
// and Bv (lb words), A winning ties, by one workgroup: two wavefronts find where the piece
// starts and ends in either run, the two pieces are read into LDS with coalesced loads, every
// thread merges kMergeItems outputs there, and the outputs leave in coalesced stores, either
// as packed words to dst + out0 or, for the last pass (skeys != null), as the final arrays of
// the slice that starts at element `base` of its index and at point id `off`; out0 is then
// the first output's position inside the slice.
struct MergeScratch {
    unsigned long long in[kMergeChunk];
    unsigned long long out[kMergeChunk];
    int64_t split[2];
};
__device__ inline void merge_piece(MergeScratch& ms, const unsigned long long* __restrict__ A, int64_t la,
                                   const unsigned long long* __restrict__ Bv, int64_t lb, int64_t d0, int64_t d1,
                                   unsigned long long* __restrict__ dst, int64_t out0, int64_t base, int64_t off,
                                   float* __restrict__ skeys, int32_t* __restrict__ sids,
                                   uint16_t* __restrict__ inv, uint16_t* __restrict__ lids) {
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int cnt = (int)(d1 - d0);
    if (wave < 2) {
        const int64_t sp = merge_split_wave(A, la, Bv, lb, wave ? d1 : d0, lane);
        if (lane == 0) ms.split[wave] = sp;
    }
    __syncthreads();
    const int64_t ia0 = ms.split[0], ia1 = ms.split[1];
    const int64_t ib0 = d0 - ia0;
    const int na = (int)(ia1 - ia0), nb = cnt - na;
    for (int j = tid; j < cnt; j += kMergeThreads)
        ms.in[j] = j < na ? A[ia0 + j] : Bv[ib0 + (j - na)];
    __syncthreads();
    {
        const unsigned long long* LA = ms.in;
        const unsigned long long* LB = ms.in + na;
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
                if (takeA) { ms.out[d + t] = va; ia++; va = ia < na ? LA[ia] : ~0ull; }
                else       { ms.out[d + t] = vb; ib++; vb = ib < nb ? LB[ib] : ~0ull; }
            }
        }
    }
    __syncthreads();
    if (!skeys) {
        for (int j = tid; j < cnt; j += kMergeThreads) dst[base + out0 + j] = ms.out[j];
    } else {
        for (int j = tid; j < cnt; j += kMergeThreads) {
            const unsigned long long w = ms.out[j];
            const int64_t e = base + out0 + j;
            skeys[e] = ord2f((uint32_t)(w >> 32));
            sids[e] = (int32_t)(off + (uint32_t)w);
            if (inv) inv[base + (uint32_t)w] = (uint16_t)(out0 + j);
            if (lids) lids[e] = (uint16_t)(uint32_t)w;
        }
    }
}

// One merge pass: within every slice, neighbouring sorted runs of length `run`
// (a multiple of kMergeChunk / 2) are merged into runs of 2*run; a workgroup
// produces kMergeChunk outputs.  The last pass (skeys != null) writes the final
// arrays instead of packed words.
__global__ __launch_bounds__(kMergeThreads) void segsort_merge_kernel(
    const unsigned long long* __restrict__ src, unsigned long long* __restrict__ dst,
    SegGeom g, int chunks, int64_t run, float* __restrict__ skeys, int32_t* __restrict__ sids,
    uint16_t* __restrict__ inv, uint16_t* __restrict__ lids) {
    __shared__ MergeScratch ms;
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
    const int64_t d0 = o0 - ps;                               // first output of this workgroup
    const int64_t d1 = min(d0 + kMergeChunk, la + lb);
    merge_piece(ms, src + base + a0, la, src + base + b0, lb, d0, d1, dst, ps + d0, base, off,
                skeys, sids, inv, lids);
}

// ---------------------------------------------------------------------------
// Appending points to a built index without sorting the old ones again.
// The partitions are the id ranges [b * ppb, (b + 1) * ppb) with ppb = ceil(n / B), so
// n0 -> n1 points moves every boundary (p0 -> p1 points per partition), and a new slice is
// made of pieces of old slices plus, in the last partitions, new points:
//   * an old slice is shorter than a new one, so it contributes to at most two new slices,
//     to each a contiguous range of its ids; taking those ids out of the slice in their
//     sorted order (a stable split in two) gives two sorted runs;
//   * the new points of a partition are sorted on their own (LDS radix sort): one more run;
//   * the runs of a new slice, laid end to end by ascending ids, are merged pairwise
//     (merge path, as in the build of long slices), the last pass writing the final arrays.
// Run r of new slice b starts at position run_start(b, r) of the slice; all of it follows
// from n0, n1, p0, p1 alone.
struct AppendGeom {
    int64_t n0, n1;     // points before and after
    int64_t p0, p1;     // points per partition before and after
    int B;
};
__host__ __device__ inline int64_t slice_len(const AppendGeom& g, int b) {
    const int64_t v = g.n1 - (int64_t)b * g.p1;
    return v < 0 ? 0 : (v < g.p1 ? v : g.p1);
}
__host__ __device__ inline int64_t old_in_slice(const AppendGeom& g, int b) {     // its points with ids below n0
    const int64_t v = g.n0 - (int64_t)b * g.p1, len = slice_len(g, b);
    return v < 0 ? 0 : (v < len ? v : len);
}
__host__ __device__ inline int slice_runs(const AppendGeom& g, int b) {
    const int64_t lo = (int64_t)b * g.p1, n_old = old_in_slice(g, b), len = slice_len(g, b);
    const int r_old = n_old > 0 ? (int)((lo + n_old - 1) / g.p0 - lo / g.p0 + 1) : 0;
    return r_old + (len > n_old ? 1 : 0);
}
__host__ __device__ inline int64_t run_start(const AppendGeom& g, int b, int r) {
    const int64_t lo = (int64_t)b * g.p1, n_old = old_in_slice(g, b), len = slice_len(g, b);
    const int r_old = n_old > 0 ? (int)((lo + n_old - 1) / g.p0 - lo / g.p0 + 1) : 0;
    if (r <= 0) return 0;
    if (r < r_old) return (lo / g.p0 + r) * g.p0 - lo;
    if (r == r_old) return n_old;
    return len;
}

// Stable split of every old slice: its (key, id) pairs leave, in their sorted order, for the
// runs of the one or two new slices their ids fall into, as packed (key, position in the new
// slice) words.  One workgroup per (simple index, old slice).
constexpr int kSplitThreads = 256;
__global__ __launch_bounds__(kSplitThreads) void append_split_kernel(
    const float* __restrict__ old_keys, const int32_t* __restrict__ old_ids, AppendGeom g,
    unsigned long long* __restrict__ packed) {
    __shared__ int s_wave[kSplitThreads / kWave][2];
    const int old_slices = (int)((g.n0 + g.p0 - 1) / g.p0);
    const int a = (int)(blockIdx.x % old_slices);
    const int64_t i = blockIdx.x / old_slices;
    const int64_t lo = (int64_t)a * g.p0;
    const int len = (int)min(g.p0, g.n0 - lo);
    const int d0 = (int)(lo / g.p1);
    const int64_t cut = (int64_t)(d0 + 1) * g.p1;                // ids from here on go to slice d0 + 1
    // where the two runs start: ids ascend along a new slice's runs
    const int64_t out_lo = i * g.n1 + (int64_t)d0 * g.p1 + (lo - (int64_t)d0 * g.p1);
    const int64_t out_hi = i * g.n1 + cut;                       // the next slice's first run
    const float* keys = old_keys + i * g.n0 + lo;
    const int32_t* ids = old_ids + i * g.n0 + lo;
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    int done_lo = 0, done_hi = 0;
    for (int j0 = 0; j0 < len; j0 += kSplitThreads) {
        const int j = j0 + tid;
        const bool real = j < len;
        const int64_t id = real ? (int64_t)ids[j] : 0;
        const uint32_t ok = real ? f2ord(keys[j]) : 0u;
        const bool hi = real && id >= cut;
        const unsigned long long m_hi = __ballot(hi), m_lo = __ballot(real && !hi);
        const unsigned long long below = (1ull << lane) - 1ull;
        if (lane == 0) { s_wave[wave][0] = __popcll(m_lo); s_wave[wave][1] = __popcll(m_hi); }
        __syncthreads();
        int before_lo = done_lo, before_hi = done_hi, all_lo = 0, all_hi = 0;
        for (int w = 0; w < kSplitThreads / kWave; w++) {
            if (w < wave) { before_lo += s_wave[w][0]; before_hi += s_wave[w][1]; }
            all_lo += s_wave[w][0]; all_hi += s_wave[w][1];
        }
        if (real) {
            if (hi) packed[out_hi + before_hi + __popcll(m_hi & below)] = ((unsigned long long)ok << 32) | (uint32_t)(id - cut);
            else packed[out_lo + before_lo + __popcll(m_lo & below)] = ((unsigned long long)ok << 32) | (uint32_t)(id - (int64_t)d0 * g.p1);
        }
        done_lo += all_lo; done_hi += all_hi;
        __syncthreads();
    }
}

// One pass over the runs of every new slice: runs 2q * step and (2q + 1) * step of level 0
// (each already a union of `step` original runs) are merged.  A workgroup produces the
// outputs [chunk * kMergeChunk, ...) of its slice, pair by pair where they straddle pairs.
// A slice whose runs this pass brings down to one gets its final arrays written at once, and
// later passes skip it: most slices have two runs and are done after the first pass.
__global__ __launch_bounds__(kMergeThreads) void append_merge_kernel(
    const unsigned long long* __restrict__ src, unsigned long long* __restrict__ dst, AppendGeom g,
    int chunks, int step, float* __restrict__ skeys, int32_t* __restrict__ sids,
    uint16_t* __restrict__ inv, uint16_t* __restrict__ lids) {
    __shared__ MergeScratch ms;
    const int64_t flat = blockIdx.x;
    const int chunk = (int)(flat % chunks);
    const int b = (int)((flat / chunks) % g.B);
    const int64_t i = flat / ((int64_t)chunks * g.B);
    const int64_t off = (int64_t)b * g.p1;
    const int64_t nseg = slice_len(g, b);
    const int64_t o0 = (int64_t)chunk * kMergeChunk, o1 = min(o0 + kMergeChunk, nseg);
    if (o0 >= nseg) return;
    const int64_t base = i * g.n1 + off;
    const int runs = slice_runs(g, b);
    if (step > 1 && step >= runs) return;                    // an earlier pass finished this slice
    if (2 * step < runs) skeys = nullptr;                    // more passes to come: packed words
    for (int q = 0; 2 * q * step < runs; q++) {
        const int64_t a0 = run_start(g, b, 2 * q * step), a1 = run_start(g, b, (2 * q + 1) * step);
        const int64_t b1 = run_start(g, b, (2 * q + 2) * step);
        if (b1 <= o0) continue;
        if (a0 >= o1) break;
        const int64_t d0 = max(o0, a0) - a0, d1 = min(o1, b1) - a0;       // this pair's outputs of this workgroup
        merge_piece(ms, src + base + a0, a1 - a0, src + base + a1, b1 - a1, d0, d1, dst, a0 + d0, base, off,
                    skeys, sids, inv, lids);
        __syncthreads();
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
    g.tail_from = -1;
    g.b_first = 0;
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
        // slices of 15 k to 19968 points: the one-word kernel, two workgroups per CU
        if (g.ppb > 15000 && g.ppb <= 512 * 39)
            return launch_radix1w<512, 39, 4>(d_keys, g, num_indices, d_skeys, d_sids, d_inv, d_lids, s);
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

// The positions of every point in simple index i, in the order of the slice of the first simple index r of
// i's composite: the batch traversal scans them for the points that stand inside the first index's visited run.
// Point ids of a partition lie in the partition, so the gather stays inside one slice of inv (L1 / L2).
__global__ __launch_bounds__(256) void positions_by_first_kernel(const int32_t* __restrict__ sids,
                                                                 const uint16_t* __restrict__ inv,
                                                                 uint16_t* __restrict__ rpos, int64_t n, int L) {
    const int m = (int)(blockIdx.y / (L - 1));
    const int h = 1 + (int)(blockIdx.y % (L - 1));
    const int64_t r = (int64_t)m * L, i = r + h;
    const int64_t e0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (e0 >= n) return;
    if (e0 + 4 <= n && (n & 3) == 0) {       // four at a time: one 16-byte read of ids, one 8-byte write
        typedef int v4i __attribute__((ext_vector_type(4)));
        typedef uint16_t v4h __attribute__((ext_vector_type(4)));
        const v4i p = *reinterpret_cast<const v4i*>(sids + r * n + e0);
        v4h o;
        o.x = inv[i * n + p.x]; o.y = inv[i * n + p.y]; o.z = inv[i * n + p.z]; o.w = inv[i * n + p.w];
        *reinterpret_cast<v4h*>(rpos + i * n + e0) = o;
    } else {
        for (int64_t e = e0; e < min(n, e0 + 4); e++) rpos[i * n + e] = inv[i * n + sids[r * n + e]];
    }
}

int fill_positions_by_first(const int32_t* d_sids, const uint16_t* d_inv, uint16_t* d_rpos, int64_t n, int M, int L,
                            hipStream_t s) {
    if (L < 2 || n <= 0) return 0;
    const int64_t bx = (n + 1023) / 1024, by = (int64_t)M * (L - 1);
    if (bx > 0x7fffffffLL || by > 65535) return fail(-1, "fill_positions_by_first: grid too large");
    hipLaunchKernelGGL(positions_by_first_kernel, dim3((unsigned)bx, (unsigned)by), dim3(256), 0, s,
                       d_sids, d_inv, d_rpos, n, L);
    DCIH_HIP(hipGetLastError());
    return 0;
}

// inv[point] = position of the point inside its sorted slice, from the slice's sorted ids.
__global__ __launch_bounds__(512) void slice_inverse_kernel(const int32_t* __restrict__ sids,
                                                            uint16_t* __restrict__ inv, int64_t n, int64_t ppb, int B) {
    extern __shared__ uint16_t pos_of[];
    const int b = (int)(blockIdx.x % B);
    const int64_t i = blockIdx.x / B;
    const int64_t off = (int64_t)b * ppb;
    const int len = (int)min(ppb, n - off);
    if (len <= 0) return;
    const int64_t base = i * n + off;
    for (int j = threadIdx.x; j < len; j += blockDim.x) pos_of[sids[base + j] - (int32_t)off] = (uint16_t)j;
    __syncthreads();
    for (int j = threadIdx.x; j < len; j += blockDim.x) inv[base + j] = pos_of[j];
}

// ---- appending -------------------------------------------------------------------
bool segsort_append_supported(int64_t n0, int64_t n1, int block_size) {
    if (n0 <= 0 || n1 <= n0 || block_size < 1) return false;
    const int64_t p0 = (n0 + block_size - 1) / block_size, p1 = (n1 + block_size - 1) / block_size;
    // the new points of a partition are sorted by one LDS pass; positions fit 16 bits
    return p1 <= kRadixMax && p1 <= 65536 && p0 <= p1;
}

size_t segsort_append_tmp_bytes(int num_indices, int64_t n1) {
    return (size_t)2 * num_indices * n1 * sizeof(unsigned long long);
}

int segsort_append(const float* d_old_skeys, const int32_t* d_old_sids, int64_t n0,
                   const float* d_keys, int64_t key_stride, int num_indices, int64_t n1, int block_size,
                   float* d_skeys, int32_t* d_sids, uint16_t* d_inv, uint16_t* d_lids, void* d_tmp,
                   hipStream_t s) {
    if (!segsort_append_supported(n0, n1, block_size)) return fail(-1, "segsort_append: shape not supported");
    if (!d_tmp) return fail(-1, "segsort_append: scratch buffer missing");
    AppendGeom ag;
    ag.n0 = n0; ag.n1 = n1; ag.B = block_size;
    ag.p0 = (n0 + block_size - 1) / block_size;
    ag.p1 = (n1 + block_size - 1) / block_size;
    unsigned long long* bufA = (unsigned long long*)d_tmp;
    unsigned long long* bufB = bufA + (size_t)num_indices * n1;
    // 1. the old slices' entries, split into the runs of the new slices
    const int64_t old_slices = (n0 + ag.p0 - 1) / ag.p0;
    if (num_indices * old_slices > 0x7fffffffLL) return fail(-1, "segsort_append: too many slices for one launch");
    hipLaunchKernelGGL(append_split_kernel, dim3((unsigned)(num_indices * old_slices)), dim3(kSplitThreads), 0, s,
                       d_old_skeys, d_old_sids, ag, bufA);
    DCIH_HIP(hipGetLastError());
    // 2. the new points of every partition that has some, sorted into one more run
    {
        SegGeom g;
        g.kstride = key_stride; g.n = n1; g.B = block_size; g.ppb = ag.p1;
        g.tiles = 1; g.tile_size = 0;
        g.tail_from = n0;
        g.b_first = (int)(n0 / ag.p1);
        int64_t longest = 0;                               // longest run of new points in one partition
        for (int b = g.b_first; b < block_size; b++)
            longest = std::max(longest, slice_len(ag, b) - old_in_slice(ag, b));
        int rc = -1;
#define DCIH_RADIX_TAIL(NT, IPT) \
    if (rc < 0 && longest <= (int64_t)(NT) * (IPT))  \
        rc = launch_radix<NT, IPT>(d_keys, g, num_indices, nullptr, nullptr, nullptr, nullptr, bufA, s)
        DCIH_RADIX_TAIL(64, 9); DCIH_RADIX_TAIL(64, 33); DCIH_RADIX_TAIL(128, 33); DCIH_RADIX_TAIL(256, 33);
        DCIH_RADIX_TAIL(256, 57); DCIH_RADIX_TAIL(512, 39); DCIH_RADIX_TAIL(512, 51); DCIH_RADIX_TAIL(512, 63);
#undef DCIH_RADIX_TAIL
        if (rc) return rc < 0 ? fail(-1, "segsort_append: no radix configuration for the new points") : rc;
    }
    // 3. pairwise merges of every slice's runs
    int most_runs = 1;
    for (int b = 0; b < block_size; b++) most_runs = std::max(most_runs, slice_runs(ag, b));
    const int chunks = (int)((ag.p1 + kMergeChunk - 1) / kMergeChunk);
    const int64_t mblocks = (int64_t)num_indices * block_size * chunks;
    if (mblocks > 0x7fffffffLL) return fail(-1, "segsort_append: too many merge chunks for one launch");
    for (int step = 1;; step *= 2) {
        const bool last = 2 * step >= most_runs;
        hipLaunchKernelGGL(append_merge_kernel, dim3((unsigned)mblocks), dim3(kMergeThreads), 0, s,
                           bufA, bufB, ag, chunks, step, d_skeys, d_sids, (uint16_t*)nullptr, d_lids);
        unsigned long long* t = bufA; bufA = bufB; bufB = t;
        if (last) break;
    }
    DCIH_HIP(hipGetLastError());
    // 4. the inverse permutation of every slice from its sorted ids, turned round in LDS so that
    // reads and writes are coalesced (written from the merge it would be a scatter of 2-byte words)
    if (d_inv) {
        const size_t lds = (size_t)ag.p1 * sizeof(uint16_t);
        static DeviceOnce once;
        const int rc = once.run([]() -> int {
            DCIH_HIP(hipFuncSetAttribute((const void*)slice_inverse_kernel,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 65536 * (int)sizeof(uint16_t)));
            return 0;
        });
        if (rc) return rc;
        hipLaunchKernelGGL(slice_inverse_kernel, dim3((unsigned)((int64_t)num_indices * block_size)), dim3(512), lds, s,
                           d_sids, d_inv, n1, ag.p1, block_size);
        DCIH_HIP(hipGetLastError());
    }
    return 0;
}

}  // namespace dcih
