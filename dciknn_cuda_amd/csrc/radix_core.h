// Least-significant-digit radix sort of NT * IPT items held in registers by a
// workgroup of NT threads, in LDS, 4 bits per pass.
#pragma once

#include "common.h"

namespace dcih {
namespace {

// On entry thread t holds items t*IPT .. t*IPT+IPT-1 (blocked): k[r] the 32-bit key,
// rp[r] a 16-bit payload in its low half.  On return the items are sorted ascending by
// key, stably, again blocked.  `stage` is LDS for IPT * NT words (its contents are
// lost), `cnt32` LDS for 8 * NT words (the digit counters, [16][NT] 16-bit values,
// digit-major), `misc` 16 more words; `varying` has a bit set wherever the keys differ (nibbles that
// are zero in it are skipped).  Thread-private counters and the digit-major scan make
// every pass stable.  All NT threads must call this; it begins and ends with the items
// in registers only (callers need a barrier before they reuse `stage`).
template <int NT, int IPT>
__device__ inline void lds_radix_passes(uint32_t (&k)[IPT], uint32_t (&rp)[IPT], uint32_t* stage,
                                        uint32_t* cnt32, uint32_t* misc, uint32_t varying) {
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    uint16_t* cnt = reinterpret_cast<uint16_t*>(cnt32);
    for (int shift = 0; shift < 32; shift += 4) {
        if (((varying >> shift) & 15u) == 0u) continue;          // same nibble everywhere
        __syncthreads();
        {   // count digits in thread-private LDS counters (no atomics, order-preserving)
#pragma unroll
            for (int w = 0; w < 8; w++) cnt32[tid + w * NT] = 0;
            __syncthreads();
            // A returning atomic on the word that holds the counter (two neighbouring
            // threads share a word): the LDS unit does the read-modify-write in issue
            // order, so the IPT updates of a thread need no round trip between them.
            const uint32_t half = (uint32_t)(tid & 1) * 16u;
            uint32_t old[IPT];
#pragma unroll
            for (int r = 0; r < IPT; r++) {
                const uint32_t a = ((k[r] >> shift) & 15u) * NT + tid;
                old[r] = atomicAdd(&cnt32[a >> 1], 1u << half);
                if ((r & 7) == 7) __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int r = 0; r < IPT; r++)
                rp[r] = (rp[r] & 0xffffu) | (((old[r] >> half) & 0xffffu) << 16);
        }
        __syncthreads();
        {   // exclusive scan of the 16*threads counters in memory order (digit-major)
            uint32_t v[8];
            uint32_t sum = 0;
#pragma unroll
            for (int w = 0; w < 8; w++) { v[w] = cnt32[tid * 8 + w]; sum += (v[w] & 0xffffu) + (v[w] >> 16); }
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
            for (int w = 0; w < 8; w++) {
                const uint32_t lo = v[w] & 0xffffu, hi = v[w] >> 16;
                cnt32[tid * 8 + w] = run | ((run + lo) << 16);
                run += lo + hi;
            }
        }
        __syncthreads();
        // an opaque copy of the shift keeps the compiler from holding all IPT counter
        // addresses of the counting loop alive across the scan
        int shift2 = shift;
        asm volatile("" : "+s"(shift2));
#pragma unroll
        for (int r = 0; r < IPT; r++) {      // all counter reads first, then all stores:
            const uint32_t a = ((k[r] >> shift2) & 15u) * NT + tid;   // interleaved they
            rp[r] += (uint32_t)cnt[a] << 16;                                      // would wait on each other
            if ((r & 7) == 7) __builtin_amdgcn_sched_barrier(0);
        }
        // (scheduling fences every 8 items keep the unrolled loops from computing all
        //  IPT addresses up front, which would spill registers)
#pragma unroll
        for (int r = 0; r < IPT; r++) {
            stage[rp[r] >> 16] = k[r];
            if ((r & 7) == 7) __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < IPT; r++) {
            k[r] = stage[tid * IPT + r];
            if ((r & 7) == 7) __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < IPT; r++) {      // ids move as whole words: 16-bit blocked reads would
            stage[rp[r] >> 16] = rp[r] & 0xffffu;                // collide on LDS banks
            if ((r & 7) == 7) __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < IPT; r++) {
            rp[r] = stage[tid * IPT + r];
            if ((r & 7) == 7) __builtin_amdgcn_sched_barrier(0);
        }
    }

}

}  // namespace
}  // namespace dcih
