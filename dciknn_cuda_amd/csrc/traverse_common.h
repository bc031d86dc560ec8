// Device helpers shared by the batch and the dense traversal kernels: the window
// streams of a simple index (dci_next_closest_proj, src/dci_cuda_kernel.cu:250-273,
// and the priority clamp, :572-590) in closed form, and searches done by lane groups.
#pragma once

#include "common.h"

namespace dcih {
namespace {

constexpr uint32_t kInfBits = 0x7f800000u;

__host__ __device__ inline int counter_bits_of(int L) {
    return L <= 15 ? 4 : (L <= 255 ? 8 : (L <= 65535 ? 16 : 32));
}

struct Stream {          // one side of one simple index within the partition
    const float* key;    // sorted keys of the slice
    int n, T, p, side;   // side: 0 = left of the query position, 1 = right
    float q;
};

// Priority of window j of a stream: |key[clamped start] - q| (:572-590).
__device__ inline uint32_t stream_prio_bits(const Stream& s, int j) {
    const int pos = s.side ? min(s.p + 1 + j * s.T, s.n - 1) : max(s.p - s.T + 1 - j * s.T, 0);
    return __builtin_bit_cast(uint32_t, fabsf(s.key[pos] - s.q));
}

// Number of windows j in [lo, hi) of the stream with priority < x (strict) or
// <= x, given that the predicate is monotone in j.
__device__ inline int count_below(const Stream& s, uint32_t x, bool strict, int lo, int hi,
                                  uint32_t& probes) {
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        const uint32_t v = stream_prio_bits(s, mid);
        probes++;
        if (strict ? v < x : v <= x) lo = mid + 1; else hi = mid;
    }
    return lo;
}

// Windows in a stream: right NR = floor((n+T-3-p)/T)+1 (0 if negative), left
// NL = ceil((p+1)/T); from the bounds of dci_next_closest_proj (:254-263).
__device__ inline int stream_windows(int n, int T, int p, int side) {
    if (side) {
        const int v = n + T - 3 - p;
        return v < 0 ? 0 : v / T + 1;
    }
    return (p + T) / T;   // ceil((p + 1) / T)
}

// Index positions [a, b) covered by windows [c0, c1) of a stream.
__device__ inline void stream_range(int n, int T, int p, int side, int c0, int c1, int& a, int& b) {
    if (side) {
        a = min((int64_t)n, (int64_t)p + 1 + (int64_t)c0 * T);
        b = min((int64_t)n, (int64_t)p + 1 + (int64_t)c1 * T);
    } else {
        a = max((int64_t)0, (int64_t)p + 1 - (int64_t)c1 * T);
        b = max((int64_t)0, (int64_t)p + 1 - (int64_t)c0 * T);
    }
}

__device__ inline unsigned long long pack_event(uint32_t time, int m, bool lane0, uint32_t local) {
    return ((unsigned long long)time << 32) | ((unsigned long long)m << 26) |
           ((unsigned long long)(lane0 ? 1u : 0u) << 25) | local;
}

// Partition point of a monotone predicate (true, then false) over [lo, hi), found by
// a group of G = 2^lg consecutive lanes that probe the midpoints of G equal parts per
// round: log_G rounds of dependent reads instead of log_2.  A group lies within one
// wavefront and starts at lane `gbase`; `g` is the lane's place in it.  Every lane of
// the wavefront must call this (the rounds are wave-uniform); lanes without a group
// pass active = false.  hi - lo must stay below 2^31 / (2 G).
template <class Pred>
__device__ inline int group_partition_point(int lo, int hi, bool active, int lg, int gbase, int g,
                                            Pred pred, uint32_t& probes) {
    const int G = 1 << lg;
    if (!active) { lo = 0; hi = 0; }
    while (__any(lo < hi)) {
        const bool busy = lo < hi;
        const uint32_t len = (uint32_t)(hi - lo);
        bool t = false;
        if (busy) {
            probes++;
            t = pred(lo + (int)((len * (uint32_t)(2 * g + 1)) >> (lg + 1)));
        }
        const unsigned long long m = __ballot(t);
        if (busy) {
            // positions rise with the lane and the predicate is monotone: the hits are a prefix
            const int hits = __popcll((m >> gbase) & ((1ull << G) - 1ull));
            const int last_hit = lo + (int)((len * (uint32_t)(2 * hits - 1)) >> (lg + 1));     // lane hits-1
            const int first_miss = lo + (int)((len * (uint32_t)(2 * hits + 1)) >> (lg + 1));   // lane hits
            if (hits < G) hi = first_miss;
            if (hits > 0) lo = last_hit + 1;
        }
    }
    return lo;
}
// Where traversals of a partition usually stop: stop_hint is [3][B] -- the sum of the stop
// steps, the sum of the promotions at the stop, and the number of stops recorded, per
// partition.  Many workgroups record at once, so the sums are formed by atomic additions; a
// partition stops recording after kHintStops stops, which makes the averages (and with them
// the sizes of the batch kernel's epochs) the same from then on.  They steer work, never results.
// All workgroups an accelerator die runs at one time work on the same partition, so their additions
// hit the same three words and queue up behind each other (a quarter more time for a whole call
// when every stop is recorded): after the first kHintEveryStop stops only every eighth query's
// stops are recorded, which spreads the same number of samples over eight times as many stops.
constexpr float kHintStops = 512.0f;
constexpr float kHintEveryStop = 64.0f;
__device__ inline void record_stop(float* stop_hint, int B, int b, int query, float steps, float promotions) {
    const float have = stop_hint[2 * B + b];
    if (have >= kHintStops || (have >= kHintEveryStop && (query & 7) != 0)) return;
    atomicAdd(&stop_hint[b], steps);
    atomicAdd(&stop_hint[B + b], promotions);
    atomicAdd(&stop_hint[2 * B + b], 1.0f);
}
// (average stop step, average promotions at the stop); zeros while nothing is recorded.  The
// three words are read at different moments, so the averages can be off by a stop's share.
__device__ inline void usual_stop(const float* stop_hint, int B, int b, float& steps, float& promotions) {
    const float stops = stop_hint[2 * B + b];
    steps = stops > 0.0f ? stop_hint[b] / stops : 0.0f;
    promotions = stops > 0.0f ? stop_hint[B + b] / stops : 0.0f;
}
// x^y for x > 0 from the hardware's log2 / exp2 approximations (epoch sizing only)
__device__ inline float fast_pow(float x, float y) { return __builtin_amdgcn_exp2f(__builtin_amdgcn_logf(x) * y); }
__host__ __device__ inline int floor_log2(int v) { int l = 0; while ((2 << l) <= v) l++; return l; }


}  // namespace
}  // namespace dcih
