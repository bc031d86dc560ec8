// Shared helpers of the gfx950 DCI engine (host + device).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

namespace dcih {

constexpr int kWave = 64;

// Records `msg` as the calling thread's last error and returns `code`.
int fail(int code, const std::string& msg);

#define DCIH_HIP(call)                                                          \
    do {                                                                        \
        hipError_t e_ = (call);                                                 \
        if (e_ != hipSuccess)                                                   \
            return ::dcih::fail(-3, std::string(#call) + ": " + hipGetErrorString(e_)); \
    } while (0)

// ---- order-preserving float <-> uint32 ------------------------------------
// Ascending unsigned order of the result equals ascending float order
// (-0.0 sorts just below +0.0; the projection kernel never emits -0.0).
__host__ __device__ inline uint32_t f2ord(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__host__ __device__ inline float ord2f(uint32_t u) {
    u = (u & 0x80000000u) ? (u & 0x7fffffffu) : ~u;
    return __builtin_bit_cast(float, u);
}

#if defined(__HIPCC__)
// ---- wavefront (64-lane) reductions ----------------------------------------
__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}
__device__ inline uint32_t wave_min_u32(uint32_t v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        uint32_t w = (uint32_t)__shfl_xor((int)v, o, kWave);
        v = w < v ? w : v;
    }
    return v;
}
__device__ inline unsigned long long wave_max_u64(unsigned long long v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        unsigned long long w = __shfl_xor(v, o, kWave);
        v = w > v ? w : v;
    }
    return v;
}
__device__ inline int lane_id() { return (int)(threadIdx.x & (kWave - 1)); }

// In-place ascending bitonic sort of `n` (a power of two) 64-bit words in LDS
// by all threads of the block.
__device__ inline void bitonic_sort_u64(unsigned long long* s, int n) {
    for (int size = 2; size <= n; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            __syncthreads();
            for (int t = threadIdx.x; t < (n >> 1); t += blockDim.x) {
                int lo = 2 * t - (t & (stride - 1));
                int hi = lo + stride;
                bool up = (lo & size) == 0;
                unsigned long long a = s[lo], b = s[hi];
                if ((a > b) == up) { s[lo] = b; s[hi] = a; }
            }
        }
    }
    __syncthreads();
}
#endif

}  // namespace dcih
