// Shared helpers of the gfx950 DCI engine (host + device).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>
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

// Runs `set_up` once per device (the current one) and remembers success: kernel
// attributes are kept per device, and several host threads may launch at once.
class DeviceOnce {
public:
    template <class F>
    int run(F set_up) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return set_up();
        std::lock_guard<std::mutex> lock(mu_);
        if (done_[dev]) return 0;
        const int rc = set_up();
        if (rc == 0) done_[dev] = true;
        return rc;
    }
private:
    static constexpr int kMaxDevices = 64;
    std::mutex mu_;
    bool done_[kMaxDevices] = {};
};

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
// ---- exchanges between the lanes of a wavefront -----------------------------------
// The value lane (l ^ O) holds, O a power of two below 64, without an address register: within
// quads by DPP, within 32 lanes by ds_swizzle with an immediate pattern, across the halves by
// v_permlane32_swap.  (__shfl_xor computes a byte address per lane from the lane number, which
// the compiler then keeps alive -- or spills -- across a whole kernel.)
template <int O>
__device__ inline uint32_t lane_xor_u32(uint32_t v) {
    static_assert(O == 1 || O == 2 || O == 4 || O == 8 || O == 16 || O == 32, "one lane bit");
    if constexpr (O == 1) {
        return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xf, 0xf, true);      // quad_perm [1,0,3,2]
    } else if constexpr (O == 2) {
        return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x4E, 0xf, 0xf, true);      // quad_perm [2,3,0,1]
    } else if constexpr (O == 32) {
        // after the swap, [0] holds in its upper half what the lower half of v held, and [1] in its
        // lower half what the upper half held
        const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
        uint32_t out;
        asm("v_cndmask_b32 %0, %1, %2, %3" : "=v"(out) : "v"(r[1]), "v"(r[0]), "s"(0xffffffff00000000ull));
        return out;
    } else {
        return (uint32_t)__builtin_amdgcn_ds_swizzle((int)v, (O << 10) | 0x1f);       // xor mask, and mask 0x1f
    }
}
template <int O> __device__ inline int lane_xor(int v) { return (int)lane_xor_u32<O>((uint32_t)v); }
template <int O> __device__ inline uint32_t lane_xor(uint32_t v) { return lane_xor_u32<O>(v); }
template <int O> __device__ inline float lane_xor(float v) {
    return __builtin_bit_cast(float, lane_xor_u32<O>(__builtin_bit_cast(uint32_t, v)));
}
template <int O> __device__ inline unsigned long long lane_xor(unsigned long long v) {
    return ((unsigned long long)lane_xor_u32<O>((uint32_t)(v >> 32)) << 32) | lane_xor_u32<O>((uint32_t)v);
}

// The same for a distance that is a constant only after loop unrolling.
__device__ inline unsigned long long lane_xor_any(unsigned long long v, int o) {
    switch (o) {
        case 1: return lane_xor<1>(v);
        case 2: return lane_xor<2>(v);
        case 4: return lane_xor<4>(v);
        case 8: return lane_xor<8>(v);
        case 16: return lane_xor<16>(v);
        default: return lane_xor<32>(v);
    }
}

// ---- wavefront (64-lane) reductions ----------------------------------------
// (levels in the order 32, 16, .., 1: the traversal kernels rely on this order for equal bits)
__device__ inline float wave_sum(float v) {
    v += lane_xor<32>(v); v += lane_xor<16>(v); v += lane_xor<8>(v);
    v += lane_xor<4>(v); v += lane_xor<2>(v); v += lane_xor<1>(v);
    return v;
}
__device__ inline uint32_t wave_min_u32(uint32_t v) {
    v = min(v, lane_xor<32>(v)); v = min(v, lane_xor<16>(v)); v = min(v, lane_xor<8>(v));
    v = min(v, lane_xor<4>(v)); v = min(v, lane_xor<2>(v)); v = min(v, lane_xor<1>(v));
    return v;
}
__device__ inline uint32_t wave_sum_u32(uint32_t v) {
    v += lane_xor<32>(v); v += lane_xor<16>(v); v += lane_xor<8>(v);
    v += lane_xor<4>(v); v += lane_xor<2>(v); v += lane_xor<1>(v);
    return v;
}
__device__ inline int wave_max_i32(int v) {
    v = max(v, lane_xor<32>(v)); v = max(v, lane_xor<16>(v)); v = max(v, lane_xor<8>(v));
    v = max(v, lane_xor<4>(v)); v = max(v, lane_xor<2>(v)); v = max(v, lane_xor<1>(v));
    return v;
}
__device__ inline unsigned long long wave_max_u64(unsigned long long v) {
    unsigned long long w;
    w = lane_xor<32>(v); v = w > v ? w : v;
    w = lane_xor<16>(v); v = w > v ? w : v;
    w = lane_xor<8>(v); v = w > v ? w : v;
    w = lane_xor<4>(v); v = w > v ? w : v;
    w = lane_xor<2>(v); v = w > v ? w : v;
    w = lane_xor<1>(v); v = w > v ? w : v;
    return v;
}
__device__ inline int lane_id() { return (int)(threadIdx.x & (kWave - 1)); }

// Euclidean distances (compute_dist_device, src/dci_cuda_kernel.cu:36-44) from R
// rows in global memory to the query held in LDS, by one wavefront.  With
// 16-byte aligned rows (vec4) lane l sums the squares of elements 4l..4l+3,
// 4l+256.., in ascending order, otherwise of elements l, l+64, ..; the lane sums
// are then added across the wavefront.  Both traversal kernels call this, so a
// point gets the same distance bits whichever kernel visits it; R > 1 only
// interleaves the reads of independent rows.
template <int R>
__device__ inline void wave_row_dists(const float* const (&rows)[R], const float* q, int dim,
                                      bool vec4, float (&dist)[R], int lane = -1) {
    if (lane < 0) lane = lane_id();      // (callers that keep their own lane number pass it)
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.f;
    if (vec4) {
        typedef float v4f __attribute__((ext_vector_type(4)));
        for (int j = lane * 4; j < dim; j += kWave * 4) {
            v4f x[R];
#pragma unroll
            for (int r = 0; r < R; r++) x[r] = *reinterpret_cast<const v4f*>(rows[r] + j);
            const float q0 = q[j], q1 = q[j + 1], q2 = q[j + 2], q3 = q[j + 3];
#pragma unroll
            for (int r = 0; r < R; r++) {
                float d = x[r].x - q0; acc[r] = __builtin_fmaf(d, d, acc[r]);
                d = x[r].y - q1; acc[r] = __builtin_fmaf(d, d, acc[r]);
                d = x[r].z - q2; acc[r] = __builtin_fmaf(d, d, acc[r]);
                d = x[r].w - q3; acc[r] = __builtin_fmaf(d, d, acc[r]);
            }
        }
    } else {
        for (int j = lane; j < dim; j += kWave) {
            const float qj = q[j];
#pragma unroll
            for (int r = 0; r < R; r++) {
                const float d = rows[r][j] - qj;
                acc[r] = __builtin_fmaf(d, d, acc[r]);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) dist[r] = sqrtf(wave_sum(acc[r]));
}
// The same sums in the same order for 16-byte aligned rows of at least 256
// elements, with no lane condition around a read: U pieces (256 elements apart) of each of
// the R rows are read at once by every lane; a lane whose piece would begin past the row's
// end reads the row's first piece again and adds nothing.  (Rows whose length is no multiple
// of 256 elements otherwise end in an extra round of reads by a few lanes.)
template <int R, int U>
__device__ inline void wave_row_dists_wide(const float* const (&rows)[R], const float* q, int dim,
                                           float (&dist)[R]) {
    typedef float v4f __attribute__((ext_vector_type(4)));
    const int lane = lane_id();
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.f;
    for (int j0 = 0; j0 < dim; j0 += U * kWave * 4) {
        v4f x[U][R];
        int jc[U];
        bool ok[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int ju = j0 + u * kWave * 4 + lane * 4;
            ok[u] = ju < dim;
            jc[u] = ok[u] ? ju : lane * 4;
#pragma unroll
            for (int r = 0; r < R; r++) x[u][r] = *reinterpret_cast<const v4f*>(rows[r] + jc[u]);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const float q0 = q[jc[u]], q1 = q[jc[u] + 1], q2 = q[jc[u] + 2], q3 = q[jc[u] + 3];
#pragma unroll
            for (int r = 0; r < R; r++) {
                float s2 = acc[r];
                float d = x[u][r].x - q0; s2 = __builtin_fmaf(d, d, s2);
                d = x[u][r].y - q1; s2 = __builtin_fmaf(d, d, s2);
                d = x[u][r].z - q2; s2 = __builtin_fmaf(d, d, s2);
                d = x[u][r].w - q3; s2 = __builtin_fmaf(d, d, s2);
                acc[r] = ok[u] ? s2 : acc[r];
            }
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) dist[r] = sqrtf(wave_sum(acc[r]));
}
// Whether every row of `data` starts on a 16-byte boundary.
__device__ inline bool rows_vec4(const float* data, int dim) {
    return (dim & 3) == 0 && (reinterpret_cast<uintptr_t>(data) & 15) == 0;
}

// In-place ascending bitonic sort of `n` (a power of two) 64-bit words in LDS
// by all threads of the block (which has at least one full wavefront).
template <int SIZE, int STRIDE>
__device__ inline void bitonic_wave_steps(unsigned long long& v, int lane, int n) {
    if (SIZE <= n) {       // (same on every lane)
        const unsigned long long o = lane_xor<STRIDE>(v);
        const bool keep_min = ((lane & STRIDE) == 0) == ((lane & SIZE) == 0);
        v = keep_min ? (v < o ? v : o) : (v > o ? v : o);
    }
    if constexpr (STRIDE > 1) bitonic_wave_steps<SIZE, STRIDE / 2>(v, lane, n);
    else if constexpr (SIZE < kWave) bitonic_wave_steps<SIZE * 2, SIZE>(v, lane, n);
}
// `tid` is the caller's thread number (a caller that hides its thread number from the
// compiler between phases passes its own copy).
__device__ inline void bitonic_sort_u64(unsigned long long* s, int n, int tid = -1) {
    if (tid < 0) tid = (int)threadIdx.x;
    if (n <= kWave) {
        // one wavefront sorts in registers with lane exchanges: no barrier per stage
        __syncthreads();
        if (tid < kWave) {
            const int lane = tid;
            unsigned long long v = lane < n ? s[lane] : ~0ull;
            bitonic_wave_steps<2, 1>(v, lane, n);
            if (lane < n) s[lane] = v;
        }
        __syncthreads();
        return;
    }
    for (int size = 2; size <= n; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            __syncthreads();
            for (int t = tid; t < (n >> 1); t += blockDim.x) {
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

// The same sort for n = 256 * E words by a workgroup of exactly 256 threads, E a power of
// two: every thread keeps E consecutive words in registers, exchanges within a thread and
// within a wavefront need neither LDS nor a barrier, and only the steps whose partners lie in
// another wavefront (two or three of them in all) go through `s`.
template <int E>
__device__ inline void bitonic_sort_u64_regs(unsigned long long* s) {
    constexpr int n = 256 * E;
    const int tid = (int)threadIdx.x;
    unsigned long long v[E];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < E; i++) v[i] = s[tid * E + i];
#pragma unroll
    for (int size = 2; size <= n; size <<= 1) {
#pragma unroll
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            if (stride >= kWave * E) {
                __syncthreads();
#pragma unroll
                for (int i = 0; i < E; i++) s[tid * E + i] = v[i];
                __syncthreads();
#pragma unroll
                for (int i = 0; i < E; i++) {
                    const int e = tid * E + i;
                    const unsigned long long o = s[e ^ stride];
                    const bool keep_min = ((e & stride) == 0) == ((e & size) == 0);
                    v[i] = keep_min ? (v[i] < o ? v[i] : o) : (v[i] > o ? v[i] : o);
                }
            } else if (stride >= E) {
#pragma unroll
                for (int i = 0; i < E; i++) {
                    const int e = tid * E + i;
                    const unsigned long long o = lane_xor_any(v[i], stride / E);
                    const bool keep_min = ((e & stride) == 0) == ((e & size) == 0);
                    v[i] = keep_min ? (v[i] < o ? v[i] : o) : (v[i] > o ? v[i] : o);
                }
            } else {
#pragma unroll
                for (int i = 0; i < E; i++) {
                    if ((i & stride) == 0) {
                        const int e = tid * E + i;
                        const bool up = (e & size) == 0;
                        const unsigned long long x = v[i], y = v[i | stride];
                        const bool swap = (x > y) == up;
                        v[i] = swap ? y : x;
                        v[i | stride] = swap ? x : y;
                    }
                }
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < E; i++) s[tid * E + i] = v[i];
    __syncthreads();
}
// n words by 256 threads: the register variant where it applies.
__device__ inline void bitonic_sort_u64_by256(unsigned long long* s, int n) {
    if (n == 256) bitonic_sort_u64_regs<1>(s);
    else if (n == 512) bitonic_sort_u64_regs<2>(s);
    else if (n == 1024) bitonic_sort_u64_regs<4>(s);
    else bitonic_sort_u64(s, n);
}
#endif

}  // namespace dcih
