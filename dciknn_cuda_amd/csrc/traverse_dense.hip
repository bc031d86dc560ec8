// Dense traversal: one workgroup per (query, partition) computes, for EVERY point
// of the partition, the outer step at which the loop of
// dci_query_single_point_by_block (src/dci_cuda_kernel.cu:401-626) would promote
// it, and from those steps the stop step, the candidates and their k best.
//
// It is the kernel for traversals that visit a large part of the index before
// they stop (hundreds or thousands of promotions per partition): there the batch
// kernel's cost per promotion (a rank by 2L binary searches, a replay) dominates,
// while the work here does not depend on where the loop stops.  Facts used, the
// same as in the batch kernel: a composite index consumes its windows in
// ascending (priority, simple index, order within the simple index), window
// number r at outer step r; a point is promoted under a composite at the step of
// the last of the L windows that hold it and is a candidate at its earliest
// (step, composite); the loop stops at the first step t with c0(t) >= k and
// (t + 1 >= outer * L or c0(t) >= max_candidates), c0 counting candidates whose
// promoting window held them in lane 0 (:598-607).
//
// Per composite index: the priorities |key[clamped window start] - q| (:572-590)
// of all its windows are laid out by (simple index, order within it) and sorted
// stably in LDS, which gives every window its step; every point then looks up the
// steps of its L windows (positions from the inverse permutation) and keeps the
// largest.  A histogram of the steps of lane-0 candidates yields the stop step;
// points promoted up to it get their exact distances (rows read by whole
// wavefronts) and go through a k-best filter.  Shapes that do not fit the tables
// are left to the other kernels through the same hand-over list.
#include <type_traits>

#include "common.h"
#include "kernels.h"
#include "radix_core.h"
#include "traverse_common.h"

namespace dcih {

namespace {

constexpr int kDT = 256;                 // threads per workgroup
constexpr int kDWaves = kDT / kWave;
constexpr uint32_t kNever = 0xffffu;     // step field of a point that is never promoted

enum DMisc {   // 32-bit scalars shared by the workgroup
    dWin = 0, dFail, dArmed, dMaxc, dCand, dProbes, dMore, dOr, dAnd, dMaxW, dWavePend0,
    dMiscWords = 16
};

struct DenseLayout {
    int ipt;          // windows per thread the sort holds (cap = 256 * ipt per composite)
    int off_idx;      // per simple index: p, qp, left start, right start   (4 * I words)
    int off_seg;      // per composite: 2L + 1 segment starts, 2L stream numbers, 2L table places of window 0
    int off_q;        // query row
    int off_time;     // uint16 per point: step << 1 | lane-0 flag
    int off_sort;     // k best + pending candidates, 64-bit words
    int off_stage;    // radix staging; later the rank table, then the step histogram
    int off_misc, off_wlist;
    int sort_cap, quota;
    int tiles;        // 1: rows of at most 128 elements, 16-byte aligned, distances wanted: whole batches of 64 rows
    size_t lds_bytes;
};

constexpr int kWlist = 2 * kWave;        // candidates a wavefront keeps listed

int dense_ipt_for(int64_t windows) {
    for (int ipt : {9, 17, 25, 33, 41})
        if (windows <= (int64_t)kDT * ipt) return ipt;
    return 0;
}

// Upper bound of the windows of one composite index: per simple index at most
// ceil((p+1)/T) + floor((n+T-3-p)/T) + 1 <= n/T + 3.
int64_t dense_max_windows(const QueryArgs& a) { return (int64_t)a.L * (a.ppb / a.T + 3); }

DenseLayout make_dense_layout(const QueryArgs& a) {
    DenseLayout y;
    const int I = a.M * a.L;
    y.ipt = dense_ipt_for(dense_max_windows(a));
    int o = dMiscWords * 4 + 64 * 4;      // scalars, then scratch of the block scans
    y.off_misc = 0;
    y.off_idx = o;      o += 4 * I * 4;
    y.off_seg = o;      o += (6 * a.L + 2) * 4;
    y.off_q = o;        o += ((a.dim + 3) & ~3) * 4;
    y.off_time = o;     o += (int)(((a.ppb + 1) & ~(int64_t)1) * 2);
    o = (o + 15) & ~15;
    // k best plus room for candidates that beat the current k-th: four wavefronts fill
    // a quota each between two merges
    // (batches of 64 rows: room for one whole batch beyond what a wavefront may hold already)
    y.tiles = (!a.blind && a.dim <= 128 && (a.dim & 3) == 0 &&
               (reinterpret_cast<uintptr_t>(a.data) & 15) == 0) ? 1 : 0;
    y.sort_cap = 64;
    while (y.sort_cap < a.kcap + 4 * (y.tiles ? 96 : 8)) y.sort_cap <<= 1;
    y.quota = (y.sort_cap - a.kcap) / kDWaves;
    y.off_sort = o;     o += y.sort_cap * 8;
    y.off_wlist = o;    o += kDWaves * kWlist * 2;
    y.off_stage = o;    o += (y.ipt + 8) * kDT * 4;      // staging words, then the digit counters
    y.lds_bytes = (size_t)o;
    return y;
}

// Sums of N rows' lane values over a group of N lanes at once: on entry lane s of the group
// holds v[r] = its share of row r; on return it holds the total of row s.  Each level pairs
// the lanes s and s ^ H and halves the rows a lane carries, adding exactly the operands the
// butterfly  v += shfl_xor(v, H)  of wave_sum adds for that row, in the same order of levels,
// so every total has the bits wave_row_dists gives (N - 1 exchanges for N rows, not N log N).
template <int N>
__device__ inline float group_row_sums(float (&v)[N], int s) {
    if constexpr (N == 1) {
        return v[0];
    } else {
        constexpr int H = N / 2;
        const bool upper = (s & H) != 0;
        float nv[H];
#pragma unroll
        for (int i = 0; i < H; i++) {
            const float send = upper ? v[i] : v[i + H];
            const float keep = upper ? v[i + H] : v[i];
            nv[i] = keep + lane_xor<H>(send);
        }
        return group_row_sums<H>(nv, s);
    }
}

typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// WPS = wavefronts per SIMD the register allocation leaves room for: three where the tables let
// three workgroups share a CU's LDS, else two (and 256 registers instead of 168).
template <int IPT, int WPS>
__global__ __launch_bounds__(kDT, WPS) void traverse_dense_kernel(QueryArgs a, DenseLayout y) {
    extern __shared__ __align__(16) unsigned char smem[];
    uint32_t* misc = reinterpret_cast<uint32_t*>(smem);
    uint32_t* scan_tmp = misc + dMiscWords;                           // 64 words
    int* s_p = reinterpret_cast<int*>(smem + y.off_idx);
    float* s_qp = reinterpret_cast<float*>(s_p + a.M * a.L);
    // per simple index: where its windows start in the step table (there they lie in the order
    // of the positions they cover), and the shift that makes (position + shift) / T a window's
    // place among them
    int* s_tabbase = reinterpret_cast<int*>(s_qp + a.M * a.L);
    int* s_shift = s_tabbase + a.M * a.L;
    int* s_seg = reinterpret_cast<int*>(smem + y.off_seg);            // 2L + 1 segment starts (layout order)
    int* s_segstream = s_seg + 2 * a.L + 1;                           // stream (2h + side) of a segment
    float* s_q = reinterpret_cast<float*>(smem + y.off_q);
    uint16_t* s_time = reinterpret_cast<uint16_t*>(smem + y.off_time);
    unsigned long long* sortbuf = reinterpret_cast<unsigned long long*>(smem + y.off_sort);
    uint32_t* stage = reinterpret_cast<uint32_t*>(smem + y.off_stage);
    uint16_t* rank16 = reinterpret_cast<uint16_t*>(stage);
    uint16_t* s_wlist = reinterpret_cast<uint16_t*>(smem + y.off_wlist);   // per wavefront: kWlist candidates
    int* s_segw = s_segstream + 2 * a.L;                              // table place of a segment's window 0

    // The thread numbers are made opaque again at the start of every phase, and every phase ends
    // in an exit that is never taken but that the compiler cannot rule out (PHASE_END): otherwise
    // each phase's lane groupings, per-thread addresses and loop-invariant loads are computed
    // once, ahead of the loop over the items, and carried through every other phase in registers
    // or scratch.
    int tid = threadIdx.x;
    int lane = tid & (kWave - 1);
    int wave = tid / kWave;
    auto fresh_thread_ids = [&]() {
        asm volatile("" : "+v"(tid));
        lane = tid & (kWave - 1);
        wave = tid / kWave;
    };
#define PHASE_END(which)                                 \
    do {                                                 \
        phase(which);                                    \
        int leave_now = 0;                               \
        asm volatile("" : "+s"(leave_now));              \
        if (leave_now) return;                           \
        fresh_thread_ids();                              \
    } while (0)
    const int I = a.M * a.L;
    const int T = a.T;
    const int X = a.xcds;
    const int xcd = (int)(blockIdx.x % X);
    const int64_t g0 = blockIdx.x / X, G = gridDim.x / X;
    const bool listed = a.dense_items != nullptr && a.mode != 3;
    const int64_t my_count = listed ? (int64_t)a.dense_count[xcd]
                                    : block_items(X, a.B, a.q_count) / X;

    // optional phase profile: thread 0 adds the 100 MHz ticks each phase took
    unsigned long long tick = 0ull;
    auto phase = [&](int which) {
        if (a.phase_ticks && tid == 0) {
            const unsigned long long now = wall_clock64();
            atomicAdd(&a.phase_ticks[which], now - tick);
            tick = now;
        }
    };

    for (int64_t slot = g0; slot < my_count; slot += G) {
        int b, qi;
        if (listed) {
            const int64_t item = a.dense_items[(int64_t)xcd * a.dense_cap + slot];
            b = (int)(item % a.B);
            qi = (int)(item / a.B);
        } else {
            if (!block_item(slot * X + xcd, X, a.B, a.q_count, b, qi)) continue;
            qi += a.q_first;
        }
        const int64_t item = (int64_t)qi * a.B + b;
        const int64_t off = (int64_t)b * a.ppb;
        const int n = (int)min(a.N - off, a.ppb);
        unsigned long long* part_out = a.part + item * a.kcap;
        __syncthreads();                         // the previous item's tables are done with
        if (n <= 0) {
            for (int j = tid; j < a.kcap; j += kDT) part_out[j] = ~0ull;
            continue;
        }

        // ---- set-up: query row, positioning searches (:279-297) -------------------
        if (a.phase_ticks) tick = wall_clock64();
        if (tid < dMiscWords) misc[tid] = 0;
        for (int j = tid; j < a.dim; j += kDT) s_q[j] = a.query[(int64_t)qi * a.dim + j];
        for (int pt = tid; pt < n; pt += kDT) s_time[pt] = (uint16_t)((kNever << 1) & 0xffffu);
        uint32_t probes = 0;
        {
            const int per_wave = (I + kDWaves - 1) / kDWaves;
            const int lg = min(3, floor_log2(kWave / per_wave > 0 ? kWave / per_wave : 1)), Gq = 1 << lg;
            const int slots = kWave >> lg;
            for (int i0 = 0; i0 < I; i0 += slots * kDWaves) {
                const int sl = lane >> lg, i = i0 + wave * slots + sl;
                const bool active = i < I;
                const float* key = a.skeys + (int64_t)(active ? i : 0) * a.N + off;
                const float qp = active ? a.qproj[(int64_t)i * a.nq + qi] : 0.f;
                const int lo = group_partition_point(0, n, active, lg, sl * Gq, lane - sl * Gq,
                                                     [&](int j) { return key[j] < qp; }, probes);
                if (active && lane == sl * Gq) { s_p[i] = lo - 1; s_qp[i] = qp; }
            }
        }
        __syncthreads();
        PHASE_END(0);

        unsigned long long maxw = 0;             // most windows any composite has
        for (int m = 0; m < a.M; m++) {
            // ---- layout of the composite's windows: per simple index its left stream, then
            // its right one; where the query lies above every key the single (ghost) right
            // window comes first, as dci_next_closest_proj orders it (:264-265)
            // (one lane per simple index, the first wavefront: L <= 64)
            if (wave == 0) {
                const int h = lane;
                int nl = 0, nr = 0, p = 0;
                if (h < a.L) {
                    p = s_p[m * a.L + h];
                    nl = stream_windows(n, T, p, 0);
                    nr = stream_windows(n, T, p, 1);
                }
                int incl = nl + nr;
#pragma unroll
                for (int o = 1; o < kWave; o <<= 1) {
                    const int t2 = __shfl_up(incl, o, kWave);
                    if (lane >= o) incl += t2;
                }
                const int at = incl - (nl + nr);
                if (h < a.L) {
                    const int i = m * a.L + h;
                    const bool corner = p == n - 1 && T >= 2;
                    // In the table the index's windows lie by the positions they cover: left
                    // window j at place nl - 1 - j, right window j at nl + j; a position pos
                    // belongs to the window at place (pos + nl * T - p - 1) / T and is its first
                    // lane where that division leaves no remainder.
                    s_tabbase[i] = at;
                    s_shift[i] = nl * T - p - 1;
                    const int w_left = at + nl - 1, w_right = at + nl;
                    if (corner) {
                        s_seg[2 * h] = at; s_segstream[2 * h] = 2 * h + 1; s_segw[2 * h] = w_right;
                        s_seg[2 * h + 1] = at + nr; s_segstream[2 * h + 1] = 2 * h; s_segw[2 * h + 1] = w_left;
                    } else {
                        s_seg[2 * h] = at; s_segstream[2 * h] = 2 * h; s_segw[2 * h] = w_left;
                        s_seg[2 * h + 1] = at + nl; s_segstream[2 * h + 1] = 2 * h + 1; s_segw[2 * h + 1] = w_right;
                    }
                }
                const int total = __shfl(incl, a.L - 1, kWave);
                if (lane == 0) {
                    s_seg[2 * a.L] = total;
                    misc[dWin] = (uint32_t)total;
                    if (total > kDT * IPT || total >= 0x7fff) misc[dFail] = 1;
                    misc[dOr] = 0; misc[dAnd] = 0xffffffffu;
                }
            }
            __syncthreads();
            if (misc[dFail]) break;
            const int W = (int)misc[dWin];
            maxw = max(maxw, (unsigned long long)W);

            // ---- priorities of the windows, blocked: thread t holds layout indices t*IPT.. ----
            uint32_t k[IPT], rp[IPT];
            {
                int seg = 0;
                const int first = tid * IPT;
                {   // the first segment that ends behind `first` (empty segments are skipped)
                    int lo = 0, hi = 2 * a.L - 1;
                    while (lo < hi) {
                        const int mid = (lo + hi) >> 1;
                        if (s_seg[mid + 1] <= first) lo = mid + 1; else hi = mid;
                    }
                    seg = lo;
                }
                // (offsets from the composite's first slice; all reads are issued before any is used)
                const float* kbase = a.skeys + (int64_t)m * a.L * a.N + off;
                uint32_t koff[IPT];
                float qv[IPT];
                // Per segment: where its windows' keys lie and which way they run.  Window j of
                // a right stream starts at position p + 1 + j * T and takes table place
                // seg_w + j; of a left stream, p - T + 1 - j * T and seg_w - j; the key read is
                // the one at that position moved into the slice.
                int seg_end, pos_cur, pos_step, w_cur, w_step;
                uint32_t h_base;
                float q_seg;
                auto enter = [&](int idx) {
                    seg_end = s_seg[seg + 1];
                    const int sidx = s_segstream[seg], j = idx - s_seg[seg], h = sidx >> 1;
                    const int p = s_p[m * a.L + h];
                    q_seg = s_qp[m * a.L + h];
                    h_base = (uint32_t)h * (uint32_t)a.N;
                    if (sidx & 1) { pos_step = T; pos_cur = p + 1 + j * T; w_step = 1; w_cur = s_segw[seg] + j; }
                    else { pos_step = -T; pos_cur = p - T + 1 - j * T; w_step = -1; w_cur = s_segw[seg] - j; }
                };
                enter(first);
#pragma unroll
                for (int r = 0; r < IPT; r++) {
                    const int idx = first + r;
                    if (idx >= seg_end && seg < 2 * a.L - 1) {
                        do { seg++; } while (seg < 2 * a.L - 1 && s_seg[seg + 1] <= idx);
                        enter(idx);
                    }
                    koff[r] = h_base + (uint32_t)(idx < W ? min(max(pos_cur, 0), n - 1) : 0);
                    qv[r] = q_seg;
                    rp[r] = (uint32_t)(idx < W ? w_cur : 0);    // the sort's payload: the window's place in the table
                    pos_cur += pos_step;
                    w_cur += w_step;
                }
                float kv[IPT];
#pragma unroll
                for (int r = 0; r < IPT; r++) kv[r] = kbase[koff[r]];
                uint32_t vor = 0, vand = 0xffffffffu;
#pragma unroll
                for (int r = 0; r < IPT; r++) {
                    const int idx = first + r;
                    const uint32_t bits = __builtin_bit_cast(uint32_t, fabsf(kv[r] - qv[r]));
                    k[r] = idx < W ? bits : 0xffffffffu;      // pads sort last and stay last
                    vor |= idx < W ? bits : 0u;
                    vand &= idx < W ? bits : 0xffffffffu;
                }
                probes += IPT;
                for (int o = 32; o > 0; o >>= 1) {
                    vor |= (uint32_t)__shfl_xor((int)vor, o, kWave);
                    vand &= (uint32_t)__shfl_xor((int)vand, o, kWave);
                }
                if (lane == 0) { atomicOr(&misc[dOr], vor); atomicAnd(&misc[dAnd], vand); }
            }
            __syncthreads();
            PHASE_END(1);
            // the step of every window: its place in the sorted order, stored doubled with bit 0
            // set: a lookup subtracts one where the point is not the window's first lane, which
            // leaves the lane-0 flag beside the step
            bool sorted_small = false;
            if constexpr (IPT == 9) {
                // Up to 1024 windows (short partitions): a bitonic sort held in registers of
                // (priority, layout index, table place) words — the layout index makes equal
                // priorities keep their order, as the stable radix passes do — takes a few
                // microseconds where eight radix passes over 2304 slots take thirty.
                if (W <= 1024) {
                    sorted_small = true;
                    const int np = W <= 256 ? 256 : (W <= 512 ? 512 : 1024);
                    unsigned long long* s64 = reinterpret_cast<unsigned long long*>(stage);
#pragma unroll
                    for (int r = 0; r < IPT; r++) {
                        const int idx = tid * IPT + r;
                        if (idx < np)
                            s64[idx] = idx < W ? ((unsigned long long)k[r] << 32) | ((unsigned long long)idx << 16) | (rp[r] & 0xffffu)
                                               : ~0ull;
                    }
                    bitonic_sort_u64_by256(s64, np);
                    unsigned long long mine[4];
                    const int per = np / kDT;
#pragma unroll
                    for (int e = 0; e < 4; e++) mine[e] = e < per ? s64[tid * per + e] : ~0ull;
                    __syncthreads();                    // the table takes the sorted words' room
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int sp = tid * per + e;
                        if (e < per && sp < W) rank16[(uint32_t)mine[e] & 0xffffu] = (uint16_t)((sp << 1) | 1);
                    }
                }
            }
            if (!sorted_small) {
                // (the pads need no pass of their own: they start behind every window, every
                //  digit of theirs is the largest, and the passes are stable)
                const uint32_t varying = misc[dOr] ^ misc[dAnd];
                lds_radix_passes<kDT, IPT>(k, rp, stage, stage + IPT * kDT, scan_tmp, varying);
                __syncthreads();
#pragma unroll
                for (int r = 0; r < IPT; r++) {
                    const int sp = tid * IPT + r;
                    if (sp < W) rank16[rp[r] & 0xffffu] = (uint16_t)((sp << 1) | 1);      // (the first W sorted items are the windows)
                }
            }
            __syncthreads();
            PHASE_END(2);

            // ---- every point: the latest of the steps of its L windows ------------------
            // A thread takes eight consecutive points at a time: their positions in one simple
            // index are one 16-byte read of the inverse permutation (slices start on 2-byte
            // boundaries; the reads need no more).  The reads for two simple indices make a
            // group, and the reads of three groups are in flight while one group is looked up
            // (the rows read for distances by the CU's other workgroup keep the memory system
            // busy: a read takes microseconds).  The last chunk of a slice is moved back to end at the
            // slice's end: some points are then looked up twice, with the same result.  The
            // phase is bound by vector-ALU issue, so the lookups are kept branch-free and short:
            // for a power-of-two T two points at a time in packed 16-bit arithmetic, otherwise
            // with 24-bit multiplies (32-bit ones run at a quarter of the rate).
            const uint16_t* invm = a.inv + (int64_t)m * a.L * a.N + off;
            auto store_time = [&](int pt, uint32_t b) __attribute__((always_inline)) {
                const uint32_t old = s_time[pt];      // ties: the earlier composite stays
                if ((b >> 1) < (old >> 1)) s_time[pt] = (uint16_t)b;
            };
            if (n < 8) {
                for (int pt = tid; pt < n; pt += kDT) {
                    uint32_t best = 0u;
                    for (int h = 0; h < a.L; h++) {
                        const int i = m * a.L + h;
                        const uint32_t x = (uint32_t)invm[(int64_t)h * a.N + pt] + (uint32_t)s_shift[i];
                        const uint32_t w = T > 1 ? __umulhi(x, a.T_magic) : x;
                        best = max(best, (uint32_t)rank16[s_tabbase[i] + w] - (x - w * (uint32_t)T != 0u ? 1u : 0u));
                    }
                    store_time(pt, best);
                }
            } else {
                auto run = [&](auto path_tag) __attribute__((always_inline)) {
                    constexpr int kPath = decltype(path_tag)::value;     // 0: T = 2^s, s >= 1; 1: any T >= 2; 2: T = 1
                    constexpr int kH = 2, kD = 4, kChunk = kDT * 8;
                    const int ngrp = (a.L + kH - 1) / kH;
                    const int NG = ((n + kChunk - 1) / kChunk) * ngrp;
                    const unsigned char* tab0 = reinterpret_cast<const unsigned char*>(rank16);
                    // path 0
                    const uint32_t sm1 = (uint32_t)floor_log2(T > 1 ? T : 2) - 1u;
                    const u16x2 sm1_pk = {(uint16_t)sm1, (uint16_t)sm1};
                    const u16x2 mask_pk = {(uint16_t)(T - 1), (uint16_t)(T - 1)};
                    const u16x2 one_pk = {1, 1};
                    // path 1: d / T for 0 <= d < 65536 is the upper 32 bits of (d << q_sh) *
                    // ceil(2^(32 - q_sh) / T); rounding the factor up adds less than 1 / T to d / T,
                    // which never reaches the next integer; q_sh = 8 serves 2 <= T <= 256, q_sh = 0
                    // the wider windows, and both factors stay below 2^24 either way.
                    const uint32_t q_sh = T <= 256 ? 8u : 0u;
                    const uint32_t q_magic = T > 1 ? (uint32_t)(((1ull << (32 - q_sh)) + (uint32_t)T - 1) / (uint32_t)T) : 0u;
                    const uint32_t q_T = (uint32_t)T << q_sh;
                    uint32_t best[kPath == 0 ? 4 : 8];     // path 0: two points a word
                    auto chunk_start = [&](int c0) { return min(c0 + 8 * tid, n - 8); };
                    auto issue = [&](int c0, int h0, u32x4 (&pv)[kH]) __attribute__((always_inline)) {
#pragma unroll
                        for (int hh = 0; hh < kH; hh++) {
                            const uint16_t* invh = invm + (int64_t)min(h0 + hh, a.L - 1) * a.N;
                            __builtin_memcpy(&pv[hh], invh + (uint32_t)chunk_start(c0), 16);
                        }
                    };
                    auto consume = [&](int c0, int h0, const u32x4 (&pv)[kH]) __attribute__((always_inline)) {
                        if (h0 == 0) {
#pragma unroll
                            for (int e = 0; e < (kPath == 0 ? 4 : 8); e++) best[e] = 0u;
                        }
                        // every table read of the group is issued before the first is used
                        uint32_t tv[kH][8];
                        u16x2 rem[kH][4];
#pragma unroll
                        for (int hh = 0; hh < kH; hh++) {
                            const int i = m * a.L + min(h0 + hh, a.L - 1);   // (past L: the last index again)
                            const uint32_t shift = (uint32_t)s_shift[i];
                            const unsigned char* tab = tab0 + 2 * s_tabbase[i];
                            const uint32_t wd[4] = {pv[hh].x, pv[hh].y, pv[hh].z, pv[hh].w};
#pragma unroll
                            for (int j = 0; j < 4; j++) {
                                if constexpr (kPath == 0) {
                                    const u16x2 shift_pk = {(uint16_t)shift, (uint16_t)shift};
                                    const u16x2 x = __builtin_bit_cast(u16x2, wd[j]) + shift_pk;
                                    // twice the window's place: the byte offset of its table entry
                                    const uint32_t w2 = __builtin_bit_cast(uint32_t, x >> sm1_pk) & 0xfffefffeu;
                                    // (spelled out: the compiler's own form of min(r, 1) is
                                    //  two compares, two selects and a byte permute)
                                    asm("v_pk_min_u16 %0, %1, %2" : "=v"(rem[hh][j]) : "v"(x & mask_pk), "v"(one_pk));
                                    tv[hh][2 * j] = *reinterpret_cast<const uint16_t*>(tab + (w2 & 0xffffu));
                                    tv[hh][2 * j + 1] = *reinterpret_cast<const uint16_t*>(tab + (w2 >> 16));
                                } else {
#pragma unroll
                                    for (int e = 0; e < 2; e++) {
                                        const uint32_t pos = e ? wd[j] >> 16 : wd[j] & 0xffffu;
                                        if constexpr (kPath == 1) {
                                            const uint32_t xs = (pos << q_sh) + (shift << q_sh);
                                            uint32_t w;
                                            asm("v_mul_hi_u32_u24 %0, %1, %2" : "=v"(w) : "s"(q_magic), "v"(xs));
                                            tv[hh][2 * j + e] = *reinterpret_cast<const uint16_t*>(tab + 2 * w);
                                            const uint32_t off_lane = (uint32_t)((uint32_t)__umul24(w, q_T) != xs);
                                            if (e) rem[hh][j].y = (uint16_t)off_lane; else rem[hh][j].x = (uint16_t)off_lane;
                                        } else {
                                            tv[hh][2 * j + e] = *reinterpret_cast<const uint16_t*>(tab + 2 * (pos + shift));
                                        }
                                    }
                                }
                            }
                        }
#pragma unroll
                        for (int hh = 0; hh < kH; hh++)
#pragma unroll
                            for (int j = 0; j < 4; j++) {
                                if constexpr (kPath == 0) {
                                    const u16x2 val =
                                        __builtin_bit_cast(u16x2, tv[hh][2 * j] | (tv[hh][2 * j + 1] << 16)) - rem[hh][j];
                                    best[j] = __builtin_bit_cast(uint32_t,
                                        __builtin_elementwise_max(__builtin_bit_cast(u16x2, best[j]), val));
                                } else if constexpr (kPath == 1) {
                                    best[2 * j] = max(best[2 * j], tv[hh][2 * j] - (uint32_t)rem[hh][j].x);
                                    best[2 * j + 1] = max(best[2 * j + 1], tv[hh][2 * j + 1] - (uint32_t)rem[hh][j].y);
                                } else {
                                    best[2 * j] = max(best[2 * j], tv[hh][2 * j]);
                                    best[2 * j + 1] = max(best[2 * j + 1], tv[hh][2 * j + 1]);
                                }
                            }
                        if (h0 + kH >= a.L) {
                            // (read, choose, write back unconditionally: a point that two threads
                            //  hold, at the moved-back end of a slice, gets the same value from both)
                            const int pt0 = chunk_start(c0);
                            uint32_t old[8];
#pragma unroll
                            for (int e = 0; e < 8; e++) old[e] = s_time[pt0 + e];
#pragma unroll
                            for (int e = 0; e < 8; e++) {
                                uint32_t b;
                                if constexpr (kPath == 0) b = (best[e >> 1] >> ((e & 1) * 16)) & 0xffffu;
                                else b = best[e];
                                // ties: the earlier composite stays
                                s_time[pt0 + e] = (uint16_t)((b >> 1) < (old[e] >> 1) ? b : old[e]);
                            }
                        }
                    };
                    // A ring of kD groups: the reads of the next kD - 1 groups are in flight while
                    // one group is looked up.  The loop body has no branch (the counters of reads
                    // under way are only exact in straight-line code): past the last group the reads
                    // repeat the slice's last chunk and the lookups change nothing that is stored.
                    int cc = 0, hc = 0, ci = 0, hi = 0;     // (chunk base, first simple index) of the group to consume / to issue
                    auto advance = [&](int& c, int& h) { h += kH; if (h >= a.L) { h = 0; c += kChunk; } };
                    u32x4 pv[kD][kH];
#pragma unroll
                    for (int d = 0; d < kD; d++) {
                        issue(ci, hi, pv[d]);
                        advance(ci, hi);
                    }
                    for (int g = 0; g < NG; g += kD) {
#pragma unroll
                        for (int d = 0; d < kD; d++) {
                            consume(cc, hc, pv[d]);
                            advance(cc, hc);
                            issue(ci, hi, pv[d]);
                            advance(ci, hi);
                        }
                    }
                };
                if (T > 1 && (T & (T - 1)) == 0) run(std::integral_constant<int, 0>{});
                else if (T > 1) run(std::integral_constant<int, 1>{});
                else run(std::integral_constant<int, 2>{});
            }
            __syncthreads();
            PHASE_END(3);
        }
        if (misc[dFail]) {      // does not fit the tables: the step-by-step kernel takes the item
            if (tid == 0) {
                const uint32_t s2 = atomicAdd(a.redo_count, 1u);
                a.redo_items[s2] = (int32_t)item;
            }
            continue;
        }

        // ---- stop step from the histogram of the steps of lane-0 candidates -----------
        const int HW = ((int)maxw + 2) / 2;                 // 32-bit words of the histogram (two steps each)
        for (int w = tid; w < HW; w += kDT) stage[w] = 0;
        if (tid == 0) { misc[dArmed] = 0xffffffffu; misc[dMaxc] = 0xffffffffu; }
        __syncthreads();
        for (int pt = tid; pt < n; pt += kDT) {
            const uint32_t v = s_time[pt];
            if ((v & 1u) && (v >> 1) != (kNever & 0x7fffu)) atomicAdd(&stage[v >> 2], 1u << (((v >> 1) & 1u) * 16));
        }
        __syncthreads();
        {
            const int per = (HW + kDT - 1) / kDT;           // words per thread, contiguous
            const int w0 = tid * per, w1 = min(HW, w0 + per);
            uint32_t sum = 0;
            for (int w = w0; w < w1; w++) { const uint32_t v = stage[w]; sum += (v & 0xffffu) + (v >> 16); }
            uint32_t incl = sum;
#pragma unroll
            for (int o = 1; o < kWave; o <<= 1) {
                const uint32_t t2 = (uint32_t)__shfl_up((int)incl, o, kWave);
                if (lane >= o) incl += t2;
            }
            if (lane == kWave - 1) scan_tmp[wave] = incl;
            __syncthreads();
            uint32_t run = incl - sum;
            for (int w2 = 0; w2 < wave; w2++) run += scan_tmp[w2];
            const uint32_t need_k = (uint32_t)a.k_stop;
            const uint32_t need_c = (uint32_t)min((int64_t)0x7fffffff, max((int64_t)1, a.max_cand));
            for (int w = w0; w < w1; w++) {
                const uint32_t v = stage[w];
                const uint32_t c_lo = run + (v & 0xffffu), c_hi = c_lo + (v >> 16);
                if (run < need_k && c_lo >= need_k) atomicMin(&misc[dArmed], (uint32_t)(2 * w));
                else if (c_lo < need_k && c_hi >= need_k) atomicMin(&misc[dArmed], (uint32_t)(2 * w + 1));
                if (run < need_c && c_lo >= need_c) atomicMin(&misc[dMaxc], (uint32_t)(2 * w));
                else if (c_lo < need_c && c_hi >= need_c) atomicMin(&misc[dMaxc], (uint32_t)(2 * w + 1));
                run = c_hi;
            }
        }
        __syncthreads();
        const uint32_t t_armed = misc[dArmed], t_maxc = misc[dMaxc];
        const bool stop = t_armed != 0xffffffffu;
        unsigned long long t_stop = ~0ull;                  // candidates: promoted at a step <= t_stop
        if (stop) {
            const unsigned long long last_needed = a.stop_at > 0 ? (unsigned long long)(a.stop_at - 1) : 0ull;
            const unsigned long long by_count = t_maxc != 0xffffffffu ? (unsigned long long)t_maxc : ~0ull;
            t_stop = max((unsigned long long)t_armed, min(last_needed, by_count));
        }
        const uint32_t t_lim = (uint32_t)min(t_stop, (unsigned long long)0x7ffe);   // every real step is below 0x7fff
        __syncthreads();                                    // the histogram's room is free again
        PHASE_END(4);

        // ---- distances of the candidates, k best ---------------------------------------
        // Every wavefront walks a quarter of the points; a candidate whose packed
        // (distance, id) does not beat the current k-th best is dropped at once, the others
        // wait in the wavefront's share of the buffer until the next merge.
        // Rows of up to 64 (128) elements are read by 16 (32) lanes each, four (two) rows
        // per load instruction and up to four such loads in flight; the lanes' partial sums
        // and the order in which they are added are those of wave_row_dists (the lanes a
        // short row leaves idle there add zeros), so the distances have the same bits.
        const bool vec4 = rows_vec4(a.data, a.dim);
        const int chunk = (n + kDWaves - 1) / kDWaves;
        int at = wave * chunk;                              // next point of this wavefront (wave-uniform)
        const int at_end = min(n, at + chunk);
        uint16_t* wl = s_wlist + wave * kWlist;             // this wavefront's candidates, listed 64 points at a time
        int list_len = 0, list_pos = 0;
        uint32_t ncand = 0;
        int topn = 0;
        // end of a round: the wavefronts' pending candidates are merged into the k best;
        // returns whether any wavefront has points left
        auto merge_round = [&](int mine, unsigned long long* my_slots) -> bool {
            for (int j = mine + lane; j < y.quota; j += kWave) my_slots[j] = ~0ull;
            const bool more = list_pos < list_len || at < at_end;
            if (lane == 0) {
                scan_tmp[8 + wave] = (uint32_t)mine;
                scan_tmp[16 + wave] = more ? 1u : 0u;
            }
            // (slots between the k best held so far and the first wavefront's share)
            for (int j = topn + tid; j < a.kcap; j += kDT) sortbuf[j] = ~0ull;
            for (int j = a.kcap + kDWaves * y.quota + tid; j < y.sort_cap; j += kDT) sortbuf[j] = ~0ull;
            __syncthreads();
            int added = 0, any_more = 0;
            for (int w2 = 0; w2 < kDWaves; w2++) { added += (int)scan_tmp[8 + w2]; any_more |= (int)scan_tmp[16 + w2]; }
            if (added > 0) {
                bitonic_sort_u64_by256(sortbuf, y.sort_cap);
                topn = min(a.kcap, topn + added);
            } else {
                __syncthreads();
            }
            return any_more != 0;
        };
        auto run_rounds = [&](auto gtag, auto rtag) {
            constexpr int GL = decltype(gtag)::value;       // lanes per row
            constexpr int R = decltype(rtag)::value;        // rows per lane group in flight
            constexpr int NG = kWave / GL;                  // lane groups
            constexpr int RB = NG * R;                      // rows per batch
            const int grp = lane / GL, sl = lane & (GL - 1);
            for (;;) {
                unsigned long long kth = ~0ull;
                if (topn >= a.kcap) kth = sortbuf[a.kcap - 1];
                int mine = 0;                               // entries this wavefront has pending
                unsigned long long* my_slots = sortbuf + a.kcap + wave * y.quota;
                for (;;) {
                    if (list_pos >= list_len) {
                        if (at >= at_end) break;
                        const int pt = at + lane;
                        const uint32_t v = pt < at_end ? (uint32_t)s_time[pt] : 0xffffu;
                        const bool is_cand = (v >> 1) <= t_lim;
                        const unsigned long long m = __ballot(is_cand);
                        if (is_cand) wl[__popcll(m & ((1ull << lane) - 1ull))] = (uint16_t)pt;
                        list_len = __popcll(m);
                        list_pos = 0;
                        at += kWave;
                        ncand += (uint32_t)list_len;
                        continue;
                    }
                    if (mine + RB > y.quota) break;         // no room for a whole batch: merge first
                    int pts[R];
                    bool valid[R];
                    unsigned long long e[R];
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        const int c = list_pos + r * NG + grp;
                        valid[r] = c < list_len;
                        pts[r] = (int)wl[min(c, list_len - 1)];
                    }
                    if (a.blind) {      // scored by the promoting step (:498-505), no row is read
#pragma unroll
                        for (int r = 0; r < R; r++)
                            e[r] = ((unsigned long long)(s_time[pts[r]] >> 1) << 32) | (uint32_t)(off + pts[r]);
                    } else {
                        const float* rows[R];
#pragma unroll
                        for (int r = 0; r < R; r++) rows[r] = a.data + (off + pts[r]) * a.dim;
                        float d[R];
                        const float* const (&crows)[R] = rows;
                        if (R > 2) wave_row_dists_wide<R, 16 / R>(crows, s_q, a.dim, d);  // (only chosen for aligned rows of 512 elements or more)
                        else wave_row_dists<R>(crows, s_q, a.dim, vec4, d);
#pragma unroll
                        for (int r = 0; r < R; r++)
                            e[r] = ((unsigned long long)__builtin_bit_cast(uint32_t, d[r]) << 32) | (uint32_t)(off + pts[r]);
                    }
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        const bool keep = valid[r] && sl == 0 && e[r] < kth;
                        const unsigned long long m = __ballot(keep);
                        if (keep) my_slots[mine + __popcll(m & ((1ull << lane) - 1ull))] = e[r];
                        mine += __popcll(m);
                    }
                    list_pos += RB;
                }
                if (!merge_round(mine, my_slots)) break;
            }
        };
        // Rows of at most 4 * GL elements: a batch is 64 candidates, GL lanes read a row (16
        // bytes each) and every lane group takes GL rows, eight loads in flight per lane; the
        // GL partial sums a lane ends up with are reduced for all its rows together, which
        // leaves lane c of the wavefront with the distance of candidate c: one comparison, one
        // ballot and one store per batch instead of one per row.
        auto run_tiles = [&](auto gtag) {
            typedef float v4f __attribute__((ext_vector_type(4)));
            constexpr int GL = decltype(gtag)::value;
            constexpr int kInFlight = 16;                   // row reads under way per lane
            const int grp = lane / GL, sl = lane & (GL - 1);
            const int j = sl * 4;
            const bool has = j < a.dim;
            float q0 = 0.f, q1 = 0.f, q2 = 0.f, q3 = 0.f;
            if (has) { q0 = s_q[j]; q1 = s_q[j + 1]; q2 = s_q[j + 2]; q3 = s_q[j + 3]; }
            const float* base = a.data + off * a.dim + (has ? j : 0);
            for (;;) {
                unsigned long long kth = ~0ull;
                if (topn >= a.kcap) kth = sortbuf[a.kcap - 1];
                int mine = 0;
                unsigned long long* my_slots = sortbuf + a.kcap + wave * y.quota;
                for (;;) {
                    // list at least a whole batch, while points are left
                    while (list_len - list_pos < kWave && at < at_end) {
                        if (list_pos > 0) {      // what is left moves to the front (one wavefront: its LDS operations keep their order)
                            const int rest = list_len - list_pos;
                            const uint16_t v = lane < rest ? wl[list_pos + lane] : (uint16_t)0;
                            if (lane < rest) wl[lane] = v;
                            list_len = rest;
                            list_pos = 0;
                        }
                        const int pt = at + lane;
                        const uint32_t v = pt < at_end ? (uint32_t)s_time[pt] : 0xffffu;
                        const bool is_cand = (v >> 1) <= t_lim;
                        const unsigned long long m = __ballot(is_cand);
                        if (is_cand) wl[list_len + __popcll(m & ((1ull << lane) - 1ull))] = (uint16_t)pt;
                        list_len += __popcll(m);
                        at += kWave;
                        ncand += (uint32_t)__popcll(m);
                    }
                    const int nb = min(kWave, list_len - list_pos);
                    if (nb <= 0) break;
                    if (mine + kWave > y.quota) break;      // no room for a whole batch: merge first
                    const uint16_t* cur = wl + list_pos;
                    float acc[GL];
#pragma unroll
                    for (int r0 = 0; r0 < GL; r0 += kInFlight) {
                        v4f x[kInFlight];
#pragma unroll
                        for (int r = 0; r < kInFlight; r++) {
                            // (lanes beyond the row's end read its head and add nothing: a load
                            //  under a condition would wait for the loads before it)
                            const int pt = (int)cur[min(grp * GL + r0 + r, nb - 1)];
                            x[r] = *reinterpret_cast<const v4f*>(base + pt * a.dim);
                        }
#pragma unroll
                        for (int r = 0; r < kInFlight; r++) {
                            float s2 = 0.f;
                            float dd = x[r].x - q0; s2 = __builtin_fmaf(dd, dd, s2);
                            dd = x[r].y - q1; s2 = __builtin_fmaf(dd, dd, s2);
                            dd = x[r].z - q2; s2 = __builtin_fmaf(dd, dd, s2);
                            dd = x[r].w - q3; s2 = __builtin_fmaf(dd, dd, s2);
                            acc[r0 + r] = has ? s2 : 0.f;
                        }
                    }
                    const float total = group_row_sums<GL>(acc, sl);      // of candidate grp * GL + sl = lane
                    const int mypt = (int)cur[min(lane, nb - 1)];
                    const unsigned long long e =
                        ((unsigned long long)__builtin_bit_cast(uint32_t, sqrtf(total)) << 32) | (uint32_t)(off + mypt);
                    const bool keep = lane < nb && e < kth;
                    const unsigned long long m = __ballot(keep);
                    if (keep) my_slots[mine + __popcll(m & ((1ull << lane) - 1ull))] = e;
                    mine += __popcll(m);
                    list_pos += nb;
                }
                if (!merge_round(mine, my_slots)) break;
            }
        };
        {
            using std::integral_constant;
            if (y.tiles && vec4 && a.dim <= 64 && y.quota >= kWave) run_tiles(integral_constant<int, 16>{});
            else if (y.tiles && vec4 && a.dim <= 128 && y.quota >= kWave) run_tiles(integral_constant<int, 32>{});
            // long rows: sixteen 16-byte reads in flight per lane, as whole 1 KiB pieces of as few rows as hold them
            else if (vec4 && !a.blind && a.dim == 512 && y.quota >= 8) run_rounds(integral_constant<int, 64>{}, integral_constant<int, 8>{});
            else if (vec4 && !a.blind && a.dim > 512 && y.quota >= 4) run_rounds(integral_constant<int, 64>{}, integral_constant<int, 4>{});
            else run_rounds(integral_constant<int, 64>{}, integral_constant<int, 2>{});
        }
        if (lane == 0) atomicAdd(&misc[dCand], ncand);
        for (int j = tid; j < a.kcap; j += kDT) part_out[j] = j < topn ? sortbuf[j] : ~0ull;
        PHASE_END(5);
        if (a.phase_ticks && tid == 0) atomicAdd(&a.phase_ticks[9], 1ull);

        // ---- hints for the batch kernel's routing, counters -----------------------------
        __syncthreads();
        const unsigned long long bound = (unsigned long long)n * a.L * T;
        unsigned long long steps = min(bound, maxw + 1);
        if (stop) steps = min(t_stop + 1, steps);
        if (a.stop_hint && tid == 0 && stop) record_stop(a.stop_hint, a.B, b, qi, (float)(t_stop + 1), (float)misc[dCand]);
        if (a.counters) {
            probes = wave_sum_u32(probes);
            if (lane == 0) atomicAdd(&misc[dProbes], probes);
            __syncthreads();
            if (tid == 0) {
                atomicAdd(&a.counters[(int64_t)qi * 4 + 0], (unsigned long long)n * I);
                atomicAdd(&a.counters[(int64_t)qi * 4 + 1], (unsigned long long)misc[dCand]);
                atomicAdd(&a.counters[(int64_t)qi * 4 + 2], (unsigned long long)misc[dProbes]);
                atomicAdd(&a.counters[(int64_t)qi * 4 + 3], steps);
            }
        }
    }
}

#undef PHASE_END

}  // namespace

bool dense_traversal_supported(const QueryArgs& a, size_t* lds_bytes) {
    if (!a.inv || a.ppb > 32766 || a.T < 1) return false;
    if (a.M > 64 || a.L > 64 || a.kcap > 512 || (int64_t)a.L * a.N >= 0x7fffffffLL) return false;
    if (dense_ipt_for(dense_max_windows(a)) == 0) return false;
    if (dense_max_windows(a) >= 0x7fff || a.ppb + (int64_t)a.T >= 65536) return false;
    if (a.xcds < 1 || a.xcds > 32 || (int64_t)a.nq * (a.B + a.xcds) >= 0x7fffffffLL) return false;
    const DenseLayout y = make_dense_layout(a);
    if (lds_bytes) *lds_bytes = y.lds_bytes;
    return y.lds_bytes <= 160 * 1024 - 512;
}

int query_dense_items(const QueryArgs& a_in, hipStream_t s) {
    QueryArgs a = a_in;
    const DenseLayout y = make_dense_layout(a);
    if (y.ipt == 0) return fail(-4, "query: this shape does not fit the dense traversal kernel");
    a.q_first = 0;
    a.q_count = a.nq;
    // enough resident workgroups to fill the device, each striding over its die's items
    const int per_cu = (int)max((size_t)1, min((size_t)4, (size_t)(160 * 1024) / y.lds_bytes));
    int64_t per_xcd = (int64_t)32 * per_cu * 2;
    const int64_t most = a.dense_items && a.mode != 3 ? (int64_t)a.dense_cap
                                                      : block_items(a.xcds, a.B, a.nq) / a.xcds;
    per_xcd = max((int64_t)1, min(per_xcd, most));
    const unsigned grid = (unsigned)(per_xcd * a.xcds);
#define DCIH_DENSE(IPT, WPS)                                                                        \
    do {                                                                                         \
        static DeviceOnce once;                                                                  \
        const int rc_attr = once.run([]() -> int {                                               \
            DCIH_HIP(hipFuncSetAttribute((const void*)traverse_dense_kernel<IPT, WPS>,             \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024)); \
            return 0;                                                                            \
        });                                                                                      \
        if (rc_attr) return rc_attr;                                                             \
        hipLaunchKernelGGL((traverse_dense_kernel<IPT, WPS>), dim3(grid), dim3(kDT), y.lds_bytes, s, a, y); \
    } while (0)
    if (y.ipt == 9 && per_cu >= 3) DCIH_DENSE(9, 3);
    else if (y.ipt == 9) DCIH_DENSE(9, 2);
    else if (y.ipt == 17) DCIH_DENSE(17, 2);
    else if (y.ipt == 25) DCIH_DENSE(25, 2);
    else if (y.ipt == 33) DCIH_DENSE(33, 2);
    else DCIH_DENSE(41, 2);
#undef DCIH_DENSE
    DCIH_HIP(hipGetLastError());
    return 0;
}

}  // namespace dcih
