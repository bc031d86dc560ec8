// Batch ("epoch") traversal: one workgroup per (query, partition), every lane
// streaming index entries.
//
// Computes exactly what the step-by-step loop of
// dci_query_single_point_by_block (src/dci_cuda_kernel.cu:401-626) computes,
// without executing it step by step.  What makes that possible:
//
//  * Inside one simple index the windows returned by dci_next_closest_proj
//    (:250-273) form two streams (left, right of the query position) whose
//    priorities (:572-590) never decrease, merged nearest-first, ties to the
//    left.  One composite index pops its L simple indices nearest-first, ties
//    to the lowest simple index (:466-478).  So composite m consumes ALL its
//    windows in ascending (priority, simple index, own order), window number r
//    of that order is visited at outer step r, and "every window with priority
//    below rho" is always a prefix of the traversal.
//  * A point is promoted by composite m at the step of the LAST of the L
//    windows that hold it; it is a candidate at its earliest (step, m) over
//    the composites; the loop stops at the first step kk with
//    c0(kk) >= k and (kk+1 >= outer*L or c0(kk) >= max_candidates), where c0
//    counts promotions whose last window held the point in lane 0 (:598-607).
//
// An epoch picks a priority bound per composite index and finds by binary search
// how many windows of every stream lie below it.  The windows a simple index has
// consumed cover one run of positions [lo, hi) of its sorted slice, so the points
// composite m has visited in all of its L simple indices are those whose position
// lies inside the run in every one of them: all lanes scan the inverse permutation
// (the position of every point in every slice, 16 bits each, eight points per
// 16-byte read) and test run membership two points per instruction in packed
// 16-bit arithmetic.  Only for the few points found the exact step is computed:
// the farthest of the point's L windows is the last one visited, and that
// window's rank is a sum of 2L binary searches.  Promotions are then replayed in
// (step, composite) order to apply the stop rule.  An epoch that promotes too
// many points at once is dropped and retried smaller.  Whatever does not fit the
// fixed LDS tables is handed to the step-by-step kernel through a redo list, so
// results never depend on which kernel produced them.
//
// Two layouts of an item's LDS state.  The full one keeps three kinds of flags as
// bits per point of the partition (accepted as a candidate; promoted under composite
// m) and runs as two or four wavefronts per item.  Where a stop is expected to take
// few promotions (the smallest tables) and the 2 m L streams fit one wavefront, the
// compact one keeps those flags as members of one small hashed set, so an item's
// LDS no longer grows with the partition, and runs as ONE wavefront per item: twice
// as many items per CU, which is what the kernel's time depends on (chains of
// dependent reads).  The few items that promote more than the set takes are listed
// and taken up again by a second launch with the full layout.
#include <cmath>
#include <type_traits>

#include "common.h"
#include "kernels.h"
#include "traverse_common.h"

namespace dcih {

namespace {

constexpr int kMaxEpochs = 100000;
constexpr int kSampleShift = 3;       // 2^shift - 1 window priorities sampled per stream and epoch
constexpr int kSamples = 1 << kSampleShift;


enum Misc {   // 32-bit scalars shared by the workgroup
    kPromoCount = 0, kEventCount, kAccCount, kFail, kStop, kC0, kStopStepLo, kStopStepHi,
    kArmedLo, kArmedHi, kScannedLo, kScannedHi, kArmed, kNumCand, kTopN, kProbes, kHintSteps, kHintPromos,
    kFirstJump, kPromoAimBits, kInvLBits, kNeedBits, kItem, kSetMarked, kListCount, kMiscWords
};

struct BlockLayout {
    int seen_words;   // one bit per point of the partition
    int flag_words;   // seen bits + per composite the points it has promoted: (M + 1) * seen_words
    int set_slots;    // 0, or: instead of those bits, one hashed set of this many words that holds the
                      // (composite, point) pairs promoted so far and the points accepted as candidates
    int set_limit;    // promotions an item may make before that set is too full (the item is then redone)
    int off_idx;      // per simple index: p, qp, and the visited run as packed 16-bit pairs (4 * I words)
    int off_stream;   // per stream: consumed, previous, total, stride (4 * 2I words)
    int off_comp;     // per composite: rho bits, K, active, previous K, sum of inverse priorities, scan flag (6 * M words)
    int off_samp;     // per stream: kSamples - 1 sampled window priorities of the current epoch's range (slot 0 unused)
    int off_promo, off_events, off_acc, off_sort, off_flags;
    int promo_cap;    // promotions one epoch may produce (table size)
    int promo_max;    // above this an epoch is dropped and halved
    int event_cap;    // promotions waiting for the other composites (= accepted candidates per replay)
    int sort_cap;     // power of two >= kcap + 128: top-k plus one batch of candidates
    size_t lds_bytes;
};

constexpr int kSetSlots = 384;
constexpr uint32_t kSetEmpty = 0xffffffffu;
constexpr uint32_t kSetSeenTag = 63u << 26;       // composites are tagged 0 .. M - 1 <= 61

// Where few promotions are expected per item (the smallest tables) and the streams fit one
// wavefront, an item is one wavefront and its per-point flags a small hashed set: LDS per
// item no longer grows with the partition, and twice as many items fit a CU.
bool block_layout_compact(const QueryArgs& a, int promo_cap) {
    return !a.full_tables && promo_cap <= 128 && 2 * a.M * a.L <= 64 && a.M <= 62;
}

BlockLayout make_block_layout(const QueryArgs& a) {
    BlockLayout y;
    const int I = a.M * a.L;
    y.seen_words = (int)((a.ppb + 31) / 32);
    y.flag_words = (a.M + 1) * y.seen_words;
    int o = kMiscWords * 4;
    y.off_idx = o;      o += 4 * I * 4;
    y.off_stream = o;   o += 4 * 2 * I * 4;
    y.off_comp = o;     o += 6 * a.M * 4;
    // small tables keep more workgroups resident per CU; an item that overflows them
    // is redone by the step-by-step kernel
    // The tables grow with the promotions a stop needs (about k * T, more when the
    // step limit rather than c0 >= k ends the traversal): fewer, larger epochs.
    // (the step limit can ask for more than k * T: a traversal that must consume the fraction f of a
    //  composite's windows before it may stop has by then promoted about f^L of the partition, unless
    //  max_candidates first-lane promotions end it earlier -- the estimate the kernel choice uses)
    const double windows = (double)a.L * ((double)a.ppb / (double)a.T);
    const double f = fmin(1.0, (double)a.stop_at / fmax(1.0, windows));
    const double by_steps = fmin((double)a.ppb * pow(f, (double)a.L), (double)a.max_cand * (double)a.T);
    const double expected = fmax((double)a.k_stop * (double)a.T, by_steps);
    y.promo_cap = 128;
    while ((double)y.promo_cap < 2.0 * expected && y.promo_cap < 2048) y.promo_cap <<= 1;
    y.promo_max = y.promo_cap * 5 / 8;
    const bool compact = block_layout_compact(a, y.promo_cap);
    y.set_slots = compact ? kSetSlots : 0;
    y.set_limit = kSetSlots * 7 / 16;     // every promotion adds at most two entries: the set stays under 7/8 full
    y.event_cap = compact ? y.promo_cap : 2 * y.promo_cap;
    y.sort_cap = 64;           // top-k plus a batch of at least 48 new candidates
    while (y.sort_cap < a.kcap + 48) y.sort_cap <<= 1;
    // the accepted candidates of a replay share the room of the priority samples and the
    // promotion list, both of which the ranking before it has finished with
    y.off_samp = o;
    y.off_acc = o;
    // (blind querying keeps the promoting step beside every accepted candidate)
    o += max(2 * I * kSamples * 4 + y.promo_cap * 4, y.event_cap * 4 * (a.blind ? 2 : 1));
    y.off_promo = y.off_samp + 2 * I * kSamples * 4;
    o = (o + 15) & ~15;
    y.off_events = o;   o += y.event_cap * 8;
    y.off_sort = o;     o += y.sort_cap * 8;
    y.off_flags = o;
    y.lds_bytes = (size_t)o + (size_t)(compact ? y.set_slots : y.flag_words) * 4;
    return y;
}

// One (query qi, partition b) item, by the whole workgroup.
template <int NT, int MINW, bool COMPACT>
__device__ __forceinline__ void traverse_block_item(const QueryArgs& a, const BlockLayout& y, const int b, const int qi) {
    extern __shared__ __align__(16) unsigned char smem[];
    uint32_t* misc = reinterpret_cast<uint32_t*>(smem);
    int* s_p = reinterpret_cast<int*>(smem + y.off_idx);
    float* s_qp = reinterpret_cast<float*>(s_p + a.M * a.L);
    uint32_t* s_lo2 = reinterpret_cast<uint32_t*>(s_qp + a.M * a.L);  // first position of the visited run, twice
    uint32_t* s_lm2 = s_lo2 + a.M * a.L;                              // its length - 1, twice
    int* s_c = reinterpret_cast<int*>(smem + y.off_stream);          // windows consumed
    int* s_cprev = s_c + 2 * a.M * a.L;                               // ... at epoch start
    int* s_ns = s_cprev + 2 * a.M * a.L;                              // windows in the stream
    int* s_stride = s_ns + 2 * a.M * a.L;                             // windows to try next epoch
    uint32_t* s_rho = reinterpret_cast<uint32_t*>(smem + y.off_comp); // per composite
    uint32_t* s_K = s_rho + a.M;
    uint32_t* s_active = s_K + a.M;
    uint32_t* s_Kprev = s_active + a.M;
    float* s_hsum = reinterpret_cast<float*>(s_Kprev + a.M);
    uint32_t* s_noscan = reinterpret_cast<uint32_t*>(s_hsum + a.M);   // some simple index of the composite has visited nothing yet
    uint32_t* s_samp = reinterpret_cast<uint32_t*>(smem + y.off_samp);
    uint32_t* promo = reinterpret_cast<uint32_t*>(smem + y.off_promo);
    uint32_t* acc = reinterpret_cast<uint32_t*>(smem + y.off_acc);
    uint32_t* acc_step = acc + y.event_cap;       // blind querying only
    unsigned long long* events = reinterpret_cast<unsigned long long*>(smem + y.off_events);
    unsigned long long* sortbuf = reinterpret_cast<unsigned long long*>(smem + y.off_sort);
    uint32_t* seen = reinterpret_cast<uint32_t*>(smem + y.off_flags);
    uint32_t* marked = seen + y.seen_words;          // [M][seen_words]: promoted under composite m in an accepted epoch
    // The compact layout keeps both kinds of flags as members of one open-addressed set in the same
    // place: (composite << 26 | point) for a promotion, (63 << 26 | point) for an accepted candidate.
    // The set never fills (set_limit), so every probe sequence ends at an empty word; the probe
    // count is bounded all the same.
    const uint32_t set_slots = (uint32_t)y.set_slots;
    // (false at compile time in the variants for the full tables; in the others left for the kernel to
    //  test: told at compile time, the compiler duplicates the phases' code around the set's probe loops
    //  and the seven-wavefront variant keeps 80 bytes per lane in scratch instead of 16)
    const bool compact = COMPACT && set_slots != 0;
    uint32_t* const hset = seen;
    auto set_home = [&](uint32_t key) { return (((key * 0x9E3779B1u) >> 16) * set_slots) >> 16; };
    auto set_has = [&](uint32_t key) {
        uint32_t h = set_home(key);
        for (uint32_t probe = 0; probe < set_slots; probe++) {
            const uint32_t v = hset[h];
            if (v == key) return true;
            if (v == kSetEmpty) return false;
            h = h + 1 == set_slots ? 0 : h + 1;
        }
        return false;
    };
    auto set_add = [&](uint32_t key) {        // true if the key was not a member yet
        uint32_t h = set_home(key);
        for (uint32_t probe = 0; probe < set_slots; probe++) {
            const uint32_t v = atomicCAS(&hset[h], kSetEmpty, key);
            if (v == kSetEmpty) return true;
            if (v == key) return false;
            h = h + 1 == set_slots ? 0 : h + 1;
        }
        misc[kFail] = 4;
        return false;
    };

    // The thread numbers are made opaque again at the start of every phase (fresh_thread_ids):
    // otherwise the compiler computes each phase's lane groupings and per-thread addresses once,
    // before the epoch loop, and keeps them all in registers (or scratch) across every phase.
    int tid = threadIdx.x;
    int lane = tid & (kWave - 1);
    int wave = tid / kWave;
    auto fresh_thread_ids = [&]() {
        asm volatile("" : "+v"(tid));
        lane = tid & (kWave - 1);
        wave = tid / kWave;
    };
    // For the same reason every phase ends in an exit that is never taken but that the compiler
    // cannot rule out (PHASE_END): loads and address arithmetic of the phases after it are then
    // not moved up across it, or out of the epoch loop.  Without the two, the five-workgroup
    // variant keeps 244 bytes per lane in scratch instead of 12 and the kernel runs a quarter slower.
#define PHASE_FENCE()                                    \
    do {                                                 \
        int leave_now = 0;                               \
        asm volatile("" : "+s"(leave_now));              \
        if (leave_now) return;                           \
        fresh_thread_ids();                              \
    } while (0)
#define PHASE_END(which)                                 \
    do {                                                 \
        phase(which);                                    \
        int leave_now = 0;                               \
        asm volatile("" : "+s"(leave_now));              \
        if (leave_now) return;                           \
        fresh_thread_ids();                              \
    } while (0)
    constexpr int kWaves = NT / kWave;
    // optional phase profile: thread 0 adds the 100 MHz ticks each phase took
    unsigned long long tick = a.phase_ticks ? wall_clock64() : 0ull;
    auto phase = [&](int which) {
        if (a.phase_ticks && tid == 0) {
            const unsigned long long now = wall_clock64();
            atomicAdd(&a.phase_ticks[which], now - tick);
            tick = now;
        }
    };
    const int I = a.M * a.L;
    const int S = 2 * I;                       // streams

    const int64_t item = (int64_t)qi * a.B + b;
    const int64_t off = (int64_t)b * a.ppb;
    const int n = (int)min(a.N - off, a.ppb);
    unsigned long long* part_out = a.part + item * a.kcap;
    if (n <= 0) {
        for (int j = tid; j < a.kcap; j += NT) part_out[j] = ~0ull;
        return;
    }
    // Traversals that need many promotions before they stop are the dense kernel's: it is
    // told so here, by the partition's record of earlier stops, or further down once this
    // traversal itself has gone that far.  Which kernel finishes an item never shows in
    // the results.
    const bool may_hand_over = a.dense_items != nullptr && a.dense_min_promos > 0;
    // An item that is already under way here is worth moving only from twice the number of
    // promotions at which a whole call is routed to the dense kernel: below that, finishing
    // it here is cheaper than starting over there.
    const int64_t hand_over_at = 2 * (int64_t)a.dense_min_promos;
    auto hand_to_dense = [&]() {
        if (threadIdx.x == 0) {
            const int x = (int)(blockIdx.x % a.xcds);
            const uint32_t sl = atomicAdd(&a.dense_count[x], 1u);
            a.dense_items[(int64_t)x * a.dense_cap + sl] = (int32_t)misc[kItem];      // (read back: no register held for it)
        }
    };
    // usual stop step and promotions at the stop: read by one thread, because other workgroups
    // are updating them and every thread must decide alike
    if (threadIdx.x < kMiscWords) misc[threadIdx.x] = 0;
    __syncthreads();
    if (threadIdx.x == 0) misc[kItem] = (uint32_t)item;
    if (threadIdx.x == 0 && a.stop_hint) {
        float steps, promotions;
        usual_stop(a.stop_hint, a.B, b, steps, promotions);
        misc[kHintSteps] = __builtin_bit_cast(uint32_t, steps);
        misc[kHintPromos] = __builtin_bit_cast(uint32_t, promotions);
    }
    __syncthreads();
    const float hint = __builtin_bit_cast(float, misc[kHintSteps]);
    const float hint_promos = __builtin_bit_cast(float, misc[kHintPromos]);
    if (may_hand_over && hint_promos >= (float)hand_over_at) {
        hand_to_dense();
        return;
    }
    // An item that the compact tables cannot finish (the set full, or the smaller event table) goes
    // to the second pass, whose tables may hold it; what the full tables cannot finish either (and
    // what the second pass's list has no room for) goes to the step-by-step kernel.
    auto hand_back = [&]() {
        if (threadIdx.x == 0) {
            bool listed = false;
            if (COMPACT && a.wide_items) {
                const uint32_t slot = atomicAdd(a.wide_count, 1u);
                listed = (int64_t)slot < a.wide_cap;
                if (listed) a.wide_items[slot] = (int32_t)misc[kItem];
            }
            if (!listed) {
                const uint32_t slot = atomicAdd(a.redo_count, 1u);
                a.redo_items[slot] = (int32_t)misc[kItem];
            }
        }
    };
    // Where stops in this partition usually need more promotions than the compact tables take,
    // the item goes to the second pass at once.
    if (COMPACT && a.wide_items && hint_promos > 0.75f * (float)y.set_limit) {
        if (threadIdx.x == 0) misc[kFail] = 4;
        __syncthreads();
        hand_back();
        return;
    }
    const int T = a.T;
    // d / T for 0 <= d < 65536 (positions inside a partition) by one multiply-high:
    // exact because the error of the rounded-up reciprocal stays below 2^-16 < 1/T
    const uint32_t T_magic = a.T_magic;
    auto div_T = [&](int d) { return T > 1 ? (int)__umulhi((uint32_t)d, T_magic) : d; };

    // ---- set-up ---------------------------------------------------------------
    if (compact) { for (int w = tid; w < y.set_slots; w += NT) hset[w] = kSetEmpty; }
    else { for (int w = tid; w < y.flag_words; w += NT) seen[w] = 0; }
    uint32_t probes = 0;
    {   // positioning search (:279-297): first position whose key is not below qp,
        // one group of lanes per simple index
        const int lg = min(3, floor_log2(kWave / ((I + kWaves - 1) / kWaves))), G = 1 << lg;
        const int slot = lane >> lg, i = wave * (kWave >> lg) + slot;
        const bool active = i < I;
        const float* key = a.skeys + (int64_t)(active ? i : 0) * a.N + off;
        const float qp = active ? a.qproj[(int64_t)i * a.nq + qi] : 0.f;
        const int lo = group_partition_point(0, n, active, lg, slot * G, lane - slot * G,
                                             [&](int j) { return key[j] < qp; }, probes);
        if (active && lane == slot * G) {
            const int p = lo - 1;
            s_p[i] = p;
            s_qp[i] = qp;
            for (int side = 0; side < 2; side++) {
                s_ns[2 * i + side] = stream_windows(n, T, p, side);
                s_c[2 * i + side] = 0;
            }
        }
    }
    __syncthreads();
    // Stride of an epoch, in windows, per stream: starts at 1/128 of the longest
    // stream; afterwards each stream's stride follows what it consumed last time
    // (its local density), scaled so that every composite lands on the same step
    // count: a composite left behind would keep the promotions of the others
    // waiting.  The total doubles from epoch to epoch until one has to be undone.
    // hint = average step at which earlier queries stopped in this partition (record_stop);
    // it only steers epoch sizes, never results.  The first jump aims
    // 12 % past it.  The number of points whose counters are complete grows like a
    // high power (L) of the steps taken, so stop steps of one partition scatter
    // little and most items finish in one epoch (12 % more steps bring about three
    // times the promotions to rank, which still costs less than a second epoch),
    // while a jump much farther overflows the tables.
    // Where the stop needs more promotions than one epoch may produce (their
    // number at earlier stops in this partition is the second hint; about k * T
    // without one), the jump is shortened by the same power law so that an epoch
    // yields about 0.6 * promo_max of them.
    constexpr float kHintGrow = 1.06f;
    const float kPromoAim = 0.6f * (float)y.promo_max;
    const float inv_L = 1.0f / (float)a.L;
    const float kHintFirst = fminf(1.12f,
        fast_pow(kPromoAim / fmaxf(1.0f, hint_promos > 0.0f ? hint_promos : (float)a.k_stop * (float)T), inv_L));
    {
        int first = 4;           // (every wavefront reduces the S <= 128 stream lengths on its own)
        for (int s = lane; s < S; s += kWave) first = max(first, s_ns[s] / 128);
        first = wave_max_i32(first);
        if (hint > 0.0f) first = max(first, (int)(kHintFirst * hint / (float)(2 * a.L)));
        if (tid < S) s_stride[tid] = first;
        if (tid < a.M) s_Kprev[tid] = 0;
        // (the later epochs' sizing reads these back from LDS instead of keeping them in registers --
        //  in scratch, in the tight variants -- across all phases)
        if (tid == 0) {
            misc[kFirstJump] = __builtin_bit_cast(uint32_t, kHintFirst);
            misc[kPromoAimBits] = __builtin_bit_cast(uint32_t, kPromoAim);
            misc[kInvLBits] = __builtin_bit_cast(uint32_t, inv_L);
            misc[kNeedBits] = __builtin_bit_cast(uint32_t, (float)(a.stop_at > 0 ? a.stop_at : 1));
        }
    }
    __syncthreads();
    PHASE_END(0);

    auto load_stream = [&](int s) {
        Stream st;
        const int i = s >> 1;
        st.key = a.skeys + (int64_t)i * a.N + off;
        st.n = n; st.T = T; st.p = s_p[i]; st.side = s & 1; st.q = s_qp[i];
        return st;
    };

    // The points an epoch promotes.  The windows simple index i has consumed so far cover the
    // positions [lo_i, hi_i) of its sorted slice (the left stream's windows end at the query
    // position, the right stream's start there), so composite m has visited a point in all of
    // its L simple indices exactly when the point's position lies in that run in every one of
    // them.  Only the points inside the run of the composite's FIRST simple index can qualify,
    // and a.rpos holds every point's positions in the order of that slice: the scan walks the
    // first index's run and tests the other L - 1 positions of the points standing there.
    // Every thread takes eight consecutive places at a time: the positions in one simple
    // index of the points standing there are ONE 16-byte read, and per pair of points
    // membership costs three packed 16-bit instructions: pos - lo (wrapping), minus
    // (length - 1) with unsigned saturation -- zero exactly when lo <= pos < hi -- and a
    // running maximum over the simple indices, which ends at zero for the points inside all
    // runs.  Those not yet promoted under m in an earlier epoch (one bit per point and
    // composite) go to the promotion list.  No state is left behind: an epoch that turns out
    // too large is simply dropped.  The loop reads (L - 1) positions per place of the run, four
    // simple indices' reads in flight per thread.
    typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(1))) const u32x4 g_u32x4;
    auto scan_epoch = [&]() {
        if (tid < a.M) s_noscan[tid] = 0;
        __syncthreads();
        if (tid < I) {
            const int64_t p1 = (int64_t)s_p[tid] + 1;
            const int lo = (int)max((int64_t)0, p1 - (int64_t)s_c[2 * tid] * T);
            const int hi = (int)min((int64_t)n, p1 + (int64_t)s_c[2 * tid + 1] * T);
            const uint32_t lm = (uint32_t)(hi - lo - 1) & 0xffffu;
            s_lo2[tid] = ((uint32_t)lo & 0xffffu) * 0x10001u;
            s_lm2[tid] = lm * 0x10001u;
            if (hi <= lo) s_noscan[tid / a.L] = 1;
        }
        __syncthreads();
        unsigned long long looked_at = 0;      // index entries read (same on every thread)
        for (int m = 0; m < a.M; m++) {
            if (s_noscan[m]) continue;
            const int64_t first_row = (int64_t)m * a.L * a.N + off;     // the composite's first simple index, this partition
            const uint32_t* lo2 = s_lo2 + m * a.L;
            const uint32_t* lm2 = s_lm2 + m * a.L;
            const uint32_t* marked_m = marked + m * y.seen_words;
            // the first index's run, in chunks of eight places that start where the reads are 16-byte
            // aligned, if the slices of all simple indices can be aligned together (N a multiple of
            // 8); else reads are unaligned
            const int run_lo = (int)(lo2[0] & 0xffffu), run_hi = run_lo + (int)(lm2[0] & 0xffffu) + 1;
            const int chunk_shift = (a.N & 7) == 0 ? (int)((off + run_lo) & 7) : 0;
            const int start = run_lo - chunk_shift;
            const int nchunks = (run_hi - start + 7) >> 3;
            const uint16_t* rp = a.rpos + first_row + start;
            // a point found inside all runs: to the promotion list unless an earlier epoch promoted it
            auto found = [&](int place) {        // place in the first index's slice
                const uint32_t local = (uint32_t)(a.sids[first_row + place] - (int32_t)off);
                if (compact ? set_has(local | ((uint32_t)m << 26)) : (bool)((marked_m[local >> 5] >> (local & 31u)) & 1u)) return;
                const uint32_t slot = atomicAdd(&misc[kPromoCount], 1u);
                if (slot < (uint32_t)y.promo_cap) promo[slot] = local | ((uint32_t)m << 26);
            };
            // rows [h_begin, h_end) of the position table for chunk c: the fields of `worst` that stay
            // zero belong to places inside the runs of all those rows (and inside the first index's run)
            auto test_chunk = [&](int c, int h_begin, int h_end, u16x2 (&worst)[4]) {
                const int first = start + 8 * c;            // place in the first index's slice of the chunk's first point
#pragma unroll
                for (int r = 0; r < 4; r++) worst[r] = u16x2{0, 0};
                if (c == 0 || c == nchunks - 1) {            // places before the run's first or past its last
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const bool out0 = first + 2 * r < run_lo || first + 2 * r >= run_hi;
                        const bool out1 = first + 2 * r + 1 < run_lo || first + 2 * r + 1 >= run_hi;
                        worst[r] = u16x2{(uint16_t)(out0 ? 0xffff : 0), (uint16_t)(out1 ? 0xffff : 0)};
                    }
                }
                // (a row's start is the same for every thread and the chunk's offset a 32-bit number:
                //  scalar base + vector offset addressing, no 64-bit address per thread and row)
                const uint32_t chunk_bytes = (uint32_t)c * 16u;
                auto group = [&](int h0, auto width) {
                    constexpr int W = decltype(width)::value;
                    u32x4 x[W];
#pragma unroll
                    for (int u = 0; u < W; u++) {
                        const char* row = reinterpret_cast<const char*>(rp + (int64_t)(h0 + u) * a.N);
                        x[u] = *(g_u32x4*)(row + chunk_bytes);
                    }
#pragma unroll
                    for (int u = 0; u < W; u++) {
                        const u16x2 lo = __builtin_bit_cast(u16x2, lo2[h0 + u]);
                        const u16x2 lm = __builtin_bit_cast(u16x2, lm2[h0 + u]);
                        const uint32_t w[4] = {x[u].x, x[u].y, x[u].z, x[u].w};
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            const u16x2 d = __builtin_bit_cast(u16x2, w[r]) - lo;
                            worst[r] = __builtin_elementwise_max(worst[r], __builtin_elementwise_sub_sat(d, lm));
                        }
                    }
                };
                // (rows per group of reads in flight: three where all rows are read in one stage, two in the
                //  two-stage form -- each measured a per cent or two ahead of the other there)
                int h0 = h_begin;
                if (!COMPACT) for (; h0 + 3 <= h_end; h0 += 3) group(h0, std::integral_constant<int, 3>());
                for (; h0 + 2 <= h_end; h0 += 2) group(h0, std::integral_constant<int, 2>());
                if (h0 < h_end) group(h0, std::integral_constant<int, 1>());
                const u16x2 m01 = __builtin_elementwise_min(worst[0], worst[1]);
                const u16x2 m23 = __builtin_elementwise_min(worst[2], worst[3]);
                const uint32_t least = __builtin_bit_cast(uint32_t, __builtin_elementwise_min(m01, m23));
                return ((least - 0x00010001u) & ~least & 0x80008000u) != 0u;     // some 16-bit field is zero
            };
            // Two stages where the composite has many simple indices (one-wavefront variants): about half
            // of the places survive each row, so after the first 0.6 L rows few are left; those are listed
            // (their distance from the run's first place, 16 bits, in the room of the priority samples,
            // which are taken after the scan) and only for them the remaining rows are read, one 2-byte
            // read per row and place -- far dearer per place than the first stage's, hence not earlier
            // (1M x 128, L = 10, 17242-point partitions: one stage 365 k queries/s; 3 / 4 / 5 / 6 / 7 rows
            // in the first stage 331 / 373 / 397 / 398 / 385 k).  The list is emptied whenever the next
            // round of chunks might overflow it.
            const int stage_rows = (3 * a.L + 2) / 5;
            uint16_t* const list = reinterpret_cast<uint16_t*>(s_samp);
            const int list_cap = 2 * I * kSamples * 2;
            if (COMPACT && a.L - 1 > stage_rows + 1 && list_cap >= 8 * NT + NT) {
                auto rest_of_rows = [&](int n_listed) {
                    for (int j = tid; j < n_listed; j += NT) {
                        const int place = run_lo + (int)list[j];
                        bool inside = true;
                        for (int h0 = 1 + stage_rows; h0 < a.L; h0 += 4) {
                            uint32_t pos[4];
#pragma unroll
                            for (int u = 0; u < 4; u++) {
                                const int h = min(h0 + u, a.L - 1);
                                pos[u] = a.rpos[first_row + (int64_t)h * a.N + place];
                            }
#pragma unroll
                            for (int u = 0; u < 4; u++) {
                                const int h = min(h0 + u, a.L - 1);
                                inside = inside && ((pos[u] - (lo2[h] & 0xffffu)) & 0xffffu) <= (lm2[h] & 0xffffu);
                            }
                        }
                        if (inside) found(place);
                    }
                };
                unsigned long long listed_total = 0;
                for (int c0 = 0; c0 < nchunks; c0 += NT) {
                    const int c = c0 + tid;
                    if (c < nchunks) {
                        u16x2 worst[4];
                        if (test_chunk(c, 1, 1 + stage_rows, worst)) {
#pragma unroll
                            for (int e = 0; e < 8; e++) {
                                const uint32_t w = __builtin_bit_cast(uint32_t, worst[e >> 1]);
                                if (((w >> ((e & 1) * 16)) & 0xffffu) != 0u) continue;
                                const uint32_t slot = atomicAdd(&misc[kListCount], 1u);
                                list[slot] = (uint16_t)(start + 8 * c + e - run_lo);
                            }
                        }
                    }
                    __syncthreads();
                    const int n_listed = (int)misc[kListCount];
                    __syncthreads();          // (every thread has the count before anyone changes it)
                    if (n_listed > list_cap - 8 * NT || c0 + NT >= nchunks) {
                        rest_of_rows(n_listed);
                        listed_total += (unsigned long long)n_listed;
                        __syncthreads();
                        if (tid == 0) misc[kListCount] = 0;
                        __syncthreads();
                    }
                }
                looked_at += (unsigned long long)nchunks * 8ull * (unsigned long long)stage_rows +
                             listed_total * (unsigned long long)(a.L - 1 - stage_rows);
                continue;
            }
            looked_at += (unsigned long long)nchunks * 8ull * (unsigned long long)(a.L - 1);
            for (int c = tid; c < nchunks; c += NT) {
                u16x2 worst[4];
                if (!test_chunk(c, 1, a.L, worst)) continue;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const uint32_t w = __builtin_bit_cast(uint32_t, worst[e >> 1]);
                    if (((w >> ((e & 1) * 16)) & 0xffffu) != 0u) continue;
                    found(start + 8 * c + e);
                }
            }
        }
        return looked_at;
    };
    auto mark_promotions = [&](uint32_t np) {
        for (uint32_t j = tid; j < np; j += NT) {
            const uint32_t local = promo[j] & 0x3ffffffu, m = promo[j] >> 26;
            if (compact) set_add(promo[j]);
            else atomicOr(&marked[m * y.seen_words + (local >> 5)], 1u << (local & 31u));
        }
    };
    bool shrunk = false;        // the previous epoch was undone
    bool undone_once = false;   // some epoch of this item was undone
    int epoch = 0;
    for (; epoch < kMaxEpochs; epoch++) {
        fresh_thread_ids();
        // ---- 1. priority bound per composite ------------------------------------
        if (tid < a.M) { s_rho[tid] = kInfBits; s_K[tid] = 0; s_active[tid] = 0; s_hsum[tid] = 0.0f; }
        __syncthreads();
        if (tid < S) {
            const int c = s_c[tid], ns = s_ns[tid];
            s_cprev[tid] = c;
            if (c < ns) {
                const int m = (tid >> 1) / a.L;
                const Stream st = load_stream(tid);
                const int64_t jp = min((int64_t)c + s_stride[tid], (int64_t)ns) - 1;
                probes++;
                const uint32_t pi = stream_prio_bits(st, (int)jp);
                atomicMin(&s_rho[m], pi);
                atomicAdd(&s_active[m], 1u);
                atomicAdd(&s_hsum[m], 1.0f / __builtin_bit_cast(float, pi));
            }
        }
        __syncthreads();
        // The smallest of the streams' stride-end priorities lets only one stream use
        // its whole stride and the epoch falls short of the steps it aimed at.  With
        // windows locally equidistant in priority, the bound at which the streams
        // together consume the sum of their strides is the harmonic mean of those
        // priorities; any bound is valid, this one lands the epoch where intended.
        // (A zero priority makes the mean 0 and a NaN makes it NaN: the minimum stays.)
        // Once an epoch had to be undone the smallest priority is kept: then no stream
        // passes its stride, and halving the strides is sure to shrink the epoch.
        if (!undone_once && tid < a.M && s_active[tid] > 0) {
            const float hm = (float)s_active[tid] / s_hsum[tid];
            if (hm > 0.0f && hm < __builtin_inff())
                s_rho[tid] = max(s_rho[tid], __builtin_bit_cast(uint32_t, hm));
        }
        __syncthreads();
        PHASE_END(1);
        // ---- 2. how far each stream goes: all windows with priority <= bound ----
        {   // one group of lanes per stream; search window by window (twice the stride,
            // then four times as much, ...) so that probes stay near where the epoch will end
            const int lg = min(3, floor_log2(kWave / ((S + kWaves - 1) / kWaves))), G = 1 << lg;
            const int slot = lane >> lg, sidx = wave * (kWave >> lg) + slot, g = lane - slot * G;
            const bool active = sidx < S;
            const int c = active ? s_c[sidx] : 0, ns = active ? s_ns[sidx] : 0;
            const int m = active ? (sidx >> 1) / a.L : 0;
            const uint32_t rho = s_rho[m];
            const Stream st = load_stream(active ? sidx : 0);
            bool more = active && c < ns && rho < kInfBits;
            const bool searched = more;
            int lo = c, hi = c;
            int64_t span = 2 * (int64_t)(active ? s_stride[sidx] : 1);
            while (__any(more)) {
                if (more) hi = (int)min((int64_t)ns, (int64_t)lo + span);
                const int r = group_partition_point(lo, hi, more, lg, slot * G, g,
                    [&](int j) { return stream_prio_bits(st, j) <= rho; }, probes);
                if (more) {
                    if (r == hi && hi < ns) { lo = hi; span *= 4; }
                    else { lo = r; more = false; }
                }
            }
            // (NaN priorities: take the rest so the epoch loop ends)
            const int cn = searched ? lo : (active && c < ns ? ns : c);
            if (active && g == 0) {
                s_c[sidx] = cn;
                atomicAdd(&s_K[m], (uint32_t)cn);
            }
        }
        __syncthreads();
        bool all_done = true;
        for (int m = 0; m < a.M; m++) all_done = all_done && s_active[m] == 0;
        if (all_done) break;      // every stream was already exhausted before this epoch
        PHASE_END(2);

        // ---- 3. the points whose L windows are now all consumed ---------------------
        {
            const unsigned long long looked_at = scan_epoch();
            if (a.counters && tid == 0) {       // (a 64-bit count in two words of the workgroup's scalars)
                const unsigned long long sum = (((unsigned long long)misc[kScannedHi] << 32) | misc[kScannedLo]) + looked_at;
                misc[kScannedLo] = (uint32_t)sum; misc[kScannedHi] = (uint32_t)(sum >> 32);
            }
        }
        __syncthreads();
        PHASE_END(3);
        const uint32_t np = misc[kPromoCount];
        // too many promotions at once (or no room left beside the ones still waiting
        // for the other composites): drop the epoch and retry with half the stride
        if (np > (uint32_t)y.promo_max || misc[kEventCount] + np > (uint32_t)y.event_cap) {
            bool minimal = true;
            for (int s2 = 0; s2 < S; s2++) minimal = minimal && s_stride[s2] <= 1;
            // Every thread has read the two counts and the strides before any of them is changed
            // below: a wavefront that came late would otherwise see the halved strides (or the
            // cleared count), decide differently and run the epoch the others are undoing.
            __syncthreads();
            if (minimal && np <= (uint32_t)y.promo_cap && misc[kEventCount] + np <= (uint32_t)y.event_cap) {
                // cannot go smaller; the tables still hold it
            } else if (minimal) {
                if (tid == 0) misc[kFail] = 2;
                __syncthreads();
                break;
            } else {
                if (tid < S) s_c[tid] = s_cprev[tid];
                if (tid < S) s_stride[tid] = max(1, s_stride[tid] / 2);
                if (tid == 0) misc[kPromoCount] = 0;
                shrunk = true;
                undone_once = true;
                __syncthreads();
                PHASE_END(4);
                continue;
            }
        }

        if (compact && misc[kSetMarked] + np > (uint32_t)y.set_limit) {     // (the same for every thread: last written before the barriers above)
            __syncthreads();
            if (tid == 0) misc[kFail] = 4;
            __syncthreads();
            break;
        }
        mark_promotions(np);      // the epoch stands: later scans skip its promotions

        // ---- 4. exact step of every promotion -----------------------------------
        if (np > 0) {     // sample every stream's new range once; all rankings of the epoch share it
            for (int idx = tid; idx < S * (kSamples - 1); idx += NT) {
                const int sidx = idx / (kSamples - 1), t = idx - sidx * (kSamples - 1) + 1;
                const int lo = s_cprev[sidx], len = s_c[sidx] - lo;
                if (len >= 32) {
                    probes++;
                    s_samp[sidx * kSamples + t] = stream_prio_bits(load_stream(sidx), lo + (int)(((uint32_t)len * (uint32_t)t) >> kSampleShift));
                }
            }
            __syncthreads();
        }
        PHASE_FENCE();
        {
            // Four lanes rank one promotion, so 16 promotions are in flight per wavefront;
            // each lane runs the binary searches of up to five streams in lockstep so that
            // their key reads overlap.
            constexpr int kGroup = 4, kPerLane = 5;
            const int gl = tid & (kGroup - 1);
            const int group = tid / kGroup;
            for (uint32_t pi = group; pi < np; pi += NT / kGroup) {
                const uint32_t pr = promo[pi];
                const uint32_t local = pr & 0x3ffffffu;
                const int m = (int)(pr >> 26);
                // farthest of the L windows that hold the point = the last one visited
                uint32_t w_bits = 0;
                int w_h = -1, w_side = 0, w_j = 0, w_t = 0;
                // (a lane's windows four at a time: first all their positions are read, then all their keys)
                constexpr int kWin = 4;
                for (int hb = gl; hb < a.L; hb += kGroup * kWin) {
                    int pos[kWin];
#pragma unroll
                    for (int u = 0; u < kWin; u++) {
                        const int h = min(hb + u * kGroup, a.L - 1);
                        pos[u] = (int)a.inv[(int64_t)(m * a.L + h) * a.N + off + local];
                    }
                    int side[kWin], j[kWin], t[kWin];
                    float kv[kWin];
#pragma unroll
                    for (int u = 0; u < kWin; u++) {
                        const int h = min(hb + u * kGroup, a.L - 1);
                        const int i = m * a.L + h;
                        const int p = s_p[i];
                        const float* key = a.skeys + (int64_t)i * a.N + off;
                        int kp;
                        if (pos[u] > p) {
                            const int d = pos[u] - (p + 1);
                            side[u] = 1; j[u] = div_T(d); t[u] = d - j[u] * T; kp = p + 1 + j[u] * T;
                        } else {
                            const int d = p - pos[u];
                            side[u] = 0; j[u] = div_T(d);
                            const int start = p - T + 1 - j[u] * T;
                            t[u] = pos[u] - start; kp = max(start, 0);
                        }
                        kv[u] = key[kp];
                    }
#pragma unroll
                    for (int u = 0; u < kWin; u++) {
                        const int h = hb + u * kGroup;
                        if (h >= a.L) continue;
                        probes++;
                        const uint32_t bits = __builtin_bit_cast(uint32_t, fabsf(kv[u] - s_qp[m * a.L + h]));
                        if (w_h < 0 || bits >= w_bits) { w_bits = bits; w_h = h; w_side = side[u]; w_j = j[u]; w_t = t[u]; }
                    }
                }
                auto farthest_of_two = [&](auto width) {      // (lane exchanges by immediate patterns: no address registers)
                    constexpr int O = decltype(width)::value;
                    const uint32_t ob = lane_xor<O>(w_bits);
                    const int oh = lane_xor<O>(w_h);
                    const int os = lane_xor<O>(w_side);
                    const int oj = lane_xor<O>(w_j);
                    const int ot = lane_xor<O>(w_t);
                    const bool take = oh >= 0 && (w_h < 0 || ob > w_bits || (ob == w_bits && oh > w_h));
                    if (take) { w_bits = ob; w_h = oh; w_side = os; w_j = oj; w_t = ot; }
                };
                static_assert(kGroup == 8 || kGroup == 4 || kGroup == 2, "exchange levels");
                if constexpr (kGroup >= 8) farthest_of_two(std::integral_constant<int, 4>());
                if constexpr (kGroup >= 4) farthest_of_two(std::integral_constant<int, 2>());
                farthest_of_two(std::integral_constant<int, 1>());
                // rank of that window = windows of the composite ordered before it
                uint32_t rank = 0;
                for (int s0 = gl; s0 < 2 * a.L; s0 += kGroup * kPerLane) {
                    // (a stream's description is read again from LDS for every probe -- cheap beside the
                    //  probe's own read -- instead of being held in registers for all the lane's streams)
                    int lo[kPerLane], hi[kPerLane];
                    bool strict[kPerLane];
#pragma unroll
                    for (int u = 0; u < kPerLane; u++) {
                        const int s2 = s0 + u * kGroup;
                        lo[u] = hi[u] = 0;
                        strict[u] = false;
                        if (s2 >= 2 * a.L) continue;
                        const int h2 = s2 >> 1, side2 = s2 & 1;
                        const int sidx = 2 * (m * a.L + h2) + side2;
                        if (h2 == w_h) {
                            const bool corner = s_p[sidx >> 1] == n - 1 && T >= 2;   // ghost window first
                            if (side2 == w_side) { lo[u] = hi[u] = w_j; continue; }
                            if (corner) { lo[u] = hi[u] = w_side ? 0 : s_ns[sidx]; continue; }
                            strict[u] = w_side == 0;
                        } else {
                            strict[u] = h2 > w_h;
                        }
                        // the epoch's range, narrowed by the sampled priorities
                        lo[u] = s_cprev[sidx]; hi[u] = s_c[sidx];
                        const int len = hi[u] - lo[u];
                        if (len >= 32) {
                            // the samples ascend: the number of them ordered before the window
                            // is the last such sample's index (independent reads, no search)
                            const uint32_t* tab = s_samp + sidx * kSamples;
                            int tl = 0;
#pragma unroll
                            for (int t2 = 1; t2 < kSamples; t2++) {
                                const uint32_t v = tab[t2];
                                tl += (strict[u] ? v < w_bits : v <= w_bits) ? 1 : 0;
                            }
                            const int base0 = lo[u];
                            if (tl > 0) lo[u] = base0 + (int)(((uint32_t)len * (uint32_t)tl) >> kSampleShift) + 1;
                            if (tl < kSamples - 1) hi[u] = base0 + (int)(((uint32_t)len * (uint32_t)(tl + 1)) >> kSampleShift);
                        }
                    }
                    for (;;) {
                        bool any = false;
#pragma unroll
                        for (int u = 0; u < kPerLane; u++) {
                            if (lo[u] < hi[u]) {
                                any = true;
                                const int mid = (lo[u] + hi[u]) >> 1;
                                int sidx = 2 * m * a.L + s0 + u * kGroup;
                                asm volatile("" : "+v"(sidx));      // (else the description is fetched once, before the loop, and kept)
                                const uint32_t v = stream_prio_bits(load_stream(sidx), mid);
                                probes++;
                                if (strict[u] ? v < w_bits : v <= w_bits) lo[u] = mid + 1; else hi[u] = mid;
                            }
                        }
                        if (!any) break;
                    }
#pragma unroll
                    for (int u = 0; u < kPerLane; u++) rank += (uint32_t)lo[u];
                }
                if constexpr (kGroup >= 8) rank += lane_xor<4>(rank);
                if constexpr (kGroup >= 4) rank += lane_xor<2>(rank);
                rank += lane_xor<1>(rank);
                if (gl == 0) {
                    const uint32_t slot = atomicAdd(&misc[kEventCount], 1u);
                    if (slot < (uint32_t)y.event_cap) events[slot] = pack_event(rank, m, w_t == 0, local);
                    else misc[kFail] = 3;
                }
            }
        }
        __syncthreads();
        PHASE_END(5);
        if (misc[kFail]) break;

        // ---- 5. replay promotions in (step, composite) order ----------------------
        const int ne = __builtin_amdgcn_readfirstlane((int)misc[kEventCount]);
        unsigned long long H = ~0ull;        // steps below H are complete for every composite
        for (int m = 0; m < a.M; m++) {      // (the lanes of a wavefront share a composite's streams)
            bool mine = true;
            for (int h = lane; h < 2 * a.L; h += kWave) {
                const int sidx = 2 * m * a.L + h;
                mine = mine && s_c[sidx] >= s_ns[sidx];
            }
            if (!__all(mine)) H = min(H, (unsigned long long)s_K[m]);
        }
        if (ne > 0) {
            int np2 = 2;
            while (np2 < ne) np2 <<= 1;
            for (int j = ne + tid; j < np2; j += NT) events[j] = ~0ull;
            bitonic_sort_u64(events, np2, tid);
        }
        PHASE_FENCE();
        if (ne <= kWave && wave == 0) {
            // Up to one event per lane: the walk below is the same as the serial one after
            // it, but reads steps and flags from registers (lane reads, ballots) instead of
            // LDS, one dependent round trip per event less; what it accepts is stored by
            // all lanes together afterwards.
            const bool have = lane < ne;
            const unsigned long long ev = have ? events[lane] : ~0ull;
            const uint32_t ev_t = (uint32_t)(ev >> 32);          // steps fit 32 bits (checked by the host)
            const uint32_t ev_e = (uint32_t)ev;
            const uint32_t local = ev_e & 0x1ffffffu;
            const bool pre = have && (compact ? set_has(kSetSeenTag | local) : (bool)((seen[local >> 5] >> (local & 31u)) & 1u));
            bool dup = false;      // the same point earlier in the list (promoted under another composite)
            for (int j = 0; j + 1 < ne; j++) {
                const uint32_t lj = (uint32_t)__builtin_amdgcn_readlane((int)local, j);
                dup = dup || (lane > j && lj == local);
            }
            const unsigned long long fresh_mask = __ballot(have && !pre && !dup);
            const unsigned long long lane0_mask = __ballot(have && (ev_e & (1u << 25)));
            // (first-lane reads tell the compiler that the walk's state is the same on every lane)
            auto uni = [](uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); };
            long long c0 = (long long)uni(misc[kC0]);
            bool armed = uni(misc[kArmed]) != 0;
            unsigned long long t_armed = ((unsigned long long)uni(misc[kArmedHi]) << 32) | uni(misc[kArmedLo]);
            bool stop = false;
            unsigned long long kk_star = 0;
            const unsigned long long last_needed = a.stop_at > 0 ? (unsigned long long)(a.stop_at - 1) : 0ull;
            int idx = 0;
            while (idx < ne) {
                const unsigned long long t = (uint32_t)__builtin_amdgcn_readlane((int)ev_t, idx);
                if (t >= H) break;
                if (armed) {
                    const unsigned long long cand = max(t_armed, last_needed);
                    if (cand < t) { stop = true; kk_star = cand; break; }
                }
                // all events of step t
                while (idx < ne && (uint32_t)__builtin_amdgcn_readlane((int)ev_t, idx) == (uint32_t)t) {
                    if ((fresh_mask >> idx) & (lane0_mask >> idx) & 1ull) c0++;
                    idx++;
                }
                if (c0 >= a.k_stop) {
                    if (!armed) { armed = true; t_armed = t; }
                    if (c0 >= a.max_cand || (long long)(t + 1) >= a.stop_at) { stop = true; kk_star = t; break; }
                }
            }
            if (!stop && armed) {
                const unsigned long long cand = max(t_armed, last_needed);
                if (cand < H) { stop = true; kk_star = cand; }
            }
            // events [0, idx) were walked: the fresh ones among them are accepted
            const unsigned long long walked = idx >= kWave ? ~0ull : ((1ull << idx) - 1ull);
            const unsigned long long take = fresh_mask & walked;
            const uint32_t nacc0 = misc[kAccCount], ncand0 = misc[kNumCand];
            if ((take >> lane) & 1ull) {
                const uint32_t slot = nacc0 + (uint32_t)__popcll(take & ((1ull << lane) - 1ull));
                acc[slot] = local;
                if (a.blind) acc_step[slot] = ev_t;
                if (compact) set_add(kSetSeenTag | local);
                else atomicOr(&seen[local >> 5], 1u << (local & 31u));
            }
            // keep what is not settled yet
            const int keep = stop ? 0 : ne - idx;
            if (!stop && lane >= idx && have) events[lane - idx] = ev;
            if (lane == 0) {
                misc[kEventCount] = (uint32_t)keep;
                misc[kC0] = (uint32_t)c0;
                misc[kArmed] = armed ? 1u : 0u;
                misc[kArmedLo] = (uint32_t)t_armed; misc[kArmedHi] = (uint32_t)(t_armed >> 32);
                misc[kAccCount] = nacc0 + (uint32_t)__popcll(take);
                misc[kNumCand] = ncand0 + (uint32_t)__popcll(take);
                misc[kStop] = stop ? 1u : 0u;
                misc[kStopStepLo] = (uint32_t)kk_star; misc[kStopStepHi] = (uint32_t)(kk_star >> 32);
                misc[kPromoCount] = 0;
                misc[kSetMarked] += np;
            }
        } else if (ne > kWave && tid == 0) {
            long long c0 = (long long)misc[kC0];
            bool armed = misc[kArmed] != 0;
            unsigned long long t_armed = ((unsigned long long)misc[kArmedHi] << 32) | misc[kArmedLo];
            uint32_t nacc = misc[kAccCount];
            uint32_t ncand = misc[kNumCand];
            bool stop = false;
            unsigned long long kk_star = 0;
            const unsigned long long last_needed = a.stop_at > 0 ? (unsigned long long)(a.stop_at - 1) : 0ull;
            int idx = 0;
            while (idx < ne) {
                const unsigned long long t = events[idx] >> 32;
                if (t >= H) break;
                if (armed) {
                    const unsigned long long cand = max(t_armed, last_needed);
                    if (cand < t) { stop = true; kk_star = cand; break; }
                }
                // all events of step t
                while (idx < ne && (events[idx] >> 32) == t) {
                    const uint32_t e = (uint32_t)events[idx];
                    const uint32_t local = e & 0x1ffffffu;
                    const uint32_t bit = 1u << (local & 31);
                    bool fresh;
                    if (compact) fresh = set_add(kSetSeenTag | local);
                    else { fresh = !(seen[local >> 5] & bit); seen[local >> 5] |= bit; }
                    if (fresh) {
                        if (a.blind) acc_step[nacc] = (uint32_t)t;
                        acc[nacc++] = local;
                        ncand++;
                        if (e & (1u << 25)) c0++;
                    }
                    idx++;
                }
                if (c0 >= a.k_stop) {
                    if (!armed) { armed = true; t_armed = t; }
                    if (c0 >= a.max_cand || (long long)(t + 1) >= a.stop_at) { stop = true; kk_star = t; break; }
                }
            }
            if (!stop && armed) {
                const unsigned long long cand = max(t_armed, last_needed);
                if (cand < H) { stop = true; kk_star = cand; }
            }
            // keep what is not settled yet
            int keep = 0;
            if (!stop) for (; idx < ne; idx++) events[keep++] = events[idx];
            misc[kEventCount] = (uint32_t)keep;
            misc[kC0] = (uint32_t)c0;
            misc[kArmed] = armed ? 1u : 0u;
            misc[kArmedLo] = (uint32_t)t_armed; misc[kArmedHi] = (uint32_t)(t_armed >> 32);
            misc[kAccCount] = nacc;
            misc[kNumCand] = ncand;
            misc[kStop] = stop ? 1u : 0u;
            misc[kStopStepLo] = (uint32_t)kk_star; misc[kStopStepHi] = (uint32_t)(kk_star >> 32);
            misc[kPromoCount] = 0;
            misc[kSetMarked] += np;
        }
        __syncthreads();
        PHASE_END(6);

        // ---- 6. distances of the accepted candidates, merged into the top-k ---------
        const int nacc = (int)misc[kAccCount];
        const bool stop = misc[kStop] != 0;
        for (int done = 0; done < nacc;) {      // in batches that fit beside the top-k
            const int topn = (int)misc[kTopN];
            const int batch = min(nacc - done, y.sort_cap - topn);
            if (a.blind) {      // scored by the promoting step (:498-505), no row is read
                for (int c = tid; c < batch; c += NT)
                    sortbuf[topn + c] = ((unsigned long long)acc_step[done + c] << 32) | (uint32_t)(off + acc[done + c]);
            }
            // two candidates per wavefront at a time: their row reads overlap
            const bool vec4 = rows_vec4(a.data, a.dim);
            for (int c = wave; c < (a.blind ? 0 : batch); c += 2 * kWaves) {
                const int c2 = c + kWaves;
                const int64_t pt0 = off + acc[done + c];
                const int64_t pt1 = c2 < batch ? off + acc[done + c2] : pt0;
                const float* const rows2[2] = {a.data + pt0 * a.dim, a.data + pt1 * a.dim};
                float d2[2];
                // (the query's row comes from global memory: it is read a few dozen times per item, and the
                //  room it took in LDS decides at some settings whether one more item fits a CU)
                wave_row_dists<2>(rows2, a.query + (int64_t)qi * a.dim, a.dim, vec4, d2, lane);
                if (lane == 0) {
                    sortbuf[topn + c] = ((unsigned long long)__builtin_bit_cast(uint32_t, d2[0]) << 32) | (uint32_t)pt0;
                    if (c2 < batch)
                        sortbuf[topn + c2] = ((unsigned long long)__builtin_bit_cast(uint32_t, d2[1]) << 32) | (uint32_t)pt1;
                }
            }
            int np2 = 2;
            while (np2 < topn + batch) np2 <<= 1;
            for (int j = topn + batch + tid; j < np2; j += NT) sortbuf[j] = ~0ull;
            bitonic_sort_u64(sortbuf, np2, tid);
            if (tid == 0) misc[kTopN] = (uint32_t)min(a.kcap, topn + batch);
            done += batch;
            __syncthreads();
        }
        if (nacc > 0) {
            if (tid == 0) misc[kAccCount] = 0;
            __syncthreads();
        }
        PHASE_END(7);
        if (stop) break;
        if (may_hand_over && misc[kNumCand] + misc[kEventCount] >= (uint32_t)hand_over_at) {
            // (the stop hints still learn from it: the dense kernel records its stops too)
            hand_to_dense();
            return;
        }
        PHASE_FENCE();
        bool mine_exhausted = true;     // every wavefront looks at all S <= 128 streams, a lane at two
        for (int s = lane; s < S; s += kWave) mine_exhausted = mine_exhausted && s_c[s] >= s_ns[s];
        if (__all(mine_exhausted)) break;     // H was unbounded: everything has been replayed
        {
            uint32_t kmax = 0, dk_lead = 1;
            for (int m = 0; m < a.M; m++)
                if (s_K[m] >= kmax) { kmax = s_K[m]; dk_lead = max(1u, s_K[m] - s_Kprev[m]); }
            // where to land next (steps per composite): just past the stop step once
            // c0 >= k; else by the hint; else twice the last stride
            const float hint_here = __builtin_bit_cast(float, misc[kHintSteps]);
            const float first_jump = __builtin_bit_cast(float, misc[kFirstJump]);
            const float aim = __builtin_bit_cast(float, misc[kPromoAimBits]);
            const float inv_L_here = __builtin_bit_cast(float, misc[kInvLBits]);
            const float S_f = (float)S;
            float k_target = (float)kmax + 2.0f * (float)dk_lead;
            const float need = __builtin_bit_cast(float, misc[kNeedBits]);
            if (misc[kArmed]) {
                const float t_armed = (float)(((unsigned long long)misc[kArmedHi] << 32) | misc[kArmedLo]);
                k_target = fmaxf(t_armed + 1.0f, need) + S_f;
            } else if (hint_here > 0.0f) {
                const float so_far = (float)max(1u, misc[kNumCand] + misc[kEventCount]);   // promotions up to here
                const float grow = fminf(kHintGrow, fast_pow(1.0f + aim / so_far, inv_L_here));
                k_target = (float)kmax < 0.9f * first_jump * hint_here ? first_jump * hint_here : grow * (float)kmax + S_f;
            }
            k_target = fminf(k_target, 2.0f * (float)kmax + 16.0f * S_f);
            if (shrunk) k_target = fminf(k_target, (float)kmax + 2.0f * (float)dk_lead);
            shrunk = false;       // the epoch after an undo was accepted: back to aimed epochs
            __syncthreads();
            if (tid < S) {
                const int m = (tid >> 1) / a.L;
                const float dk = (float)max(1u, s_K[m] - s_Kprev[m]);
                const float scale = fminf(16.0f, fmaxf(0.0f, k_target - (float)s_K[m]) / dk);
                const float want = ceilf((float)max(1, s_c[tid] - s_cprev[tid]) * scale);
                s_stride[tid] = (int)fminf(fmaxf(want, 1.0f), 16777216.0f);
            }
            __syncthreads();
            if (tid < a.M) s_Kprev[tid] = s_K[tid];
            __syncthreads();
        }
    }
    __syncthreads();

    if (misc[kFail] || epoch >= kMaxEpochs) {
        // hand the item to the step-by-step kernel
        if (a.phase_ticks && tid == 0) {
            atomicAdd(&a.phase_ticks[10], 1ull);
            atomicAdd(&a.phase_ticks[11 + min(3u, misc[kFail])], 1ull);
            a.phase_ticks[15] = ((unsigned long long)item << 32) | ((unsigned long long)misc[kEventCount] << 16) | misc[kPromoCount];
        }
        hand_back();
        return;
    }

    if (a.phase_ticks && tid == 0) {
        atomicAdd(&a.phase_ticks[8], (unsigned long long)epoch + 1);
        atomicAdd(&a.phase_ticks[9], 1ull);
    }
    if (a.stop_hint && tid == 0 && misc[kStop])
        record_stop(a.stop_hint, a.B, b, qi, (float)((((unsigned long long)misc[kStopStepHi] << 32) | misc[kStopStepLo]) + 1),
                    (float)(misc[kNumCand] + misc[kEventCount]));
    // ---- results -------------------------------------------------------------------
    const int topn = (int)misc[kTopN];
    for (int j = tid; j < a.kcap; j += NT) part_out[j] = j < topn ? sortbuf[j] : ~0ull;
    if (a.counters) {
        probes = wave_sum_u32(probes);
        if (lane == 0) atomicAdd(&misc[kProbes], probes);
        __syncthreads();
        if (tid == 0) {
            unsigned long long steps;   // outer steps the loop would have run (:458, :598-609)
            const unsigned long long bound = (unsigned long long)n * a.L * T;
            unsigned long long maxw = 0;
            for (int m = 0; m < a.M; m++) {
                unsigned long long w = 0;
                for (int h = 0; h < 2 * a.L; h++) w += (unsigned long long)s_ns[2 * m * a.L + h];
                maxw = max(maxw, w);
            }
            if (misc[kStop]) {
                steps = (((unsigned long long)misc[kStopStepHi] << 32) | misc[kStopStepLo]) + 1;
                steps = min(steps, min(bound, maxw + 1));
            } else {
                steps = min(bound, maxw + 1);
            }
            const unsigned long long st = ((unsigned long long)misc[kScannedHi] << 32) | misc[kScannedLo];
            atomicAdd(&a.counters[(int64_t)qi * 4 + 0], st);
            atomicAdd(&a.counters[(int64_t)qi * 4 + 1], (unsigned long long)misc[kNumCand]);
            atomicAdd(&a.counters[(int64_t)qi * 4 + 2], (unsigned long long)misc[kProbes]);
            atomicAdd(&a.counters[(int64_t)qi * 4 + 3], steps);
        }
    }
}

// MINW = waves per SIMD the register allocation must leave room for: LDS decides how
// many workgroups fit a CU, and the kernel should not be the tighter limit.
// Which (partition, query) a workgroup works on: see block_item (one partition's slices stay
// in the L2 of the XCD that works through its queries).
template <int NT, int MINW, bool COMPACT>
__global__ __launch_bounds__(NT, MINW) void traverse_block_kernel(QueryArgs a, BlockLayout y) {
    int b, qi;
    if (!block_item((int64_t)blockIdx.x, a.xcds, a.B, a.q_count, b, qi)) return;
    traverse_block_item<NT, MINW, COMPACT>(a, y, b, qi + a.q_first);
}
// Second pass: the workgroups stride over the list of items the compact variants handed back
// (its length is only known on the device, so the grid is a fixed number of resident workgroups).
template <int NT, int MINW>
__global__ __launch_bounds__(NT, MINW) void traverse_block_list_kernel(QueryArgs a, BlockLayout y) {
    const uint32_t listed = *a.block_list_count;
    const uint32_t count = (int64_t)listed < a.wide_cap ? listed : (uint32_t)a.wide_cap;
    for (uint32_t w = blockIdx.x; w < count; w += gridDim.x) {
        const int32_t item = a.block_list[w];
        traverse_block_item<NT, MINW, false>(a, y, item % a.B, item / a.B);
        __syncthreads();          // the next item reuses the tables
    }
}

constexpr int kBlockThreads = 256;
constexpr int kNarrowThreads = 128;     // workgroups of two wavefronts: more (query, partition) items per CU
constexpr int kLeadQueries = 32;

#undef PHASE_END
#undef PHASE_FENCE

}  // namespace

bool block_traversal_supported(const QueryArgs& a, size_t* lds_bytes) {
    const BlockLayout y = make_block_layout(a);
    if (lds_bytes) *lds_bytes = y.lds_bytes;
    const int I = a.M * a.L;
    if (!a.inv || !a.rpos || !a.rpos_ready || a.ppb > 65536) return false;   // positions inside a slice are 16-bit values
    if (4 * I > kBlockThreads || a.M > 64) return false;   // lane groups per stream in the searches; composite number in 6 bits
    if (a.kcap > 512) return false;
    if (a.ppb >= (1 << 25)) return false;
    if ((int64_t)a.L * (a.ppb + 2 * (int64_t)a.T) >= 0x7fffffffLL) return false;   // steps fit 32 bits
    if ((int64_t)a.ppb + 2 * (int64_t)a.T >= 0x7fffffffLL) return false;
    if (a.xcds < 1 || block_queries_per_launch(a.xcds, a.B, a.nq) < 1) return false;
    return y.lds_bytes <= 160 * 1024 - 512;
}

// One launch of the kernel variant that suits the layout: `items` workgroups.
static int launch_block(const QueryArgs& a, const BlockLayout& y, int64_t items, hipStream_t s) {
    const int fit = (int)(160 * 1024 / y.lds_bytes);      // workgroups per CU by LDS
#define DCIH_LAUNCH_KERNEL(KERNEL, NT, GRID)                                                      \
    do {                                                                                           \
        static DeviceOnce once;                                                                    \
        const int rc_attr = once.run([]() -> int {                                                 \
            DCIH_HIP(hipFuncSetAttribute((const void*)KERNEL,                                      \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024)); \
            return 0;                                                                              \
        });                                                                                        \
        if (rc_attr) return rc_attr;                                                               \
        hipLaunchKernelGGL(KERNEL, dim3((unsigned)(GRID)), dim3(NT), y.lds_bytes, s, a, y);        \
    } while (0)
#define DCIH_LAUNCH_COMPACT(MW) DCIH_LAUNCH_KERNEL((traverse_block_kernel<kWave, MW, true>), kWave, items)
    // (the second pass: as many workgroups as the device holds at a time, striding over the list)
    const int64_t resident = std::min(items, (int64_t)a.xcds * 32 * std::max(1, fit));
#define DCIH_LAUNCH(NT, MW)                                                                        \
    do {                                                                                           \
        if (a.block_list) DCIH_LAUNCH_KERNEL((traverse_block_list_kernel<NT, MW>), NT, resident);  \
        else DCIH_LAUNCH_KERNEL((traverse_block_kernel<NT, MW, false>), NT, items);                \
    } while (0)
    // The kernel's time is chains of dependent reads, so what counts is how many items a CU holds: as
    // many as LDS lets in, with the registers that leaves (wavefronts per SIMD = the second template
    // argument).  Full layout: two wavefronts per item where LDS lets ten or more items into a CU (and the
    // streams fit their lane groups), else four.  Measured on 1M x 128, thread_size 2: 17242-point
    // partitions, four wavefronts per item, 5 / 6 / 7 workgroups per CU 275 / 301 / 309 k queries/s; two
    // wavefronts, ten / twelve / thirteen workgroups 326 / 349 / 354 k; with fewer items per CU two
    // wavefronts lose to four (287 against 300 k at 26316 points, 79.5 against 88.0 k with eight or nine
    // items at 26316 points, thread_size 3, 5000 iterations); with the 256-entry tables of the reference's
    // default setting (10000-point partitions, thread_size 10) two wavefronts give 88.4 against 76.0 k.
    // One wavefront with the full layout, thirteen items, 260 k; one wavefront with the compact layout,
    // twenty-six items, 366 k.
    if (y.set_slots) {      // compact layout: one wavefront per item
        const int w = fit >= 25 ? 7 : (fit >= 21 ? 6 : (fit >= 17 ? 5 : 4));
        if (w == 7) DCIH_LAUNCH_COMPACT(7); else if (w == 6) DCIH_LAUNCH_COMPACT(6);
        else if (w == 5) DCIH_LAUNCH_COMPACT(5); else DCIH_LAUNCH_COMPACT(4);
        DCIH_HIP(hipGetLastError());
        return 0;
    }
    const bool narrow = 4 * a.M * a.L <= kNarrowThreads && fit >= 10;
    int minw = narrow ? (fit * (kNarrowThreads / 64) + 3) / 4 : fit;      // wavefronts per SIMD
    minw = minw >= 7 ? 7 : (minw < 3 ? 3 : minw);
    if (narrow) {
        if (minw >= 7) DCIH_LAUNCH(kNarrowThreads, 7); else if (minw == 6) DCIH_LAUNCH(kNarrowThreads, 6);
        else if (minw == 5) DCIH_LAUNCH(kNarrowThreads, 5); else if (minw == 4) DCIH_LAUNCH(kNarrowThreads, 4);
        else DCIH_LAUNCH(kNarrowThreads, 3);
    } else {
        if (minw >= 7) DCIH_LAUNCH(kBlockThreads, 7); else if (minw == 6) DCIH_LAUNCH(kBlockThreads, 6);
        else if (minw == 5) DCIH_LAUNCH(kBlockThreads, 5); else if (minw == 4) DCIH_LAUNCH(kBlockThreads, 4);
        else DCIH_LAUNCH(kBlockThreads, 3);
    }
#undef DCIH_LAUNCH
#undef DCIH_LAUNCH_COMPACT
#undef DCIH_LAUNCH_KERNEL
    DCIH_HIP(hipGetLastError());
    return 0;
}

int query_block(const QueryArgs& a_in, hipStream_t s) {
    const BlockLayout y = make_block_layout(a_in);
    // as many queries per launch as the launch limit allows (nearly always all of them)
    const int per_launch = block_queries_per_launch(a_in.xcds, a_in.B, a_in.nq);
    if (per_launch < 1) return fail(-4, "query: block_size too large for the batch traversal kernel");
    // The items that outgrow the compact tables are taken up again with the full ones, if those fit
    // LDS (else they go to the step-by-step kernel like everything else the kernel hands back).
    QueryArgs second = a_in;
    second.full_tables = 1;
    second.block_list = a_in.wide_items;
    second.block_list_count = a_in.wide_count;
    second.wide_items = nullptr;
    second.q_first = 0;
    second.q_count = a_in.nq;
    const BlockLayout y2 = make_block_layout(second);
    const bool two_passes = y.set_slots != 0 && a_in.wide_items != nullptr && a_in.wide_cap > 0 &&
                            y2.lds_bytes <= 160 * 1024 - 512;
    // With nothing known yet about where traversals stop, a few queries go ahead in a launch of
    // their own: their stops are on record when the others start, which then size their first
    // epoch from them instead of feeling their way forward (the first resident round of every
    // partition would otherwise do that in the middle of the large launch).  Results do not depend on it.
    const int lead = a_in.hints_cold && a_in.stop_hint && a_in.nq >= 8 * kLeadQueries ? kLeadQueries : 0;
    for (int q0 = 0; q0 < a_in.nq; q0 += (q0 < lead ? lead : per_launch)) {
        QueryArgs a = a_in;
        if (!two_passes) a.wide_items = nullptr;
        a.q_first = q0;
        a.q_count = q0 < lead ? lead : min(per_launch, a_in.nq - q0);
        const int rc = launch_block(a, y, block_items(a.xcds, a.B, a.q_count), s);
        if (rc) return rc;
    }
    if (two_passes) {
        const int64_t most = min(a_in.wide_cap, (int64_t)a_in.nq * a_in.B);
        const int rc = launch_block(second, y2, most, s);
        if (rc) return rc;
    }
    return 0;
}

}  // namespace dcih
