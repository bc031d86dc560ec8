// Host side of libdci_hip.so: the C-ABI declared in include/dci_hip.h (and the
// inspection entry points of include/dci_hip_debug.h).
//
// Mirrors the host functions of the reference (dci_init, dci_add, dci_query,
// dci_clear, dci_reset, dci_free: src/dci_cuda_kernel.cu:77-187, :777-899) but
// returns status codes instead of asserting, takes a stream, frees what it
// allocates, and launches a constant number of kernels per call instead of
// several per query.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <new>
#include <string>
#include <vector>

#include "../../include/dci_hip.h"
#include "../../include/dci_hip_debug.h"
#include "common.h"
#include "kernels.h"

namespace dcih {

static thread_local std::string g_last_error;

int fail(int code, const std::string& msg) {
    g_last_error = msg;
    return code;
}

namespace {

// splitmix64 -> xoshiro256** -> Box-Muller in double: the same seed gives the
// same directions on every machine.
struct Rng {
    uint64_t s[4];
    bool have_spare = false;
    double spare = 0.0;
    explicit Rng(uint64_t seed) {
        uint64_t x = seed;
        for (int i = 0; i < 4; i++) {
            x += 0x9e3779b97f4a7c15ull;
            uint64_t z = x;
            z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
            z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
            s[i] = z ^ (z >> 31);
        }
    }
    static uint64_t rotl(uint64_t v, int k) { return (v << k) | (v >> (64 - k)); }
    uint64_t next() {
        const uint64_t r = rotl(s[1] * 5, 7) * 9;
        const uint64_t t = s[1] << 17;
        s[2] ^= s[0]; s[3] ^= s[1]; s[1] ^= s[2]; s[0] ^= s[3];
        s[2] ^= t; s[3] = rotl(s[3], 45);
        return r;
    }
    double uniform() { return ((next() >> 11) + 0.5) * (1.0 / 9007199254740992.0); }  // (0,1)
    double normal() {
        if (have_spare) { have_spare = false; return spare; }
        const double u = uniform(), v = uniform();
        const double r = std::sqrt(-2.0 * std::log(u));
        const double th = 6.283185307179586476925 * v;
        spare = r * std::sin(th);
        have_spare = true;
        return r * std::cos(th);
    }
};

struct DeviceGuard {
    int prev = -1;
    bool ok;
    explicit DeviceGuard(int dev) {
        ok = hipGetDevice(&prev) == hipSuccess && hipSetDevice(dev) == hipSuccess;
    }
    ~DeviceGuard() { if (prev >= 0) (void)hipSetDevice(prev); }
};

}  // namespace
}  // namespace dcih

using namespace dcih;

// Scratch of dcih_query_noalloc: part of the code object, so every device the library
// runs on holds its own copy from the moment the library is loaded there until the
// process ends.  Host code never uses this name as an address (on the host it is only a
// stand-in for the symbol): dcih_create asks the runtime where the array lives on its
// device and keeps that pointer.  (The host code's use of the name below is what gives the
// device symbol external linkage, which the runtime's lookup by name needs: a `used`
// attribute would keep it local to the code object and the lookup would abort.)
constexpr size_t kScratchBytes = DCIH_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
constexpr int kMaxXcds = 32;      // dies per device the query scratch has list lengths for (256 bytes: 1 + 32 words used)
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on `device`, which must be the current device.
int resolve_scratch(int device) {
    if (device < 0 || device >= kMaxDevices) return fail(DCIH_EINVAL, "device number out of range");
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (g_scratch_ptr[device]) return 0;
    void* ptr = nullptr;
    DCIH_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return fail(DCIH_EHIP, "hipGetSymbolAddress returned no address for the scratch array");
    g_scratch_ptr[device] = ptr;
    return 0;
}

void* scratch_of(int device) {
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    return device >= 0 && device < kMaxDevices ? g_scratch_ptr[device] : nullptr;
}
}  // namespace

struct dcih_index {
    int dim = 0, M = 0, L = 0, device = 0;
    int xcds = 8;                       // accelerator dies of the device
    uint64_t seed = 0;
    uint64_t draws = 0;                 // direction sets drawn so far
    std::vector<float> h_dirs;          // [I][dim]
    float* d_dirs = nullptr;
    const float* d_data = nullptr;      // borrowed
    int64_t n = 0;
    int block_size = 0;
    float* d_skeys = nullptr;           // [I][n]
    int32_t* d_sids = nullptr;          // [I][n]
    uint16_t* d_inv = nullptr;          // [I][n] position of each point in its sorted slice (partitions <= 65536 points)
    uint16_t* d_rpos = nullptr;         // [I][n] the same, in the order of each composite's first simple index (room kept by the
                                        // build, filled by the first query that runs the batch traversal kernel)
    int rpos_ready = 0;
    float* d_own = nullptr;             // rows copied in by dcih_append (the index owns these)
    float* d_ukeys = nullptr;           // [I][own_rows] unsorted projections of the rows in d_own
    int64_t own_rows = 0;               // capacity of d_own / d_ukeys in rows
    int64_t ukeys_rows = 0;             // leading rows of d_own whose projections d_ukeys holds
    float* d_stop_hint = nullptr;       // [3][block_size] epoch-size hints learnt from earlier queries
    int hint_k = 0, hint_outer = 0, hint_T = 0, hint_maxc = 0;   // query shape the hints belong to
    int traversal = 0;                  // DCIH_OPT_TRAVERSAL value
    int dense_min_promos = 160;         // DCIH_OPT_DENSE_MIN_PROMOTIONS value
    int append_mode = 0;                // DCIH_OPT_APPEND value
    unsigned long long* d_phase_ticks = nullptr;   // optional profile of the batch kernel
    // grow-only workspace: query scratch, and the unsorted keys during a build
    void* ws = nullptr;
    size_t ws_bytes = 0;
    // grow-only arenas the sorted arrays and the hint table are carved from; kept
    // across dcih_clear so that a rebuild allocates nothing.  The index lives in
    // arena[cur]; dcih_append builds the next one in the other and then switches, so
    // a failed append leaves the index as it was.
    void* arena[2] = {nullptr, nullptr};
    size_t arena_bytes[2] = {0, 0};
    int cur = 0;
    // optional per-kernel timing: ev[2*t], ev[2*t+1] bracket timer t
    bool profiling = false;
    hipEvent_t ev[2 * DCIH_NUM_TIMERS] = {};
    bool ev_valid[DCIH_NUM_TIMERS] = {};
};

namespace {

int num_indices(const dcih_index* h) { return h->M * h->L; }

// Draws direction set number h->draws from the handle's seed and uploads it.
int draw_directions(dcih_index* h) {
    const int I = num_indices(h);
    Rng rng(h->seed + 0x632be59bd9b4e019ull * h->draws);
    h->draws++;
    h->h_dirs.resize((size_t)I * h->dim);
    for (auto& v : h->h_dirs) v = (float)rng.normal();
    // unit rows: sequential fp32 sum of squares, sqrtf, divide
    // (normalize_proj_vecs, src/dci_cuda_kernel.cu:52-73)
    for (int r = 0; r < I; r++) {
        float* row = h->h_dirs.data() + (size_t)r * h->dim;
        float sq = 0.0f;
        for (int k = 0; k < h->dim; k++) sq += row[k] * row[k];
        const float norm = sqrtf(sq);
        for (int k = 0; k < h->dim; k++) row[k] /= norm;
    }
    DCIH_HIP(hipMemcpy(h->d_dirs, h->h_dirs.data(), h->h_dirs.size() * sizeof(float),
                       hipMemcpyHostToDevice));
    return 0;
}

// Drops the sorted arrays (their arena stays allocated for the next build) but keeps the rows.
int release_sorted(dcih_index* h) {
    h->d_skeys = nullptr;
    h->d_sids = nullptr;
    h->d_inv = nullptr;
    h->d_rpos = nullptr;
    h->rpos_ready = 0;
    h->d_stop_hint = nullptr;
    return 0;
}

int release_arena(dcih_index* h) {
    (void)release_sorted(h);
    for (int j = 0; j < 2; j++)
        if (h->arena[j]) { (void)hipFree(h->arena[j]); h->arena[j] = nullptr; h->arena_bytes[j] = 0; }
    return 0;
}

int release_index(dcih_index* h) {
    const int rc = release_sorted(h);
    if (h->d_own) { (void)hipFree(h->d_own); h->d_own = nullptr; }
    if (h->d_ukeys) { (void)hipFree(h->d_ukeys); h->d_ukeys = nullptr; }
    h->own_rows = h->ukeys_rows = 0;
    h->d_data = nullptr;
    h->n = 0;
    h->block_size = 0;
    return rc;
}

// True while `s` is recording into a graph: nothing may be allocated or freed then.
bool capturing(hipStream_t s) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    return hipStreamIsCapturing(s, &st) == hipSuccess && st != hipStreamCaptureStatusNone;
}

int ensure_ws(dcih_index* h, size_t bytes, hipStream_t s) {
    if (bytes <= h->ws_bytes) return 0;
    if (capturing(s))
        return fail(DCIH_ESTATE, "the workspace would have to grow while the stream is being captured: "
                                 "run the same call once outside the capture first");
    if (h->ws) { DCIH_HIP(hipFree(h->ws)); h->ws = nullptr; h->ws_bytes = 0; }
    DCIH_HIP(hipMalloc(&h->ws, bytes));
    h->ws_bytes = bytes;
    return 0;
}

size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

// Makes arena `which` at least `bytes` large.  Growing frees that arena first, so it must
// not hold the live index.
int ensure_arena(dcih_index* h, int which, size_t bytes) {
    if (bytes <= h->arena_bytes[which]) return 0;
    if (h->arena[which]) { DCIH_HIP(hipFree(h->arena[which])); h->arena[which] = nullptr; h->arena_bytes[which] = 0; }
    DCIH_HIP(hipMalloc(&h->arena[which], bytes));
    h->arena_bytes[which] = bytes;
    return 0;
}

// Where the arrays of an index of n points lie inside an arena.
struct ArenaLayout {
    size_t keys, ids, inv, rpos, hint, total;   // byte offsets, and the size of it all
    bool small_parts;                           // partitions of at most 65536 points: 16-bit tables exist
};
ArenaLayout arena_layout(int I, int64_t n, int block_size) {
    ArenaLayout y;
    const size_t cells = (size_t)I * (size_t)n;
    y.small_parts = (n + block_size - 1) / block_size <= 65536;
    const size_t b_keys = align_up(cells * sizeof(float));
    const size_t b_ids = align_up(cells * sizeof(int32_t));
    // +16: the traversal reads whole 16-byte chunks of positions, also at the very end
    const size_t b_inv = y.small_parts ? align_up((cells + 16) * sizeof(uint16_t)) : 0;
    const size_t b_hint = align_up((size_t)3 * block_size * sizeof(float));   // stop step, promotions at the stop, stops seen
    y.keys = 0;
    y.ids = b_keys;
    y.inv = y.ids + b_ids;
    y.rpos = y.inv + b_inv;
    y.hint = y.rpos + b_inv;
    y.total = y.hint + b_hint;
    return y;
}

// Records the start (which = 0) or end (1) event of timer t when profiling.
void mark(dcih_index* h, int t, int which, hipStream_t s) {
    if (!h->profiling) return;
    (void)hipEventRecord(h->ev[2 * t + which], s);
    if (which) h->ev_valid[t] = true;
}

}  // namespace

extern "C" {

const char* dcih_last_error(void) { return g_last_error.c_str(); }

int dcih_abi_version(void) { return 2; }

int dcih_create(int dim, int num_comp_indices, int num_simp_indices, int device,
                uint64_t seed, dcih_index** out) {
    if (!out) return fail(DCIH_EINVAL, "dcih_create: out is null");
    *out = nullptr;
    if (dim <= 0 || num_comp_indices <= 0 || num_simp_indices <= 0)
        return fail(DCIH_EINVAL, "dcih_create: dim and index counts must be positive");
    if ((int64_t)num_comp_indices * num_simp_indices > (1 << 20))
        return fail(DCIH_EINVAL, "dcih_create: too many simple indices");
    int ndev = 0;
    DCIH_HIP(hipGetDeviceCount(&ndev));
    if (device < 0 || device >= ndev) return fail(DCIH_EINVAL, "dcih_create: no such device");
    DeviceGuard guard(device);
    if (!guard.ok) return fail(DCIH_EHIP, "dcih_create: cannot select device");
    dcih_index* h = new (std::nothrow) dcih_index();
    if (!h) return fail(DCIH_EHIP, "dcih_create: out of host memory");
    h->dim = dim; h->M = num_comp_indices; h->L = num_simp_indices;
    h->device = device; h->seed = seed;
    {   // dies with an L2 of their own: the batch traversal orders its work by them
        int xcds = 0;
        // (the per-die list lengths of the query scratch have room for kMaxXcds dies; a device
        //  that reports more, or none, is treated as one of 8)
        if (hipDeviceGetAttribute(&xcds, hipDeviceAttributeNumberOfXccs, device) == hipSuccess &&
            xcds >= 1 && xcds <= kMaxXcds)
            h->xcds = xcds;
        (void)hipGetLastError();
    }
    if (const int rc_s = resolve_scratch(device)) { delete h; return rc_s; }
    const size_t bytes = (size_t)num_indices(h) * dim * sizeof(float);
    if (hipMalloc(&h->d_dirs, bytes) != hipSuccess) {
        delete h;
        return fail(DCIH_EHIP, "dcih_create: hipMalloc of the directions failed");
    }
    const int rc = draw_directions(h);
    if (rc) { (void)hipFree(h->d_dirs); delete h; return rc; }
    *out = h;
    return DCIH_OK;
}

int dcih_get_directions(const dcih_index* h, float* h_dirs) {
    if (!h || !h_dirs) return fail(DCIH_EINVAL, "dcih_get_directions: null argument");
    std::memcpy(h_dirs, h->h_dirs.data(), h->h_dirs.size() * sizeof(float));
    return DCIH_OK;
}

int dcih_set_directions(dcih_index* h, const float* h_dirs) {
    if (!h || !h_dirs) return fail(DCIH_EINVAL, "dcih_set_directions: null argument");
    if (h->n > 0) return fail(DCIH_ESTATE, "dcih_set_directions: index is not empty");
    DeviceGuard guard(h->device);
    std::memcpy(h->h_dirs.data(), h_dirs, h->h_dirs.size() * sizeof(float));
    DCIH_HIP(hipMemcpy(h->d_dirs, h_dirs, h->h_dirs.size() * sizeof(float), hipMemcpyHostToDevice));
    return DCIH_OK;
}

// Sorts the projections of `num_points` rows (index i's at d_keys + i * key_stride) into
// arena `which`, which must already be large enough, and makes the result the handle's
// index over the rows at d_data.  Synchronises the stream before returning; on failure the
// handle's fields are untouched.
// With merge_from > 0 the live index (over the first merge_from points, in the other arena) is
// merged with the sorted new points instead of everything being sorted again.
static int sort_into(dcih_index* h, int which, const float* d_keys, int64_t key_stride,
                     int64_t num_points, const float* d_data, int block_size, void* d_tmp,
                     hipStream_t s, int64_t merge_from = 0) {
    const int I = num_indices(h);
    const ArenaLayout y = arena_layout(I, num_points, block_size);
    char* base = (char*)h->arena[which];
    float* skeys = (float*)(base + y.keys);
    int32_t* sids = (int32_t*)(base + y.ids);
    uint16_t* inv = y.small_parts ? (uint16_t*)(base + y.inv) : nullptr;
    float* hint = (float*)(base + y.hint);
    // (the table's room is a multiple of 256 bytes, so whole 64-bit words may be cleared)
    int rc = zero_words64(hint, (int64_t)(((size_t)3 * block_size * sizeof(float) + 7) / 8), s);
    if (rc == DCIH_OK) {
        mark(h, DCIH_T_SEGSORT, 0, s);
        if (merge_from > 0)
            rc = segsort_append(h->d_skeys, h->d_sids, merge_from, d_keys, key_stride, I, num_points, block_size,
                                skeys, sids, inv, nullptr, d_tmp, s);
        else
            rc = segsort(d_keys, key_stride, I, num_points, block_size, skeys, sids, inv, nullptr, d_tmp, s);
        mark(h, DCIH_T_SEGSORT, 1, s);
    }
    // like the reference's dci_add, the call returns when the index is complete
    const hipError_t se = hipStreamSynchronize(s);
    if (rc == DCIH_OK && se != hipSuccess)
        rc = fail(DCIH_EHIP, std::string("build: ") + hipGetErrorString(se));
    if (rc) return rc;
    h->d_skeys = skeys; h->d_sids = sids; h->d_inv = inv; h->d_stop_hint = hint;
    h->d_rpos = y.small_parts ? (uint16_t*)(base + y.rpos) : nullptr;
    h->rpos_ready = 0;
    h->cur = which;
    h->d_data = d_data;
    h->n = num_points;
    h->block_size = block_size;
    h->hint_k = h->hint_outer = h->hint_T = h->hint_maxc = 0;
    return DCIH_OK;
}

int dcih_add(dcih_index* h, int dim, int64_t num_points, const float* d_data,
             int block_size, int thread_size, void* stream) {
    if (!h) return fail(DCIH_EINVAL, "dcih_add: null handle");
    if (dim != h->dim) return fail(DCIH_EINVAL, "dcih_add: dim differs from the index's");
    if (h->n > 0) return fail(DCIH_ESTATE, "dcih_add: index already holds points; clear it first");
    if (num_points <= 0 || !d_data) return fail(DCIH_EINVAL, "dcih_add: no points given");
    if (num_points > 0x7fffffffLL) return fail(DCIH_EINVAL, "dcih_add: more than 2^31-1 points");
    if (block_size <= 0 || thread_size <= 0)
        return fail(DCIH_EINVAL, "dcih_add: block_size and thread_size must be positive");
    DeviceGuard guard(h->device);
    hipStream_t s = (hipStream_t)stream;
    const int I = num_indices(h);
    // one arena for what the index keeps, the workspace for what only the build needs
    // (the unsorted keys): a rebuild of the same size allocates and frees nothing
    const size_t b_keys = align_up((size_t)I * num_points * sizeof(float));
    const size_t tmp_bytes = segsort_tmp_bytes(I, num_points, block_size);
    int rc = ensure_arena(h, h->cur, arena_layout(I, num_points, block_size).total);
    if (rc == DCIH_OK) rc = ensure_ws(h, b_keys + align_up(tmp_bytes), s);
    if (rc == DCIH_OK) {
        float* d_keys = (float*)h->ws;
        mark(h, DCIH_T_PROJECT, 0, s);
        rc = project(h->d_dirs, I, d_data, num_points, dim, d_keys, num_points, s);
        mark(h, DCIH_T_PROJECT, 1, s);
        if (rc == DCIH_OK)
            rc = sort_into(h, h->cur, d_keys, num_points, num_points, d_data, block_size,
                           tmp_bytes ? (void*)((char*)h->ws + b_keys) : nullptr, s);
        else
            (void)hipStreamSynchronize(s);
    }
    if (rc) (void)release_index(h);
    return rc;
}

int dcih_append(dcih_index* h, int dim, int64_t num_points, const float* d_data,
                int block_size, int thread_size, void* stream) {
    if (!h) return fail(DCIH_EINVAL, "dcih_append: null handle");
    if (dim != h->dim) return fail(DCIH_EINVAL, "dcih_append: dim differs from the index's");
    if (num_points <= 0 || !d_data) return fail(DCIH_EINVAL, "dcih_append: no points given");
    if (block_size <= 0 || thread_size <= 0)
        return fail(DCIH_EINVAL, "dcih_append: block_size and thread_size must be positive");
    if (h->n > 0 && block_size != h->block_size)
        return fail(DCIH_EINVAL, "dcih_append: block_size differs from the one the index was built with");
    const int64_t total = h->n + num_points;
    if (total > 0x7fffffffLL) return fail(DCIH_EINVAL, "dcih_append: more than 2^31-1 points");
    DeviceGuard guard(h->device);
    hipStream_t s = (hipStream_t)stream;
    const int I = num_indices(h);
    const size_t row_bytes = (size_t)dim * sizeof(float);

    // Everything that can fail for lack of memory happens before the index is touched:
    // room for the rows and their projections (both owned by the index, capacity doubles
    // so that copies amortise), for the next index in the spare arena, and for the sort.
    float* rows = h->d_own;
    float* ukeys = h->d_ukeys;
    int64_t cap = h->own_rows;
    int64_t have_keys = (h->n > 0 && h->d_data == h->d_own) ? std::min(h->ukeys_rows, h->n) : 0;
    const int spare = 1 - h->cur;
    // Merging the old slices with the sorted new points instead of sorting everything again.
    // Both are built; left to choose, the append sorts: the one-pass LDS sort moves 16 bytes per
    // index entry, split + merge + inverse move 40, and on an MI355X the sort is the faster of the
    // two at every size of the incremental workload (8.7 against 9.0 ms for 1M onto 19M points).
    const bool merge = h->n > 0 && h->append_mode == 2 && h->d_inv != nullptr &&
                       segsort_append_supported(h->n, total, block_size);
    if (h->append_mode == 2 && h->n > 0 && !merge)
        return fail(DCIH_EUNSUPPORTED, "dcih_append: this shape cannot be appended by merging (partitions too long)");
    float* fresh_rows = nullptr;
    float* fresh_keys = nullptr;
    if (!rows || cap < total) {
        cap = std::max<int64_t>(total, 2 * h->own_rows);
        if (hipMalloc(&fresh_rows, (size_t)cap * row_bytes) != hipSuccess ||
            hipMalloc(&fresh_keys, (size_t)I * cap * sizeof(float)) != hipSuccess) {
            (void)hipGetLastError();
            if (fresh_rows) (void)hipFree(fresh_rows);
            return fail(DCIH_EHIP, "dcih_append: out of device memory for the rows (the index is unchanged)");
        }
        rows = fresh_rows;
        ukeys = fresh_keys;
    }
    const size_t tmp_bytes = merge ? segsort_append_tmp_bytes(I, total) : segsort_tmp_bytes(I, total, block_size);
    int rc = ensure_arena(h, h->n > 0 ? spare : h->cur,
                          std::max(arena_layout(I, total, block_size).total,
                                   arena_layout(I, cap, block_size).total));
    if (rc == DCIH_OK && tmp_bytes) rc = ensure_ws(h, align_up(tmp_bytes), s);
    hipError_t e = hipSuccess;
    if (rc == DCIH_OK && h->n > 0 && rows != h->d_data)        // rows (and projections) indexed so far
        e = hipMemcpyAsync(rows, h->d_data, (size_t)h->n * row_bytes, hipMemcpyDeviceToDevice, s);
    if (rc == DCIH_OK && e == hipSuccess && have_keys > 0 && ukeys != h->d_ukeys)
        e = hipMemcpy2DAsync(ukeys, (size_t)cap * sizeof(float), h->d_ukeys, (size_t)h->own_rows * sizeof(float),
                             (size_t)have_keys * sizeof(float), (size_t)I, hipMemcpyDeviceToDevice, s);
    if (rc == DCIH_OK && e == hipSuccess)
        e = hipMemcpyAsync(rows + (size_t)h->n * dim, d_data, (size_t)num_points * row_bytes,
                           hipMemcpyDeviceToDevice, s);
    if (rc == DCIH_OK && e != hipSuccess) rc = fail(DCIH_EHIP, std::string("dcih_append: ") + hipGetErrorString(e));
    if (rc == DCIH_OK) {
        // only rows without kept projections are projected: the new ones, after a plain
        // dcih_add (which keeps none) all of them
        mark(h, DCIH_T_PROJECT, 0, s);
        rc = project(h->d_dirs, I, rows + (size_t)have_keys * dim, total - have_keys, dim,
                     ukeys + have_keys, cap, s);
        mark(h, DCIH_T_PROJECT, 1, s);
    }
    if (rc == DCIH_OK)
        // the partition boundaries move with the total, so every slice is formed again
        rc = sort_into(h, h->n > 0 ? spare : h->cur, ukeys, cap, total, rows, block_size,
                       tmp_bytes ? h->ws : nullptr, s, merge ? h->n : 0);
    else
        (void)hipStreamSynchronize(s);
    if (rc) {       // the index stays as it was
        if (fresh_rows) (void)hipFree(fresh_rows);
        if (fresh_keys) (void)hipFree(fresh_keys);
        return rc;
    }
    if (fresh_rows) {
        if (h->d_own) (void)hipFree(h->d_own);
        if (h->d_ukeys) (void)hipFree(h->d_ukeys);
        h->d_own = fresh_rows;
        h->d_ukeys = fresh_keys;
        h->own_rows = cap;
    }
    h->ukeys_rows = total;
    return DCIH_OK;
}

// dcih_query and dcih_query_noalloc.  `fixed` = take every byte of scratch from the
// device's static array and refuse what does not fit, instead of growing the handle's
// workspace.
static int query_impl(dcih_index* h, int dim, int num_queries, const float* d_query,
                      int num_neighbours, int blind, int num_outer_iterations,
                      int max_num_candidates, int block_size, int thread_size,
                      int32_t* d_nn, float* d_dists, uint64_t* d_counters, void* stream,
                      bool fixed, const char* who) {
    const std::string me(who);
    if (!h) return fail(DCIH_EINVAL, me + ": null handle");
    if (dim != h->dim) return fail(DCIH_EINVAL, me + ": dim differs from the index's");
    if (h->n <= 0) return fail(DCIH_ESTATE, me + ": index is empty");
    if (num_neighbours <= 0 || num_neighbours > h->n)
        return fail(DCIH_EINVAL, me + ": num_neighbours must be in [1, num_points]");
    if (num_queries < 0 || (num_queries > 0 && (!d_query || !d_nn || (!blind && !d_dists))))
        return fail(DCIH_EINVAL, me + ": null buffer");
    // blind: as many candidates per query as the reference's result buffer holds (:782-783)
    const int64_t num_results =
        blind ? std::min<int64_t>(max_num_candidates, num_outer_iterations) : num_neighbours;
    if (num_results <= 0)
        return fail(DCIH_EINVAL, me + ": blind querying needs positive max_num_candidates and num_outer_iterations");
    if (thread_size <= 0) return fail(DCIH_EINVAL, me + ": thread_size must be positive");
    if (block_size != h->block_size)
        return fail(DCIH_EINVAL, me + ": block_size differs from the one the index was built with");
    if (num_queries == 0) return DCIH_OK;
    DeviceGuard guard(h->device);
    hipStream_t s = (hipStream_t)stream;
    const int I = num_indices(h);
    // the scratch of this call: the handle's workspace, grown as needed, or the static array
    char* ws_base = nullptr;
    auto get_ws = [&](size_t bytes) -> int {
        if (!fixed) {
            const int rc = ensure_ws(h, bytes, s);
            ws_base = (char*)h->ws;
            return rc;
        }
        ws_base = (char*)scratch_of(h->device);
        if (!ws_base) return fail(DCIH_ESTATE, me + ": the scratch array of this device was not located");
        if (bytes > kScratchBytes)
            return fail(DCIH_EINVAL, me + ": this call needs " + std::to_string(bytes) +
                                     " bytes of scratch and the fixed array holds " +
                                     std::to_string(kScratchBytes) + "; pass fewer queries per call");
        return 0;
    };

    h->ev_valid[DCIH_T_BATCH] = h->ev_valid[DCIH_T_DENSE] = false;
    QueryArgs a;
    a.skeys = h->d_skeys; a.sids = h->d_sids; a.inv = h->d_inv; a.data = h->d_data; a.query = d_query;
    a.rpos = h->d_rpos; a.rpos_ready = &h->rpos_ready;
    a.hints_cold = 0;
    a.mode = h->traversal; a.item_list = nullptr; a.item_count = nullptr; a.dense = nullptr;
    a.xcds = h->xcds; a.q_first = 0; a.q_count = num_queries;
    a.dense_items = nullptr; a.dense_count = nullptr; a.dense_cap = 0;
    a.wide_items = nullptr; a.wide_count = nullptr; a.wide_cap = 0;
    a.block_list = nullptr; a.block_list_count = nullptr; a.full_tables = 0;
    a.dense_min_promos = h->dense_min_promos;
    a.phase_ticks = h->d_phase_ticks;
    // the hints describe where traversals of one query shape stop; forget them when it
    // changes (cleared by a kernel: a memset node is not safe in a captured graph)
    if (h->hint_k != num_neighbours || h->hint_outer != num_outer_iterations ||
        h->hint_T != thread_size || h->hint_maxc != max_num_candidates) {
        const int rc = zero_words64(h->d_stop_hint, (int64_t)(((size_t)3 * block_size * sizeof(float) + 7) / 8), s);
        if (rc) return rc;
        h->hint_k = num_neighbours; h->hint_outer = num_outer_iterations;
        h->hint_T = thread_size; h->hint_maxc = max_num_candidates;
        a.hints_cold = 1;
    }
    a.stop_hint = h->d_stop_hint;
    a.N = h->n;
    a.ppb = (h->n + block_size - 1) / block_size;
    a.dim = dim; a.M = h->M; a.L = h->L; a.B = block_size; a.T = thread_size;
    a.T_magic = thread_size > 1 ? (unsigned)((0x100000000ull + (unsigned)thread_size - 1u) / (unsigned)thread_size) : 0u;
    a.nq = num_queries; a.k = (int)std::min<int64_t>(num_results, 0x7fffffff);
    a.k_stop = num_neighbours; a.blind = blind ? 1 : 0;
    a.kcap = (int)std::min<int64_t>(num_results, a.ppb);
    a.stop_at = (int64_t)num_outer_iterations * h->L;
    a.max_cand = max_num_candidates;
    a.counters = (unsigned long long*)d_counters;
    a.out_ids = d_nn; a.out_dists = d_dists;

    if (fixed && num_results > 8192)
        return fail(DCIH_EUNSUPPORTED, me + ": more than 8192 results per query need the row-per-query "
                                            "workspace of dcih_query");
    if (num_results > 8192 &&
        (blind || num_neighbours < a.ppb || (num_neighbours == a.ppb && d_counters))) {
        // More results than the top-k tables hold while partitions may still stop early: the
        // step-by-step traversal records every candidate in a dense row per query, which is
        // then sorted like the full ranking below.
        const int chunk = exhaustive_chunk(h->n, num_queries);
        QueryArgs probe = a;
        probe.nq = chunk; probe.kcap = 1;
        const size_t qp_bytes = align_up((size_t)I * chunk * sizeof(float));
        const size_t rank_bytes = align_up(exhaustive_ws_bytes(h->n, chunk));
        const size_t gs_bytes = align_up(query_gscratch_bytes(probe));
        int rc = get_ws(qp_bytes + rank_bytes + gs_bytes);
        if (rc) return rc;
        a.gscratch = gs_bytes ? (uint32_t*)(ws_base + qp_bytes + rank_bytes) : nullptr;
        mark(h, DCIH_T_TRAVERSE, 0, s);
        rc = query_dense(a, h->d_dirs, ws_base, chunk, s);
        mark(h, DCIH_T_TRAVERSE, 1, s);
        return rc;
    }
    // The stop rule (:598-607) can also never fire when a partition has fewer points than
    // max_num_candidates and fewer windows per simple index (at most ppb / T + 3) than
    // num_outer_iterations: the loop then runs every partition dry, as in the reference's own
    // example (3000 points in 100 partitions, 5000 iterations).  Left to pick, the engine
    // computes that answer directly as well (not with the fixed scratch, which a million
    // points per query would overrun: there the traversal kernels give the same neighbours).
    const bool runs_dry = !blind && !fixed && h->traversal == 0 && a.ppb < (int64_t)max_num_candidates &&
                          a.ppb / thread_size + 4 < (int64_t)num_outer_iterations;
    if (!blind && (num_neighbours > 8192 || runs_dry)) {
        // With more neighbours asked for than a partition holds, no partition can stop early
        // (c0 counts promotions of one partition, :598-607), so the answer is the full ranking
        // and is computed as such.  (With exactly as many, the results are the same but the
        // last step may end the loop before its idle pass: the counters then come from the
        // traversal above.)
        const int chunk = exhaustive_chunk(h->n, num_queries);
        const size_t qp_bytes = d_counters ? align_up((size_t)I * num_queries * sizeof(float)) : 0;
        int rc = get_ws(qp_bytes + exhaustive_ws_bytes(h->n, chunk));
        if (rc) return rc;
        if (d_counters) {
            rc = project(h->d_dirs, I, d_query, num_queries, dim, (float*)ws_base, num_queries, s);
            if (rc) return rc;
            a.qproj = (float*)ws_base;
        }
        mark(h, DCIH_T_TRAVERSE, 0, s);
        rc = query_exhaustive(a, ws_base + qp_bytes, chunk, s);
        mark(h, DCIH_T_TRAVERSE, 1, s);
        return rc;
    }

    const size_t qp_bytes = align_up((size_t)I * num_queries * sizeof(float));
    const size_t part_bytes = align_up(query_part_bytes(a));
    const size_t gs_bytes = align_up(query_gscratch_bytes(a));
    const size_t redo_bytes = align_up((size_t)num_queries * block_size * sizeof(int32_t));
    // per die one list of the items the batch kernel leaves to the dense kernel
    a.dense_cap = (int64_t)num_queries * (block_size / h->xcds + 1) + 64;
    const bool dense_lists = h->traversal == 0 && h->dense_min_promos > 0 && !blind &&
                             dense_traversal_supported(a, nullptr) && block_traversal_supported(a, nullptr);
    const size_t dense_bytes = dense_lists ? align_up((size_t)h->xcds * a.dense_cap * sizeof(int32_t)) : 0;
    // (the second pass may have to take every item, up to what one launch of 256-thread workgroups covers)
    a.wide_cap = std::min((int64_t)num_queries * block_size, (int64_t)1 << 23);
    const size_t wide_bytes = align_up((size_t)a.wide_cap * sizeof(int32_t));
    int rc = get_ws(qp_bytes + part_bytes + gs_bytes + redo_bytes + 256 + dense_bytes + wide_bytes);
    if (rc) return rc;
    char* base = ws_base;
    float* d_qproj = (float*)base;
    a.qproj = d_qproj;
    a.part = (unsigned long long*)(base + qp_bytes);
    a.gscratch = gs_bytes ? (uint32_t*)(base + qp_bytes + part_bytes) : nullptr;
    a.redo_items = (int32_t*)(base + qp_bytes + part_bytes + gs_bytes);
    a.redo_count = (uint32_t*)(base + qp_bytes + part_bytes + gs_bytes + redo_bytes);
    a.dense_count = a.redo_count + 1;         // one length per die, cleared together with redo_count
    a.dense_items = dense_lists ? (int32_t*)(base + qp_bytes + part_bytes + gs_bytes + redo_bytes + 256) : nullptr;
    a.wide_count = a.redo_count + kListCountWords - 1;      // (the last of the list lengths that are cleared together)
    a.wide_items = (int32_t*)(base + qp_bytes + part_bytes + gs_bytes + redo_bytes + 256 + dense_bytes);

    mark(h, DCIH_T_QPROJECT, 0, s);
    rc = project(h->d_dirs, I, d_query, num_queries, dim, d_qproj, num_queries, s);
    mark(h, DCIH_T_QPROJECT, 1, s);
    if (rc) return rc;
    // events in the order query() records them: traversal start, batch kernel end, dense
    // kernel end, traversal end, merge end
    hipEvent_t qev[5] = {h->ev[2 * DCIH_T_TRAVERSE], h->ev[2 * DCIH_T_BATCH + 1], h->ev[2 * DCIH_T_DENSE + 1],
                         h->ev[2 * DCIH_T_TRAVERSE + 1], h->ev[2 * DCIH_T_MERGE + 1]};
    bool ran[2] = {false, false};
    rc = query(a, s, h->profiling ? qev : nullptr, ran);
    if (rc == DCIH_OK && h->profiling) {
        h->ev_valid[DCIH_T_TRAVERSE] = h->ev_valid[DCIH_T_MERGE] = true;
        h->ev_valid[DCIH_T_BATCH] = ran[0];
        h->ev_valid[DCIH_T_DENSE] = ran[1];
    }
    return rc;
}

int dcih_query(dcih_index* h, int dim, int num_queries, const float* d_query,
               int num_neighbours, int blind, int num_outer_iterations,
               int max_num_candidates, int block_size, int thread_size,
               int32_t* d_nn, float* d_dists, uint64_t* d_counters, void* stream) {
    return query_impl(h, dim, num_queries, d_query, num_neighbours, blind, num_outer_iterations,
                      max_num_candidates, block_size, thread_size, d_nn, d_dists, d_counters, stream,
                      false, "dcih_query");
}

int dcih_query_noalloc(dcih_index* h, int dim, int num_queries, const float* d_query,
                       int num_neighbours, int blind, int num_outer_iterations,
                       int max_num_candidates, int block_size, int thread_size,
                       int32_t* d_nn, float* d_dists, uint64_t* d_counters, void* stream) {
    return query_impl(h, dim, num_queries, d_query, num_neighbours, blind, num_outer_iterations,
                      max_num_candidates, block_size, thread_size, d_nn, d_dists, d_counters, stream,
                      true, "dcih_query_noalloc");
}

int64_t dcih_debug_launch_map(int xcds, int block_size, int num_queries, int64_t block,
                              int* b, int* q, int* queries_per_launch) {
    if (xcds < 1 || block_size < 1 || num_queries < 1) return -1;
    const int per_launch = block_queries_per_launch(xcds, block_size, num_queries);
    if (queries_per_launch) *queries_per_launch = per_launch;
    if (per_launch < 1) return -1;
    const int nq = std::min(per_launch, num_queries);
    const int64_t items = block_items(xcds, block_size, nq);
    if (b && q && block >= 0 && block < items) {
        int bb = -1, qq = -1;
        if (!block_item(block, xcds, block_size, nq, bb, qq)) bb = qq = -1;
        *b = bb; *q = qq;
    }
    return items;
}

int dcih_debug_positions(dcih_index* h, uint16_t* d_inv, uint16_t* d_rpos, void* stream) {
    if (!h) return fail(DCIH_EINVAL, "dcih_debug_positions: null handle");
    if (h->n <= 0) return fail(DCIH_ESTATE, "dcih_debug_positions: the index is empty");
    if (!h->d_inv || !h->d_rpos) return fail(DCIH_EUNSUPPORTED, "dcih_debug_positions: this index keeps no position tables");
    DeviceGuard guard(h->device);
    hipStream_t s = (hipStream_t)stream;
    const size_t cells = (size_t)num_indices(h) * (size_t)h->n;
    if (d_inv) DCIH_HIP(hipMemcpyAsync(d_inv, h->d_inv, cells * sizeof(uint16_t), hipMemcpyDeviceToDevice, s));
    if (d_rpos) {
        if (!h->rpos_ready) {
            // (rows of the first simple indices are never written: clear the table so that they read as zeros)
            DCIH_HIP(hipMemsetAsync(h->d_rpos, 0, cells * sizeof(uint16_t), s));
            const int rc = fill_positions_by_first(h->d_sids, h->d_inv, h->d_rpos, h->n, h->M, h->L, s);
            if (rc) return rc;
            h->rpos_ready = 1;
        }
        DCIH_HIP(hipMemcpyAsync(d_rpos, h->d_rpos, cells * sizeof(uint16_t), hipMemcpyDeviceToDevice, s));
    }
    DCIH_HIP(hipStreamSynchronize(s));
    return DCIH_OK;
}

int dcih_set_option(dcih_index* h, int option, int value) {
    if (!h) return fail(DCIH_EINVAL, "dcih_set_option: null handle");
    if (option == DCIH_OPT_TRAVERSAL && value >= 0 && value <= 3) {
        h->traversal = value;
        return DCIH_OK;
    }
    if (option == DCIH_OPT_DENSE_MIN_PROMOTIONS && value >= 0) {
        h->dense_min_promos = value;
        return DCIH_OK;
    }
    if (option == DCIH_OPT_APPEND && value >= 0 && value <= 2) {
        h->append_mode = value;
        return DCIH_OK;
    }
    if (option == DCIH_OPT_FORGET_HINTS) {
        h->hint_k = h->hint_outer = h->hint_T = h->hint_maxc = 0;     // the next query clears the table
        return DCIH_OK;
    }
    return fail(DCIH_EINVAL, "dcih_set_option: unknown option or value");
}

int dcih_phase_profile(dcih_index* h, uint64_t* d_ticks) {
    if (!h) return fail(DCIH_EINVAL, "dcih_phase_profile: null handle");
    h->d_phase_ticks = (unsigned long long*)d_ticks;
    return DCIH_OK;
}

int dcih_profile(dcih_index* h, int enable) {
    if (!h) return fail(DCIH_EINVAL, "dcih_profile: null handle");
    DeviceGuard guard(h->device);
    if (enable && !h->ev[0]) {
        for (auto& e : h->ev) DCIH_HIP(hipEventCreate(&e));
    }
    h->profiling = enable != 0;
    for (auto& v : h->ev_valid) v = false;
    return DCIH_OK;
}

int dcih_last_timings(dcih_index* h, float* h_ms) {
    if (!h || !h_ms) return fail(DCIH_EINVAL, "dcih_last_timings: null argument");
    if (!h->profiling) return fail(DCIH_ESTATE, "dcih_last_timings: profiling is off");
    DeviceGuard guard(h->device);
    for (int t = 0; t < DCIH_NUM_TIMERS; t++) {
        h_ms[t] = -1.0f;
        if (!h->ev_valid[t]) continue;
        // timers that start where another one ends: the merge after the traversal, the batch
        // kernel at the traversal's start, the dense kernel after the batch kernel
        hipEvent_t a = h->ev[2 * t];
        if (t == DCIH_T_MERGE) a = h->ev[2 * DCIH_T_TRAVERSE + 1];
        if (t == DCIH_T_BATCH) a = h->ev[2 * DCIH_T_TRAVERSE];
        if (t == DCIH_T_DENSE) a = h->ev_valid[DCIH_T_BATCH] ? h->ev[2 * DCIH_T_BATCH + 1] : h->ev[2 * DCIH_T_TRAVERSE];
        hipEvent_t b = h->ev[2 * t + 1];
        DCIH_HIP(hipEventSynchronize(b));
        DCIH_HIP(hipEventElapsedTime(&h_ms[t], a, b));
    }
    return DCIH_OK;
}

int dcih_get_index(const dcih_index* h, float* h_keys, int32_t* h_ids) {
    if (!h) return fail(DCIH_EINVAL, "dcih_get_index: null handle");
    if (h->n <= 0) return fail(DCIH_ESTATE, "dcih_get_index: index is empty");
    DeviceGuard guard(h->device);
    const size_t cells = (size_t)num_indices(h) * h->n;
    DCIH_HIP(hipDeviceSynchronize());
    if (h_keys) DCIH_HIP(hipMemcpy(h_keys, h->d_skeys, cells * sizeof(float), hipMemcpyDeviceToHost));
    if (h_ids) DCIH_HIP(hipMemcpy(h_ids, h->d_sids, cells * sizeof(int32_t), hipMemcpyDeviceToHost));
    return DCIH_OK;
}

int64_t dcih_num_points(const dcih_index* h) { return h ? h->n : 0; }

int dcih_clear(dcih_index* h) {
    if (!h) return fail(DCIH_EINVAL, "dcih_clear: null handle");
    DeviceGuard guard(h->device);
    DCIH_HIP(hipDeviceSynchronize());
    return release_index(h);
}

int dcih_reset(dcih_index* h) {
    const int rc = dcih_clear(h);
    if (rc) return rc;
    DeviceGuard guard(h->device);
    return draw_directions(h);
}

int dcih_free(dcih_index* h) {
    if (!h) return DCIH_OK;
    DeviceGuard guard(h->device);
    (void)hipDeviceSynchronize();
    (void)release_index(h);
    (void)release_arena(h);
    if (h->ws) (void)hipFree(h->ws);
    if (h->d_dirs) (void)hipFree(h->d_dirs);
    for (auto& e : h->ev) if (e) (void)hipEventDestroy(e);
    delete h;
    return DCIH_OK;
}

int dcih_project(const float* d_dirs, int num_idx, const float* d_rows, int64_t num_rows,
                 int dim, float* d_out, void* stream) {
    if (!d_dirs || !d_rows || !d_out || num_idx <= 0 || num_rows < 0 || dim <= 0)
        return fail(DCIH_EINVAL, "dcih_project: bad argument");
    return project(d_dirs, num_idx, d_rows, num_rows, dim, d_out, num_rows, (hipStream_t)stream);
}

int dcih_segsort(const float* d_keys, int num_idx, int64_t num_points, int block_size,
                 float* d_skeys, int32_t* d_sids, void* stream) {
    if (!d_keys || !d_skeys || !d_sids || num_idx <= 0 || num_points <= 0 || block_size <= 0)
        return fail(DCIH_EINVAL, "dcih_segsort: bad argument");
    hipStream_t s = (hipStream_t)stream;
    const size_t tmp_bytes = segsort_tmp_bytes(num_idx, num_points, block_size);
    void* d_tmp = nullptr;
    if (tmp_bytes) DCIH_HIP(hipMalloc(&d_tmp, tmp_bytes));
    const int rc = segsort(d_keys, num_points, num_idx, num_points, block_size, d_skeys, d_sids, nullptr, nullptr, d_tmp, s);
    if (d_tmp) {
        (void)hipStreamSynchronize(s);
        (void)hipFree(d_tmp);
    }
    return rc;
}

}  // extern "C"
