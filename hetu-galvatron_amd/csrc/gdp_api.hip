// Host side of libgalvatron_dp_hip.so: the C ABI declared in include/galvatron_dp_hip.h.
//
// A plan owns one device allocation, one stream and the events used for timing while it lives, so
// calls from different threads never touch common mutable state -- but for the cache of device
// allocations below, which is behind a mutex.
#include "../../include/galvatron_dp_hip.h"
#include "gdp_kernels.h"
#include "gdp_host.h"

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <condition_variable>
#include <mutex>
#include <new>
#include <string>
#include <unordered_map>
#include <vector>

// ---- shared with gdp_static.hip (declared in gdp_host.h) ---------------------------------------------
namespace {
thread_local char g_err[320] = "";   // a fixed buffer: reporting an error allocates nothing
}

void gdp_clear_error() { g_err[0] = 0; }

int gdp_fail(int code, const char *msg)
{
    snprintf(g_err, sizeof g_err, "%s", msg ? msg : "");
    return code;
}

int gdp_fail_hip(hipError_t e, const char *what)
{
    // a failed allocation is reported as such; everything else as a runtime error
    const int code = (e == hipErrorOutOfMemory || e == hipErrorMemoryAllocation) ? GDP_E_NOMEM : GDP_E_HIP;
    snprintf(g_err, sizeof g_err, "%s: %s", what, hipGetErrorString(e));
    return code;
}

namespace {

int fail(int code, const char *msg) { return gdp_fail(code, msg); }
int fail_hip(hipError_t e, const char *what) { return gdp_fail_hip(e, what); }

#define GDP_HIP(call)                                    \
    do {                                                 \
        hipError_t e_ = (call);                          \
        if (e_ != hipSuccess) return fail_hip(e_, #call); \
    } while (0)

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// ---- cache of device allocations -----------------------------------------------------------------
// Getting fresh device memory costs far more than filling it (94 GB for 256 Llama-7B-like instances:
// 2.7 s to allocate, 0.05 s to solve), and the search engine solves thousands of DPs in a row.  The
// allocation of a finished plan is therefore kept for the next plan on that device instead of being
// freed: up to GALVATRON_DP_CACHE_MB (default 20480 or an eighth of the device memory, whichever is less; 0 = keep nothing) in total -- room for the two
// allocations of GALVATRON_DP_ARENA_MB that a batch solved in parts works in, and the small ones of
// single solves between such batches --, the ones given back longest ago given up first when that is
// exceeded, all of them on an out-of-memory error or gdp_cache_trim().
struct Arena {
    int device;
    char *ptr;
    size_t bytes;
};
std::mutex g_arena_mu;
std::vector<Arena> g_arenas;

size_t env_mb(const char *name, size_t dflt_mb)
{
    const char *e = getenv(name);
    if (!e || !*e) return dflt_mb << 20;
    const long long v = atoll(e);
    return v <= 0 ? 0 : (size_t)v << 20;
}

void arena_trim(int device /* -1: every device */)
{
    std::vector<Arena> drop;
    {
        std::lock_guard<std::mutex> lk(g_arena_mu);
        for (size_t i = 0; i < g_arenas.size();) {
            if (device < 0 || g_arenas[i].device == device) {
                drop.push_back(g_arenas[i]);
                g_arenas.erase(g_arenas.begin() + (long)i);
            } else {
                ++i;
            }
        }
    }
    int cur = 0;
    (void)hipGetDevice(&cur);
    for (const Arena &a : drop) {
        (void)hipSetDevice(a.device);
        (void)hipFree(a.ptr);
    }
    (void)hipSetDevice(cur);
}

// The smallest kept allocation of `device` that holds `need` bytes, or a fresh one.
hipError_t arena_take(int device, size_t need, char **ptr, size_t *bytes)
{
    // test aid: requests above GALVATRON_DP_DEVICE_LIMIT_MB are answered like a device that is full
    if (getenv("GALVATRON_DP_DEVICE_LIMIT_MB") && need > env_mb("GALVATRON_DP_DEVICE_LIMIT_MB", 0)) {
        *ptr = nullptr;
        return hipErrorOutOfMemory;
    }
    {
        std::lock_guard<std::mutex> lk(g_arena_mu);
        size_t best = g_arenas.size();
        for (size_t i = 0; i < g_arenas.size(); ++i)
            if (g_arenas[i].device == device && g_arenas[i].bytes >= need &&
                (best == g_arenas.size() || g_arenas[i].bytes < g_arenas[best].bytes))
                best = i;
        if (best != g_arenas.size()) {
            *ptr = g_arenas[best].ptr;
            *bytes = g_arenas[best].bytes;
            g_arenas.erase(g_arenas.begin() + (long)best);
            return hipSuccess;
        }
    }
    hipError_t e = hipMalloc((void **)ptr, need);
    if (e == hipErrorOutOfMemory || e == hipErrorMemoryAllocation) {
        (void)hipGetLastError();
        arena_trim(device);  // what is kept may be what is missing
        e = hipMalloc((void **)ptr, need);
    }
    *bytes = need;
    return e;
}

// What may stay cached on `device`: GALVATRON_DP_CACHE_MB if set, else 20 GB but never more than an
// eighth of the device's memory (a process that shares the device with other work can set it to 0, or
// call gdp_cache_trim() when its search is over).
size_t cache_cap(int device)
{
    const char *e = getenv("GALVATRON_DP_CACHE_MB");
    if (e && *e) return env_mb("GALVATRON_DP_CACHE_MB", 0);
    static std::mutex mu;
    static std::vector<size_t> total;  // per device, 0 = not asked yet
    std::lock_guard<std::mutex> lk(mu);
    if (device >= 0 && (size_t)device >= total.size()) total.resize((size_t)device + 1, 0);
    if (device >= 0 && total[(size_t)device] == 0) {
        size_t t = 0;
        if (hipDeviceTotalMem(&t, device) != hipSuccess || t == 0) {
            (void)hipGetLastError();
            t = (size_t)64 << 30;
        }
        total[(size_t)device] = t;
    }
    const size_t eighth = device >= 0 ? total[(size_t)device] / 8 : (size_t)8 << 30;
    return std::min((size_t)20480 << 20, eighth);
}

void arena_give(int device, char *ptr, size_t bytes)
{
    const size_t cap = cache_cap(device);
    std::vector<Arena> drop;
    if (bytes > cap) {
        drop.push_back({device, ptr, bytes});
    } else {
        std::lock_guard<std::mutex> lk(g_arena_mu);
        g_arenas.push_back({device, ptr, bytes});
        size_t total = 0;
        for (const Arena &a : g_arenas) total += a.bytes;
        while (total > cap) {  // the one given back longest ago first (they are kept in that order)
            total -= g_arenas.front().bytes;
            drop.push_back(g_arenas.front());
            g_arenas.erase(g_arenas.begin());
        }
    }
    for (const Arena &a : drop) (void)hipFree(a.ptr);  // same device as the caller's plan
}

// ---- streams kept between plans --------------------------------------------------------------------
// Creating and destroying a stream costs more than solving a small DP (0.14 ms against 0.4 ms), and
// a search makes thousands of such calls in a row.  A finished plan therefore hands its stream, its
// two events and its page-locked read-back buffer to the next plan on that device; at most
// LANES_KEPT wait here, gdp_cache_trim() releases them.
struct Lane {
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev_begin = nullptr, ev_end = nullptr;
    hipEvent_t ev_back = nullptr;  // after the copy of the results (a flow run queues more work behind it)
    hipStream_t side = nullptr;    // second stream: the upload of a small plan's inputs runs beside the kernel that
    hipEvent_t ev_side = nullptr;  // prepares its cost buffers; the event joins it to the main stream
    char *back = nullptr;  // page-locked host memory the results are copied into
    size_t back_bytes = 0;
    char *up = nullptr;    // page-locked host memory the inputs' device layout is built in (may be absent)
    size_t up_bytes = 0;
};
constexpr size_t LANES_KEPT = 64;
std::mutex g_lane_mu;
std::vector<Lane> g_lanes;

void lane_release(Lane &ln)  // the lane's device is current
{
    if (ln.ev_begin) (void)hipEventDestroy(ln.ev_begin);
    if (ln.ev_end) (void)hipEventDestroy(ln.ev_end);
    if (ln.ev_back) (void)hipEventDestroy(ln.ev_back);
    if (ln.ev_side) (void)hipEventDestroy(ln.ev_side);
    if (ln.side) (void)hipStreamDestroy(ln.side);
    if (ln.stream) (void)hipStreamDestroy(ln.stream);
    if (ln.back) (void)hipHostFree(ln.back);
    if (ln.up) (void)hipHostFree(ln.up);
    ln = Lane();
}

// Page-locked memory of at least `bytes` behind *ptr (grown in steps of `grain`, contents not kept).
hipError_t pinned_reserve(char **ptr, size_t *have, size_t bytes, size_t grain)
{
    if (*have >= bytes) return hipSuccess;
    if (*ptr) (void)hipHostFree(*ptr);
    *ptr = nullptr;
    *have = 0;
    const size_t want = align_up(bytes, grain);
    const hipError_t e = hipHostMalloc((void **)ptr, want, hipHostMallocDefault);
    if (e == hipSuccess) *have = want;
    return e;
}

// Inputs up to this size are laid out in page-locked memory: the upload then is one asynchronous DMA
// (a 0.4 MB upload from pageable memory holds the calling thread for 0.17 ms).  Larger ones are
// built in ordinary memory; their upload is a small part of their solve.
constexpr size_t UPLOAD_PINNED_MAX = (size_t)16 << 20;

hipError_t lane_take(int device, size_t back_bytes, size_t up_bytes, Lane *out)
{
    Lane ln;
    {
        std::lock_guard<std::mutex> lk(g_lane_mu);
        for (size_t i = g_lanes.size(); i-- > 0;)
            if (g_lanes[i].device == device) {
                ln = g_lanes[i];
                g_lanes.erase(g_lanes.begin() + (long)i);
                break;
            }
    }
    hipError_t e = hipSuccess;
    if (!ln.stream) {
        ln.device = device;
        e = hipStreamCreateWithFlags(&ln.stream, hipStreamNonBlocking);
        if (e == hipSuccess) e = hipEventCreate(&ln.ev_begin);
        if (e == hipSuccess) e = hipEventCreate(&ln.ev_end);
        if (e == hipSuccess) e = hipEventCreateWithFlags(&ln.ev_back, hipEventDisableTiming);
        if (e == hipSuccess) e = hipStreamCreateWithFlags(&ln.side, hipStreamNonBlocking);
        if (e == hipSuccess) e = hipEventCreateWithFlags(&ln.ev_side, hipEventDisableTiming);
    }
    if (e == hipSuccess) e = pinned_reserve(&ln.back, &ln.back_bytes, back_bytes, 65536);
    if (e == hipSuccess && up_bytes <= UPLOAD_PINNED_MAX) e = pinned_reserve(&ln.up, &ln.up_bytes, up_bytes, (size_t)1 << 20);
    if (e != hipSuccess) {
        lane_release(ln);
        return e;
    }
    *out = ln;
    return hipSuccess;
}

void lane_give(Lane &ln)  // the lane's device is current and its stream idle
{
    if (!ln.stream) return;
    {
        std::lock_guard<std::mutex> lk(g_lane_mu);
        if (g_lanes.size() < LANES_KEPT && ln.back_bytes <= ((size_t)64 << 20)) {  // up_bytes is bounded anyway
            g_lanes.push_back(ln);
            ln = Lane();
            return;
        }
    }
    lane_release(ln);
}

void lane_trim()
{
    std::vector<Lane> drop;
    {
        std::lock_guard<std::mutex> lk(g_lane_mu);
        drop.swap(g_lanes);
    }
    int cur = 0;
    (void)hipGetDevice(&cur);
    for (Lane &ln : drop) {
        (void)hipSetDevice(ln.device);
        lane_release(ln);
    }
    (void)hipSetDevice(cur);
}

// One fused launch at a time.  Its workgroups wait, while resident, for earlier workgroups of the same
// launch.  Alone on the device that cannot block: every XCD starts its share of the workgroups in
// order, so the oldest unfinished one is resident and waits for nothing.  Two such launches side by
// side can fill an XCD each with workgroups waiting for one that needs a place on the other XCD;
// the bounded wait then runs out (seconds) and both fall back to per-layer launches.  Launches
// without such waits (one per layer) may run beside a fused one: their workgroups always finish.
// The turn is a flag under a mutex, not a held mutex: a run may be started by one thread and waited for
// (or its plan destroyed) by another.  It orders the threads of ONE process; another process on the same
// device is not seen (its fused launches and these can then block each other until the bounded wait of
// one of them runs out, after which that plan continues with one launch per layer).
std::mutex g_fused_mu;
std::condition_variable g_fused_cv;
bool g_fused_busy = false;

void fused_turn_take()
{
    std::unique_lock<std::mutex> lk(g_fused_mu);
    g_fused_cv.wait(lk, [] { return !g_fused_busy; });
    g_fused_busy = true;
}

// The turn if it is free.  A flow plan that finds it taken does not queue up for it: it runs that solve
// with one launch per layer, beside the launch that holds the turn (threads that call the plugin side by
// side, as the reference's parallel search does, then overlap instead of taking turns).
// When a launch whose workgroups wait was given up although nobody had shortened its waits, something else
// holds places on the device -- most likely another process with such launches of its own (the turn above
// orders the threads of this process only).  Every further launch of that kind would risk the same
// wait of a good part of a second, so for the next while the library chooses launches that never wait
// (one per layer) where the choice is its own; a caller's explicit request still counts.
// How long a waiting wave keeps polling before its launch is given up, when the caller has set no limit of
// its own: WAIT_BOUND_FACTOR times what the plan's relaxations take at a rate every healthy launch exceeds
// (a wave of a healthy launch waits for less than the launch lasts), no less than WAIT_BOUND_MIN_S and no
// more than WAIT_BOUND_MAX_S.  A solve of 0.1 ms gives up after 5 ms, one of 3 ms after a quarter of a second.
constexpr double WAIT_BOUND_FACTOR = 50.0, WAIT_BOUND_RATE = 5e12 /* relaxations per second */;
constexpr double WAIT_BOUND_MIN_S = 5e-3, WAIT_BOUND_MAX_S = 1.0;
// Time between two looks of a waiting wave: a sleep of 3.5 us in a launch with completion counters; the round
// trip of an agent-scope load, at least 1 us, in a flow launch (see wait_tiles and flow_poll in gdp_kernels.hip).
constexpr double POLL_S_FUSED = 3.5e-6, POLL_S_FLOW = 1e-6;
std::atomic<int64_t> g_last_give_up_ms{-1};   // steady clock, milliseconds; -1: never

// For how long after a give-up launches that wait are avoided (GALVATRON_DP_SHARED_BACKOFF_MS; default 30 s).
int64_t shared_backoff_ms()
{
    const char *e = getenv("GALVATRON_DP_SHARED_BACKOFF_MS");
    if (e && *e) return std::max<long long>(0, atoll(e));
    return 30000;
}

int64_t steady_ms()
{
    return std::chrono::duration_cast<std::chrono::milliseconds>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

bool device_seems_shared()
{
    const int64_t t = g_last_give_up_ms.load(std::memory_order_relaxed);
    return t >= 0 && steady_ms() - t < shared_backoff_ms();
}

bool fused_turn_try_take()
{
    std::lock_guard<std::mutex> lk(g_fused_mu);
    if (g_fused_busy) return false;
    g_fused_busy = true;
    return true;
}

void fused_turn_give()
{
    {
        std::lock_guard<std::mutex> lk(g_fused_mu);
        g_fused_busy = false;
    }
    g_fused_cv.notify_one();
}

// gdp_batch_stats_begin / _end: what the batches of the process did in between.
std::mutex g_stats_mu;
bool g_stats_on = false;
gdp_batch_stats g_stats = {};

struct HostInst {
    int orig;  // index in the caller's arrays
    int L, V, S, SP, SU, P, ntile, n_key, n_inter, variant, nbuf;
    int64_t ld, ldm;
    uint32_t flags;
    int key_begin;  // first entry in the key table
    int res_begin;  // first element in the result array
    // byte offsets inside the device allocation
    size_t off_H, off_M, off_inter, off_intra, off_index, off_roff, off_mem;
    bool has_zero = false;  // some memory cost is 0 (see gdp_launch_zero_pass)
    size_t off_zcols = 0;
    // a dense [L,S,S] transition array whose equal matrices are kept once (share_equal_matrices):
    std::vector<int32_t> mat_of;   // layer -> kept matrix
    std::vector<int32_t> mat_src;  // kept matrix -> the layer whose copy is taken
    int matrix(const gdp_problem *q, int l) const { return q->inter_index ? q->inter_index[l] : mat_of[(size_t)l]; }
    // where the caller keeps kept matrix t
    const double *matrix_at(const gdp_problem *q, int t) const
    {
        return q->inter + (size_t)(q->inter_index ? t : mat_src[(size_t)t]) * (size_t)S * (size_t)S;
    }
    int tables_of = -1;   // an earlier instance of the plan (sorted order) whose device copy of the matrices this one reads
    // The caller's initial costs where they are not all zero (gdp_problem.f0), one row per strategy -- the
    // layout of a cost buffer; kept for the life of the plan, because a plan with two cost buffers writes
    // over buffer 0 in every run and gets them uploaded again before the next.
    std::vector<double> f0t;
};

// The reference's callers pass one transition matrix per layer, and almost all of them are copies of a
// few (galvatron/core/search_engine/dynamic_programming.py:368-372: one matrix per layer type, repeated
// for its layers, the first layer's zeroed).  Matrices with the same bytes are kept once: the layers in
// flight then share their transition costs in the caches instead of each fetching its own copy
// (measured per call from host arrays, 32 equal matrices of 44 x 44: 0.81 -> 0.60 ms; 48 of 88 x 88:
// 6.65 -> 6.26 ms), and the upload shrinks.  A layer is compared with the matrix of the layer before it
// and, failing that, with the first few kept ones; comparisons of different matrices end at the first
// byte that differs, so an array of L different matrices costs next to nothing to look through.
void share_equal_matrices(const gdp_problem *q, HostInst &h)
{
    constexpr size_t LOOKED_AT = 8;
    const size_t bytes = sizeof(double) * (size_t)q->S * q->S;
    auto mat = [&](int l) { return reinterpret_cast<const char *>(q->inter) + (size_t)l * bytes; };
    h.mat_of.assign((size_t)q->L, 0);
    h.mat_src.clear();
    for (int l = 0; l < q->L; ++l) {
        int found = -1;
        const int before = l > 0 ? h.mat_of[(size_t)l - 1] : -1;
        if (before >= 0 && memcmp(mat(l), mat(h.mat_src[(size_t)before]), bytes) == 0) found = before;
        for (size_t t = 0; found < 0 && t < std::min(h.mat_src.size(), LOOKED_AT); ++t)
            if ((int)t != before && memcmp(mat(l), mat(h.mat_src[t]), bytes) == 0) found = (int)t;
        if (found < 0) {
            found = (int)h.mat_src.size();
            h.mat_src.push_back(l);
        }
        h.mat_of[(size_t)l] = found;
    }
    h.n_inter = (int)h.mat_src.size();
}

struct Group {  // instances with the same S, sorted by L descending
    int first, count, SP, S, max_L, max_ntile, variant, ntb, nbt;   // ntb: wave tasks per tile (with the parts of split tasks)
    int split = 1;            // fused launches: waves that share the source strategies of a task (1, or 2: see relax_task)
    int xcd_group = 1;        // consecutive block tasks handed to one XCD (whole tiles)
    int slots = 0;            // workgroups per XCD, instance and layer of a fused launch
    int64_t max_ld;
    std::vector<int> active;  // active[l] = number of instances with L > l
    std::vector<int64_t> live_blocks;  // block tasks of layer l that carry arithmetic, over its instances
    struct Segment { int first, layers; unsigned lds_bytes; };
    std::vector<Segment> segments;  // fused launches: runs of layers with the same active set, or -- chunked --
                                    // runs of at most 65535 entries of the row table
    std::vector<char> zero_layer;   // [max_L] some instance of the group has a strategy with mem == 0 in layer l
    int max_V = 0;
    int latency = 0;                // per-layer launches use the variant for launches with few waves: 0, or the
                                    // number of waves (1, 2, 4) that share the source strategies of a task
    bool any_fill = false;          // some layer of some instance has rows below its band that are filled once per plan
    int flow_nsrc = 0;              // flow launch: source strategies per wave (SU = flow_nsrc * latency)
    bool lat_ok = true;             // SU suits the latency variant of the per-layer kernel (a multiple of 8 * latency)
    int flow_blocks = 0;            // flow launch: workgroups of the widest band (wave tasks incl. the parts of split ones)
    int chunk = 0;                  // instances taken through all their layers together; >= count: not chunked
    std::vector<int32_t> rows;      // chunked: {first instance, instances, layer} per grid row
    size_t off_rows = 0;
    GdpSched sched = {};      // argument of the fused launches (device pointers inside)
    bool latency_possible(bool keep_marks) const
    {
        return !keep_marks && GDP_VARIANTS[variant].ts == GDP_LAT_TS && GDP_VARIANTS[variant].r == GDP_LAT_R;
    }
    size_t off_active, off_cnt, off_lay;  // byte offsets in the device allocation
};

// Target-tile width.  With enough work to go round -- `tiles` row tiles of 64 rows in flight together
// give every wave slot of the device a task -- the width that covers S with the fewest target
// blocks, of those the one that pads S least, of those the widest (S = 44: three blocks of 15;
// S = 64: four of 16; S = 36: three of 12).  A problem too small for that is short of parallelism, not
// of load bandwidth: it takes the next larger block count that fills the device (one instance of S = 44,
// V = 65536: four blocks of 11, 0.50 ms against 0.67 ms with three of 15), or failing that the most
// blocks there are.  marks: only among the variants built with the argmin table, by least padding.
// GALVATRON_DP_TILE_TS forces a width (tuning aid).
int pick_ts(int S, bool marks, int64_t tiles, int64_t wave_slots)
{
    const char *forced = getenv("GALVATRON_DP_TILE_TS");
    struct Cand { int ts; size_t blocks, sp; };
    std::vector<Cand> cands;
    for (int v = 0; v < GDP_NUM_VARIANTS; ++v) {
        if (marks && !GDP_VARIANTS[v].marks) continue;
        const int ts = GDP_VARIANTS[v].ts;
        if (forced && ts == atoi(forced)) return ts;
        const size_t sp = align_up((size_t)S, (size_t)ts);
        cands.push_back({ts, sp / (size_t)ts, sp});
    }
    if (marks) {
        // five vector instructions per relaxation: the arithmetic binds, so the least padding decides
        // (S = 64: eight blocks of 8, 5.9 ms; six of 11, padded to 66, 6.3 ms)
        const Cand *best = &cands[0];
        for (const Cand &c : cands)
            if (c.sp < best->sp || (c.sp == best->sp && c.ts > best->ts)) best = &c;
        return best->ts;
    }
    std::sort(cands.begin(), cands.end(), [](const Cand &a, const Cand &b) {
        if (a.blocks != b.blocks) return a.blocks < b.blocks;
        if (a.sp != b.sp) return a.sp < b.sp;
        return a.ts > b.ts;
    });
    for (const Cand &c : cands)
        if (tiles * (int64_t)c.blocks >= wave_slots) return c.ts;
    const size_t most = cands.back().blocks;  // not enough work whatever the width: the most tasks
    for (const Cand &c : cands)
        if (c.blocks == most) return c.ts;
    return cands.back().ts;
}

int gcd_int(int a, int b) { return b == 0 ? a : gcd_int(b, a % b); }

}  // namespace

int gdp_find_variant(int ts, int r)
{
    for (int v = 0; v < GDP_NUM_VARIANTS; ++v)
        if (GDP_VARIANTS[v].ts == ts && GDP_VARIANTS[v].r == r) return v;
    return -1;
}

namespace {
int find_variant(int ts, int r) { return gdp_find_variant(ts, r); }
}  // namespace

struct gdp_plan {
    int n = 0;
    int device = 0;
    std::vector<HostInst> inst;  // sorted order
    std::vector<Group> groups;
    char *dbase = nullptr;
    size_t dbytes = 0;       // bytes laid out
    size_t dalloc = 0;       // bytes of the allocation behind dbase (a kept one may be larger)
    size_t off_insts = 0, off_keys = 0, off_out = 0, off_res = 0;
    int n_key_total = 0;
    size_t n_res_total = 0;
    int max_L = 0;
    Lane lane;                   // stream, events and read-back buffer, taken from / returned to the pool
    hipStream_t stream = nullptr;    // = lane.stream
    hipEvent_t ev_begin = nullptr, ev_end = nullptr;
    std::vector<hipEvent_t> ev_relax;  // pairs
    // What a run copies back in one piece: abort flag, per-key outputs, strategy lists (device offsets
    // off_abort .. off_res + its size; the same offsets relative to off_abort inside lane.back).
    size_t back_bytes = 0;
    const GdpDevOut *h_out = nullptr;
    const int32_t *h_res = nullptr;
    std::vector<char> stage;     // host copy of the inputs' device layout when it is too large for lane.up;
                                 // the upload reads it asynchronously
    double relaxations = 0, relax_bytes = 0;
    double executed = 0;     // relaxations actually carried out (tiles inside the bands)
    bool skip = true;        // GDP_OPT_SKIP: use the bands (off: every tile of every layer is computed)
    bool ran = false;
    bool flow_clean = false;      // every cell a flow launch writes holds NaN and the abort flag zero (nothing has run since)
    bool one_shot = false;        // the plan runs once (gdp_solve_batch): nothing is prepared for a next run
    bool wait_back = false;       // the last run queued work behind its results: run_finish waits for lane.ev_back only
    bool holds_fused = false;     // between run_enqueue and run_finish of a fused run: this plan has the turn
    bool fused = true;            // one launch for all layers instead of one per layer
    bool flow = false;            // one launch for all layers whose tasks wait on the cost cells themselves (small
                                  // plans; see gdp_relax_flow_kernel); only with fused off
    bool split_upload = false;    // the per-instance inputs were uploaded on the lane's second stream
    bool run_flow = false;        // the run in flight (or the last one) is a flow launch: a flow plan that does not
                                  // get the turn runs that solve with one launch per layer
    bool flow_ready = false;      // the plan was laid out for it: closed bands, latency tile, NaN in the bands
    int flow_override = -1;       // GALVATRON_DP_FLOW=0|1: never / wherever the layout allows
    bool keep_marks = false;      // store the argmin table while relaxing (two cost buffers are then enough);
                                  // otherwise all L+1 cost buffers are kept and the backtrack recomputes it
    int64_t spin_limit = 0;       // polls a waiting wave makes before the launch is abandoned, if the caller has set
                                  // them (GDP_OPT_SPIN_LIMIT, GALVATRON_DP_SPIN_LIMIT); 0: from wait_bound_s
    double wait_bound_s = WAIT_BOUND_MAX_S;  // ... else for this long (set from the plan's size when it is laid out)
    bool scheme_fused = false, scheme_flow = false;  // the launch scheme the plan was given (fused / flow are what it
                                  // runs with now: both off after a give-up, until the plan is armed again)
    int64_t gave_up_ms = -1;      // when a waiting launch of this plan was last given up (steady clock)
    size_t off_zero = 0, zero_words = 0, off_abort = 0;
    int num_cu = 0;
    size_t lds_per_cu = 0;
    bool can_fuse = true;    // cost buffers were laid out one per layer
    bool rezero = false;     // buffer 0 is overwritten during a run and must be zeroed before each
    bool fused_gave_up = false;  // a fused launch was abandoned and the plan switched to per-layer launches
    bool no_fallback = false;    // GDP_OPT_NO_FALLBACK: report that instead of switching (tests)
    bool debug_stall = false;    // GDP_OPT_DEBUG_STALL: the first layer of a waiting launch does not signal (tests)
    bool no_occupancy_cap = false;  // GALVATRON_DP_OCCUPANCY_CAP=0 (tuning aid)
    int occupancy_cap_override = 0; // GALVATRON_DP_OCCUPANCY_CAP=n: n workgroups per CU in fused launches
    int chunk_override = 0;         // GALVATRON_DP_CHUNK=n: n instances at a time in fused launches
    int tile_r_override = 0; // GALVATRON_DP_TILE_R: force the register tile height (tuning aid)
    int latency_override = -1;  // GALVATRON_DP_LATENCY_VARIANT=0|1|2|4: never / wherever it exists, sources of a
                                // task on as many waves as the rule says / on 2 / on 4 (tuning aid)
    bool poison = false;     // test aid: NaN-fill the not-yet-written cost buffers before each run
    // gdp_debug_check_layout: the plan is laid out for a device that is only described (CUs, LDS per CU);
    // nothing is allocated, uploaded or launched, dbase is an address that is never dereferenced, and the
    // host copy of the tables always lives in `stage`
    bool has_zero = false;   // some instance has a memory cost of 0: one launch per layer, each followed by the
                             // pass that redoes those strategies in the reference's in-place order
    bool dry = false;
    size_t small_bytes = 0;  // bytes of the tables at the start of the allocation (what `stage` / lane.up hold)
    int dry_num_cu = 0;
    size_t dry_lds_per_cu = 0;
};

// Looks through n costs: false if a NaN or -inf is among them, else *maxabs = the largest finite magnitude
// (+inf entries are allowed and do not count).  Eight independent running maxima and no early exit, so that
// the loop runs at the speed of the loads (the dense transition array of a Galvatron-sized call is 0.36 MB,
// and looking through it was a third of the host's share of such a call).
static bool scan_costs(const double *q, size_t n, double *maxabs)
{
    double m[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    uint64_t bad[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    size_t k = 0;
    for (; k + 8 <= n; k += 8)
        for (int j = 0; j < 8; ++j) {
            const double x = q[k + j];
            const double a = std::fabs(x);
            const double fin = a < INFINITY ? a : 0.0;   // NaN and the infinities count as 0 here
            m[j] = fin > m[j] ? fin : m[j];
            bad[j] |= (uint64_t)(x != x) | (uint64_t)(x == -INFINITY);
        }
    double mm = 0;
    uint64_t b = 0;
    for (int j = 0; j < 8; ++j) {
        mm = std::max(mm, m[j]);
        b |= bad[j];
    }
    for (; k < n; ++k) {
        const double x = q[k];
        if (x != x || x == -INFINITY) b = 1;
        else if (x != INFINITY) mm = std::max(mm, std::fabs(x));
    }
    *maxabs = mm;
    return b == 0;
}

// The caller's initial costs (gdp_problem.f0): *live says whether anything but +0.0 is in there (an array of
// zeros is what every caller of the reference passes, and is treated like no array), *maxabs the largest
// finite magnitude.  The common case is one pass over the array that ORs its words.
static int scan_f0(const gdp_problem *p, bool *live, double *maxabs)
{
    *live = false;
    *maxabs = 0;
    if (!p->f0) return 0;
    const size_t n = (size_t)p->V * (size_t)p->S;
    uint64_t any = 0;
    size_t k = 0;
    for (; k + 64 <= n && !any; k += 64)
        for (int j = 0; j < 64; ++j) {
            uint64_t w;
            memcpy(&w, p->f0 + k + j, sizeof w);
            any |= w;
        }
    for (; k < n && !any; ++k) {
        uint64_t w;
        memcpy(&w, p->f0 + k, sizeof w);
        any |= w;
    }
    if (!any) return 0;
    *live = true;
    double m = 0;
    for (k = 0; k < n; ++k) {
        const double x = p->f0[k];
        if (x != x || x == -INFINITY) return 1;
        if (x == 0 && std::signbit(x)) return 2;
        if (x != INFINITY) m = std::max(m, std::fabs(x));
    }
    *maxabs = m;
    return 0;
}

// The magnitudes of the cost arrays may add up to COST_BOUND and those of the initial costs reach it, so that
// no partial sum can overflow.
static constexpr double COST_BOUND = 5e299;

int gdp_validate_f0(const gdp_problem *p, int i, bool *f0_live)
{
    char buf[200];
    bool live = false;
    double m = 0;
    const int what = scan_f0(p, &live, &m);
    if (f0_live) *f0_live = live;
    if (what == 0 && m < COST_BOUND) return GDP_OK;
    snprintf(buf, sizeof buf, "instance %d: %s", i,
             what == 1 ? "NaN or -inf in f0"
             : what == 2 ? "-0.0 in f0 (the sign of a zero cost would depend on the order of evaluation)"
                         : "cost magnitudes could overflow binary64 (f0)");
    return gdp_fail(what == 2 ? GDP_E_BADARG : GDP_E_NONFINITE, buf);
}

int gdp_validate(const gdp_problem *p, int i)
{
    char buf[160];
    auto bad = [&](int code, const char *why) {
        snprintf(buf, sizeof buf, "instance %d: %s", i, why);
        return fail(code, buf);
    };
    if (!p) return bad(GDP_E_BADARG, "null problem");
    if (p->L < 1 || p->V < 1 || p->S < 1) return bad(GDP_E_BADARG, "L, V and S must be >= 1");
    if (p->V > GDP_MAX_V) return bad(GDP_E_BADARG, "V exceeds GDP_MAX_V");
    if (p->L > GDP_MAX_L) return bad(GDP_E_BADARG, "L exceeds GDP_MAX_L");
    if (p->S > GDP_MAX_S) return bad(GDP_E_BADARG, "S exceeds GDP_MAX_S");
    if (p->S > GDP_MAX_S_MARKS && (p->flags & (GDP_KEEP_MARKS | GDP_EXPORT_MARK)))
        return bad(GDP_E_BADARG, "S exceeds GDP_MAX_S_MARKS and the argmin table was asked for");
    if (!p->mem || !p->intra || !p->inter) return bad(GDP_E_BADARG, "null input array");
    if (p->n_key < 0 || (p->n_key > 0 && (!p->other_mem || !p->other_time)))
        return bad(GDP_E_BADARG, "bad key arrays");
    const int T = p->inter_index ? p->n_inter : p->L;
    if (T < 1) return bad(GDP_E_BADARG, "n_inter must be >= 1");
    const size_t LS = (size_t)p->L * p->S;
    for (size_t k = 0; k < LS; ++k) {
        if (p->mem[k] < 0) return bad(GDP_E_BADARG, "negative mem entry");
    }
    if (p->inter_index)
        for (int l = 0; l < p->L; ++l)
            if (p->inter_index[l] < 0 || p->inter_index[l] >= T) return bad(GDP_E_BADARG, "inter_index out of range");
    // NaN and -inf make the reference's result depend on evaluation order; reject them, and
    // make sure no partial sum can overflow to an infinity of either sign.
    double bound = 0;
    for (int l = 0; l < p->L; ++l) {
        double m = 0;
        if (!scan_costs(p->intra + (size_t)l * p->S, (size_t)p->S, &m)) return bad(GDP_E_NONFINITE, "NaN or -inf in intra");
        bound += m;
    }
    // This function allocates nothing: the per-matrix maxima live in a small fixed table, and with more
    // matrices than that a matrix shared by several layers is simply scanned once per layer.
    const size_t SS = (size_t)p->S * p->S;
    auto matrix_max = [&](int t, double *m_out) { return scan_costs(p->inter + (size_t)t * SS, SS, m_out); };
    constexpr int TMAX_KEPT = 1024;   // 8 KB of stack
    double tmax[TMAX_KEPT];
    const bool kept = p->inter_index && T <= TMAX_KEPT;
    if (p->inter_index)  // every matrix is checked, also one that no layer uses
        for (int t = 0; t < T; ++t) {
            double m = 0;
            if (!matrix_max(t, &m)) return bad(GDP_E_NONFINITE, "NaN or -inf in inter");
            if (kept) tmax[t] = m;
        }
    for (int l = 0; l < p->L; ++l) {
        double m = 0;
        if (kept) m = tmax[p->inter_index[l]];
        else if (!matrix_max(p->inter_index ? p->inter_index[l] : l, &m))
            return bad(GDP_E_NONFINITE, "NaN or -inf in inter");
        bound += m;
    }
    for (int k = 0; k < p->n_key; ++k) {
        const double x = p->other_time[k];
        if (x != x || x == -INFINITY) return bad(GDP_E_NONFINITE, "NaN or -inf in other_time");
        // start row V-1-other_mem (csrc/dp_core.cpp:82): a negative entry puts it above the table, where the
        // reference reads out of bounds; an entry above V-1 is an infeasible key and is answered as such
        if (p->other_mem[k] < 0) return bad(GDP_E_BADARG, "negative other_mem entry (start row above the table)");
    }
    if (!(bound < COST_BOUND)) return bad(GDP_E_NONFINITE, "cost magnitudes could overflow binary64");
    return GDP_OK;
}

namespace {

// Looks through the initial costs of all problems; f0_live[i] != 0 where problem i brings some other than zeros.
int validate_f0_all(int32_t n, const gdp_problem *const *p, std::vector<char> &f0_live)
{
    f0_live.assign((size_t)n, 0);
    for (int i = 0; i < n; ++i) {
        bool live = false;
        const int rc = gdp_validate_f0(p[i], i, &live);
        if (rc != GDP_OK) return rc;
        f0_live[(size_t)i] = live ? 1 : 0;
    }
    return GDP_OK;
}

// Validates all problems, initial costs included.
int validate_all(int32_t n, const gdp_problem *const *p, std::vector<char> &f0_live)
{
    for (int i = 0; i < n; ++i) {
        const int rc = gdp_validate(p[i], i);
        if (rc != GDP_OK) return rc;
    }
    return validate_f0_all(n, p, f0_live);
}

void destroy(gdp_plan *pl)
{
    if (!pl) return;
    if (pl->dry) {
        delete pl;
        return;
    }
    if (pl->dbase || pl->lane.stream) (void)hipSetDevice(pl->device);
    if (pl->lane.stream) (void)hipStreamSynchronize(pl->lane.stream);  // the upload may still read its host copy
    if (pl->split_upload && pl->lane.side) (void)hipStreamSynchronize(pl->lane.side);   // (joined to the main stream: idle by now)
    if (pl->holds_fused) {  // a run that was started and never waited for: its launch has ended by now
        pl->holds_fused = false;
        fused_turn_give();
    }
    if (pl->dbase) arena_give(pl->device, pl->dbase, pl->dalloc);
    for (hipEvent_t e : pl->ev_relax) (void)hipEventDestroy(e);
    lane_give(pl->lane);
    delete pl;
}

// Per layer: how far down a reader reaches, and the band of tiles that has to be computed.
//  lo: source rows u < reach = sum_{k<l} min{mem[k][s] : mem < V, intra finite} hold +inf for every
//      strategy (by induction over the layers), so tiles entirely below `reach` need no arithmetic.
//  hi: a cell written from source row u at layer l lies on a path to start row v0 only if
//      u + sum_{k>=l} mem[k][s_k] = v0 for some choice, hence u <= max v0 - sum_{k>=l} min_s mem[k][s];
//      rows above are never read by a row inside the band of the next layer, nor by the epilogue.
// `skip` off (or exports requested, for hi) gives the full range.
// closed: hi is raised, where needed, to the tile that holds the highest row read by the band of the
//      next layer.  (A tile is computed whole, so the band of layer l+1 reads up to tile_rows - 1 rows
//      beyond what any path needs; those cells matter to no result, but a flow launch waits for every
//      cell it reads and must find each of them written.)
void fill_bands(const gdp_problem *q, const HostInst &h, int tile_rows, bool skip, int32_t *dep, double *executed,
                bool closed = false)
{
    std::vector<int64_t> minfin((size_t)h.L), minany((size_t)h.L);
    for (int l = 0; l < h.L; ++l) {
        int maxm = 0;
        int64_t mf = h.V, ma = h.V;
        for (int s = 0; s < h.S; ++s) {
            const int m = q->mem[(size_t)l * h.S + s];
            if (m >= h.V) continue;
            maxm = std::max(maxm, m);
            ma = std::min<int64_t>(ma, m);
            if (q->intra[(size_t)l * h.S + s] < INFINITY) mf = std::min<int64_t>(mf, m);
        }
        minfin[(size_t)l] = mf;
        minany[(size_t)l] = ma;
        dep[3 * l] = (maxm + tile_rows - 1) / tile_rows;
    }
    int64_t v0max = -1;
    for (int k = 0; k < h.n_key; ++k) v0max = std::max<int64_t>(v0max, (int64_t)h.V - 1 - q->other_mem[k]);
    const bool full = !skip || (h.flags & (GDP_EXPORT_F | GDP_EXPORT_MARK));
    int64_t reach = 0;  // first row of the previous layer's output that can be finite
    std::vector<int64_t> ub((size_t)h.L + 1);
    ub[(size_t)h.L] = v0max;
    for (int l = h.L - 1; l >= 0; --l) ub[(size_t)l] = ub[(size_t)l + 1] - minany[(size_t)l];
    if (closed && !full)   // layer l+1 reads row u - mem[l][s'] of layer l's output for every row u of its own band
        for (int l = h.L - 2; l >= 0; --l) {
            if (ub[(size_t)l + 1] < 0) continue;
            const int64_t top = std::min<int64_t>(h.ntile - 1, ub[(size_t)l + 1] / tile_rows) * tile_rows + tile_rows - 1;
            ub[(size_t)l] = std::max(ub[(size_t)l], top - minany[(size_t)l]);
        }
    for (int l = 0; l < h.L; ++l) {
        int64_t lo = skip ? std::min<int64_t>(reach, h.V) / tile_rows : 0;
        int64_t hi = h.ntile - 1;
        if (!full) hi = ub[(size_t)l] < 0 ? -1 : std::min<int64_t>(hi, ub[(size_t)l] / tile_rows);
        if (lo > h.ntile) lo = h.ntile;
        dep[3 * l + 1] = (int32_t)lo;
        dep[3 * l + 2] = (int32_t)hi;  // -1: nothing to compute
        if (hi >= lo) {
            const int64_t rows = std::min<int64_t>(h.V, (hi + 1) * tile_rows) - lo * tile_rows;
            *executed += (double)std::max<int64_t>(rows, 0) * (double)h.S * h.S;
        }
        reach = std::min<int64_t>(reach + minfin[(size_t)l], h.V);
    }
}

// Device bytes one instance takes in the costs-only layout, to within the padding of the rows.
size_t footprint(const gdp_problem *q)
{
    int maxm = 1;
    for (size_t k = 0; k < (size_t)q->L * q->S; ++k)
        if (q->mem[k] < q->V) maxm = std::max(maxm, q->mem[k]);
    const size_t ld = (size_t)q->V + (size_t)maxm + 1024;
    return sizeof(double) * ((size_t)q->L + 1) * ((size_t)q->S + 1) * ld;
}

// Internal return code: the costs-only layout (one cost buffer per layer) does not fit in device memory;
// the caller starts over with force_marks, i.e. two cost buffers and the argmin table.
constexpr int GDP_RETRY_WITH_MARKS = 1 << 20;

// The initial costs of the instances that brought some, into the data region of their buffer 0 (behind
// whatever zeroed it on the plan's stream).
int upload_f0(gdp_plan *pl)
{
    for (const HostInst &h : pl->inst) {
        if (h.f0t.empty()) continue;
        double *dst = reinterpret_cast<double *>(pl->dbase + h.off_H) + h.P;
        GDP_HIP(hipMemcpy2DAsync(dst, sizeof(double) * (size_t)h.ld, h.f0t.data(), sizeof(double) * (size_t)h.V,
                                 sizeof(double) * (size_t)h.V, (size_t)h.S, hipMemcpyHostToDevice, pl->stream));
    }
    return GDP_OK;
}

// Lays a plan out and brings it onto the device, one step after the other (create() below runs them in order).
// What more than one step needs lives here; everything that outlasts the creation is written into the plan.
struct PlanBuilder {
    int32_t n;
    const gdp_problem *const *p;
    gdp_plan *pl;
    bool force_marks;      // start over with the argmin table (the costs-only layout did not fit the device)
    const char *f0_live;   // null, or per problem whether its f0 holds anything but zeros (validate_all)

    bool fused_preset = false;   // the launch scheme was asked for (environment, flags): it is not the library's choice
    bool marks_preset = false;
    std::vector<HostInst> inst;  // sorted by S, then by L descending; moved into the plan at the end
    int64_t wave_slots = 0;      // wave slots of the device at 4 resident waves per SIMD
    double band_frac = 1.0;      // share of the relaxations that lie inside the bands
    size_t off = 0;              // next free byte of the device allocation while it is laid out
    int nk = 0;                  // keys / strategy-list entries of all instances
    size_t nres = 0;
    size_t small_bytes = 0;      // tables and per-instance inputs: what is built on the host and uploaded
    size_t fixed_bytes = 0;      // ... plus counters and results: everything in front of the cost buffers
    int max_S = 0;
    struct { char *p; char *data() const { return p; } } stage = {nullptr};   // host copy of the first small_bytes
    std::vector<std::vector<int32_t>> h_band;   // per instance {tiles a reader reaches down, first, last tile to compute} per layer
    bool turn_free = false;      // a flow plan whose first run will most likely flow (nobody holds the turn)
    bool prepared_early = false; // ... and whose cost buffers are already being prepared by a kernel fed with arguments
    GdpDevInst *di = nullptr;    // instance and key records inside `stage`
    GdpDevKey *dk = nullptr;

    size_t take(size_t bytes)
    {
        const size_t o = off;
        off = align_up(off + bytes, 256);
        return o;
    }
    int read_presets();
    int describe_device();
    void describe_instances();
    int form_groups();
    struct FlowPick { int K, nsrc; double resident; };
    FlowPick flow_pick(const Group &g) const;
    void choose_launch_scheme();
    int lay_out_tables();
    int allocate();
    int take_stage();
    void compute_bands();
    int32_t fill_from_of(int i, int l) const;
    int prepare_early();
    void build_instance_tables();
    void build_group_tables();
    int upload();
};

// Options of the plan: presets from the environment, then what the problems' flags ask for.
int PlanBuilder::read_presets()
{
    pl->n = n;
    if (!pl->dry) GDP_HIP(hipGetDevice(&pl->device));
    // defaults of the plan options can be preset from the environment
    if (const char *e = getenv("GALVATRON_DP_FUSED")) {
        pl->fused = atoi(e) != 0;
        fused_preset = true;
    }
    if (const char *e = getenv("GALVATRON_DP_KEEP_MARKS")) {
        pl->keep_marks = atoi(e) != 0;
        marks_preset = true;
    }
    if (const char *e = getenv("GALVATRON_DP_POISON")) pl->poison = atoi(e) != 0;
    if (const char *e = getenv("GALVATRON_DP_SKIP")) pl->skip = atoi(e) != 0;
    if (const char *e = getenv("GALVATRON_DP_TILE_R")) pl->tile_r_override = atoi(e);
    if (const char *e = getenv("GALVATRON_DP_LATENCY_VARIANT")) pl->latency_override = std::max(0, atoi(e));
    if (const char *e = getenv("GALVATRON_DP_CHUNK")) pl->chunk_override = atoi(e);
    if (const char *e = getenv("GALVATRON_DP_FLOW")) pl->flow_override = atoi(e) != 0;
    if (const char *e = getenv("GALVATRON_DP_OCCUPANCY_CAP")) {
        pl->no_occupancy_cap = atoi(e) == 0;
        pl->occupancy_cap_override = atoi(e);
    }
    if (const char *e = getenv("GALVATRON_DP_SPIN_LIMIT")) {
        const long long v = atoll(e);
        if (v >= 1) pl->spin_limit = v;
    }
    for (int i = 0; i < n; ++i) {
        if (p[i]->flags & GDP_COMPUTE_ALL) pl->skip = false;
        if ((p[i]->flags & GDP_KEEP_MARKS) && !marks_preset) pl->keep_marks = true;
        if (p[i]->flags & GDP_EXPORT_MARK) pl->keep_marks = true;  // the table itself is asked for
    }
    for (int i = 0; i < n && !fused_preset; ++i) {  // an explicit request of the caller
        if (p[i]->flags & GDP_LAUNCH_FUSED) { pl->fused = true; fused_preset = true; }
        else if (p[i]->flags & GDP_LAUNCH_PER_LAYER) { pl->fused = false; fused_preset = true; }
    }
    for (int i = 0; i < n && !pl->has_zero; ++i)
        for (size_t k = 0; k < (size_t)p[i]->L * p[i]->S; ++k)
            if (p[i]->mem[k] == 0) {
                pl->has_zero = true;
                break;
            }
    if (force_marks || pl->has_zero) {
        if (force_marks) pl->keep_marks = true;
        pl->fused = false;    // (mem == 0: a cell then depends on cells of its own layer, which the counters of a
        fused_preset = true;  //  fused launch do not order)
    }
    return GDP_OK;
}

// Compute units and LDS per unit of the device the plan is for.
int PlanBuilder::describe_device()
{
    if (pl->dry) {
        pl->num_cu = pl->dry_num_cu;
        pl->lds_per_cu = pl->dry_lds_per_cu;
    } else {
        // asked once per device: the call costs as much as laying out a small plan
        static std::mutex mu;
        static std::vector<std::pair<int, size_t>> known;   // per device: {CUs, LDS bytes per CU}, {0, 0} = not asked yet
        std::lock_guard<std::mutex> lk(mu);
        if ((size_t)pl->device >= known.size()) known.resize((size_t)pl->device + 1, {0, 0});
        if (known[(size_t)pl->device].first == 0) {
            hipDeviceProp_t prop;
            GDP_HIP(hipGetDeviceProperties(&prop, pl->device));
            known[(size_t)pl->device] = {prop.multiProcessorCount, (size_t)prop.maxSharedMemoryPerMultiProcessor};
        }
        pl->num_cu = known[(size_t)pl->device].first;
        pl->lds_per_cu = known[(size_t)pl->device].second;
    }
    return GDP_OK;
}

// Shapes of the instances, their equal transition matrices, their initial costs; sorted into groups of one S.
void PlanBuilder::describe_instances()
{
    inst.assign((size_t)n, HostInst());
    for (int i = 0; i < n; ++i) {
        const gdp_problem *q = p[i];
        HostInst &h = inst[(size_t)i];
        h.orig = i;
        h.L = q->L; h.V = q->V; h.S = q->S;
        h.SU = (int)align_up((size_t)q->S, GDP_SRC_UNROLL);
        h.n_key = q->n_key;
        h.n_inter = q->inter_index ? q->n_inter : q->L;
        if (!q->inter_index) share_equal_matrices(q, h);
        h.flags = q->flags;
        int maxm = 0;
        for (size_t k = 0; k < (size_t)q->L * q->S; ++k) {
            if (q->mem[k] < q->V) maxm = std::max(maxm, q->mem[k]);
            if (q->mem[k] == 0) h.has_zero = true;
        }
        h.P = (int)align_up((size_t)std::max(maxm, 1), 64);
        if (f0_live && f0_live[i] && q->f0 && !pl->dry) {   // [V][S] -> one row per strategy
            h.f0t.resize((size_t)q->S * (size_t)q->V);
            for (int v = 0; v < q->V; ++v)
                for (int s2 = 0; s2 < q->S; ++s2) h.f0t[(size_t)s2 * q->V + v] = q->f0[(size_t)v * q->S + s2];
        }
    }
    // group by S, then by L descending (stable, so equal shapes keep the caller's order)
    std::stable_sort(inst.begin(), inst.end(), [](const HostInst &a, const HostInst &b) {
        if (a.S != b.S) return a.S < b.S;
        return a.L > b.L;
    });
}

// One group per S: register tile, chunking of fused launches, row lengths, per-layer activity.
int PlanBuilder::form_groups()
{
    wave_slots = (int64_t)pl->num_cu * 4 * 4;  // 4 SIMDs x 4 resident waves
    for (int i = 0; i < n;) {
        Group g;
        g.first = i; g.S = inst[(size_t)i].S;
        int j = i;
        while (j < n && inst[(size_t)j].S == g.S) ++j;
        g.count = j - i;
        // Register tile.  Width: pick_ts.  Height: the tallest whose first layer still gives every
        // resident wave at least two tasks, so that the stores of one task drain under the arithmetic
        // of the next; small problems get the shortest (most parallel) one.
        int64_t tiles64 = 0;
        for (int k = i; k < j; ++k) tiles64 += ((int64_t)inst[(size_t)k].V + 63) / 64;
        const int ts = pick_ts(g.S, pl->keep_marks, tiles64, wave_slots);
        const int ntb = (int)align_up((size_t)g.S, (size_t)ts) / ts;
        // A fused launch can take `chunk` instances at a time through all their layers (in the sorted
        // order, so mostly instances of one depth) instead of the whole batch layer by layer: as many as
        // keep two cost buffers each -- the layer being read and the one being written -- within
        // GALVATRON_DP_CHUNK_MB (default 144) of the 256 MB memory-side cache, so that a layer's output
        // is still there when the next layer reads it.  Fewer instances in flight also means less work
        // between a layer and the next, i.e. more waiting; what wins was measured (batches of 96-256
        // instances, times per solve, layer by layer -> chunked):
        //   8- and 11-wide tiles, S >= 36: S = 36 14.1 -> 10.8 ms, S = 40 (V = 29493, L = 28) 26.6 -> 21.1,
        //   S = 44 (V = 65536) 46.8 -> 43.3, S = 56 21.8 -> 16.2, S = 72 25.0 -> 18.1, S = 88 20.5 -> 17.7;
        //   never slower in 20 shapes; one instance at a time is always slower;
        //   16-wide tiles (S = 32, 48, 64): 6.4 -> 6.6, 23.2 -> 23.4, 5.7 -> 7.2 -- they issue half the
        //   cost-row loads per relaxation and do not wait for memory in the first place;
        //   S = 22..30: 5.0 -> 5.6, 13.4 -> 14.7, 13.9 -> 13.1 -- a block task is over in 2-3 us, and the
        //   per-task cost of waiting and signalling weighs more than the memory.
        // So: narrow tiles, at least 36 strategies, and at least two instances that fit.  (With the widths
        // 12 to 16 picked for S >= 36 by now, this happens only where a narrow tile is forced; with those
        // widths chunking changed the same batches by -9 % to +9 %, so it is left to GALVATRON_DP_CHUNK.)
        {
            size_t pair = 0;  // bytes of two cost buffers of the largest instance
            for (int k = i; k < j; ++k)
                pair = std::max(pair, 2 * sizeof(double) * ((size_t)g.S + 1) *
                                          ((size_t)inst[(size_t)k].V + (size_t)inst[(size_t)k].P));
            const size_t fit = env_mb("GALVATRON_DP_CHUNK_MB", 144) / std::max<size_t>(pair, 1);
            g.chunk = g.count;  // not chunked
            if (g.S >= 36 && ts <= 11 && !pl->keep_marks && fit >= 2 && fit < (size_t)g.count) g.chunk = (int)fit;
            if (pl->chunk_override > 0) g.chunk = std::min(g.count, pl->chunk_override);
        }
        int best_r = 0;
        {
            // variants of one width are listed tallest first
            for (int v = 0; v < GDP_NUM_VARIANTS; ++v) {
                if (GDP_VARIANTS[v].ts != ts) continue;
                const int r = GDP_VARIANTS[v].r;
                int64_t tasks = 0;  // of the instances that are in flight together
                for (int k = i; k < i + g.chunk; ++k) tasks += ((int64_t)inst[(size_t)k].V + 64 * r - 1) / (64 * r) * ntb;
                best_r = r;
                if (tasks >= 2 * wave_slots) break;
            }
        }
        if (pl->tile_r_override > 0 && find_variant(ts, pl->tile_r_override) >= 0) best_r = pl->tile_r_override;
        g.variant = find_variant(ts, best_r);
        if (g.variant < 0) return fail(GDP_E_BADARG, "no kernel variant for the requested tile/scan override");
        const int tile_rows = 64 * best_r;
        g.SP = ntb * ts;
        g.ntb = ntb;
        // A group whose layers hold no more wave tasks than the device has wave slots (one instance of middling
        // size) is short of waves, not of work per wave: the sources of a task then go on two waves -- twice the
        // waves, each half as long, so that the start of one task (a chain of dependent loads) lies behind the
        // arithmetic of another.  Measured, relaxation time per solve, one wave -> two, every cell / with row
        // skipping (ms): L=32 S=44 V=65536 0.441 -> 0.398 / 0.431 -> 0.386; L=28 S=40 V=65536 0.366 -> 0.322 /
        // 0.53 -> 0.30; L=16 S=88 V=32768 0.345 -> 0.310 / 0.319 -> 0.281; L=48 S=36 V=65536 0.573 -> 0.525 /
        // 0.80 -> 0.45; L=24 S=22 V=131072 0.280 -> 0.262 / 0.307 -> 0.243.  Not with the 16-wide tile (its
        // exchange buffer of 32 KB holds a CU to five workgroups: L=16 S=64 V=65536 0.339 -> 0.351), and not where
        // a layer fills the slots anyway (L=32 S=44 V=131072 0.709 -> 0.807).  GALVATRON_DP_SPLIT=1|2 overrides.
        // (Not the narrowest tile either: plans that get it run as flow launches or with the latency variant, which
        // split their sources in their own way and pad SU for that.)
        if (!pl->keep_marks && best_r == GDP_SPLIT_R && ts != GDP_LAT_TS) {
            int64_t tasks = 0;
            for (int k = i; k < j; ++k) tasks += ((int64_t)inst[(size_t)k].V + tile_rows - 1) / tile_rows * ntb;
            if (g.S >= 16 && ts <= 15 && tasks <= wave_slots) g.split = 2;
            if (const char *e = getenv("GALVATRON_DP_SPLIT")) g.split = atoi(e) == 2 ? 2 : 1;
        }
        g.ntb = ntb * g.split;
        g.max_L = 0; g.max_ntile = 0; g.max_ld = 0;
        for (int k = i; k < j; ++k) {
            HostInst &h = inst[(size_t)k];
            h.variant = g.variant;
            h.SP = g.SP;
            if (g.split > 1) h.SU = (int)align_up((size_t)h.S, (size_t)GDP_SRC_UNROLL * g.split);
            h.ntile = (h.V + tile_rows - 1) / tile_rows;
            h.ldm = (int64_t)align_up((size_t)h.ntile * tile_rows, 256);
            h.ld = h.P + h.ldm;
            g.max_L = std::max(g.max_L, h.L);
            g.max_ntile = std::max(g.max_ntile, h.ntile);
            g.max_ld = std::max(g.max_ld, h.ld);
        }
        g.active.assign((size_t)g.max_L, 0);
        g.zero_layer.assign((size_t)g.max_L, 0);
        for (int k = i; k < j; ++k) {
            g.max_V = std::max(g.max_V, inst[(size_t)k].V);
            for (int l = 0; l < inst[(size_t)k].L; ++l) {
                g.active[(size_t)l]++;
                if (inst[(size_t)k].has_zero)
                    for (int s2 = 0; s2 < g.S; ++s2)
                        if (p[inst[(size_t)k].orig]->mem[(size_t)l * g.S + s2] == 0) g.zero_layer[(size_t)l] = 1;
            }
        }
        g.nbt = (g.max_ntile * g.ntb + GDP_WAVES_PER_BLOCK - 1) / GDP_WAVES_PER_BLOCK;
        // Whole tiles per XCD turn: the fewest whose wave tasks fill whole workgroups.  (Longer turns
        // would save some of the cache lines that neighbouring tiles share -- a tile's source rows start
        // at any 8-byte offset -- from being fetched into two L2s, but measured slower: cfg3 49.5 ms with
        // one tile per turn, 50.7 with two or four, 54 with eight.)
        g.xcd_group = GDP_WAVES_PER_BLOCK / gcd_int(g.ntb, GDP_WAVES_PER_BLOCK) * g.ntb / GDP_WAVES_PER_BLOCK;
        g.slots = ((g.nbt + g.xcd_group - 1) / g.xcd_group + 7) / 8 * g.xcd_group;
        pl->max_L = std::max(pl->max_L, g.max_L);
        pl->groups.push_back(g);
        i = j;
    }
    return GDP_OK;
}

// Which of the three launch schemes the plan runs with, where the caller has not said (see the comments
// inside), and with it the variant of the per-layer kernel and how a task's sources are split over waves.
void PlanBuilder::choose_launch_scheme()
{
    if (!fused_preset || pl->flow_override != 0) {
        // One launch for all layers pays off once a layer holds about two block tasks that carry
        // arithmetic per CU (measured: 950 per layer, 0.48 ms against 0.58 ms; 128 per layer, 0.23 ms
        // against 0.17 ms): the launch gaps and the ramp up and down of every layer go away, and layers
        // overlap where their dependencies allow.  Below that a layer is over before signalling through
        // memory has paid for itself, and a launch per layer is quicker.
        double first_layer = 0, all = 0, live = 0;
        std::vector<int32_t> band;
        for (const Group &g : pl->groups) {
            first_layer += (double)g.active[0] * g.nbt;
            for (int k = g.first; k < g.first + g.count; ++k) {
                const HostInst &h = inst[(size_t)k];
                band.assign((size_t)h.L * 3, 0);
                fill_bands(p[h.orig], h, 64 * GDP_VARIANTS[h.variant].r, pl->skip, band.data(), &live);
                all += (double)h.L * h.V * (double)h.S * h.S;
            }
        }
        band_frac = all > 0 ? live / all : 1.0;
        if (!fused_preset) pl->fused = first_layer * band_frac >= 2.0 * pl->num_cu && !device_seems_shared();
    }
    // Launches that small run one or two waves per SIMD, and what they wait for is memory latency, not
    // instruction issue: their narrowest tile has a variant built for that (measured, 16 layers, one
    // instance: S=22 V=16384 0.176 -> 0.126 ms, S=44 V=16384 0.241 -> 0.208, S=64 V=4096 0.284 -> 0.192;
    // with all layers in one launch, or on larger problems, it is the slower one).
    // Small and middling plans run all their layers in one launch that waits on the cost cells themselves
    // (gdp_relax_flow_kernel) -- unless the caller asked for a launch scheme: per-layer launches are also
    // what a shared device wants, since they never wait.  A flow task asks for all its cost rows at once,
    // at most 32 per wave (they wait in registers), so its sources go on 1, 2 or 4 waves.  More waves
    // shorten the task -- as long as the next layers' tasks still find room on the device beside the layer
    // at work: the start of a task (four dependent round trips to memory before it reaches its gate) then
    // lies behind it when its cost rows appear.  So: the most waves per task that keep two layers' tasks
    // resident, else what keeps the most (ms per solve, 1 / 2 / 4 waves: S=22 V=16384 L=24 0.099 / 0.091 /
    // 0.081; S=40 V=29493 L=28 - / 0.163 / 0.194).  It exists for the narrowest tile only, which is what a
    // plan has when it is too small to fill the device with wider ones; for such plans it beat the launch
    // with completion counters at every size measured (flow against it, by the share of a layer's tasks
    // that is resident: S=22 V=65536 L=24, 1.0: 0.16 against 0.23 ms; S=44 V=32768 L=32, 0.5: 0.38 against
    // 0.55; S=64 V=32768 L=16, 0.31: 0.31 against 0.35; S=88 V=16384 L=16, 0.27: 0.27 against 0.39; S=96
    // V=16384 L=48, 0.25: 0.87 against 1.72).  Plans that get a wider tile run faster with the counters
    // (forced onto the narrow tile and the flow launch: S=44 V=65536 L=32 0.63 against 0.64 ms, S=44
    // V=131072 1.22 against 0.83, S=64 V=65536 L=16 0.62 against 0.45).  GALVATRON_DP_FLOW=1 asks for it
    // wherever the layout allows (costs only, no memory cost of 0, the tile of the latency variant).
    bool want_flow = pl->flow_override >= 0 ? pl->flow_override == 1 && !(fused_preset && pl->fused)
                                            : !fused_preset && !device_seems_shared();
    want_flow = want_flow && !pl->keep_marks && !pl->has_zero && pl->max_L <= 65534;
    for (const Group &g : pl->groups) {
        want_flow = want_flow && g.latency_possible(pl->keep_marks) && g.count <= 65535 && g.S <= GDP_FLOW_MAX_S;
        if (want_flow && pl->flow_override != 1) want_flow = flow_pick(g).resident >= 0.1;
    }
    pl->flow = pl->flow_ready = want_flow;
    if (want_flow) pl->fused = false;
    for (Group &g : pl->groups) {
        const GdpVariant &v = GDP_VARIANTS[g.variant];
        bool on = !pl->fused && !pl->keep_marks && v.ts == GDP_LAT_TS && v.r == GDP_LAT_R;
        if (pl->latency_override >= 0) on = g.latency_possible(pl->keep_marks) && pl->latency_override != 0;
        if (pl->flow_ready) on = true;
        g.latency = 0;
        if (on) {
            // With many sources and wave slots to spare, the sources of a task are split over 2 or 4 waves:
            // the chain of dependent steps of a layer gets that much shorter.  Measured per solve, 1 / 2 / 4
            // waves: S=44 V=8192 L=32 0.317 / 0.242 / 0.250 ms, S=64 V=4096 L=16 0.190 / 0.142 / 0.132,
            // S=44 V=16384 L=16 0.208 / 0.188 / 0.231; no gain or a loss with few sources (S=22 V=16384 L=24
            // 0.180 / 0.196 / 0.188) or once the waves pass three per SIMD (S=40 V=29493 L=28 0.321 / 0.319 /
            // 0.388, S=64 V=16384 L=16 0.253 / 0.260 / 0.276).
            int64_t tasks = 0;
            for (int k = g.first; k < g.first + g.count; ++k) tasks += (int64_t)inst[(size_t)k].ntile * g.ntb;
            const int64_t room = (int64_t)pl->num_cu * 4 * 3;  // three waves per SIMD
            g.latency = g.S < 32 ? 1 : tasks * 4 <= room ? 4 : tasks * 2 <= room ? 2 : 1;
            if (pl->latency_override >= 1) g.latency = pl->latency_override >= 4 ? 4 : pl->latency_override >= 2 ? 2 : 1;
            int su = (int)align_up((size_t)g.S, (size_t)GDP_SRC_UNROLL_LAT * g.latency);
            if (pl->flow_ready) {
                const FlowPick fp = flow_pick(g);
                g.latency = fp.K;
                g.flow_nsrc = fp.nsrc;
                su = fp.nsrc * fp.K;
            }
            g.lat_ok = su % (GDP_SRC_UNROLL_LAT * g.latency) == 0;
            for (int k = g.first; k < g.first + g.count; ++k) inst[(size_t)k].SU = su;
        }
    }
}

// Flow launch: waves per task (4, 2, 1) and sources per wave for a group -- the most waves that keep two
// layers' tasks resident, else what keeps the most.
PlanBuilder::FlowPick PlanBuilder::flow_pick(const Group &g) const
{
    {
        auto waves_per_simd = [](int nsrc) { return nsrc <= 12 ? 8 : nsrc <= 16 ? 7 : nsrc <= 20 ? 6 : nsrc <= 28 ? 5 : 4; };  // by their registers (38 + 2 per source)
        auto nsrc_for = [&](int K) {
            for (int c : GDP_FLOW_NSRC)
                if (c * K >= g.S) return c;
            return 0;
        };
        double band_tiles = 0;   // of an average layer, over the group
        for (int k = g.first; k < g.first + g.count; ++k) band_tiles += (double)inst[(size_t)k].ntile * band_frac;
        const int ntb8 = (g.S + GDP_LAT_TS - 1) / GDP_LAT_TS;
        FlowPick best = {0, 0, -1.0};
        for (int K : {4, 2, 1}) {
            const int c = nsrc_for(K);
            if (!c) continue;
            const double res = (double)pl->num_cu * 4 * waves_per_simd(c) / std::max(1.0, band_tiles * ntb8 * K);
            if (pl->latency_override >= 1 && K == (pl->latency_override >= 4 ? 4 : pl->latency_override >= 2 ? 2 : 1))
                return FlowPick{K, c, res};
            if (res >= 2.0 && best.resident < 2.0) best = {K, c, res};
            if (best.resident < 2.0 && res > best.resident) best = {K, c, res};
        }
        return best;
    }
}

// Device layout, first part: [tables | per-instance inputs] (uploaded in one copy), then the words every run
// resets and the results (copied back in one piece).
int PlanBuilder::lay_out_tables()
{
    off = 0;
    nk = 0;
    nres = 0;
    {
        // the key table and the array of strategy lists are indexed with 32-bit offsets on the device
        size_t keys = 0, lists = 0;
        for (const auto &h : inst) {
            keys += (size_t)h.n_key;
            lists += (size_t)h.n_key * (size_t)h.L;
        }
        if (keys > (size_t)INT32_MAX || lists > (size_t)INT32_MAX)
            return fail(GDP_E_BADARG, "more than 2^31-1 keys or strategy-list entries in one plan");
    }
    for (auto &h : inst) {
        h.key_begin = nk; nk += h.n_key;
        h.res_begin = (int)nres; nres += (size_t)h.n_key * h.L;
    }
    pl->n_key_total = nk;
    pl->n_res_total = nres;
    pl->off_insts = take(sizeof(GdpDevInst) * (size_t)n);
    pl->off_keys = take(sizeof(GdpDevKey) * (size_t)std::max(nk, 1));
    for (auto &g : pl->groups) {
        g.off_active = take(sizeof(int32_t) * (size_t)g.max_L);
        g.off_lay = take(sizeof(GdpDevLayer) * (size_t)g.count * (size_t)g.max_L);
        g.rows.clear();
        if (g.chunk < g.count)
            for (int i0 = 0; i0 < g.count; i0 += g.chunk) {
                const int cnt = std::min(g.chunk, g.count - i0);
                for (int l = 0; l < inst[(size_t)(g.first + i0)].L; ++l) {  // the deepest of a chunk comes first
                    g.rows.push_back(i0);
                    g.rows.push_back(cnt);
                    g.rows.push_back(l);
                }
            }
        g.off_rows = take(sizeof(int32_t) * std::max<size_t>(g.rows.size(), 1));
    }
    // Instances that were handed the very same transition matrices (same addresses: the instances of a sweep
    // that differ in their memory and intra costs only, the stages of one pipeline degree) read ONE device
    // copy: workgroups of different instances that run side by side on a CU then find each other's
    // transition costs in the scalar cache instead of evicting them.
    std::unordered_map<const double *, std::vector<int>> owners;   // first kept matrix -> instances with a copy of their own
    for (size_t i = 0; i < inst.size(); ++i) {
        HostInst &h = inst[i];
        const gdp_problem *q = p[h.orig];
        std::vector<int> &cands = owners[h.matrix_at(q, 0)];
        h.tables_of = -1;
        for (int j : cands) {
            const HostInst &o = inst[(size_t)j];
            if (o.S != h.S || o.n_inter != h.n_inter || o.SU != h.SU || o.SP != h.SP) continue;
            bool same = true;
            for (int t = 1; same && t < h.n_inter; ++t) same = o.matrix_at(p[o.orig], t) == h.matrix_at(q, t);
            if (same) {
                h.tables_of = j;
                break;
            }
        }
        if (h.tables_of >= 0) {
            h.off_inter = inst[(size_t)h.tables_of].off_inter;
        } else {
            h.off_inter = take(sizeof(double) * (size_t)h.n_inter * (h.SU + GDP_SRC_PAD) * h.SP);
            cands.push_back((int)i);
        }
        h.off_intra = take(sizeof(double) * (size_t)h.L * h.SP);
        h.off_index = take(sizeof(int32_t) * (size_t)h.L);
        h.off_roff = take(sizeof(int64_t) * (size_t)(h.L + 1) * (h.SU + GDP_SRC_PAD));
        h.off_mem = take(sizeof(int32_t) * (size_t)h.L * h.S);
        h.off_zcols = h.has_zero ? take(sizeof(int32_t) * (size_t)h.L * (size_t)(h.S + 1)) : 0;
    }
    small_bytes = off;
    pl->small_bytes = small_bytes;
    // words that every fused run resets to zero: completion counters, abort flag
    pl->off_zero = off;
    for (auto &g : pl->groups) {
        g.off_cnt = take(sizeof(int32_t) * (size_t)g.count * g.max_L * g.max_ntile);
    }
    pl->off_abort = take(sizeof(int32_t));
    pl->zero_words = (off - pl->off_zero) / sizeof(int32_t);
    // abort flag, per-key outputs and strategy lists lie together: a run copies them back in one piece
    pl->off_out = take(sizeof(GdpDevOut) * (size_t)std::max(nk, 1));
    pl->off_res = take(sizeof(int32_t) * std::max<size_t>(nres, 1));
    pl->back_bytes = off - pl->off_abort;
    fixed_bytes = off;
    return GDP_OK;
}

// Device layout, second part: the cost buffers (and the argmin table), and the allocation itself.
int PlanBuilder::allocate()
{
    // One cost buffer per layer lets all layers share a launch and lets the backtrack recompute the
    // argmin of the cells it visits, so that the relaxation does not have to track it.  If that does
    // not fit in device memory: two cost buffers, the argmin table, one launch per layer.
    max_S = 0;
    for (const auto &h : inst) max_S = std::max(max_S, h.S);
    if (pl->keep_marks && max_S > GDP_MAX_S_MARKS)  // preset from the environment
        return fail(GDP_E_BADARG, "S exceeds GDP_MAX_S_MARKS and the argmin table is to be kept");
    for (int attempt = 0; attempt < 2; ++attempt) {
        off = fixed_bytes;
        pl->can_fuse = (pl->fused || !pl->keep_marks) && !pl->has_zero;
        pl->rezero = false;
        for (auto &h : inst) {
            h.nbuf = (pl->can_fuse || !pl->keep_marks) ? h.L + 1 : 2;   // costs only: the backtrack needs every layer's costs
            if (h.nbuf < h.L + 1) pl->rezero = true;
            h.off_H = take(sizeof(double) * (size_t)h.nbuf * (size_t)(h.S + 1) * (size_t)h.ld);
            h.off_M = pl->keep_marks ? take((size_t)h.L * h.S * (size_t)h.ldm) : 0;
        }
        pl->dbytes = off;
        if (pl->dry) {
            pl->dbase = reinterpret_cast<char *>((uintptr_t)1 << 44);  // never dereferenced
            pl->dalloc = pl->dbytes;
            break;
        }
        hipError_t e = arena_take(pl->device, pl->dbytes, &pl->dbase, &pl->dalloc);
        if (e == hipSuccess) break;
        pl->dbase = nullptr;
        (void)hipGetLastError();
        if ((e == hipErrorOutOfMemory || e == hipErrorMemoryAllocation) && !pl->keep_marks && max_S <= GDP_MAX_S_MARKS)
            return GDP_RETRY_WITH_MARKS;  // tile widths and paddings differ with the table: start over
        if ((e == hipErrorOutOfMemory || e == hipErrorMemoryAllocation) && pl->can_fuse && pl->keep_marks) {
            pl->fused = false;            // table kept and all layers in one launch: drop the latter
            continue;
        }
        char buf[128];
        snprintf(buf, sizeof buf, "hipMalloc of %zu bytes", pl->dbytes);
        return fail_hip(e, buf);
    }
    return GDP_OK;
}

// Stream, events and page-locked buffers of the plan, and the host memory the tables are built in.
int PlanBuilder::take_stage()
{
    if (!pl->dry) {
        const hipError_t e = lane_take(pl->device, pl->back_bytes, small_bytes, &pl->lane);
        if (e == hipErrorOutOfMemory || e == hipErrorMemoryAllocation) {
            (void)hipGetLastError();
            return fail(GDP_E_NOMEM, "page-locked host memory for inputs and results");
        }
        GDP_HIP(e);
        pl->stream = pl->lane.stream;
        pl->ev_begin = pl->lane.ev_begin;
        pl->ev_end = pl->lane.ev_end;
    }
    stage.p = pl->lane.up;
    if (small_bytes > UPLOAD_PINNED_MAX || pl->dry) {
        try {
            pl->stage.assign(small_bytes, 0);
        } catch (const std::bad_alloc &) {
            return fail(GDP_E_NOMEM, "host staging allocation failed");
        }
        stage.p = pl->stage.data();
    } else {
        // the previous plan of this lane has been destroyed, i.e. its stream waited for: nothing reads
        // the buffer any more
        memset(stage.p, 0, small_bytes);
    }
    return GDP_OK;
}

// The band of tiles every layer of every instance has to compute.
void PlanBuilder::compute_bands()
{
    h_band.assign((size_t)n, std::vector<int32_t>());
    for (int i = 0; i < n; ++i) {
        const HostInst &h = inst[(size_t)i];
        h_band[(size_t)i].assign((size_t)h.L * 3, 0);
        fill_bands(p[h.orig], h, 64 * GDP_VARIANTS[h.variant].r, pl->skip, h_band[(size_t)i].data(), &pl->executed,
                   pl->flow_ready);
    }
}

// Rows of a layer's output below its band are +inf and are filled once per plan -- those that something
// reads: the band of the next layer reaches down by at most this layer's largest memory cost (the
// backtrack reads what the relaxation read), the epilogue and the pass for memory costs of 0 read anywhere.
// The first such row of layer l of instance i.
int32_t PlanBuilder::fill_from_of(int i, int l) const
{
    const HostInst &h = inst[(size_t)i];
    if (l + 1 >= h.L || h.has_zero) return 0;
    const int64_t lo_next = h_band[(size_t)i][3 * (size_t)(l + 1) + 1];
    const int64_t reach = (int64_t)h_band[(size_t)i][3 * (size_t)l];   // tiles
    return (int32_t)std::max<int64_t>(0, (lo_next - reach) * (64 * GDP_VARIANTS[h.variant].r));
}

// A small plan laid out for the flow launch, the turn free right now (its first run will most likely
// flow): the kernel that prepares its cost buffers -- pads, zeros, the filled rows, NaN into the bands --
// gets what it needs with its arguments and starts here, before the tables have even been built; it runs
// beside the host's work on them and beside their upload (which then goes over the second stream in one
// piece).  (A Galvatron-like call: upload 15 us, then this kernel 42 us, then the first launch; now the
// kernel is under way 30 us earlier.)
int PlanBuilder::prepare_early()
{
    turn_free = false;
    if (!pl->dry && pl->flow_ready) {
        std::lock_guard<std::mutex> lk(g_fused_mu);
        turn_free = !g_fused_busy;
    }
    prepared_early = false;
    if (turn_free && n <= GDP_PREP_MAX_INST) {
        int layers = 0;
        for (const auto &h : inst) layers += h.L;
        if (layers <= GDP_PREP_MAX_LAYERS) {
            GdpPrepArgs A;
            memset(&A, 0, sizeof A);
            int e = 0;
            for (int i = 0; i < n; ++i) {
                const HostInst &h = inst[(size_t)i];
                GdpPrepArgs::Inst &a = A.inst[i];
                a.H = reinterpret_cast<double *>(pl->dbase + h.off_H);
                a.hstride = (int64_t)(h.S + 1) * h.ld;
                a.ld = h.ld;
                a.P = h.P;
                a.S = h.S;
                a.L = h.L;
                a.tile_rows = 64 * GDP_VARIANTS[h.variant].r;
                a.first_layer = e;
                for (int l = 0; l < h.L; ++l, ++e) {
                    A.lo[e] = h_band[(size_t)i][3 * (size_t)l + 1];
                    A.hi[e] = h_band[(size_t)i][3 * (size_t)l + 2];
                    A.fill_from[e] = fill_from_of(i, l);
                }
            }
            A.abort_flag = reinterpret_cast<int32_t *>(pl->dbase + pl->off_abort);
            A.n_inst = n;
            A.nan_bands = 1;
            GDP_HIP(gdp_launch_prepare_args(A, pl->stream));
            prepared_early = true;
        }
    }
    return GDP_OK;
}

// The host copy of the per-instance device tables: instance and key records, transition matrices, intra
// costs, row offsets.
void PlanBuilder::build_instance_tables()
{
    di = reinterpret_cast<GdpDevInst *>(stage.data() + pl->off_insts);
    dk = reinterpret_cast<GdpDevKey *>(stage.data() + pl->off_keys);
    for (int i = 0; i < n; ++i) {
        const HostInst &h = inst[(size_t)i];
        const gdp_problem *q = p[h.orig];
        GdpDevInst &d = di[i];
        d.H = reinterpret_cast<double *>(pl->dbase + h.off_H);
        d.hstride = (int64_t)(h.S + 1) * h.ld;
        d.nbuf = h.nbuf;
        d.M = pl->keep_marks ? reinterpret_cast<uint8_t *>(pl->dbase + h.off_M) : nullptr;
        d.inter = reinterpret_cast<const double *>(pl->dbase + h.off_inter);
        d.intra = reinterpret_cast<const double *>(pl->dbase + h.off_intra);
        d.inter_index = reinterpret_cast<const int32_t *>(pl->dbase + h.off_index);
        d.roff = reinterpret_cast<const int64_t *>(pl->dbase + h.off_roff);
        d.mem = reinterpret_cast<const int32_t *>(pl->dbase + h.off_mem);
        d.ld = h.ld; d.ldm = h.ldm;
        d.L = h.L; d.V = h.V; d.S = h.S; d.SP = h.SP; d.SU = h.SU; d.P = h.P; d.ntile = h.ntile;
        const int rows = h.SU + GDP_SRC_PAD;  // source rows per matrix / offsets per layer
        // inter: [T][rows][SP], zero padded
        double *it = reinterpret_cast<double *>(stage.data() + h.off_inter);
        for (int t = 0; t < (h.tables_of >= 0 ? 0 : h.n_inter); ++t) {
            const double *from = h.matrix_at(q, t);
            for (int a = 0; a < h.S; ++a)
                memcpy(it + ((size_t)t * rows + a) * h.SP, from + (size_t)a * h.S, sizeof(double) * (size_t)h.S);
        }
        double *ia = reinterpret_cast<double *>(stage.data() + h.off_intra);
        for (int l = 0; l < h.L; ++l)
            memcpy(ia + (size_t)l * h.SP, q->intra + (size_t)l * h.S, sizeof(double) * (size_t)h.S);
        int32_t *ix = reinterpret_cast<int32_t *>(stage.data() + h.off_index);
        for (int l = 0; l < h.L; ++l) ix[l] = h.matrix(q, l);
        memcpy(stage.data() + h.off_mem, q->mem, sizeof(int32_t) * (size_t)h.L * h.S);
        d.zcols = nullptr;
        if (h.has_zero) {
            d.zcols = reinterpret_cast<const int32_t *>(pl->dbase + h.off_zcols);
            int32_t *z = reinterpret_cast<int32_t *>(stage.data() + h.off_zcols);
            for (int l = 0; l < h.L; ++l) {
                int32_t *row = z + (size_t)l * (h.S + 1);
                row[0] = 0;
                for (int s = 0; s < h.S; ++s)
                    if (q->mem[(size_t)l * h.S + s] == 0) row[++row[0]] = s;
            }
        }
        // roff[l][s']: where row 0 of "f after layer l-1, strategy s'" sits in a cost buffer
        int64_t *ro = reinterpret_cast<int64_t *>(stage.data() + h.off_roff);
        const int64_t inf_row = (int64_t)h.S * h.ld + h.P;
        for (int l = 0; l <= h.L; ++l) {
            int64_t *row = ro + (size_t)l * rows;
            for (int s = 0; s < h.S; ++s) {
                if (l == 0) {
                    row[s] = (int64_t)s * h.ld + h.P;  // zeros: the caller's initial f
                } else {
                    const int m = q->mem[(size_t)(l - 1) * h.S + s];
                    row[s] = (m >= h.V) ? inf_row : (int64_t)s * h.ld + h.P - m;
                }
            }
            for (int s = h.S; s < rows; ++s) row[s] = inf_row;  // padding sources and prefetch targets
        }
        for (int k = 0; k < h.n_key; ++k) {
            GdpDevKey &key = dk[h.key_begin + k];
            key.other_mem = q->other_mem[k];
            key.other_time = q->other_time[k];
            key.inst = i;
            key.res_off = h.res_begin + k * h.L;
        }
        pl->relaxations += (double)h.L * h.V * (double)h.S * h.S;
        pl->relax_bytes += (double)h.L * h.V * (double)h.S * (8 + 8 + (pl->keep_marks ? 1 : 0));
    }
}

// The host copy of the per-group tables: one record per (instance, layer), and what a fused launch needs --
// slots per XCD, the runs of layers that share a launch, the occupancy cap of each.
void PlanBuilder::build_group_tables()
{
    // grid.y of a launch; GALVATRON_DP_MAX_GRID_ROWS lowers it (test aid: splits launches of small cases)
    int max_grid_rows = 65535;
    if (const char *e = getenv("GALVATRON_DP_MAX_GRID_ROWS")) max_grid_rows = std::min(65535, std::max(1, atoi(e)));
    for (auto &g : pl->groups) {
        GdpSched *sc = &g.sched;
        // the per-(instance, layer) records; entries of layers an instance does not have stay zero but for hi
        GdpDevLayer *lay = reinterpret_cast<GdpDevLayer *>(stage.data() + g.off_lay);
        sc->lay = reinterpret_cast<const GdpDevLayer *>(pl->dbase + g.off_lay);
        g.live_blocks.assign((size_t)g.max_L, 0);
        for (int k = 0; k < g.count; ++k) {
            const HostInst &h = inst[(size_t)(g.first + k)];
            const gdp_problem *q = p[h.orig];
            const GdpDevInst &d = di[g.first + k];
            const int rows = h.SU + GDP_SRC_PAD;
            for (int l = 0; l < g.max_L; ++l) {
                GdpDevLayer &y = lay[(size_t)k * g.max_L + l];
                y.hi = -1;
                if (l >= h.L) continue;
                const int mat = h.matrix(q, l);
                y.src = d.H + (int64_t)(l % h.nbuf) * d.hstride;
                y.dst = d.H + (int64_t)((l + 1) % h.nbuf) * d.hstride + h.P;
                y.ro = d.roff + (int64_t)l * rows;
                memcpy(y.ro_head, reinterpret_cast<const int64_t *>(stage.data() + h.off_roff) + (size_t)l * rows,
                       sizeof(y.ro_head));
                y.it = d.inter + (int64_t)mat * rows * h.SP;
                y.ia = d.intra + (int64_t)l * h.SP;
                y.m = d.M ? d.M + (int64_t)l * h.S * h.ldm : nullptr;
                y.ld = h.ld; y.ldm = h.ldm;
                y.S = h.S; y.SU = h.SU; y.SP = h.SP; y.ntile = h.ntile;
                y.gate = 0;
                if (pl->flow_ready && l >= 1)
                    for (int part = 0; part < g.latency; ++part) {
                        int best_s = 0, best_m = INT32_MAX;
                        for (int u = 0; u < g.flow_nsrc; ++u) {
                            const int s2 = part * g.flow_nsrc + u;
                            if (s2 >= h.S) break;
                            const int m = q->mem[(size_t)(l - 1) * h.S + s2];
                            if (m < h.V && m < best_m) { best_m = m; best_s = u; }
                        }
                        y.gate |= (uint32_t)best_s << (8 * part);
                    }
                y.fill_from = fill_from_of(g.first + k, l);
                y.dep = h_band[(size_t)(g.first + k)][3 * (size_t)l];
                if ((int64_t)h_band[(size_t)(g.first + k)][3 * (size_t)l + 1] * (64 * GDP_VARIANTS[h.variant].r) > y.fill_from)
                    g.any_fill = true;
                y.lo = h_band[(size_t)(g.first + k)][3 * (size_t)l + 1];
                y.hi = h_band[(size_t)(g.first + k)][3 * (size_t)l + 2];
                if (y.hi >= y.lo)
                    g.flow_blocks = std::max<int>(g.flow_blocks, (int)(((int64_t)(y.hi - y.lo + 1) * g.ntb * std::max(g.latency, 1) +
                                                                         GDP_WAVES_PER_BLOCK - 1) / GDP_WAVES_PER_BLOCK));
                if (y.hi >= y.lo)
                    g.live_blocks[(size_t)l] += ((int64_t)(y.hi - y.lo + 1) * g.ntb + GDP_WAVES_PER_BLOCK - 1) /
                                                GDP_WAVES_PER_BLOCK;
            }
        }
        sc->cnt = reinterpret_cast<int32_t *>(pl->dbase + g.off_cnt);
        sc->abort_flag = reinterpret_cast<int32_t *>(pl->dbase + pl->off_abort);
        sc->n_active = reinterpret_cast<const int32_t *>(pl->dbase + g.off_active);
        sc->max_L = g.max_L; sc->max_ntile = g.max_ntile; sc->ntb = g.ntb;
        sc->group = g.xcd_group;
        if (!pl->keep_marks) {
            // Costs only: a fused launch holds the block tasks of the bands alone (the rows below a
            // band are filled once, below; the rows above it are never read).  Slots per XCD: the widest
            // band of the group, counted in groups of whole tiles from the group its first tile is in.
            int64_t widest = 1;
            for (int k = 0; k < g.count; ++k) {
                const HostInst &h = inst[(size_t)(g.first + k)];
                for (int l = 0; l < h.L; ++l) {
                    const int64_t lo = h_band[(size_t)(g.first + k)][3 * (size_t)l + 1];
                    const int64_t hi = h_band[(size_t)(g.first + k)][3 * (size_t)l + 2];
                    if (hi < lo) continue;
                    const int64_t bt_lo = lo * g.ntb / GDP_WAVES_PER_BLOCK;
                    const int64_t bt_hi = ((hi + 1) * g.ntb - 1) / GDP_WAVES_PER_BLOCK;
                    widest = std::max(widest, bt_hi / g.xcd_group - bt_lo / g.xcd_group + 1);
                }
            }
            g.slots = (int)((widest + 7) / 8 * g.xcd_group);
        }
        sc->slots = g.slots;
        sc->spin_limit = 0;   // (set per launch: wait_polls)
        int32_t *act = reinterpret_cast<int32_t *>(stage.data() + g.off_active);
        for (int l = 0; l < g.max_L; ++l) act[l] = g.active[(size_t)l];
        sc->rows = nullptr;
        g.segments.clear();
        if (!g.rows.empty()) {
            // chunked: the grid rows follow the table, at most 65535 per launch
            memcpy(stage.data() + g.off_rows, g.rows.data(), sizeof(int32_t) * g.rows.size());
            sc->rows = reinterpret_cast<const int32_t *>(pl->dbase + g.off_rows);
            const int n_rows = (int)(g.rows.size() / 3);
            for (int r0 = 0; r0 < n_rows; r0 += max_grid_rows)
                g.segments.push_back({r0, std::min(max_grid_rows, n_rows - r0), 0u});
        }
        // Otherwise one fused launch per run of layers with the same number of active instances
        // (grid.y <= 65535); a batch with very many different depths merges the shortest runs into
        // their predecessors.
        for (int l = 0; l < g.max_L && g.rows.empty(); ++l) {
            if (!g.segments.empty() && g.active[(size_t)l] == g.active[(size_t)g.segments.back().first] &&
                g.segments.back().layers < max_grid_rows)
                g.segments.back().layers++;
            else
                g.segments.push_back({l, 1, 0u});
        }
        while (g.segments.size() > 32) {
            size_t best = 1;
            for (size_t i = 1; i < g.segments.size(); ++i)
                if (g.segments[i].layers < g.segments[best].layers) best = i;
            g.segments[best - 1].layers += g.segments[best].layers;
            g.segments.erase(g.segments.begin() + (long)best);
        }
        // Workgroups are dispatched in order, so the ones resident at any time are a window of
        // consecutive ones.  A window wider than the arithmetic of one layer reaches into the next
        // layer, whose workgroups can only wait, and they take the places of ones that could run on
        // CUs that then sit idle.  Dynamic LDS that the kernel never touches holds the number of
        // workgroups per CU to just under (arithmetic-carrying block tasks of an average layer) / CUs,
        // between 2 and the 8 that fit anyway.
        for (auto &seg : g.segments) {
            int64_t sum = 0, grid_rows = seg.layers;
            if (g.rows.empty()) {
                for (int l = seg.first; l < seg.first + seg.layers; ++l) sum += g.live_blocks[(size_t)l];
            } else {  // an average grid row: `chunk` instances of an average (instance, layer)
                int64_t pairs = 0;
                for (int l = 0; l < g.max_L; ++l) { sum += g.live_blocks[(size_t)l]; pairs += g.active[(size_t)l]; }
                sum = sum * g.chunk / std::max<int64_t>(pairs, 1);
                grid_rows = 1;
            }
            // ... and strictly fewer than one layer's worth: with exactly a layer resident, all its workgroups
            // start together, finish together, and the next layer's start together again, each paying the
            // chain of dependent loads at its start with nothing to hide it behind; a narrower window
            // makes layers overlap at their seams (measured, every cell computed, workgroups per CU ->
            // ms: one instance L=32 S=44 V=65536, 4 per layer and CU: 3 -> 0.45, 4 -> 0.57, 5 -> 0.83, no
            // limit 0.70; L=28 S=40 V=29493, 2.25 per layer and CU: 2 -> 0.38, 3 -> 0.55, no limit 0.53).
            const int64_t cus = std::max(pl->num_cu, 1);
            const int64_t per_layer = sum / grid_rows;
            int64_t per_cu = std::max<int64_t>(2, (per_layer + cus - 1) / cus - 1);
            if (pl->occupancy_cap_override >= 1) per_cu = pl->occupancy_cap_override;
            seg.lds_bytes = 0;
            if (per_cu < 8 && pl->lds_per_cu >= 65536 && !pl->no_occupancy_cap)
                seg.lds_bytes = (unsigned)std::min<size_t>(pl->lds_per_cu / (size_t)per_cu - 1024, 65536 - 1024);
            // (split tasks exchange their partial minima through static LDS, which counts towards the same limit)
            const unsigned xch = (unsigned)GDP_SPLIT_LDS_BYTES(GDP_VARIANTS[g.variant].ts);
            if (g.split > 1) seg.lds_bytes = seg.lds_bytes > xch ? seg.lds_bytes - xch : 0u;
        }
    }
}

// The tables onto the device, and the parts of the cost buffers that no run ever overwrites.
int PlanBuilder::upload()
{
    // A flow plan (small): the tables go first, the kernel that prepares the cost buffers needs nothing else;
    // the per-instance inputs follow on a second stream, beside that kernel.
    size_t tables_bytes = small_bytes;
    bool &split_upload = pl->split_upload;
    split_upload = turn_free;
    if (prepared_early) {
        tables_bytes = 0;      // everything over the second stream, beside the kernel that is already running
    } else if (split_upload) {
        for (const auto &h : inst) tables_bytes = std::min(tables_bytes, h.off_inter);
        split_upload = tables_bytes > 0 && tables_bytes < small_bytes;
    }
    if (!prepared_early)
        GDP_HIP(hipMemcpyAsync(pl->dbase, stage.data(), split_upload ? tables_bytes : small_bytes, hipMemcpyHostToDevice,
                               pl->stream));
    if (split_upload) {
        // (the side stream is idle: whatever it last carried was joined to a main stream that has been waited for)
        GDP_HIP(hipMemcpyAsync(pl->dbase + tables_bytes, stage.data() + tables_bytes, small_bytes - tables_bytes,
                               hipMemcpyHostToDevice, pl->lane.side));
        GDP_HIP(hipEventRecord(pl->lane.ev_side, pl->lane.side));
    }
    {   // the parts of the cost buffers that no run ever overwrites
        const GdpDevInst *d_insts = reinterpret_cast<const GdpDevInst *>(pl->dbase + pl->off_insts);
        // A plan laid out for the flow launch gets NaN into its bands here if the turn is free right now (its
        // first run will most likely flow), else when a run first takes that way: a plan that finds the turn
        // taken every time never pays for it.
        const bool nan_bands = split_upload;
        for (const Group &g : pl->groups) {
            if (prepared_early) continue;
            if (!nan_bands)   // (one launch instead of three pays only where the three are short)
                GDP_HIP(gdp_launch_init(d_insts + g.first, g.count, g.max_ld, g.S, g.sched.lay, g.max_L,
                                        64 * GDP_VARIANTS[g.variant].r,
                                        GDP_INIT_PADS | GDP_INIT_ZERO | (pl->keep_marks || !g.any_fill ? 0 : GDP_INIT_FILL),
                                        pl->stream));
            else
                GDP_HIP(gdp_launch_prepare(d_insts + g.first, g.count, g.max_ld, g.S, g.sched.lay, g.max_L,
                                           64 * GDP_VARIANTS[g.variant].r, nan_bands, g.sched.abort_flag, pl->stream));
        }
        pl->flow_clean = nan_bands;
        if (split_upload) GDP_HIP(hipStreamWaitEvent(pl->stream, pl->lane.ev_side, 0));
    }
    // no wait here: the stream orders the upload and these fills before the first run, the host copy
    // stays alive as long as the plan, and an error of theirs is reported by the run
    return GDP_OK;
}

// f0_live: null, or per problem whether its f0 holds anything but zeros (validate_all).
int create(int32_t n, const gdp_problem *const *p, gdp_plan *pl, bool force_marks, const char *f0_live)
{
    PlanBuilder b{n, p, pl, force_marks, f0_live};
    int rc = b.read_presets();
    if (rc == GDP_OK) rc = b.describe_device();
    if (rc != GDP_OK) return rc;
    b.describe_instances();
    rc = b.form_groups();
    if (rc != GDP_OK) return rc;
    b.choose_launch_scheme();
    rc = b.lay_out_tables();
    if (rc == GDP_OK) rc = b.allocate();     // (may ask to start over with the argmin table: GDP_RETRY_WITH_MARKS)
    if (rc == GDP_OK) rc = b.take_stage();
    if (rc != GDP_OK) return rc;
    b.compute_bands();
    rc = b.prepare_early();
    if (rc != GDP_OK) return rc;
    b.build_instance_tables();
    b.build_group_tables();
    pl->scheme_fused = pl->fused;
    pl->scheme_flow = pl->flow;
    pl->wait_bound_s = std::min(WAIT_BOUND_MAX_S, std::max(WAIT_BOUND_MIN_S, WAIT_BOUND_FACTOR * pl->executed / WAIT_BOUND_RATE));
    if (!pl->dry) rc = b.upload();
    pl->inst.swap(b.inst);
    if (rc == GDP_OK && !pl->dry) rc = upload_f0(pl);
    return rc;
}



// ---- audit of a laid-out plan (gdp_debug_check_layout) -----------------------------------------------
// Every address the kernels form from these tables, bounded against the sub-allocation it must stay
// in.  The bounds restate what the kernels touch:
//   relaxation (relax_task, relax_task_lat): source elements src + roff[l][s'] + u, u in [0, ntile * tile
//     rows), s' in [0, SU + GDP_SRC_PAD) (the entries from SU on are the targets of the last prefetches);
//     transition rows it + s' * SP + column, the same s', columns [0, SP); intra ia + [0, SP);
//     destination dst + s * ld + u and argmin m + s * ldm + u, s in [0, S), the same u;
//   fill of the rows below a band: dst-side elements [0, lo * tile rows) of rows [0, S) of buffer l + 1;
//   fused launches: counters cnt + (instance * max_L + layer) * max_ntile + tile;
//   epilogue: H + (L % nbuf) * hstride + roff[L][s] + v0 with v0 in [0, V), the argmin table
//     M + (l * S + s) * ldm + v, v in [0, V), strategy lists res + res_off + [0, L).
// The audit derives every bound on its own, from the plan's shapes and the caller's arrays, and compares it
// with what the builder wrote into the tables: sharing the builder's arithmetic would check nothing.
int audit_bad(const char *what, long long a, long long b, long long c)
{
    char buf[256];
    snprintf(buf, sizeof buf, "layout audit: %s (%lld, %lld, %lld)", what, a, b, c);
    return fail(GDP_E_HIP, buf);
}

long long audit_off(const gdp_plan *pl, const void *q)
{
    return (long long)(reinterpret_cast<uintptr_t>(q) - reinterpret_cast<uintptr_t>(pl->dbase));
}

// The sub-allocations lie inside the allocation and do not overlap.
int audit_sub_allocations(const gdp_plan *pl)
{
    auto bad = audit_bad;
    // sub-allocations: inside the allocation and disjoint
    struct Span { size_t lo, hi; };
    std::vector<Span> spans;
    auto span = [&](size_t lo, size_t bytes) { spans.push_back({lo, lo + bytes}); };
    span(pl->off_insts, sizeof(GdpDevInst) * (size_t)pl->n);
    span(pl->off_keys, sizeof(GdpDevKey) * (size_t)std::max(pl->n_key_total, 1));
    span(pl->off_out, sizeof(GdpDevOut) * (size_t)std::max(pl->n_key_total, 1));
    span(pl->off_res, sizeof(int32_t) * std::max<size_t>(pl->n_res_total, 1));
    span(pl->off_abort, sizeof(int32_t));
    for (const Group &g : pl->groups) {
        span(g.off_active, sizeof(int32_t) * (size_t)g.max_L);
        span(g.off_lay, sizeof(GdpDevLayer) * (size_t)g.count * (size_t)g.max_L);
        span(g.off_rows, sizeof(int32_t) * std::max<size_t>(g.rows.size(), 1));
        span(g.off_cnt, sizeof(int32_t) * (size_t)g.count * g.max_L * g.max_ntile);
    }
    for (const HostInst &h : pl->inst) {
        const size_t rows = (size_t)h.SU + GDP_SRC_PAD;
        if (h.tables_of < 0) {
            span(h.off_inter, sizeof(double) * (size_t)h.n_inter * rows * h.SP);
        } else {
            const int j = h.tables_of;
            if (j < 0 || j >= pl->n) return bad("owner of shared transition matrices", j, pl->n, 0);
            const HostInst &o = pl->inst[(size_t)j];
            if (o.tables_of >= 0 || o.off_inter != h.off_inter || o.n_inter != h.n_inter || o.S != h.S || o.SU != h.SU || o.SP != h.SP)
                return bad("shared transition matrices", j, (long long)o.off_inter, (long long)h.off_inter);
        }
        span(h.off_intra, sizeof(double) * (size_t)h.L * h.SP);
        span(h.off_index, sizeof(int32_t) * (size_t)h.L);
        span(h.off_roff, sizeof(int64_t) * (size_t)(h.L + 1) * rows);
        span(h.off_mem, sizeof(int32_t) * (size_t)h.L * h.S);
        if (h.has_zero) span(h.off_zcols, sizeof(int32_t) * (size_t)h.L * (size_t)(h.S + 1));
        span(h.off_H, sizeof(double) * (size_t)h.nbuf * (size_t)(h.S + 1) * (size_t)h.ld);
        if (pl->keep_marks) span(h.off_M, (size_t)h.L * h.S * (size_t)h.ldm);
    }
    std::sort(spans.begin(), spans.end(), [](const Span &a, const Span &b) { return a.lo < b.lo; });
    for (size_t i = 0; i < spans.size(); ++i) {
        if (spans[i].hi > pl->dbytes) return bad("sub-allocation beyond the allocation", (long long)spans[i].lo, (long long)spans[i].hi, (long long)pl->dbytes);
        if (i && spans[i].lo < spans[i - 1].hi) return bad("sub-allocations overlap", (long long)spans[i - 1].lo, (long long)spans[i - 1].hi, (long long)spans[i].lo);
    }
    return GDP_OK;
}

// Instance records, row offsets, matrix indices and key records.
int audit_instances(const gdp_plan *pl, const gdp_problem *const *p)
{
    auto bad = audit_bad;
    auto off_of = [&](const void *q) { return audit_off(pl, q); };
    const char *stage = pl->stage.data();
    const GdpDevInst *di = reinterpret_cast<const GdpDevInst *>(stage + pl->off_insts);
    const GdpDevKey *dk = reinterpret_cast<const GdpDevKey *>(stage + pl->off_keys);
    for (int i = 0; i < pl->n; ++i) {
        const HostInst &h = pl->inst[(size_t)i];
        const gdp_problem *q = p[h.orig];
        const GdpDevInst &d = di[i];
        const int tile_rows = 64 * GDP_VARIANTS[h.variant].r;
        const long long rows = (long long)h.SU + GDP_SRC_PAD;
        const long long span_u = (long long)h.ntile * tile_rows;      // source rows a launch touches
        const long long buf_elems = (long long)(h.S + 1) * h.ld;
        if (h.SP % GDP_VARIANTS[h.variant].ts || h.SP < h.S || h.SU < h.S) return bad("strategy padding", h.SP, h.SU, h.S);
        if (span_u < h.V || h.ldm < span_u || h.ld < h.P + span_u) return bad("row length", h.ld, h.ldm, span_u);
        if (off_of(d.H) != (long long)h.off_H || d.hstride != buf_elems || d.nbuf != h.nbuf || h.nbuf < 2)
            return bad("cost buffers of the instance record", off_of(d.H), d.hstride, d.nbuf);
        if (off_of(d.inter) != (long long)h.off_inter || off_of(d.intra) != (long long)h.off_intra ||
            off_of(d.inter_index) != (long long)h.off_index || off_of(d.roff) != (long long)h.off_roff ||
            off_of(d.mem) != (long long)h.off_mem || (pl->keep_marks && off_of(d.M) != (long long)h.off_M))
            return bad("table pointers of the instance record", i, 0, 0);
        // row offsets: every source element a task or the epilogue can form stays inside one cost buffer
        const int64_t *ro = reinterpret_cast<const int64_t *>(stage + h.off_roff);
        for (int l = 0; l <= h.L; ++l)
            for (long long s = 0; s < rows; ++s) {
                const long long o = ro[(size_t)l * rows + s];
                if (o < 0 || o + span_u > buf_elems) return bad("row offset leaves the cost buffer", l, s, o);
                // a real strategy reads its own row shifted down by its memory cost, or the +inf row
                if (s < h.S && l > 0) {
                    const int m = q->mem[(size_t)(l - 1) * h.S + s];
                    const long long want = m >= h.V ? (long long)h.S * h.ld + h.P : s * h.ld + h.P - m;
                    if (o != want || (m < h.V && m > h.P)) return bad("row offset of a strategy", l, s, o);
                }
            }
        const int32_t *ix = reinterpret_cast<const int32_t *>(stage + h.off_index);
        for (int l = 0; l < h.L; ++l)
            if (ix[l] < 0 || ix[l] >= h.n_inter) return bad("transition-matrix index", l, ix[l], h.n_inter);
        for (int k = 0; k < h.n_key; ++k) {
            const GdpDevKey &key = dk[h.key_begin + k];
            if (key.inst != i) return bad("instance of a key", i, k, key.inst);
            if (key.res_off < 0 || (size_t)key.res_off + (size_t)h.L > pl->n_res_total) return bad("strategy list of a key", i, k, key.res_off);
            if (key.other_mem < 0) return bad("start row above the table", i, k, (long long)key.other_mem);
        }
    }
    return GDP_OK;
}

// Layer records, bands, and the grids of the three launch schemes.
int audit_groups(const gdp_plan *pl, const gdp_problem *const *p)
{
    auto bad = audit_bad;
    auto off_of = [&](const void *q) { return audit_off(pl, q); };
    const char *stage = pl->stage.data();
    for (const Group &g : pl->groups) {
        const GdpDevLayer *lay = reinterpret_cast<const GdpDevLayer *>(stage + g.off_lay);
        const int tile_rows = 64 * GDP_VARIANTS[g.variant].r;
        if (g.split < 1 || g.ntb % g.split || g.ntb / g.split * GDP_VARIANTS[g.variant].ts != g.SP)
            return bad("target blocks of a group", g.ntb, g.SP, g.split);
        if (g.split > 1)
            for (int k = 0; k < g.count; ++k)
                if (pl->inst[(size_t)(g.first + k)].SU % (GDP_SRC_UNROLL * g.split) || pl->keep_marks ||
                    GDP_VARIANTS[g.variant].r != GDP_SPLIT_R)
                    return bad("sources of a split task", k, pl->inst[(size_t)(g.first + k)].SU, g.split);
        if (off_of(g.sched.lay) != (long long)g.off_lay || off_of(g.sched.cnt) != (long long)g.off_cnt ||
            off_of(g.sched.n_active) != (long long)g.off_active || off_of(g.sched.abort_flag) != (long long)pl->off_abort ||
            g.sched.max_L != g.max_L || g.sched.max_ntile != g.max_ntile)
            return bad("launch record of a group", g.first, 0, 0);
        for (int k = 0; k < g.count; ++k) {
            const HostInst &h = pl->inst[(size_t)(g.first + k)];
            const long long rows = (long long)h.SU + GDP_SRC_PAD;
            if (h.ntile > g.max_ntile || h.L > g.max_L || h.SP != g.SP) return bad("instance against its group", k, h.ntile, h.L);
            for (int l = 0; l < g.max_L; ++l) {
                const GdpDevLayer &y = lay[(size_t)k * g.max_L + l];
                if (l >= h.L) {
                    if (y.hi >= y.lo) return bad("a layer the instance does not have is not empty", k, l, y.hi);
                    continue;
                }
                const long long H0 = (long long)h.off_H, buf_bytes = (long long)sizeof(double) * (h.S + 1) * h.ld;
                const long long src = off_of(y.src) - H0, dst = off_of(y.dst) - H0 - (long long)sizeof(double) * h.P;
                if (src < 0 || src % buf_bytes || src / buf_bytes >= h.nbuf) return bad("source buffer of a layer", k, l, src);
                if (dst < 0 || dst % buf_bytes || dst / buf_bytes >= h.nbuf || dst == src) return bad("destination buffer of a layer", k, l, dst);
                if (src / buf_bytes != l % h.nbuf || dst / buf_bytes != (l + 1) % h.nbuf) return bad("buffer order of a layer", k, l, 0);
                if (off_of(y.ro) != (long long)h.off_roff + (long long)sizeof(int64_t) * l * rows) return bad("row offsets of a layer", k, l, 0);
                const long long mat = (off_of(y.it) - (long long)h.off_inter) / ((long long)sizeof(double) * rows * h.SP);
                if (off_of(y.it) != (long long)h.off_inter + mat * (long long)sizeof(double) * rows * h.SP || mat < 0 || mat >= h.n_inter)
                    return bad("transition matrix of a layer", k, l, mat);
                if (off_of(y.ia) != (long long)h.off_intra + (long long)sizeof(double) * l * h.SP) return bad("intra row of a layer", k, l, 0);
                if (pl->keep_marks ? off_of(y.m) != (long long)h.off_M + (long long)l * h.S * h.ldm : y.m != nullptr)
                    return bad("argmin rows of a layer", k, l, 0);
                if (y.ld != h.ld || y.ldm != h.ldm || y.S != h.S || y.SU != h.SU || y.SP != h.SP || y.ntile != h.ntile)
                    return bad("shape fields of a layer", k, l, 0);
                if (y.lo < 0 || y.lo > h.ntile || y.hi < -1 || y.hi >= h.ntile || y.dep < 0) return bad("band of a layer", y.lo, y.hi, y.dep);
                if ((long long)y.lo * tile_rows > h.ldm) return bad("filled rows beyond a row", k, l, y.lo);
                if (y.fill_from < 0) return bad("first filled row of a layer", k, l, y.fill_from);   // (at or above the band: nothing to fill)
                // What the band of this layer reads of the previous layer's output (rows u - mem[l-1][s'] for
                // every row u of the band): in the pads, in the rows filled once per plan, or -- costs only --
                // in the previous band.  A flow launch waits for every such cell, so each must get written;
                // with the bands not closed (other launch schemes) the rows beyond the previous band belong
                // to lanes whose results nobody reads.
                if (l >= 1 && y.hi >= y.lo && !pl->keep_marks && !h.has_zero) {
                    const GdpDevLayer &prev = lay[(size_t)k * g.max_L + (l - 1)];
                    const gdp_problem *q = p[h.orig];
                    long long mn = -1, mx = -1;
                    for (int s2 = 0; s2 < h.S; ++s2) {
                        const long long m = q->mem[(size_t)(l - 1) * h.S + s2];
                        if (m >= h.V) continue;
                        mn = mn < 0 ? m : std::min(mn, m);
                        mx = std::max(mx, m);
                    }
                    if (mx >= 0) {
                        const long long lowest = (long long)y.lo * tile_rows - mx;
                        const long long highest = (long long)(y.hi + 1) * tile_rows - 1 - mn;
                        if (lowest < -(long long)h.P) return bad("a band reads below the pad", k, l, lowest);
                        if (lowest >= 0 && lowest < prev.fill_from) return bad("a band reads below the filled rows", k, l, lowest);
                        const long long written_to = prev.hi >= prev.lo ? (long long)(prev.hi + 1) * tile_rows : (long long)prev.lo * tile_rows;
                        if (pl->flow_ready && highest >= written_to) return bad("a band of a flow plan reads above the previous band", k, l, highest);
                    }
                }
            }
        }
        for (size_t r = 0; r + 2 < g.rows.size(); r += 3) {
            const int first = g.rows[r], cnt = g.rows[r + 1], layer = g.rows[r + 2];
            if (first < 0 || cnt < 1 || first + cnt > g.count || layer < 0 || layer >= pl->inst[(size_t)(g.first + first)].L)
                return bad("row of a chunked launch", first, cnt, layer);
        }
        for (const auto &seg : g.segments) {
            const long long rows_total = g.rows.empty() ? g.max_L : (long long)(g.rows.size() / 3);
            if (seg.first < 0 || seg.layers < 1 || seg.layers > 65535 || seg.first + seg.layers > rows_total)
                return bad("segment of fused launches", seg.first, seg.layers, rows_total);
            const long long grid_x = 8LL * (g.rows.empty() ? g.active[(size_t)seg.first] : g.chunk) * g.slots;
            if (grid_x < 1 || grid_x > 0x7fffffffLL || g.slots < 1) return bad("grid of a fused launch", grid_x, g.slots, 0);
            if (seg.lds_bytes > 65536u) return bad("dynamic LDS of a fused launch", seg.lds_bytes, 0, 0);
        }
        if (pl->flow_ready) {
            // flow launch: grid = (workgroups of the widest band, layers, instances); a task's row offsets are
            // ro[part * nsrc + u], u < nsrc (inside the SU entries checked below), its cost rows and gate cells
            // the elements a per-layer task reads
            if (g.flow_blocks < 0 || g.max_L > 65535 || g.count > 65535) return bad("grid of a flow launch", g.flow_blocks, g.max_L, g.count);
            bool known = false;
            for (int c : GDP_FLOW_NSRC) known = known || c == g.flow_nsrc;
            if (!known || 2 * g.flow_nsrc > 64) return bad("sources per wave of a flow task", g.flow_nsrc, 0, 0);
        }
        const long long tasks = (long long)g.max_ntile * g.ntb * (g.latency > 1 ? g.latency : 1);
        if (tasks / GDP_WAVES_PER_BLOCK + 16 > 0x7fffffffLL || g.count > 65535) return bad("grid of a per-layer launch", tasks, g.count, 0);
        if (g.latency && (g.latency != 1 && g.latency != 2 && g.latency != 4)) return bad("latency variant", g.latency, 0, 0);
        if (g.latency)
            for (int k = 0; k < g.count; ++k) {
                const int su = pl->inst[(size_t)(g.first + k)].SU;
                if (g.lat_ok && su % (GDP_SRC_UNROLL_LAT * g.latency)) return bad("source padding of the latency variant", k, g.latency, 0);
                if (su % GDP_SRC_UNROLL) return bad("source padding", k, su, 0);
                if (pl->flow_ready && (su != g.flow_nsrc * g.latency || su < g.S)) return bad("sources of a flow task", k, su, g.flow_nsrc);
            }
    }
    return GDP_OK;
}

int audit(const gdp_plan *pl, const gdp_problem *const *p)
{
    if (pl->stage.size() < pl->small_bytes)
        return audit_bad("host copy of the tables is short", (long long)pl->stage.size(), (long long)pl->small_bytes, 0);
    int rc = audit_sub_allocations(pl);
    if (rc == GDP_OK) rc = audit_instances(pl, p);
    if (rc == GDP_OK) rc = audit_groups(pl, p);
    return rc;
}

int run(gdp_plan *pl, int32_t mode, gdp_timing *t);

size_t relax_launches(const gdp_plan *pl)
{
    size_t launches = 0;
    for (const Group &g : pl->groups) launches += pl->fused ? g.segments.size() : pl->run_flow ? 1 : (size_t)g.max_L;
    return launches;
}

// Everything of a run that does not wait: the launches and the copy of the results into the plan's
// page-locked buffer, on the plan's stream.
int run_enqueue(gdp_plan *pl, int32_t mode)
{
    GDP_HIP(hipSetDevice(pl->device));
    const GdpDevInst *d_insts = reinterpret_cast<const GdpDevInst *>(pl->dbase + pl->off_insts);
    const GdpDevKey *d_keys = reinterpret_cast<const GdpDevKey *>(pl->dbase + pl->off_keys);
    GdpDevOut *d_out = reinterpret_cast<GdpDevOut *>(pl->dbase + pl->off_out);
    int32_t *d_res = reinterpret_cast<int32_t *>(pl->dbase + pl->off_res);
    pl->run_flow = false;
    // A plan that gave a waiting launch up runs with one launch per layer -- until the time has passed for which
    // the library avoids such launches after a give-up; then it is armed again with the scheme it was given.
    if (pl->fused_gave_up && !pl->no_fallback && steady_ms() - pl->gave_up_ms >= shared_backoff_ms() && !device_seems_shared()) {
        pl->fused_gave_up = false;
        pl->fused = pl->scheme_fused;
        pl->flow = pl->scheme_flow;
    }
    if (pl->fused && !pl->holds_fused) {
        fused_turn_take();  // until run_finish has waited for the launch
        pl->holds_fused = true;
    } else if (pl->flow && !pl->fused) {
        // (GALVATRON_DP_FLOW_WAIT=1: queue up for the turn like a fused plan does)
        static const bool wait_turn = getenv("GALVATRON_DP_FLOW_WAIT") && atoi(getenv("GALVATRON_DP_FLOW_WAIT")) != 0;
        if (pl->holds_fused) pl->run_flow = true;
        else if (wait_turn) { fused_turn_take(); pl->holds_fused = pl->run_flow = true; }
        else pl->holds_fused = pl->run_flow = fused_turn_try_take();
    }
    const size_t launches = relax_launches(pl);
    if (mode >= 2)
        while (pl->ev_relax.size() < 2 * launches) {
            hipEvent_t e;
            GDP_HIP(hipEventCreate(&e));
            pl->ev_relax.push_back(e);
        }
    if (mode >= 1) GDP_HIP(hipEventRecord(pl->ev_begin, pl->stream));
    {
        // (the poison would cover the rows that are filled once per plan: they are filled again after it)
        const int what = (pl->rezero ? GDP_INIT_ZERO : 0) | (pl->poison ? GDP_INIT_POISON : 0) |
                         (pl->poison && !pl->keep_marks ? GDP_INIT_FILL : 0);
        if (what)
            for (const Group &g : pl->groups)
                GDP_HIP(gdp_launch_init(d_insts + g.first, g.count, g.max_ld, g.S, g.sched.lay, g.max_L,
                                        64 * GDP_VARIANTS[g.variant].r, g.any_fill ? what : (what & ~GDP_INIT_FILL), pl->stream));
        if (pl->rezero) {
            const int rc = upload_f0(pl);
            if (rc != GDP_OK) return rc;
        }
    }
    size_t li = 0;
    auto wait_polls = [&](double poll_s) {
        return pl->spin_limit > 0 ? pl->spin_limit : std::max<int64_t>(1, (int64_t)(pl->wait_bound_s / poll_s));
    };

    if (pl->fused) {
        GDP_HIP(gdp_launch_zero(reinterpret_cast<int32_t *>(pl->dbase + pl->off_zero), (int64_t)pl->zero_words,
                                pl->stream));
        for (const Group &g : pl->groups)
            for (const auto &seg : g.segments) {
                const int grid_x = 8 * (g.rows.empty() ? g.active[(size_t)seg.first] : g.chunk) * g.slots;
                if (mode >= 2) GDP_HIP(hipEventRecord(pl->ev_relax[2 * li], pl->stream));
                GdpSched sched = g.sched;
                sched.spin_limit = wait_polls(POLL_S_FUSED);
                sched.debug_stall = pl->debug_stall ? 1 : 0;
                GDP_HIP(gdp_launch_relax_fused(g.variant, pl->keep_marks, g.split,
                                               sched, grid_x,
                                               seg.first, seg.layers, seg.lds_bytes, pl->stream));
                if (mode >= 2) GDP_HIP(hipEventRecord(pl->ev_relax[2 * li + 1], pl->stream));
                ++li;
            }
    } else if (pl->run_flow) {
        if (!pl->flow_clean)   // (every flow run of a plan that runs again leaves them clean; nothing else does)
            for (const Group &g : pl->groups)
                GDP_HIP(gdp_launch_flow_reset(d_insts + g.first, g.count, g.max_ld, g.S, g.sched.lay, g.max_L,
                                              64 * GDP_VARIANTS[g.variant].r, g.sched.abort_flag, pl->stream));
        for (const Group &g : pl->groups) {
            if (mode >= 2) GDP_HIP(hipEventRecord(pl->ev_relax[2 * li], pl->stream));
            if (g.flow_blocks > 0)
                GDP_HIP(gdp_launch_relax_flow(g.flow_nsrc, g.latency, g.sched.lay, g.max_L, g.count, g.flow_blocks, g.SP, 0, g.max_L,
                                              g.sched.abort_flag, wait_polls(POLL_S_FLOW), pl->debug_stall, pl->stream));
            if (mode >= 2) GDP_HIP(hipEventRecord(pl->ev_relax[2 * li + 1], pl->stream));
            ++li;
        }
    } else {
        for (int l = 0; l < pl->max_L; ++l)
            for (const Group &g : pl->groups) {
                if (l >= g.max_L) continue;
                if (mode >= 2) GDP_HIP(hipEventRecord(pl->ev_relax[2 * li], pl->stream));
                GDP_HIP(gdp_launch_relax(g.variant, pl->keep_marks, pl->keep_marks || !g.lat_ok ? 0 : g.latency,
                                         reinterpret_cast<const GdpDevLayer *>(pl->dbase + g.off_lay), g.max_L,
                                         g.active[(size_t)l], g.max_ntile, g.SP, l, pl->stream));
                if (g.zero_layer[(size_t)l])
                    GDP_HIP(gdp_launch_zero_pass(pl->keep_marks, d_insts + g.first, g.sched.lay, g.max_L,
                                                 64 * GDP_VARIANTS[g.variant].r, g.active[(size_t)l], g.max_V, l, pl->stream));
                if (mode >= 2) GDP_HIP(hipEventRecord(pl->ev_relax[2 * li + 1], pl->stream));
                ++li;
            }
    }
    GDP_HIP(gdp_launch_epilogue(pl->keep_marks, d_insts, d_keys, pl->n_key_total, d_out, d_res, pl->stream));
    if (mode >= 1) GDP_HIP(hipEventRecord(pl->ev_end, pl->stream));
    GDP_HIP(hipMemcpyAsync(pl->lane.back, pl->dbase + pl->off_abort, pl->back_bytes, hipMemcpyDeviceToHost,
                           pl->stream));
    pl->wait_back = false;
    pl->flow_clean = false;
    bool exports = false;   // gdp_plan_fetch then reads the cost buffers: they are cleaned before the next run instead
    for (const HostInst &h : pl->inst) exports = exports || (h.flags & (GDP_EXPORT_F | GDP_EXPORT_MARK));
    if (pl->run_flow && !pl->one_shot && !exports) {
        // NaN again into what the run wrote, behind the results: the caller does not wait for it, the
        // next run on this stream (or the destruction of the plan) does
        GDP_HIP(hipEventRecord(pl->lane.ev_back, pl->stream));
        pl->wait_back = true;
        for (const Group &g : pl->groups)
            GDP_HIP(gdp_launch_flow_reset(d_insts + g.first, g.count, g.max_ld, g.S, g.sched.lay, g.max_L,
                                          64 * GDP_VARIANTS[g.variant].r, g.sched.abort_flag, pl->stream));
        pl->flow_clean = true;
    }
    return GDP_OK;
}

// Waits for what run_enqueue started; repeats the run with one launch per layer if a fused launch gave up.
int run_finish(gdp_plan *pl, int32_t mode, gdp_timing *t)
{
    GDP_HIP(hipSetDevice(pl->device));
    const size_t launches = relax_launches(pl);
    const hipError_t waited = pl->wait_back ? hipEventSynchronize(pl->lane.ev_back) : hipStreamSynchronize(pl->stream);
    if (pl->holds_fused) {
        pl->holds_fused = false;
        fused_turn_give();
    }
    GDP_HIP(waited);
    pl->h_out = reinterpret_cast<const GdpDevOut *>(pl->lane.back + (pl->off_out - pl->off_abort));
    pl->h_res = reinterpret_cast<const int32_t *>(pl->lane.back + (pl->off_res - pl->off_abort));
    // the flag is cleared and written by fused launches only
    const int32_t aborted = (pl->fused || pl->run_flow) ? *reinterpret_cast<const int32_t *>(pl->lane.back) : 0;
    if (aborted) {
        // Not every block of the fused launch was resident (the device is shared) or a wait ran out:
        // nothing of that run is kept; do the same work with one launch per layer instead.
        pl->ran = false;
        pl->fused = false;
        pl->flow = false;
        pl->fused_gave_up = true;
        pl->gave_up_ms = steady_ms();
        // nobody had shortened the waits: something else holds places on the device
        if (pl->spin_limit == 0) g_last_give_up_ms.store(pl->gave_up_ms, std::memory_order_relaxed);
        if (pl->no_fallback)
            return fail(GDP_E_HIP, "fused launch: a bounded wait ran out before its tiles were finished");
        return run(pl, mode, t);
    }
    pl->ran = true;
    if (t) {
        memset(t, 0, sizeof *t);
        t->relaxations = pl->relaxations;
        t->executed = pl->executed;
        t->relax_bytes = pl->relax_bytes;
        t->relax_launches = (int32_t)launches;
        t->fused = pl->fused ? 1 : 0;
        t->flow = pl->run_flow ? 1 : 0;
        if (!pl->groups.empty()) {
            const Group &g0 = pl->groups.front();
            t->tile_ts = GDP_VARIANTS[g0.variant].ts;
            t->tile_r = GDP_VARIANTS[g0.variant].r;
            t->chunk = (pl->fused && g0.chunk < g0.count) ? g0.chunk : 0;
            t->latency_variant = pl->fused || (!pl->run_flow && !g0.lat_ok) ? 0 : g0.latency;
            t->fused_split = pl->fused ? g0.split : 1;
        }
        t->keep_marks = pl->keep_marks ? 1 : 0;
        if (mode >= 1) GDP_HIP(hipEventElapsedTime(&t->total_ms, pl->ev_begin, pl->ev_end));
        if (mode >= 2) {
            float sum = 0;
            for (size_t k = 0; k < launches; ++k) {
                float ms = 0;
                GDP_HIP(hipEventElapsedTime(&ms, pl->ev_relax[2 * k], pl->ev_relax[2 * k + 1]));
                sum += ms;
            }
            t->relax_ms = sum;
        }
    }
    return GDP_OK;
}

int run(gdp_plan *pl, int32_t mode, gdp_timing *t)
{
    const int rc = run_enqueue(pl, mode);
    if (rc != GDP_OK && pl->holds_fused) {  // a launch failed: nothing to wait for
        (void)hipStreamSynchronize(pl->stream);
        pl->holds_fused = false;
        fused_turn_give();
    }
    return rc == GDP_OK ? run_finish(pl, mode, t) : rc;
}

int fetch(gdp_plan *pl, gdp_result *const *r)
{
    if (!pl->ran) return fail(GDP_E_BADARG, "gdp_plan_fetch before gdp_plan_run");
    GDP_HIP(hipSetDevice(pl->device));
    // the run has already copied the outputs into the plan's page-locked buffer
    const GdpDevInst *d_insts = reinterpret_cast<const GdpDevInst *>(pl->dbase + pl->off_insts);
    for (int i = 0; i < pl->n; ++i) {
        const HostInst &h = pl->inst[(size_t)i];
        gdp_result *out = r[h.orig];
        if (!out) return fail(GDP_E_BADARG, "null result");
        if (h.n_key > 0 && (!out->total || !out->remaining || !out->res)) return fail(GDP_E_BADARG, "null result array");
        for (int k = 0; k < h.n_key; ++k) {
            const GdpDevOut &o = pl->h_out[(size_t)(h.key_begin + k)];
            out->total[k] = o.total;
            out->remaining[k] = o.remaining;
            if (o.feasible)
                memcpy(out->res + (size_t)k * h.L, pl->h_res + h.res_begin + (size_t)k * h.L,
                       sizeof(int32_t) * (size_t)h.L);
        }
        if ((h.flags & GDP_EXPORT_F) && out->f_out) {
            double *tmp = nullptr;
            const size_t bytes = sizeof(double) * (size_t)h.V * h.S;
            GDP_HIP(hipMalloc((void **)&tmp, bytes));
            hipError_t e = gdp_launch_export_f(d_insts + i, tmp, h.V, h.S, pl->stream);
            if (e == hipSuccess) e = hipMemcpyAsync(out->f_out, tmp, bytes, hipMemcpyDeviceToHost, pl->stream);
            if (e == hipSuccess) e = hipStreamSynchronize(pl->stream);
            (void)hipFree(tmp);
            if (e != hipSuccess) return fail_hip(e, "export f");
        }
        if ((h.flags & GDP_EXPORT_MARK) && out->mark_out) {
            int32_t *tmp = nullptr;
            const size_t bytes = sizeof(int32_t) * (size_t)h.V * h.S;
            GDP_HIP(hipMalloc((void **)&tmp, bytes));
            hipError_t e = hipSuccess;
            for (int l = 0; l < h.L && e == hipSuccess; ++l) {
                e = gdp_launch_export_mark(d_insts + i, l, tmp, h.V, h.S, pl->stream);
                if (e == hipSuccess)
                    e = hipMemcpyAsync(out->mark_out + (size_t)l * h.V * h.S, tmp, bytes, hipMemcpyDeviceToHost,
                                       pl->stream);
                if (e == hipSuccess) e = hipStreamSynchronize(pl->stream);
            }
            (void)hipFree(tmp);
            if (e != hipSuccess) return fail_hip(e, "export mark");
        }
    }
    return GDP_OK;
}

// A plan for problems that validate_all() has accepted.
int create_checked(int32_t n, const gdp_problem *const *p, const char *f0_live, gdp_plan **out)
{
    *out = nullptr;
    for (int attempt = 0; attempt < 2; ++attempt) {
        gdp_plan *pl = new (std::nothrow) gdp_plan();
        if (!pl) return fail(GDP_E_NOMEM, "plan allocation failed");
        int rc;
        try {
            rc = create(n, p, pl, attempt == 1, f0_live);
        } catch (const std::bad_alloc &) {
            rc = fail(GDP_E_NOMEM, "host allocation failed");
        }
        if (rc == GDP_OK) {
            *out = pl;
            return GDP_OK;
        }
        destroy(pl);
        if (rc != GDP_RETRY_WITH_MARKS || attempt == 1) return rc == GDP_RETRY_WITH_MARKS ? fail(GDP_E_NOMEM, "device memory") : rc;
    }
    return fail(GDP_E_NOMEM, "device memory");
}

}  // namespace

extern "C" {

int gdp_plan_create(int32_t n, const gdp_problem *const *p, gdp_plan **out)
{
    gdp_clear_error();
    if (!out) return fail(GDP_E_BADARG, "null plan pointer");
    *out = nullptr;
    if (n < 1 || !p) return fail(GDP_E_BADARG, "need at least one problem");
    if (n > 65535) return fail(GDP_E_BADARG, "at most 65535 instances per plan");
    try {
        std::vector<char> f0_live;
        const int rc = validate_all(n, p, f0_live);
        if (rc != GDP_OK) return rc;
        return create_checked(n, p, f0_live.data(), out);
    } catch (const std::bad_alloc &) {
        return fail(GDP_E_NOMEM, "host allocation failed");
    }
}

int gdp_plan_run(gdp_plan *plan, int32_t timing_mode, gdp_timing *timing)
{
    gdp_clear_error();
    if (!plan) return fail(GDP_E_BADARG, "null plan");
    return run(plan, timing ? timing_mode : 0, timing);
}

int gdp_plan_fetch(gdp_plan *plan, gdp_result *const *r)
{
    gdp_clear_error();
    if (!plan || !r) return fail(GDP_E_BADARG, "null plan or results");
    return fetch(plan, r);
}

int gdp_plan_set_option(gdp_plan *plan, int32_t option, int64_t value)
{
    gdp_clear_error();
    if (!plan) return fail(GDP_E_BADARG, "null plan");
    switch (option) {
        case GDP_OPT_FUSED:
            if (value != 0 && !plan->can_fuse)
                return fail(GDP_E_BADARG, "plan was laid out for per-layer launches only (two cost buffers, or a memory cost of 0)");
            plan->fused = plan->scheme_fused = value != 0;
            plan->flow = plan->scheme_flow = false;
            plan->fused_gave_up = false;
            return GDP_OK;
        case GDP_OPT_FLOW:
            if (value != 0 && !plan->flow_ready)
                return fail(GDP_E_BADARG, "plan was not laid out for a flow launch (see GALVATRON_DP_FLOW)");
            plan->flow = plan->scheme_flow = value != 0;
            if (plan->flow) plan->fused = plan->scheme_fused = false;
            plan->fused_gave_up = false;
            return GDP_OK;
        case GDP_OPT_POISON:
            plan->poison = value != 0;
            return GDP_OK;
        case GDP_OPT_NO_FALLBACK:
            plan->no_fallback = value != 0;
            return GDP_OK;
        case GDP_OPT_DEBUG_STALL:
            plan->debug_stall = value != 0;
            return GDP_OK;
        case GDP_OPT_SPIN_LIMIT: {
            if (value < 1) return fail(GDP_E_BADARG, "spin limit must be >= 1");
            plan->spin_limit = value;
            return GDP_OK;
        }
        default:
            return fail(GDP_E_BADARG, "unknown option");
    }
}

void gdp_plan_destroy(gdp_plan *plan) { destroy(plan); }

int gdp_debug_check_layout(int32_t n, const gdp_problem *const *p, int32_t num_cu, int64_t lds_per_cu)
{
    gdp_clear_error();
    if (n < 1 || !p) return fail(GDP_E_BADARG, "need at least one problem");
    if (n > 65535) return fail(GDP_E_BADARG, "at most 65535 instances per plan");
    if (num_cu < 1 || lds_per_cu < 0) return fail(GDP_E_BADARG, "bad device description");
    for (int i = 0; i < n; ++i) {
        int rc = gdp_validate(p[i], i);
        if (rc == GDP_OK) rc = gdp_validate_f0(p[i], i, nullptr);
        if (rc != GDP_OK) return rc;
    }
    for (int attempt = 0; attempt < 2; ++attempt) {     // costs only first, then with the argmin table where S allows
        gdp_plan *pl = new (std::nothrow) gdp_plan();
        if (!pl) return fail(GDP_E_NOMEM, "plan allocation failed");
        pl->dry = true;
        pl->dry_num_cu = num_cu;
        pl->dry_lds_per_cu = (size_t)lds_per_cu;
        int rc;
        try {
            rc = create(n, p, pl, attempt == 1, nullptr);   // (initial costs change no address)
            if (rc == GDP_OK) rc = audit(pl, p);
        } catch (const std::bad_alloc &) {
            rc = fail(GDP_E_NOMEM, "host allocation failed");
        }
        destroy(pl);
        if (rc != GDP_OK) return rc;
        bool marks_possible = true;
        for (int i = 0; i < n; ++i) marks_possible = marks_possible && p[i]->S <= GDP_MAX_S_MARKS;
        if (!marks_possible) break;
    }
    return GDP_OK;
}

void gdp_debug_shared_device(int32_t seems_shared)
{
    g_last_give_up_ms.store(seems_shared ? steady_ms() : -1, std::memory_order_relaxed);
}

void gdp_batch_stats_begin(void)
{
    std::lock_guard<std::mutex> lk(g_stats_mu);
    g_stats = gdp_batch_stats();
    g_stats_on = true;
}

int gdp_batch_stats_end(gdp_batch_stats *out)
{
    gdp_clear_error();
    if (!out) return fail(GDP_E_BADARG, "null statistics record");
    std::lock_guard<std::mutex> lk(g_stats_mu);
    g_stats_on = false;
    *out = g_stats;
    return GDP_OK;
}

void gdp_cache_trim(void)
{
    arena_trim(-1);
    lane_trim();
}

// The parts of gdp_solve_batch.  f0_live: per problem, whether its initial costs are to be uploaded.
// scan_f0_late: the initial costs have not been looked at yet -- the batch is one part, and they are looked
// through while the device works on it; *f0_found says afterwards whether any hold more than zeros (or are
// refused: then the return code says so), in which case nothing has been written to the results.
static int solve_parts(int32_t n, const gdp_problem *const *p, gdp_result *const *r, size_t budget, std::vector<char> &f0_live,
                       bool scan_f0_late, bool *f0_found)
{
    int begin = 0, prev_begin = 0;
    gdp_plan *prev = nullptr;
    bool stats = false;
    {
        std::lock_guard<std::mutex> lk(g_stats_mu);
        stats = g_stats_on;
    }
    const int mode = stats ? 1 : 0;   // events around the kernels of every part
    auto finish = [&](gdp_plan *pl) {
        gdp_timing t;
        const int rc = run_finish(pl, mode, stats ? &t : nullptr);
        if (rc == GDP_OK && stats) {
            std::lock_guard<std::mutex> lk(g_stats_mu);
            g_stats.relaxations += t.relaxations;
            g_stats.executed += t.executed;
            g_stats.device_ms += t.total_ms;
            g_stats.instances += pl->n;
            g_stats.parts += 1;
            (t.flow ? g_stats.flow_parts : t.fused ? g_stats.fused_parts : g_stats.per_layer_parts) += 1;
        }
        return rc;
    };
    while (begin < n) {
        int end = begin;
        size_t bytes = 0;
        while (end < n && end - begin < 65535) {
            const size_t b = footprint(p[end]);
            if (end > begin && bytes + b > budget) break;
            bytes += b;
            ++end;
        }
        // The next part is laid out and uploaded, and the constant parts of its cost buffers are filled
        // (on a stream of its own), while the previous part still runs; it is launched as soon as that
        // one has finished, before that one's results are handed out.
        gdp_plan *pl = nullptr;
        int rc = create_checked(end - begin, p + begin, f0_live.data() + begin, &pl);
        int rp = prev ? finish(prev) : GDP_OK;
        if (rc == GDP_OK && rp == GDP_OK) {
            pl->one_shot = true;
            rc = run_enqueue(pl, mode);
            if (rc != GDP_OK && pl->holds_fused) {
                (void)hipStreamSynchronize(pl->stream);
                pl->holds_fused = false;
                fused_turn_give();
            }
        }
        if (prev) {
            if (rp == GDP_OK) rp = fetch(prev, r + prev_begin);
            destroy(prev);
            prev = nullptr;
            if (rc == GDP_OK) rc = rp;
        }
        if (rc != GDP_OK) {
            destroy(pl);
            return rc;
        }
        prev = pl;
        prev_begin = begin;
        begin = end;
    }
    int rs = GDP_OK;
    if (scan_f0_late) {
        rs = validate_f0_all(n, p, f0_live);
        for (char c : f0_live) *f0_found = *f0_found || c != 0;
    }
    int rc = finish(prev);
    if (rs != GDP_OK) rc = rs;
    if (rc == GDP_OK && !*f0_found) rc = fetch(prev, r + prev_begin);
    destroy(prev);
    return rc;
}

int gdp_solve_batch(int32_t n, const gdp_problem *const *p, gdp_result *const *r)
{
    gdp_clear_error();
    if (!r) return fail(GDP_E_BADARG, "null results");
    if (n < 1 || !p) return fail(GDP_E_BADARG, "need at least one problem");
    bool any_f0 = false;
    for (int i = 0; i < n; ++i) {  // all of them first: nothing is written when one is rejected
        const int rc = gdp_validate(p[i], i);
        if (rc != GDP_OK) return rc;
        any_f0 = any_f0 || p[i]->f0 != nullptr;
    }
    // A batch whose cost buffers would take more than GALVATRON_DP_ARENA_MB (default 8192) of device
    // memory is solved in consecutive parts that reuse one allocation: the time to obtain device
    // memory grows with its size, the time to solve a part does not grow faster than its share.
    const size_t budget = std::max<size_t>(env_mb("GALVATRON_DP_ARENA_MB", 8192), (size_t)1 << 20);
    try {
        std::vector<char> f0_live((size_t)n, 0);
        // Initial costs (gdp_problem.f0) are zeros in every call the reference's own code makes, and looking
        // through V x S doubles takes as long as solving a small instance.  A batch of one part is therefore
        // started as if they were zeros and the arrays are looked through while the device works; should one
        // of them hold anything else, that solve is dropped and the batch solved again with them.
        size_t bytes = 0;
        for (int i = 0; i < n && bytes <= budget; ++i) bytes += footprint(p[i]);
        const bool late = any_f0 && n <= 65535 && bytes <= budget;
        if (any_f0 && !late) {
            const int rc = validate_f0_all(n, p, f0_live);
            if (rc != GDP_OK) return rc;
        }
        bool f0_found = false;
        int rc = solve_parts(n, p, r, budget, f0_live, late, &f0_found);
        if (rc == GDP_OK && f0_found) {
            f0_found = false;
            rc = solve_parts(n, p, r, budget, f0_live, false, &f0_found);
        }
        return rc;
    } catch (const std::bad_alloc &) {
        return fail(GDP_E_NOMEM, "host allocation failed");
    }
}

int gdp_solve(const gdp_problem *p, gdp_result *r)
{
    const gdp_problem *pp[1] = {p};
    gdp_result *rr[1] = {r};
    return gdp_solve_batch(1, pp, rr);
}

const char *gdp_last_error(void) { return g_err; }

int gdp_version(void) { return GDP_VERSION; }

int gdp_device_info(char *buf, size_t len)
{
    gdp_clear_error();
    if (!buf || len == 0) return fail(GDP_E_BADARG, "null buffer");
    int dev = 0;
    GDP_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    GDP_HIP(hipGetDeviceProperties(&prop, dev));
    snprintf(buf, len, "%s;%s;%d;%zu", prop.name, prop.gcnArchName, prop.multiProcessorCount,
             (size_t)prop.totalGlobalMem);
    return GDP_OK;
}

}  // extern "C"
