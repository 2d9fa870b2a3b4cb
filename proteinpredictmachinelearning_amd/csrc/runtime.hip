// Device selection, error text and the per-shape call statistics of the backend.
#include "common.hpp"

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <optional>
#include <string>
#include <tuple>
#include <vector>

namespace ppmlhip {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
}

int check_launch(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return RC_OK;
    set_error("%s: %s", what, hipGetErrorString(e));
    return RC_LAUNCH;
}

// Mirrors the reference's MUL_MAT statistics (include/ppml/MulMatStats.h:39-169 and the event
// fold-in of src/cuda/CUDAKernels.cu:1693-1732): a histogram keyed by (path, M, K, N) with a call
// count and the accumulated milliseconds of the launches, measured with a pair of events recorded on
// the launcher's stream so that nothing waits.  The elapsed times are folded in when the table is
// read or dumped (and at exit).  Switched on by PPML_MULMAT_STATS=1 or ppml_hip_mulmat_stats_enable.
// Unlike the reference's key (20 bits per dimension, MulMatStats.h:70-74) the key keeps whole values.
namespace {

struct StatKey {
    std::string path;
    int64_t M, K, N;
    bool operator<(const StatKey& o) const { return std::tie(path, M, K, N) < std::tie(o.path, o.M, o.K, o.N); }
};
struct StatVal { int64_t calls = 0; double ms = 0.0; };
struct Pending { StatKey key; hipEvent_t e0, e1; };

struct Stats {
    std::mutex mu;
    std::map<StatKey, StatVal> table;
    std::vector<Pending> pending;
    std::vector<hipEvent_t> spare;                     // events to use again
    std::optional<std::chrono::steady_clock::time_point> first_call;   // the clock the report's wall time runs on
};
Stats& stats() {
    static Stats* s = new Stats();                     // never destroyed: the exit handler still reads it
    return *s;
}
std::atomic<int> g_stats_on{-1};

// Elapsed times of finished launches go into the table; with `wait` the unfinished ones are waited for.
void fold_pending_locked(Stats& s, bool wait) {
    size_t keep = 0;
    for (size_t i = 0; i < s.pending.size(); ++i) {
        Pending& p = s.pending[i];
        hipError_t e = wait ? hipEventSynchronize(p.e1) : hipEventQuery(p.e1);
        if (e == hipErrorNotReady) { s.pending[keep++] = p; continue; }
        float ms = 0.0f;
        if (e == hipSuccess && hipEventElapsedTime(&ms, p.e0, p.e1) == hipSuccess) s.table[p.key].ms += ms;
        else (void)hipGetLastError();
        s.spare.push_back(p.e0);
        s.spare.push_back(p.e1);
    }
    s.pending.resize(keep);
}

// The report in two steps: the table folded three ways (whole, per kernel family, per shape by time), then printed.
// Only the look of the lines is shared with the reference's report (include/ppml/MulMatStats.h:86-145): tools that
// grep "[MULMAT-STAT]" keep working.
struct Report {
    struct Line { std::string path; int64_t M = 0, K = 0, N = 0, calls = 0; double ms = 0.0; };
    Line whole;
    std::vector<Line> families;                        // one per path, by name
    std::vector<Line> shapes;                          // one per (path, M, K, N), most device time first
    double wall_ms = 0.0;
};

Report summarise(const Stats& s) {
    Report r;
    if (s.first_call) r.wall_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - *s.first_call).count();
    for (const auto& [key, val] : s.table) {           // the map is ordered by path first
        if (r.families.empty() || r.families.back().path != key.path) r.families.push_back(Report::Line{key.path});
        for (Report::Line* into : {&r.whole, &r.families.back()}) { into->calls += val.calls; into->ms += val.ms; }
        r.shapes.push_back(Report::Line{key.path, key.M, key.K, key.N, val.calls, val.ms});
    }
    std::stable_sort(r.shapes.begin(), r.shapes.end(), [](const Report::Line& a, const Report::Line& b) { return a.ms > b.ms; });
    return r;
}

void print_report(const Report& r, std::FILE* to) {
    constexpr size_t TOP = 12;
    const double share = r.wall_ms > 0.0 ? 100.0 * r.whole.ms / r.wall_ms : 0.0;
    std::fprintf(to, "\n[MULMAT-STAT] ===== MUL_MAT shapes and times (PPML_MULMAT_STATS=1) =====\n");
    std::fprintf(to, "[MULMAT-STAT] total calls=%lld device time=%.3f ms | wall since the first call=%.0f ms (%.1f%%)\n",
                 (long long)r.whole.calls, r.whole.ms, r.wall_ms, share);
    for (const Report::Line& f : r.families)
        std::fprintf(to, "[MULMAT-STAT]   %-24s calls=%-7lld time=%10.3f ms\n", f.path.c_str(), (long long)f.calls, f.ms);
    std::fprintf(to, "[MULMAT-STAT] top shapes by accumulated time (M = output rows, K = contracted, N = output columns):\n");
    size_t rank = 0;
    for (const Report::Line& sh : r.shapes) {
        if (++rank > TOP) break;
        std::fprintf(to, "[MULMAT-STAT]   #%-2zu %-24s M=%-8lld K=%-8lld N=%-8lld calls=%-7lld time=%10.3f ms\n", rank, sh.path.c_str(),
                     (long long)sh.M, (long long)sh.K, (long long)sh.N, (long long)sh.calls, sh.ms);
    }
    std::fprintf(to, "[MULMAT-STAT] ===== end =====\n");
}

void dump_locked(Stats& s) { print_report(summarise(s), stderr); }

void stats_at_exit() {
    Stats& s = stats();
    std::lock_guard<std::mutex> lock(s.mu);
    if (s.table.empty()) return;
    fold_pending_locked(s, true);
    dump_locked(s);
}

}  // namespace

bool stats_enabled() {
    int on = g_stats_on.load(std::memory_order_relaxed);
    if (on < 0) {
        const char* e = std::getenv("PPML_MULMAT_STATS");
        on = (e && e[0] && std::strcmp(e, "0") != 0) ? 1 : 0;      // the reference's rule, MulMatStats.h:39-45
        g_stats_on.store(on, std::memory_order_relaxed);
    }
    return on == 1;
}

StatsScope::StatsScope(const char* path, int64_t M, int64_t K, int64_t N, hipStream_t stream)
    : path_(path), M_(M), K_(K), N_(N), stream_(stream) {
    if (!stats_enabled()) return;
    on_ = true;
    // events cannot be recorded into a stream that is being captured: count the call only
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess) { (void)hipGetLastError(); cap = hipStreamCaptureStatusNone; }
    if (cap != hipStreamCaptureStatusNone) return;
    Stats& s = stats();
    {
        std::lock_guard<std::mutex> lock(s.mu);
        for (hipEvent_t* e : {&e0_, &e1_}) {
            if (!s.spare.empty()) { *e = s.spare.back(); s.spare.pop_back(); }
        }
    }
    if (!e0_ && hipEventCreate(&e0_) != hipSuccess) { (void)hipGetLastError(); e0_ = nullptr; }
    if (!e1_ && hipEventCreate(&e1_) != hipSuccess) { (void)hipGetLastError(); e1_ = nullptr; }
    timed_ = e0_ && e1_ && hipEventRecord(e0_, stream) == hipSuccess;
    if (!timed_) (void)hipGetLastError();
}

StatsScope::~StatsScope() {
    if (!on_) return;
    if (timed_ && hipEventRecord(e1_, stream_) != hipSuccess) { (void)hipGetLastError(); timed_ = false; }
    Stats& s = stats();
    std::lock_guard<std::mutex> lock(s.mu);
    static const bool registered = [] { std::atexit(stats_at_exit); return true; }();
    (void)registered;
    if (!s.first_call) s.first_call = std::chrono::steady_clock::now();
    StatKey key{path_ ? path_ : "unknown", M_, K_, N_};
    ++s.table[key].calls;
    if (timed_) {
        s.pending.push_back(Pending{key, e0_, e1_});
        if (s.pending.size() >= 4096) fold_pending_locked(s, false);
    } else {
        if (e0_) s.spare.push_back(e0_);
        if (e1_) s.spare.push_back(e1_);
    }
}

// Stream-ordered workspace of the launchers that need one (the split planes of the large f32 contractions,
// the partial sums of repeat_back): a pool of this library's own per device, which keeps what it
// has allocated (release threshold at the maximum), so after the first call an allocation is a list
// operation ordered on the caller's stream; freeing is ordered on that stream as well, which makes reuse
// from other streams safe without the library tracking anything.  Returns null when the device has no pool.
hipMemPool_t workspace_pool() {
    constexpr int MAX_DEVICES = 64;
    static std::mutex mu;
    static hipMemPool_t pools[MAX_DEVICES];
    static bool tried[MAX_DEVICES];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) { (void)hipGetLastError(); return nullptr; }
    std::lock_guard<std::mutex> guard(mu);
    if (!tried[dev]) {
        tried[dev] = true;
        hipMemPoolProps props{};
        props.allocType = hipMemAllocationTypePinned;
        props.handleTypes = hipMemHandleTypeNone;
        props.location.type = hipMemLocationTypeDevice;
        props.location.id = dev;
        if (hipMemPoolCreate(&pools[dev], &props) != hipSuccess) {
            (void)hipGetLastError();
            pools[dev] = nullptr;
        } else {
            uint64_t keep = ~0ull;
            (void)hipMemPoolSetAttribute(pools[dev], hipMemPoolAttrReleaseThreshold, &keep);
        }
    }
    return pools[dev];
}

Workspace workspace_take(size_t bytes, hipStream_t stream) {
    Workspace ws;
    if (bytes == 0) return ws;
    // A stream under capture gets no workspace, and nothing here touches the pool for it: an allocation made while the
    // graph is recorded is released again before the graph ever runs, and the recorded kernels would keep its address
    // (a replay then reads and writes memory that is not theirs -- an illegal access on the device).  The caller takes
    // the form of its operation that needs no workspace; mul_mat_tn_noalloc_hip brings the forms that do to recorded code.
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (stream != nullptr && stream != hipStreamPerThread && hipStreamIsCapturing(stream, &capturing) != hipSuccess) {
        (void)hipGetLastError();
        capturing = hipStreamCaptureStatusActive;        // (cannot tell: treat it as the careful case)
    }
    if (capturing != hipStreamCaptureStatusNone) return ws;
    hipMemPool_t pool = workspace_pool();
    if (!pool) return ws;
    if (stream == hipStreamPerThread) {
        // one name for many streams: allocate for this call only
        if (hipMallocFromPoolAsync(reinterpret_cast<void**>(&ws.ptr), bytes, pool, stream) != hipSuccess) { (void)hipGetLastError(); ws.ptr = nullptr; }
        ws.call_owned = ws.ptr != nullptr;
        return ws;
    }
    struct Kept { uint8_t* ptr = nullptr; size_t cap = 0; std::mutex turn; };
    static std::mutex mu;
    static std::map<std::pair<int, hipStream_t>, Kept> kept;       // (nodes of a map stay where they are)
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return ws; }
    Kept* entry;
    {
        std::lock_guard<std::mutex> guard(mu);
        entry = &kept[{dev, stream}];
    }
    Kept& k = *entry;
    k.turn.lock();                                       // until workspace_give()
    if (k.cap < bytes) {
        if (k.ptr && hipFreeAsync(k.ptr, stream) != hipSuccess) (void)hipGetLastError();
        k.ptr = nullptr; k.cap = 0;
        const size_t want = (bytes + (bytes >> 2) + ((1u << 20) - 1)) & ~static_cast<size_t>((1u << 20) - 1);    // a quarter more, whole MiB
        if (hipMallocFromPoolAsync(reinterpret_cast<void**>(&k.ptr), want, pool, stream) == hipSuccess) k.cap = want;
        else { (void)hipGetLastError(); k.ptr = nullptr; }
    }
    ws.ptr = k.ptr;
    if (ws.ptr) ws.turn = &k.turn;
    else k.turn.unlock();
    return ws;
}

void workspace_give(const Workspace& ws, hipStream_t stream) {
    if (ws.call_owned && ws.ptr && hipFreeAsync(ws.ptr, stream) != hipSuccess) (void)hipGetLastError();
    if (ws.turn) static_cast<std::mutex*>(ws.turn)->unlock();
}

// compute units of the device the library first ran on (256 on the part this library is built for)
int device_cu_count() {
    static const int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            n = 256;
        }
        return n;
    }();
    return cus;
}

// which kernel family served the calling thread's last mul_mat_q8 call
static thread_local int g_q8_path = 0;
void set_q8_path(int path) { g_q8_path = path; }

}  // namespace ppmlhip

using namespace ppmlhip;

extern "C" int ppml_hip_abi_version(void) { return PPML_HIP_ABI_VERSION; }

extern "C" const char* ppml_hip_last_error(void) { return g_err; }

extern "C" int ppml_hip_init(int device) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        set_error("ppml_hip_init: no HIP device visible");
        return RC_NO_DEVICE;
    }
    if (device < 0 || device >= n) { set_error("ppml_hip_init: device %d out of range (%d visible)", device, n); return RC_BAD_ARGS; }
    if (hipSetDevice(device) != hipSuccess) { (void)hipGetLastError(); set_error("ppml_hip_init: hipSetDevice(%d) failed", device); return RC_NO_DEVICE; }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) != hipSuccess) { (void)hipGetLastError(); set_error("ppml_hip_init: cannot query device %d", device); return RC_NO_DEVICE; }
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        set_error("ppml_hip_init: device %d is %s, this library holds gfx950 code only", device, prop.gcnArchName);
        return RC_NO_DEVICE;
    }
    // set-up of the entry point that allocates nothing: the address of its static workspace on this device
    return noalloc_scratch_setup(nullptr);
}

extern "C" int ppml_hip_synchronize(void) {
    const hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) { set_error("ppml_hip_synchronize: %s", hipGetErrorString(e)); return RC_LAUNCH; }
    return RC_OK;
}

extern "C" int ppml_hip_mulmat_stats_enable(int on) {
    const int before = stats_enabled() ? 1 : 0;
    if (on == 0 || on == 1) g_stats_on.store(on, std::memory_order_relaxed);
    return before;
}

extern "C" int ppml_hip_mulmat_stats(int64_t* rows, int cap) {
    Stats& s = stats();
    std::lock_guard<std::mutex> lock(s.mu);
    std::map<std::tuple<int64_t, int64_t, int64_t>, int64_t> shapes;      // summed over the paths
    for (const auto& kv : s.table) shapes[std::make_tuple(kv.first.M, kv.first.K, kv.first.N)] += kv.second.calls;
    int i = 0;
    for (const auto& kv : shapes) {
        if (rows && i < cap) {
            rows[4 * i + 0] = std::get<0>(kv.first);
            rows[4 * i + 1] = std::get<1>(kv.first);
            rows[4 * i + 2] = std::get<2>(kv.first);
            rows[4 * i + 3] = kv.second;
        }
        ++i;
    }
    return i;
}

extern "C" int ppml_hip_mulmat_stats_rows(ppml_hip_mulmat_stat* rows, int cap) {
    Stats& s = stats();
    std::lock_guard<std::mutex> lock(s.mu);
    fold_pending_locked(s, true);
    int i = 0;
    for (const auto& kv : s.table) {
        if (rows && i < cap) {
            std::snprintf(rows[i].path, sizeof rows[i].path, "%s", kv.first.path.c_str());
            rows[i].M = kv.first.M; rows[i].K = kv.first.K; rows[i].N = kv.first.N;
            rows[i].calls = kv.second.calls;
            rows[i].ms = kv.second.ms;
        }
        ++i;
    }
    return i;
}

extern "C" void ppml_hip_mulmat_stats_dump(void) {
    Stats& s = stats();
    std::lock_guard<std::mutex> lock(s.mu);
    fold_pending_locked(s, true);
    dump_locked(s);
}

extern "C" void ppml_hip_mulmat_stats_reset(void) {
    Stats& s = stats();
    std::lock_guard<std::mutex> lock(s.mu);
    fold_pending_locked(s, true);
    s.table.clear();
    s.first_call.reset();
}

extern "C" int ppml_hip_q8_last_path(void) { return g_q8_path; }
