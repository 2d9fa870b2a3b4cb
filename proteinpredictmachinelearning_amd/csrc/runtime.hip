// Device selection, error text and the per-shape call statistics of the backend.
#include "common.hpp"

#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>

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

// Mirrors mulmat_stats_record (include/ppml/MulMatStats.h:154-169): a histogram keyed by shape,
// switched on by PPML_MULMAT_STATS=1.  Only call counts are kept; kernel times come from rocprof.
static std::mutex g_stats_mtx;
static std::map<uint64_t, int64_t> g_stats;

static bool stats_enabled() {
    static const bool on = [] {
        const char* e = std::getenv("PPML_MULMAT_STATS");
        return e && e[0] && e[0] != '0';
    }();
    return on;
}

void stats_record(int64_t M, int64_t K, int64_t N) {
    if (!stats_enabled()) return;
    const uint64_t key = (static_cast<uint64_t>(M) << 40) | (static_cast<uint64_t>(K) << 20) | static_cast<uint64_t>(N);
    std::lock_guard<std::mutex> lock(g_stats_mtx);
    ++g_stats[key];
}

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
    return RC_OK;
}

extern "C" int ppml_hip_synchronize(void) {
    const hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) { set_error("ppml_hip_synchronize: %s", hipGetErrorString(e)); return RC_LAUNCH; }
    return RC_OK;
}

extern "C" int ppml_hip_mulmat_stats(int64_t* rows, int cap) {
    std::lock_guard<std::mutex> lock(g_stats_mtx);
    int i = 0;
    for (const auto& kv : g_stats) {
        if (rows && i < cap) {
            rows[4 * i + 0] = static_cast<int64_t>(kv.first >> 40);
            rows[4 * i + 1] = static_cast<int64_t>((kv.first >> 20) & 0xfffff);
            rows[4 * i + 2] = static_cast<int64_t>(kv.first & 0xfffff);
            rows[4 * i + 3] = kv.second;
        }
        ++i;
    }
    return i;
}
