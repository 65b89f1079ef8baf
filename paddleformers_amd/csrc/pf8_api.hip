// pf8_api.hip -- library-wide state: version, thread-local error text, compute-unit budget.
#include "pf8_host.h"

#include <atomic>
#include <cstdio>
#include <cstdlib>

namespace {
thread_local char g_err[512] = "";
std::atomic<int> g_num_cus{0};
constexpr int MAX_DEVICES = 64;
std::atomic<int> g_dev_cus[MAX_DEVICES];   // compute units of each device, 0 = not asked yet
}  // namespace

int pf8_fail(int code, const char* where, const char* msg) {
    snprintf(g_err, sizeof(g_err), "%s: %s", where, msg);
    return code;
}

int pf8_check_launch(const char* where) {
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) return PF8_OK;
    snprintf(g_err, sizeof(g_err), "%s: HIP launch failed: %s", where, hipGetErrorString(e));
    return PF8_ELAUNCH;
}

// compute units of the CURRENT device, asked once per device
static int device_cus() {
    int d = 0;
    if (hipGetDevice(&d) != hipSuccess || d < 0) d = 0;
    const int slot = d % MAX_DEVICES;
    int n = g_dev_cus[slot].load(std::memory_order_relaxed);
    if (n <= 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, d) != hipSuccess || n <= 0) n = 256;
        g_dev_cus[slot].store(n, std::memory_order_relaxed);
    }
    return n;
}
int pf8_effective_cus() {
    const int dev = device_cus(), cap = g_num_cus.load();
    return (cap > 0 && cap < dev) ? cap : dev;
}
bool pf8_cus_capped() {
    const int cap = g_num_cus.load();
    return cap > 0 && cap < device_cus();
}

void pf8_note_once(int id, const char* msg) {
    static std::atomic<uint32_t> raised{0};
    const uint32_t bit = 1u << (id & 31);
    if (raised.fetch_or(bit) & bit) return;
    const char* q = getenv("PF8_QUIET");
    if (q && q[0] == '1') return;
    fprintf(stderr, "pf8: %s\n", msg);
}

extern "C" int pf8_version(void) { return 100; }
extern "C" const char* pf8_last_error(void) { return g_err; }
extern "C" int pf8_set_num_cus(int n) {
    int prev = g_num_cus.exchange(n < 0 ? 0 : n);
    return prev;
}
extern "C" int pf8_get_num_cus(void) { return g_num_cus.load(); }

// experts at least this many 128-row blocks long take the 256x256-tile weight-gradient kernel
static std::atomic<int> g_wgrad_tile256_min_blocks{6};
int pf8_wgrad_tile256_min_blocks() { return g_wgrad_tile256_min_blocks.load(); }
extern "C" int pf8_debug_set_wgrad_tile256_min_blocks(int blocks) { return g_wgrad_tile256_min_blocks.exchange(blocks < 0 ? 0 : blocks); }
extern "C" int pf8_effective_num_cus(void) { return pf8_effective_cus(); }
