// pf8_api.hip -- library-wide state: version, thread-local error text, compute-unit budget.
#include "pf8_host.h"

#include <atomic>
#include <cstdio>

namespace {
thread_local char g_err[512] = "";
std::atomic<int> g_num_cus{0};
std::atomic<int> g_dev_cus{-1};
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

int pf8_effective_cus() {
    int dev = g_dev_cus.load();
    if (dev < 0) {
        int d = 0, n = 0;
        if (hipGetDevice(&d) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, d) != hipSuccess || n <= 0)
            n = 256;
        g_dev_cus.store(n);
        dev = n;
    }
    int cap = g_num_cus.load();
    return (cap > 0 && cap < dev) ? cap : dev;
}

extern "C" int pf8_version(void) { return 100; }
extern "C" const char* pf8_last_error(void) { return g_err; }
extern "C" int pf8_set_num_cus(int n) {
    int prev = g_num_cus.exchange(n < 0 ? 0 : n);
    return prev;
}
extern "C" int pf8_get_num_cus(void) { return g_num_cus.load(); }
