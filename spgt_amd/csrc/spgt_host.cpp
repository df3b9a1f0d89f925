// Error state and version of the C ABI.
#include "spgt_host.h"

#include <atomic>
#include <mutex>
#include <stdio.h>
#include <string.h>
#include <vector>

namespace spgt {

namespace {
thread_local char g_last_error[512] = "";
}

int fail(int code, const char* msg) {
    snprintf(g_last_error, sizeof(g_last_error), "%s", msg);
    return code;
}

int check_launch(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return SPGT_OK;
    snprintf(g_last_error, sizeof(g_last_error), "%s: kernel launch failed: %s", what, hipGetErrorString(e));
    return SPGT_ERR_LAUNCH;
}

int device_cu_count() {
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

bool allow_dynamic_lds(const void* fn, size_t bytes) {
    if (bytes <= 64 * 1024) return true;
    struct Granted {
        int dev;
        const void* fn;
        size_t bytes;
    };
    static std::mutex mu;
    static std::vector<Granted> granted;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return false;
    std::lock_guard<std::mutex> lock(mu);
    for (Granted& g : granted)
        if (g.dev == dev && g.fn == fn) {
            if (g.bytes >= bytes) return true;
            if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) return false;
            g.bytes = bytes;
            return true;
        }
    if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    granted.push_back(Granted{dev, fn, bytes});
    return true;
}

}  // namespace spgt

extern "C" int spgt_version(void) { return 100; }

extern "C" const char* spgt_last_error(void) { return spgt::g_last_error; }
