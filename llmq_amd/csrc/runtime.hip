// Host-side support of the C ABI: thread-local error text, device property cache, version strings.
#include <cstdarg>
#include <cstring>
#include <mutex>

#include "common.hpp"

namespace llmq {

static thread_local char tl_error[512] = "";

int set_error(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(tl_error, sizeof(tl_error), fmt, ap);
    va_end(ap);
    return code;
}

int cu_count() {
    static int cached[64];
    static std::mutex mu;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    std::lock_guard<std::mutex> lock(mu);
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

int xcd_count() {
    static int cached[64];
    static std::mutex mu;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 8;
    std::lock_guard<std::mutex> lock(mu);
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeNumberOfXccs, dev) != hipSuccess || n <= 0) n = 8;
        cached[dev] = n;
    }
    return cached[dev];
}

}  // namespace llmq

extern "C" const char* llmq_last_error(void) { return llmq::tl_error; }
extern "C" const char* llmq_version(void) { return "llmq-fp8-gfx950 0.1"; }
extern "C" const char* llmq_target_arch(void) { return "gfx950"; }
