// Error reporting, per-device workspace and small utility entry points.
#include "common.h"

#include <mutex>

namespace pxh {

namespace {
thread_local char g_error[512] = "";

struct DeviceScratch {
    void* ptr = nullptr;
    size_t bytes = 0;
};
constexpr int kMaxDevices = 16;
DeviceScratch g_scratch[kMaxDevices];
std::mutex g_scratch_mutex;
}  // namespace

void set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int fail_invalid(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return PXH_ERR_INVALID_ARGUMENT;
}

int check_launch(const char* what)
{
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        set_error("%s: %s", what, hipGetErrorString(err));
        return static_cast<int>(err);
    }
    return PXH_OK;
}

void* library_workspace(size_t bytes)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    DeviceScratch& s = g_scratch[dev];
    if (s.bytes >= bytes && s.ptr) return s.ptr;
    // Grow: work queued on the old buffer must finish before it is released.
    if (s.ptr) {
        if (hipDeviceSynchronize() != hipSuccess) return nullptr;
        (void) hipFree(s.ptr);
        s.ptr = nullptr;
        s.bytes = 0;
    }
    // 16 MB covers every shape of a YOLOv3-sized network, so the buffer rarely grows after the first
    // call (growing synchronises the device, which a call inside a graph capture must not do)
    size_t want = bytes < (16u << 20) ? (16u << 20) : bytes;
    if (hipMalloc(&s.ptr, want) != hipSuccess) {
        s.ptr = nullptr;
        return nullptr;
    }
    s.bytes = want;
    return s.ptr;
}

int resolve_workspace(void* user, size_t user_bytes, size_t need, void** out)
{
    if (user) {
        if (user_bytes < need) {
            set_error("workspace too small: %zu bytes given, %zu needed", user_bytes, need);
            return PXH_ERR_WORKSPACE;
        }
        if (!aligned16(user)) {
            set_error("workspace must be 16-byte aligned");
            return PXH_ERR_WORKSPACE;
        }
        *out = user;
        return PXH_OK;
    }
    void* p = library_workspace(need);
    if (!p) {
        set_error("could not allocate %zu bytes of device workspace", need);
        return PXH_ERR_WORKSPACE;
    }
    *out = p;
    return PXH_OK;
}

}  // namespace pxh

extern "C" {

const char* pxh_last_error(void) { return pxh::g_error; }

int pxh_abi_version(void) { return 1; }

// Host-only check hook for the multiply-high division used by the indexing code.
unsigned pxh_debug_fastdiv(unsigned n, unsigned d)
{
    pxh::FastDiv f(d);
    return f.div(n);
}

}
