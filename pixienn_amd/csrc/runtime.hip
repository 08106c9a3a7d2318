// Error reporting, per-device workspace and small utility entry points.
#include "common.h"
#include "pixienn_hip_test.h"

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

// The per-device buffer behind every call that passes no workspace.  A block that has been handed
// out is never freed: work already queued, and graphs that were captured with its address, may still
// use it after a later call has asked for more and been given a larger block.  Growing allocates, so
// it is refused while `stream` is being captured; pxh_reserve_workspace sizes the buffer beforehand.
int library_workspace(size_t bytes, hipStream_t stream, bool may_grow_in_capture, void** out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        set_error("library workspace: no usable current device (%s)", hipGetErrorString(e));
        return PXH_ERR_WORKSPACE;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    DeviceScratch& s = g_scratch[dev];
    if (s.bytes >= bytes && s.ptr) {
        *out = s.ptr;
        return PXH_OK;
    }
    if (!may_grow_in_capture) {
        hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
        // (asking about the null stream while another stream of the thread captures is itself an error of the
        // capture kind: that, too, means no allocation now)
        const hipError_t asked = hipStreamIsCapturing(stream, &status);
        if (asked == hipErrorStreamCaptureImplicit || (asked == hipSuccess && status != hipStreamCaptureStatusNone)) {
            (void) hipGetLastError();
            set_error("the library's workspace holds %zu bytes and this call needs %zu: it cannot grow while the "
                      "stream is being captured; call pxh_reserve_workspace(%zu) before the capture, or pass a "
                      "workspace", s.bytes, bytes, bytes);
            return PXH_ERR_WORKSPACE;
        }
        (void) hipGetLastError();
    }
    // 16 MB covers every shape of a YOLOv3-sized network, so the buffer rarely grows after the first call;
    // when it does it at least doubles, so that the blocks left behind (they are never freed, see above) add up
    // to less than the live one however slowly the requests rise
    size_t want = bytes < (16u << 20) ? (16u << 20) : bytes;
    if (want < 2 * s.bytes) want = 2 * s.bytes;
    void* fresh = nullptr;
    e = hipMalloc(&fresh, want);
    if (e != hipSuccess) {
        set_error("could not allocate %zu bytes of device workspace: %s", want, hipGetErrorString(e));
        return PXH_ERR_WORKSPACE;
    }
    // the outgrown block stays allocated until the process ends (see above)
    s.ptr = fresh;
    s.bytes = want;
    *out = s.ptr;
    return PXH_OK;
}

int resolve_workspace(void* user, size_t user_bytes, size_t need, void** out, hipStream_t stream)
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
    return library_workspace(need, stream, false, out);
}

}  // namespace pxh

extern "C" {

const char* pxh_last_error(void) { return pxh::g_error; }

int pxh_abi_version(void) { return 2; }

int pxh_reserve_workspace(size_t bytes)
{
    // Growing allocates, so this is a call for before a capture.  It takes no stream and cannot ask whether
    // the thread is capturing one (on this runtime the question, put to the null stream, itself invalidates a
    // capture in progress): inside a capture the allocation fails and the failure is reported.
    void* p = nullptr;
    return pxh::library_workspace(bytes, nullptr, true, &p);
}

// Test hook: the address of the current device's library workspace once it holds `bytes`.
void* pxh_debug_library_workspace(size_t bytes)
{
    void* p = nullptr;
    return pxh::library_workspace(bytes, nullptr, true, &p) == PXH_OK ? p : nullptr;
}

// Host-only check hook for the multiply-high division used by the indexing code.
unsigned pxh_debug_fastdiv(unsigned n, unsigned d)
{
    pxh::FastDiv f(d);
    return f.div(n);
}

}
