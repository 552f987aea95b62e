// Host-side services every entry point uses: the thread's error text, launch checks, the gfx950 check and
// the once-per-kernel LDS attribute; cw_version / cw_last_error / cw_device_arch. Linked into the library
// and into the measurement library (which shares no other object with it).
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <unordered_map>

#include "cw_common.h"

namespace cw {

namespace {
thread_local char g_error[512] = "";
thread_local char g_arch[128] = "";
}  // namespace

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return CW_OK;
    return fail(CW_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
}

namespace {
constexpr int kMaxDevices = 64;
std::atomic<int> g_arch_ok[kMaxDevices];  // 0 = not asked yet, 1 = gfx950, -1 = something else
std::mutex g_lds_mutex;
std::unordered_map<const void*, int> g_lds_limit[kMaxDevices];  // kernel -> largest limit set on that device
}  // namespace

int require_gfx950(const char* who) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0) {
        (void)hipGetLastError();
        return fail(CW_ERR_DEVICE, "%s: no HIP device is current (this library runs on gfx950 only)", who);
    }
    if (dev < kMaxDevices) {
        const int known = g_arch_ok[dev].load(std::memory_order_relaxed);
        if (known == 1) return CW_OK;
    }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
        (void)hipGetLastError();
        return fail(CW_ERR_DEVICE, "%s: cannot query device %d", who, dev);
    }
    const bool ok = strncmp(prop.gcnArchName, "gfx950", 6) == 0;
    if (dev < kMaxDevices) g_arch_ok[dev].store(ok ? 1 : -1, std::memory_order_relaxed);
    if (!ok)
        return fail(CW_ERR_DEVICE, "%s: device %d is %s; this library holds code objects for gfx950 only", who, dev,
                    prop.gcnArchName);
    return CW_OK;
}

int ensure_dynamic_lds(const void* kernel, int bytes, const char* what) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        dev = -1;
    }
    if (dev >= 0) {
        std::lock_guard<std::mutex> lock(g_lds_mutex);
        auto it = g_lds_limit[dev].find(kernel);
        if (it != g_lds_limit[dev].end() && it->second >= bytes) return CW_OK;
    }
    const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(CW_ERR_LAUNCH, "hipFuncSetAttribute(%s, %d bytes of LDS): %s", what, bytes, hipGetErrorString(e));
    }
    if (dev >= 0) {
        std::lock_guard<std::mutex> lock(g_lds_mutex);
        int& slot = g_lds_limit[dev][kernel];
        if (slot < bytes) slot = bytes;
    }
    return CW_OK;
}

}  // namespace cw

using namespace cw;

extern "C" const char* cw_version(void) { return "cubework-hip 0.1.0 (gfx950)"; }

extern "C" const char* cw_last_error(void) { return g_error; }

extern "C" const char* cw_device_arch(void) {
    g_arch[0] = '\0';
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return g_arch;
    }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
        (void)hipGetLastError();
        return g_arch;
    }
    strncpy(g_arch, prop.gcnArchName, sizeof(g_arch) - 1);
    g_arch[sizeof(g_arch) - 1] = '\0';
    return g_arch;
}
