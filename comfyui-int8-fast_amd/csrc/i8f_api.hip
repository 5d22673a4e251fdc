// Version, status text, per-thread HIP error and the device check shared by all entry points.
#include <atomic>
#include <cstring>

#include "i8f_common.hpp"

namespace i8f {

int &last_hip_error_slot() {
    static thread_local int slot = 0;
    return slot;
}

// 0 = unknown, 1 = gfx950, 2 = something else.  The architecture of a device
// never changes, so this cache is a read-only fact once filled.
static std::atomic<int> g_arch_of_device[64];

int check_device() {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        last_hip_error_slot() = (int)e;
        return I8F_ERR_HIP;
    }
    if (dev < 0 || dev >= 64) return I8F_ERR_DEVICE;
    int st = g_arch_of_device[dev].load(std::memory_order_relaxed);
    if (st == 0) {
        hipDeviceProp_t prop;
        e = hipGetDeviceProperties(&prop, dev);
        if (e != hipSuccess) {
            last_hip_error_slot() = (int)e;
            return I8F_ERR_HIP;
        }
        st = std::strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 2;
        g_arch_of_device[dev].store(st, std::memory_order_relaxed);
    }
    return st == 1 ? I8F_OK : I8F_ERR_DEVICE;
}

}  // namespace i8f

extern "C" int i8f_version(void) { return I8F_VERSION; }

extern "C" const char *i8f_status_string(int status) {
    switch (status) {
    case I8F_OK: return "ok";
    case I8F_ERR_INVALID: return "invalid argument";
    case I8F_ERR_UNSUPPORTED: return "unsupported shape or option";
    case I8F_ERR_HIP: return "HIP runtime error (see i8f_last_hip_error)";
    case I8F_ERR_DEVICE: return "current device is not gfx950";
    default: return "unknown status";
    }
}

extern "C" int i8f_last_hip_error(void) { return i8f::last_hip_error_slot(); }
