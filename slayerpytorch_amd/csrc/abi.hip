// Library-level entry points of libslayer_hip: version, status text, error bookkeeping.
#include "common.h"

#include <atomic>

namespace slayer {

static thread_local char g_last_error[256] = "";
static std::atomic<int> g_force_generic{0};

int note_hip_error(hipError_t err)
{
    if (err == hipSuccess) return SLAYER_OK;
    const char *text = hipGetErrorString(err);
    int i = 0;
    for (; text && text[i] && i < 255; ++i) g_last_error[i] = text[i];
    g_last_error[i] = '\0';
    return SLAYER_ELAUNCH;
}

int compute_units()
{
    int device = 0, cus = 0;
    if (hipGetDevice(&device) != hipSuccess) return 256;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0)
        return 256;
    return cus;
}

bool generic_forced() { return g_force_generic.load(std::memory_order_relaxed) != 0; }

}  // namespace slayer

extern "C" int slayer_hip_abi_version(void) { return SLAYER_HIP_ABI_VERSION; }

extern "C" const char *slayer_status_string(int status)
{
    switch (status) {
        case SLAYER_OK: return "ok";
        case SLAYER_EINVAL: return "invalid argument";
        case SLAYER_EUNSUPPORTED: return "size not supported";
        case SLAYER_ELAUNCH: return "HIP launch failed";
        default: return "unknown status";
    }
}

extern "C" const char *slayer_last_hip_error(void) { return slayer::g_last_error; }

extern "C" int slayer_force_generic_kernels(int on)
{
    return slayer::g_force_generic.exchange(on ? 1 : 0);
}
