// Library-level services of the C-ABI: version, thread-local error slot, device facts.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "common.h"

namespace mhip {

static thread_local char g_err[512] = {0};

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(MHIP_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return MHIP_OK;
}

int tune_int(const char* name, int fallback) {
    const char* v = getenv(name);
    if (!v || !*v) return fallback;
    char* end = nullptr;
    const long r = strtol(v, &end, 10);
    return (end && *end == 0 && r > 0 && r < (1 << 20)) ? (int)r : fallback;
}

int compute_units() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

}  // namespace mhip

using namespace mhip;

extern "C" const char* mhip_version(void) { return "0.1.0-gfx950"; }

extern "C" const char* mhip_last_error(void) { return g_err; }

extern "C" int mhip_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

extern "C" int mhip_device_info(int device, int* out_cus, int* out_lds_bytes, char* arch,
                                size_t arch_len) {
    if (mhip_device_count() <= device || device < 0)
        return fail(MHIP_ERR_NO_DEVICE, "mhip_device_info: no HIP device %d", device);
    hipDeviceProp_t p;
    hipError_t e = hipGetDeviceProperties(&p, device);
    if (e != hipSuccess) return fail(MHIP_ERR_NO_DEVICE, "hipGetDeviceProperties: %s", hipGetErrorString(e));
    if (out_cus) *out_cus = p.multiProcessorCount;
    if (out_lds_bytes) *out_lds_bytes = (int)p.sharedMemPerBlock;
    if (arch && arch_len) {
        strncpy(arch, p.gcnArchName, arch_len - 1);
        arch[arch_len - 1] = 0;
    }
    return MHIP_OK;
}
