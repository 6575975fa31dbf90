// Error reporting, device query and ABI version of libdaxq.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "daxq_common.h"

namespace daxq {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(DAXQ_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return DAXQ_OK;
}

}  // namespace daxq

extern "C" {

int daxq_abi_version(void) { return DAXQ_ABI_VERSION; }

const char* daxq_last_error(void) { return daxq::g_err; }

int daxq_device_info(int device, int* cu_count, int* clock_khz, int* lds_bytes, char* arch, int arch_len) {
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return daxq::fail(DAXQ_ERR_DEVICE, "hipGetDeviceProperties(%d): %s", device, hipGetErrorString(e));
    if (cu_count) *cu_count = prop.multiProcessorCount;
    if (clock_khz) *clock_khz = prop.clockRate;
    if (lds_bytes) *lds_bytes = (int)prop.maxSharedMemoryPerMultiProcessor;
    if (arch && arch_len > 0) {
        strncpy(arch, prop.gcnArchName, (size_t)arch_len - 1);
        arch[arch_len - 1] = 0;
    }
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return daxq::fail(DAXQ_ERR_DEVICE, "device %d is %s; libdaxq is built for gfx950 only", device, prop.gcnArchName);
    return DAXQ_OK;
}

}  // extern "C"
