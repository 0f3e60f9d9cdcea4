// Status text, thread-local error message and device query of the C ABI.
#include "q8_host.h"
#include <string.h>

namespace q8 {
char* last_error_buf() {
    static thread_local char buf[256] = {0};
    return buf;
}
}  // namespace q8

extern "C" const char* q8_strerror(int status) {
    switch (status) {
        case Q8_OK: return "ok";
        case Q8_ERR_NULL: return "null pointer";
        case Q8_ERR_DTYPE: return "unsupported element type";
        case Q8_ERR_SHAPE: return "unsupported shape";
        case Q8_ERR_ALIGN: return "misaligned pointer or stride";
        case Q8_ERR_LAUNCH: return "kernel launch failed";
        case Q8_ERR_FLAGS: return "unknown flags";
        default: return "unknown status";
    }
}

extern "C" const char* q8_last_error(void) { return q8::last_error_buf(); }

extern "C" int q8_device_info(int* cu_count, int* clock_mhz, int64_t* hbm_bytes, char* arch_name) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) {
        (void)hipGetLastError();
        return q8::fail(Q8_ERR_LAUNCH, "q8_device_info: no HIP device");
    }
    if (cu_count) *cu_count = prop.multiProcessorCount;
    if (clock_mhz) *clock_mhz = prop.clockRate / 1000;
    if (hbm_bytes) *hbm_bytes = (int64_t)prop.totalGlobalMem;
    if (arch_name) {
        strncpy(arch_name, prop.gcnArchName, 31);
        arch_name[31] = 0;
    }
    return Q8_OK;
}
