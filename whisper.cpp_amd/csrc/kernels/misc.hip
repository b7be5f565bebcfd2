// Library identity and device probing.
#include "common.h"
#include <string.h>

extern "C" int mi355x_abi_version(void) { return 1; }

extern "C" int mi355x_device_is_gfx950(int device) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) != hipSuccess) { (void) hipGetLastError(); return -1; }
    return strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 0;
}

extern "C" const char * mi355x_status_string(int status) {
    switch (status) {
        case MI355X_OK:              return "ok";
        case MI355X_ERR_UNSUPPORTED: return "unsupported type or layout";
        case MI355X_ERR_INVALID:     return "invalid argument";
        case MI355X_ERR_WORKSPACE:   return "workspace missing or too small";
        case MI355X_ERR_HIP:         return "HIP launch error";
        default:                     return "unknown status";
    }
}
