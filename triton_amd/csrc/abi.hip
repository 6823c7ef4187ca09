// Library-level entry points: version, status names, device check.
#include "common.h"
#include <string.h>

extern "C" int trn_version(void) { return 100; }  // 0.1.0

extern "C" const char* trn_status_name(int status) {
    switch (status) {
        case TRN_OK: return "TRN_OK";
        case TRN_E_NULL: return "TRN_E_NULL";
        case TRN_E_SHAPE: return "TRN_E_SHAPE";
        case TRN_E_STRIDE: return "TRN_E_STRIDE";
        case TRN_E_ALIGN: return "TRN_E_ALIGN";
        case TRN_E_UNSUPPORTED: return "TRN_E_UNSUPPORTED";
        case TRN_E_LAUNCH: return "TRN_E_LAUNCH";
        case TRN_E_ARCH: return "TRN_E_ARCH";
        default: return "TRN_E_UNKNOWN";
    }
}

extern "C" int trn_check_device(void) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return TRN_E_ARCH;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return TRN_E_ARCH;
    return strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? TRN_OK : TRN_E_ARCH;
}
