// Status strings and version of the C ABI.
#include "../../include/hk355.h"

extern "C" const char* hk_status_string(int status) {
    switch (status) {
        case HK_OK: return "ok";
        case HK_ERR_NULL_POINTER: return "null pointer";
        case HK_ERR_BAD_SHAPE: return "bad shape";
        case HK_ERR_BAD_ALIGNMENT: return "pointer not 16-byte aligned";
        case HK_ERR_WORKSPACE: return "workspace missing or too small";
        case HK_ERR_LAUNCH: return "HIP launch error";
        case HK_ERR_UNSUPPORTED: return "unsupported parameters";
        default: return "unknown status";
    }
}

extern "C" int hk_version(void) { return 100; }
