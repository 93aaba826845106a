// Library identity and error strings.
#include "common.h"

extern "C" int om_version(void) { return 100; }  // major*10000 + minor*100 + patch

extern "C" const char *om_arch(void) { return "gfx950"; }

extern "C" const char *om_strerror(int code) {
    switch (code) {
        case OM_OK: return "ok";
        case OM_ERR_NULL: return "a required pointer is NULL";
        case OM_ERR_DTYPE: return "unsupported dtype code for this entry point";
        case OM_ERR_SHAPE: return "sizes violate a documented constraint";
        case OM_ERR_ALIGN: return "pointer or row pitch is not 16-byte aligned";
        case OM_ERR_LAUNCH: return "the HIP runtime rejected a kernel launch";
        case OM_ERR_WORKSPACE: return "workspace too small";
        default: return "unknown error code";
    }
}
