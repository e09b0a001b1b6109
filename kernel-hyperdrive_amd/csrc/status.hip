// Status strings and ABI version of the C interface.
#include "ck_device.h"

extern "C" const char* ck_status_string(int status) {
    switch (status) {
        case CK_OK: return "ok";
        case CK_ERR_DTYPE: return "unsupported dtype";
        case CK_ERR_SHAPE: return "unsupported size or stride";
        case CK_ERR_NULL: return "required pointer is NULL";
        case CK_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
        case CK_ERR_LAUNCH: return "kernel launch failed";
        case CK_ERR_ALIGN: return "pointer not aligned to its element size";
        case CK_ERR_SCRATCH: return "problem too large for the library's built-in scratch buffer";
        case CK_ERR_RUNTIME: return "HIP runtime query failed";
        default: return "unknown status";
    }
}

extern "C" int ck_abi_version(void) { return 3; }
