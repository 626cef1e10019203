// Version and status strings of the C ABI.
#include "../../include/diffulex_amd.h"

extern "C" int dfx_abi_version(void) { return DFX_ABI_VERSION; }

extern "C" const char* dfx_status_string(int status) {
    switch (status) {
        case DFX_OK: return "ok";
        case DFX_ERR_INVALID_ARG: return "invalid argument";
        case DFX_ERR_UNSUPPORTED: return "unsupported shape";
        case DFX_ERR_WORKSPACE: return "workspace missing or too small";
        case DFX_ERR_LAUNCH: return "HIP launch failed";
        case DFX_ERR_SCRATCH_LIMIT: return "shape exceeds the static scratch limit";
        default: return "unknown status";
    }
}
