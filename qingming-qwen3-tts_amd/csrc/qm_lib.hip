// qm_lib.hip — library identification and error strings of the C ABI.

#include "qm_host.h"

extern "C" int32_t qm_abi_version(void) { return 1; }

extern "C" const char* qm_target_arch(void) { return "gfx950"; }

extern "C" const char* qm_error_string(int32_t code) {
    switch (code) {
        case QM_OK: return "ok";
        case QM_ERR_NULL: return "required pointer is NULL";
        case QM_ERR_GEOMETRY: return "unsupported head/page geometry or misaligned pointer";
        case QM_ERR_SLOT_RANGE: return "cache position beyond the capacity of the page table";
        case QM_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
        case QM_ERR_ARGUMENT: return "invalid argument";
        case QM_ERR_NO_DEVICE: return "no usable gfx950 device";
        default: break;
    }
    if (code <= QM_ERR_HIP_BASE) return hipGetErrorString(static_cast<hipError_t>(QM_ERR_HIP_BASE - code));
    return "unknown error";
}
