// mxq_common.hip — status strings, version, last-error slot.
#include "mxq_host.h"

namespace mxq {
thread_local int g_last_hip_error = 0;
}

extern "C" {

const char* mx_status_string(int status) {
    switch (status) {
        case MX_OK: return "ok";
        case MX_ERR_NULL: return "required pointer is NULL";
        case MX_ERR_SHAPE: return "dimension violates a precondition";
        case MX_ERR_ALIGN: return "pointer violates the required alignment";
        case MX_ERR_LAUNCH: return "HIP runtime error";
        case MX_ERR_UNSUPPORTED: return "combination not built";
        case MX_ERR_IO: return "file could not be opened or mapped";
        case MX_ERR_FORMAT: return "file violates its format";
        case MX_ERR_NOT_FOUND: return "no entry of that name";
        case MX_ERR_WORKSPACE: return "workspace smaller than this launch needs (see the *_ws_bytes query)";
    }
    return "unknown status";
}

int mx_last_hip_error(void) { return mxq::g_last_hip_error; }

int mx_version(void) { return 110; }

int mx_init(void) {
    if (int rc = mxq::gemv_init_device()) return rc;
    return mxq::gemm_init_device();
}

}  // extern "C"
