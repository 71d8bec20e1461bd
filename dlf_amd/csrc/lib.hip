// Library-level entry points: version, status text, last HIP error.
#include "common.hip.h"

namespace dlfx {

static thread_local int g_last_hip_error = 0;

int record_hip_error(hipError_t e) {
    g_last_hip_error = static_cast<int>(e);
    return DLFX_ERR_LAUNCH;
}

}  // namespace dlfx

namespace dlfx {
bool set_scan_tuning(const char* key, int64_t value);
bool set_sort_tuning(const char* key, int64_t value);
bool set_topk_tuning(const char* key, int64_t value);
}

extern "C" int dlfx_set_tuning(const char* key, int64_t value) {
    if (!key) return DLFX_ERR_INVALID_ARGUMENT;
    if (dlfx::set_scan_tuning(key, value) || dlfx::set_sort_tuning(key, value) || dlfx::set_topk_tuning(key, value)) return DLFX_OK;
    return DLFX_ERR_UNKNOWN_OP;
}

extern "C" int dlfx_version(void) { return 100; }

extern "C" int dlfx_last_hip_error(void) { return dlfx::g_last_hip_error; }

extern "C" const char* dlfx_status_string(int status) {
    switch (status) {
    case DLFX_OK: return "ok";
    case DLFX_ERR_INVALID_ARGUMENT: return "invalid argument";
    case DLFX_ERR_UNSUPPORTED_DTYPE: return "unsupported element type for this operation";
    case DLFX_ERR_UNKNOWN_OP: return "unknown operation name";
    case DLFX_ERR_SCRATCH_TOO_SMALL: return "scratch buffer too small";
    case DLFX_ERR_RANK: return "view rank exceeds DLFX_MAX_RANK";
    case DLFX_ERR_LAUNCH: return "HIP launch failed";
    case DLFX_ERR_TOO_LARGE: return "extent too large for this kernel";
    case DLFX_ERR_CAPTURING: return "the first call on a device cannot be recorded into a graph";
    default: return "unknown status";
    }
}
