// Device context: error bookkeeping and creation/destruction.
#include "ctx.h"

namespace altius {

namespace {
thread_local std::string g_error;
}

void set_global_error(const std::string &msg) { g_error = msg; }
const char *global_error() { return g_error.c_str(); }

int DeviceCtx::fail(int code, const std::string &msg) {
    last_error = msg;
    return code;
}

int DeviceCtx::check(hipError_t e, const char *what) {
    if (e == hipSuccess) return AHIP_OK;
    last_error = std::string(what) + ": " + hipGetErrorString(e);
    return e == hipErrorOutOfMemory ? AHIP_ERR_OOM : AHIP_ERR_HIP;
}

}  // namespace altius
