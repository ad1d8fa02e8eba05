// Version, status strings and the thread-local error message of the C ABI.
#include <stdarg.h>
#include <stdio.h>

#include "ka_common.h"

namespace ka {

static thread_local char g_error[512] = "";

int fail(int status, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return status;
}

int check_hip(hipError_t err, const char *what) {
    if (err == hipSuccess) return KA_OK;
    return fail(KA_ERR_HIP, "%s: %s", what, hipGetErrorString(err));
}

}  // namespace ka

KA_EXPORT const char *ka_version(void) { return "kernel_align_hip 0.4 (gfx950)"; }

KA_EXPORT int ka_abi_revision(void) { return KA_ABI_REVISION; }

KA_EXPORT const char *ka_last_error(void) { return ka::g_error; }

KA_EXPORT const char *ka_status_string(int status) {
    switch (status) {
        case KA_OK: return "KA_OK";
        case KA_ERR_BAD_ARG: return "KA_ERR_BAD_ARG";
        case KA_ERR_UNSUPPORTED: return "KA_ERR_UNSUPPORTED";
        case KA_ERR_WORKSPACE: return "KA_ERR_WORKSPACE";
        case KA_ERR_HIP: return "KA_ERR_HIP";
        default: return "KA_ERR_UNKNOWN";
    }
}
