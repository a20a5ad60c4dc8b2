// Error plumbing shared by every C-ABI entry point of libhs_attn.
#include <stdarg.h>
#include <stdio.h>

#include "common.hpp"

namespace hs {

static thread_local char g_last_error[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HS_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
    return HS_OK;
}

}  // namespace hs

extern "C" {

const char *hs_attn_last_error(void) { return hs::g_last_error; }

int hs_attn_abi_version(void) { return HS_ATTN_ABI_VERSION; }

}  // extern "C"
