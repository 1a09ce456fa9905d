// jl_error.hip — error plumbing of the layer-kernel libraries; linked into each of them, so that each keeps its own last message.
#include "jl_common.h"

static thread_local char g_err[512] = "";

int jl_fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}
int jl_check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return jl_fail(JL_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return JL_OK;
}
extern "C" int jl_version(void) { return JL_VERSION; }
extern "C" const char *jl_last_error(void) { return g_err; }
