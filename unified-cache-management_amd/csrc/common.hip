#include "common.h"

namespace ucm {

char* error_buffer()
{
    static thread_local char buf[512] = {0};
    return buf;
}

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

int check_hip(hipError_t e, const char* what)
{
    if (e == hipSuccess) { return UCM_OK; }
    return fail(UCM_EHIP, "%s: %s", what, hipGetErrorString(e));
}

}  // namespace ucm

extern "C" int ucm_version(void) { return 100; }

extern "C" const char* ucm_last_error(void) { return ucm::error_buffer(); }
