// Library-wide state of the C-ABI layer: version and the per-thread error text.
#include "host_utils.hpp"

#include <cstring>

namespace trtamd
{
namespace
{
thread_local char gLastError[512] = "";
}

int set_error(int status, char const* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(gLastError, sizeof(gLastError), fmt, ap);
    va_end(ap);
    return status;
}
} // namespace trtamd

extern "C" int trtamd_version(void)
{
    return 100; // 0.1.0
}

extern "C" char const* trtamd_last_error(void)
{
    return trtamd::gLastError;
}
