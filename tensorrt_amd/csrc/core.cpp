// Library-wide state of the C-ABI layer: version, the per-thread error text and the tuning switches.
#include "host_utils.hpp"

#include "trtamd_test_hooks.h"

#include <atomic>
#include <cstdlib>
#include <cstring>
#include <mutex>

namespace trtamd
{
namespace
{
thread_local char gLastError[512] = "";

struct TuningEntry
{
    char const* name;
    int fallback;
};
constexpr TuningEntry kTuning[(int) Tuning::kCount] = {
    {"TRTAMD_LINEAR_PARTIAL_ROUND", 50}, {"TRTAMD_LINEAR_PERSISTENT", 1}, {"TRTAMD_LINEAR_DIRECT", 1},
    {"TRTAMD_LINEAR_PIECES", 50},
    {"TRTAMD_FMHA_GENERIC", 0}, {"TRTAMD_FMHA_QSPLIT", 0}, {"TRTAMD_FMHA_RANKED", -1}, {"TRTAMD_UNFUSED_SPLIT", 0},
};
constexpr int kUnset = INT32_MIN;
std::atomic<int> gTuningOverride[(int) Tuning::kCount];
std::atomic<int> gTuningEnv[(int) Tuning::kCount];
std::once_flag gTuningOnce;

void read_tuning_env()
{
    for (int i = 0; i < (int) Tuning::kCount; ++i)
    {
        char const* e = getenv(kTuning[i].name);
        gTuningEnv[i].store(e ? atoi(e) : kTuning[i].fallback, std::memory_order_relaxed);
        gTuningOverride[i].store(kUnset, std::memory_order_relaxed);
    }
}
} // namespace

int num_cus()
{
    static int const n = [] {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess
            || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        {
            cus = 256;
        }
        return cus;
    }();
    return n;
}

int tuning(Tuning which)
{
    std::call_once(gTuningOnce, read_tuning_env);
    int const o = gTuningOverride[(int) which].load(std::memory_order_relaxed);
    return o != kUnset ? o : gTuningEnv[(int) which].load(std::memory_order_relaxed);
}

namespace
{
int set_tuning(char const* name, int value, bool set)
{
    std::call_once(gTuningOnce, read_tuning_env);
    for (int i = 0; name && i < (int) Tuning::kCount; ++i)
    {
        if (strcmp(name, kTuning[i].name) == 0)
        {
            gTuningOverride[i].store(set ? value : kUnset, std::memory_order_relaxed);
            return TRTAMD_STATUS_SUCCESS;
        }
    }
    return set_error(TRTAMD_STATUS_BAD_PARAM, "unknown tuning switch: %s", name ? name : "(null)");
}
} // namespace

int set_error(int status, char const* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(gLastError, sizeof(gLastError), fmt, ap);
    va_end(ap);
    return status;
}
} // namespace trtamd

extern "C" int trtamd_test_set_tuning(char const* name, int32_t value)
{
    return trtamd::set_tuning(name, value, true);
}

extern "C" int trtamd_test_reset_tuning(char const* name)
{
    return trtamd::set_tuning(name, 0, false);
}

extern "C" int trtamd_version(void)
{
    return 100; // 0.1.0
}

extern "C" char const* trtamd_last_error(void)
{
    return trtamd::gLastError;
}
