// Host-side helpers of the C-ABI layer: per-thread error text and launch checking.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "trtamd_bert_kernels.h"

namespace trtamd
{

// Stores a printf-style message retrievable through trtamd_last_error() and returns `status`.
int set_error(int status, char const* fmt, ...) __attribute__((format(printf, 2, 3)));

// Status of the launch that was just issued (hipPeekAtLastError semantics of the reference's
// PLUGIN_CHECK(cudaPeekAtLastError()) without terminating the process).
inline int check_launch(char const* what)
{
    hipError_t const e = hipGetLastError();
    if (e != hipSuccess)
    {
        return set_error(TRTAMD_STATUS_FAILURE, "%s: %s", what, hipGetErrorString(e));
    }
    return TRTAMD_STATUS_SUCCESS;
}

inline hipStream_t as_stream(trtamd_stream_t s)
{
    return reinterpret_cast<hipStream_t>(s);
}

inline bool aligned16(void const* p)
{
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

// Tuning switches: kernel variants other than the default choice, selectable with an environment variable (read once
// per process, at the first use of the switch) or, from the tests, with trtamd_test_set_tuning (which wins).  A
// launcher reads a switch once per call and hands the decision down, so a change between two reads cannot split a call.
enum class Tuning : int
{
    kLinearPartialRound = 0, // TRTAMD_LINEAR_PARTIAL_ROUND=<percent>, default 50
    kLinearPersistent,       // TRTAMD_LINEAR_PERSISTENT=0/1, default 1
    kLinearDirect,           // TRTAMD_LINEAR_DIRECT=0/1, default 1
    kLinearPieces,           // TRTAMD_LINEAR_PIECES=<percent>, default 50
    kFmhaGeneric,            // TRTAMD_FMHA_GENERIC=0/1, default 0
    kFmhaQsplit,             // TRTAMD_FMHA_QSPLIT=<n>, default 0 (chosen from the launch size)
    kFmhaRanked,             // TRTAMD_FMHA_RANKED=0/1, default -1 (chosen from the launch size)
    kUnfusedSplit,           // TRTAMD_UNFUSED_SPLIT=0/1, default 0
    kCount
};
int tuning(Tuning which);

// Compute units of the current device, asked once per process (256 when the query fails).
int num_cus();

template <typename T>
constexpr T ceil_div(T a, T b)
{
    return (a + b - 1) / b;
}

} // namespace trtamd
