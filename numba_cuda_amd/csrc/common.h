// Internal helpers shared by the translation units of libnbhip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "nbhip.h"

#define NBH_TRY(expr)                     \
    do {                                  \
        hipError_t nbh_err_ = (expr);     \
        if (nbh_err_ != hipSuccess)       \
            return (int)nbh_err_;         \
    } while (0)

// Reports a failed launch configuration right away; execution faults surface at
// the next synchronisation, as with any asynchronous HIP work.
static inline int nbh_launch_status() { return (int)hipGetLastError(); }

static inline hipStream_t nbh_hip_stream(nbh_stream_t s) { return (hipStream_t)s; }

// Number of compute units of the current device (cached per device).
int nbh_cu_count();

// dst[0:nbytes] = src[0:nbytes] with the flat copy kernel of nbh_assign, on `stream`
// (asynchronous).  Both ranges must be memory the current device can address.
int nbh_flat_copy(void *dst, const void *src, int64_t nbytes, hipStream_t stream);
