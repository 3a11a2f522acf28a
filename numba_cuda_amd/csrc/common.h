// Internal helpers shared by the translation units of libnbhip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

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

// Launching threads (launchq.hip, opt-in): a launch handed to a stream's thread is not in
// the stream yet when the call returns, so whoever is about to put something else into that
// stream waits for its queue first - here, where every entry point turns its stream argument
// into the runtime's.  One relaxed load when the feature has never been switched on.
extern std::atomic<int> nbh_queue_in_use;
void nbh_queue_drain(nbh_stream_t stream);     // a default stream (0 included) stands for all streams
void nbh_queue_forget(nbh_stream_t stream);    // before the stream is destroyed
int nbh_queue_take_status(nbh_stream_t stream);
static inline void nbh_queue_drain_all()
{
    if (nbh_queue_in_use.load(std::memory_order_relaxed))
        nbh_queue_drain(nullptr);
}
static inline hipStream_t nbh_hip_stream(nbh_stream_t s)
{
    if (nbh_queue_in_use.load(std::memory_order_relaxed))
        nbh_queue_drain(s);
    return (hipStream_t)s;
}

// Number of compute units of the current device (cached per device).
int nbh_cu_count();

// The caching pool (pool.hip) must know which streams have had work submitted: every
// entry point that takes a stream reports it (a no-op until the pool is in use).
void nbh_pool_note_stream(hipStream_t stream);
void nbh_pool_forget_stream(hipStream_t stream);
// The report has to come AFTER the work is in the stream's queue (a block freed by
// another thread in between must not be covered by an event recorded too early):
// declare one of these at the top of an entry point and it reports on the way out.
struct nbh_stream_report {
    hipStream_t stream;
    explicit nbh_stream_report(hipStream_t s) : stream(s) {}
    ~nbh_stream_report() { nbh_pool_note_stream(stream); }
    nbh_stream_report(const nbh_stream_report &) = delete;
    nbh_stream_report &operator=(const nbh_stream_report &) = delete;
};

// Large copies between pageable host memory and the device through a
// ring of page-locked buffers and a few copy threads (hostcopy.hip).  0: done;
// -1: not a case for the pipeline, use hipMemcpy; otherwise a hipError_t.
int nbh_staged_d2h(void *dst, const void *src, size_t nbytes, hipStream_t stream);
int nbh_staged_h2d(void *dst, const void *src, size_t nbytes, hipStream_t stream);

// dst[0:nbytes] = src[0:nbytes] with the flat copy kernel of nbh_assign, on `stream`
// (asynchronous).  Both ranges must be memory the current device can address.
int nbh_flat_copy(void *dst, const void *src, int64_t nbytes, hipStream_t stream);

// Sixteen bytes at an address that is only A-byte aligned, moved as one vector:
// global memory takes 128-bit accesses at any alignment, and the under-aligned
// vector type tells the compiler exactly what it may assume.  NT = non-temporal.
typedef uint32_t nbh_u32x4 __attribute__((ext_vector_type(4)));
template <int A> struct nbh_packet;
template <> struct nbh_packet<1> { typedef nbh_u32x4 type __attribute__((aligned(1))); };
template <> struct nbh_packet<2> { typedef nbh_u32x4 type __attribute__((aligned(2))); };
template <> struct nbh_packet<4> { typedef nbh_u32x4 type __attribute__((aligned(4))); };
template <> struct nbh_packet<8> { typedef nbh_u32x4 type __attribute__((aligned(8))); };
template <> struct nbh_packet<16> { typedef nbh_u32x4 type __attribute__((aligned(16))); };
template <int A, bool NT> __device__ __forceinline__ nbh_u32x4 nbh_load16(const void *p)
{
    const typename nbh_packet<A>::type *q = static_cast<const typename nbh_packet<A>::type *>(p);
    if (NT)
        return __builtin_nontemporal_load(q);
    return *q;
}
template <int A, bool NT> __device__ __forceinline__ void nbh_store16(void *p, nbh_u32x4 v)
{
    typename nbh_packet<A>::type *q = static_cast<typename nbh_packet<A>::type *>(p);
    if (NT)
        __builtin_nontemporal_store(v, q);
    else
        *q = v;
}
