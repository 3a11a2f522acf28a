// A caching device-memory pool (host code): nbh_pool_malloc / nbh_pool_free.
//
// hipMalloc + hipFree cost 17 us for a kilobyte and 300 us for 64 MiB on an MI355X
// box, and hipFree waits for the whole device; a 64 MiB transpose takes 25 us.  Code
// that allocates per call (`a.T`, `cuda.to_device` in a loop) spends its time in the
// allocator.  The pool keeps freed blocks and hands them out again.
//
// When is a freed block safe to hand out?  The owner dropped it, but kernels that
// use it may still be queued.  hipFree answers by waiting for the device.  Here every
// entry point of the library that puts work on a stream marks that stream as used
// (nbh_pool_note_stream); when a block is freed, an event is recorded on each stream
// used since its last such event, and the block waits in the pool until those events
// have completed (checked with hipEventQuery when an allocation looks at the block:
// no host-side wait, no device-wide synchronisation).  The legacy default stream is
// treated like any other stream, so an event is recorded on it - which makes it a
// barrier for the blocking streams - only if the caller has been using it anyway.
// Work that reaches a stream WITHOUT passing through this library (another library
// launching on a shared stream) is invisible here: memory handed to such code must be
// kept alive until that work is known to have finished, as with any pooling allocator.
//
// Sizes: multiples of 512 B up to 1 MiB, multiples of 1/8 of the enclosing power of
// two above (at most 12.5 % slack); a request is served by a block of exactly its size
// class.  When hipMalloc runs out of memory, every idle block is returned to the
// driver and the allocation retried once.
#include "common.h"
#include "pool_core.h"

#include <pthread.h>

#include <atomic>
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace {

struct HipBackend {
    using Event = hipEvent_t;
    static bool event_record(Event *out, hipStream_t s)
    {
        hipEvent_t ev = nullptr;
        if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        if (hipEventRecord(ev, s) != hipSuccess) {
            (void)hipGetLastError();
            (void)hipEventDestroy(ev);
            return false;
        }
        *out = ev;
        return true;
    }
    static bool event_done(Event e)
    {
        const hipError_t rc = hipEventQuery(e);
        if (rc == hipSuccess)
            return true;
        if (rc != hipErrorNotReady)
            (void)hipGetLastError();
        return false;
    }
    static void event_destroy(Event e) { (void)hipEventDestroy(e); }
    static void device_synchronize() { (void)hipDeviceSynchronize(); }
    static bool is_per_thread(hipStream_t s) { return s == hipStreamPerThread; }
    static uint64_t thread_id() { return (uint64_t)pthread_self(); }
};
using Tracker = nbh_pool::Tracker<HipBackend, hipStream_t>;

struct Block {
    void *ptr;
    std::vector<Tracker::EventRef> waits;
};

struct DevicePool {
    std::map<size_t, std::vector<Block>> idle;  // size class -> blocks
    std::unordered_map<void *, size_t> live;    // handed out: ptr -> size class
    Tracker tracker;
    size_t idle_bytes = 0, live_bytes = 0;
    uint64_t hits = 0, misses = 0;
};

std::mutex g_mu;
DevicePool g_pools[64];
std::atomic<bool> g_enabled{false};  // set by the first nbh_pool_malloc

using nbh_pool::size_class;

int current_pool(DevicePool **out)
{
    int dev = 0;
    NBH_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64)
        return (int)hipErrorInvalidDevice;
    *out = &g_pools[dev];
    return 0;
}

// hipFree every idle block (they may still be waited on: hipFree itself waits).
void release_idle(DevicePool &p)
{
    for (auto &cls : p.idle)
        for (Block &b : cls.second)
            (void)hipFree(b.ptr);
    p.idle.clear();
    p.idle_bytes = 0;
}

}  // namespace

void nbh_pool_note_stream(hipStream_t stream)
{
    if (!g_enabled.load(std::memory_order_relaxed))
        return;
    DevicePool *p = nullptr;
    if (current_pool(&p))
        return;
    std::lock_guard<std::mutex> lock(g_mu);
    p->tracker.note_stream(stream);
}

void nbh_pool_forget_stream(hipStream_t stream)
{
    if (!g_enabled.load(std::memory_order_relaxed))
        return;
    DevicePool *p = nullptr;
    if (current_pool(&p))
        return;
    std::lock_guard<std::mutex> lock(g_mu);
    p->tracker.forget_stream(stream);  // blocks keep their own references to its events
}

extern "C" {

int nbh_pool_malloc(void **ptr, size_t nbytes)
{
    if (!ptr)
        return (int)hipErrorInvalidValue;
    g_enabled.store(true, std::memory_order_relaxed);
    DevicePool *p = nullptr;
    if (int rc = current_pool(&p))
        return rc;
    const size_t cls = size_class(nbytes);
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = p->idle.find(cls);
    if (it != p->idle.end()) {
        std::vector<Block> &blocks = it->second;
        for (size_t i = blocks.size(); i-- > 0;) {  // most recently freed first
            if (Tracker::ready(blocks[i].waits)) {
                void *got = blocks[i].ptr;
                blocks[i] = std::move(blocks.back());
                blocks.pop_back();
                if (blocks.empty())
                    p->idle.erase(it);
                p->idle_bytes -= cls;
                p->live[got] = cls;
                p->live_bytes += cls;
                ++p->hits;
                *ptr = got;
                return 0;
            }
        }
    }
    ++p->misses;
    void *fresh = nullptr;
    hipError_t e = hipMalloc(&fresh, cls);
    if (e == hipErrorOutOfMemory) {
        (void)hipGetLastError();
        release_idle(*p);
        e = hipMalloc(&fresh, cls);
    }
    if (e != hipSuccess)
        return (int)e;
    p->live[fresh] = cls;
    p->live_bytes += cls;
    *ptr = fresh;
    return 0;
}

int nbh_pool_free(void *ptr)
{
    if (!ptr)
        return 0;
    nbh_queue_drain_all();  // the events recorded below must come after every launch that names the block
    DevicePool *p = nullptr;
    if (int rc = current_pool(&p))
        return rc;
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = p->live.find(ptr);
    if (it == p->live.end())
        return (int)hipErrorInvalidValue;  // not from this device's pool
    const size_t cls = it->second;
    p->live.erase(it);
    p->live_bytes -= cls;
    Block b{ptr, p->tracker.waits_for_a_free()};
    p->idle[cls].push_back(std::move(b));
    p->idle_bytes += cls;
    return 0;
}

int nbh_pool_trim(void)
{
    DevicePool *p = nullptr;
    if (int rc = current_pool(&p))
        return rc;
    std::lock_guard<std::mutex> lock(g_mu);
    release_idle(*p);
    return 0;
}

int nbh_pool_stats(size_t *idle_bytes, size_t *live_bytes, uint64_t *hits, uint64_t *misses)
{
    DevicePool *p = nullptr;
    if (int rc = current_pool(&p))
        return rc;
    std::lock_guard<std::mutex> lock(g_mu);
    if (idle_bytes)
        *idle_bytes = p->idle_bytes;
    if (live_bytes)
        *live_bytes = p->live_bytes;
    if (hits)
        *hits = p->hits;
    if (misses)
        *misses = p->misses;
    return 0;
}

}  // extern "C"
