// Launching threads for small reductions (opt-in, off by default).
//
// The runtime's kernel-launch path costs 2.4 - 3.0 us per launch on one host thread, and that is
// what a loop of Reduce(...)(row, res=slot, stream=s) calls waits for; from several host threads
// the launches run side by side (4096 launches over four streams: 2.6 - 3.1 us per call from one
// thread, 0.9 us issued / 1.9 us finished with a thread per stream).  With nbh_launch_threads(1)
// nbh_reduce_queued() hands the launch to a thread that belongs to the stream and returns:
//   * one queue and one thread per stream, so launches keep the order of the calls;
//   * every entry point of this library that takes a stream waits until that stream's queue
//     has been launched before it goes on (nbh_hip_stream() in common.h), and everything that
//     concerns the whole device - the default streams, synchronous copies, releasing memory,
//     device synchronisation - waits for all queues (nbh_queue_drain(0));
//   * a launch that fails is reported by the next nbh_stream_synchronize of its stream.
// WHAT IT CANNOT COVER: code outside this library that was handed the stream (through
// __cuda_array_interface__ or an external-stream wrapper) does not know about the queue; a
// caller who mixes the two must call nbh_stream_synchronize or nbh_queue_drain first.  Hence
// opt-in.  The default streams (0, legacy, per-thread) are never queued.
// A forked child has none of the threads and may hold a copy of a locked lock: a
// pthread_atfork handler empties the child's list of queues and switches the feature off
// there, so that no entry point waits for a thread that does not exist.  At the end of a
// process nbh_launch_threads(-1) (called by the Python layer from an exit hook, before the
// runtime's own exit handlers run) launches what is queued and joins the threads; the static
// destructor below only catches what was never stopped that way.
#include "common.h"

#include <atomic>
#include <condition_variable>
#include <cstring>
#include <mutex>
#include <thread>
#include <vector>

#include <new>

#include <pthread.h>
#include <unistd.h>

std::atomic<int> nbh_queue_in_use{0};

namespace {

struct Job {
    int op, dtype;
    const void *in;
    int64_t n, stride;
    alignas(16) unsigned char init[16];
    void *out, *scratch;
    size_t scratch_bytes;
};

constexpr uint64_t kRing = 1024;  // jobs a queue holds before the caller has to wait
constexpr int kSpins = 20000;     // polls of an empty queue (some tens of microseconds) before the thread sleeps

struct Lane {
    nbh_stream_t stream = nullptr;
    int device = 0;
    pid_t owner = 0;              // the process that started the thread (a forked child has none)
    bool has_thread = false;      // set once, before the lane is published
    Job ring[kRing];
    std::atomic<uint64_t> pushed{0}, issued{0};
    std::atomic<int> status{0};   // first failure since the last report
    std::atomic<bool> stop{false}, asleep{false};
    std::atomic<bool> direct{false};  // the stream's handle has left the library: launches go straight to the runtime
    std::mutex push_lock;         // several host threads may use one stream
    std::mutex sleep_lock;
    std::condition_variable wake;
    std::thread worker;
};

std::atomic<bool> g_enabled{false};
std::mutex g_lock;               // guards g_lanes
std::vector<Lane *> g_lanes;     // lanes of living streams
std::atomic<uint64_t> g_generation{1};  // bumped whenever g_lanes changes: invalidates the per-thread caches
thread_local bool t_is_launcher = false;

inline void cpu_relax() { __builtin_ia32_pause(); }

size_t item_bytes(int dtype)
{
    switch (dtype) {
    case NBH_I8: case NBH_U8: return 1;
    case NBH_I16: case NBH_U16: case NBH_F16: return 2;
    case NBH_I32: case NBH_U32: case NBH_F32: return 4;
    case NBH_I64: case NBH_U64: case NBH_F64: case NBH_C64: return 8;
    case NBH_C128: return 16;
    default: return 0;
    }
}

void run(Lane *lane)
{
    t_is_launcher = true;
    (void)hipSetDevice(lane->device);
    int idle = 0;
    for (;;) {
        // asked to stop: whoever asks has waited for the queue first (nbh_queue_forget) or is
        // ending the process, when nothing more may be launched
        if (lane->stop.load(std::memory_order_acquire))
            return;
        const uint64_t at = lane->issued.load(std::memory_order_relaxed);
        if (at != lane->pushed.load(std::memory_order_acquire)) {
            const Job &job = lane->ring[at % kRing];
            const int rc = nbh_reduce(job.op, job.dtype, job.in, job.n, job.stride, job.init, job.out, job.scratch,
                                      job.scratch_bytes, lane->stream);
            if (rc) {
                int none = 0;
                lane->status.compare_exchange_strong(none, rc);
            }
            lane->issued.store(at + 1, std::memory_order_release);
            idle = 0;
            continue;
        }
        if (++idle < kSpins) {
            cpu_relax();
            continue;
        }
        std::unique_lock<std::mutex> hold(lane->sleep_lock);
        lane->asleep.store(true);  // sequentially consistent, like the load in push(): one of the two sees the other
        lane->wake.wait(hold, [&] {
            return lane->stop.load() || lane->pushed.load() != lane->issued.load(std::memory_order_relaxed);
        });
        lane->asleep.store(false);
        idle = 0;
    }
}

void rouse(Lane *lane)
{
    if (lane->asleep.load()) {
        std::lock_guard<std::mutex> hold(lane->sleep_lock);
        lane->wake.notify_one();
    }
}

// The lane of a stream, from a small per-thread cache; made (with its thread) on first use.
Lane *lane_of(nbh_stream_t stream, bool make, bool with_thread = true)
{
    struct Cached {
        nbh_stream_t stream;
        Lane *lane;
    };
    thread_local Cached cache[8];
    thread_local uint64_t cache_generation = 0;
    thread_local int cache_next = 0;
    const uint64_t now = g_generation.load(std::memory_order_acquire);
    if (cache_generation != now) {
        for (auto &c : cache)
            c = Cached{nullptr, nullptr};
        cache_generation = now;
    }
    // a cached "no lane" is good too: making a lane bumps the generation
    for (const auto &c : cache)
        if (c.stream == stream && (c.lane || !make))
            return c.lane;
    Lane *found = nullptr;
    {
        std::lock_guard<std::mutex> hold(g_lock);
        for (Lane *l : g_lanes)
            if (l->stream == stream)
                found = l;
        if (!found && make) {
            found = new Lane;
            found->stream = stream;
            found->owner = getpid();
            if (hipGetDevice(&found->device) != hipSuccess)
                found->device = 0;
            found->has_thread = with_thread;
            if (with_thread)
                found->worker = std::thread(run, found);
            else
                found->direct.store(true);
            g_lanes.push_back(found);
            g_generation.fetch_add(1, std::memory_order_release);  // other threads may have cached "no lane"
        }
    }
    if (stream) {  // slot 0..7 in turn; an empty slot is {nullptr, nullptr} and never matches a stream
        cache[cache_next] = Cached{stream, found};
        cache_next = (cache_next + 1) % 8;
    }
    return found;
}

void wait_launched(Lane *lane)
{
    if (lane->owner != getpid() || !lane->has_thread)
        return;  // a forked child, or a lane that never had a thread: nothing is queued
    const uint64_t upto = lane->pushed.load(std::memory_order_acquire);
    if (lane->issued.load(std::memory_order_acquire) >= upto)
        return;
    rouse(lane);
    while (lane->issued.load(std::memory_order_acquire) < upto)
        cpu_relax();
}

void retire(Lane *lane)
{
    if (lane->owner != getpid()) {  // a forked child: the thread does not exist here
        if (lane->worker.joinable())
            lane->worker.detach();
        return;                     // the lane is left behind
    }
    lane->stop.store(true, std::memory_order_release);
    {
        std::lock_guard<std::mutex> hold(lane->sleep_lock);
        lane->wake.notify_one();
    }
    if (lane->worker.joinable())
        lane->worker.join();
    delete lane;
}

// In the child of a fork: forget the queues (their threads are the parent's), take a fresh lock
// in place of one that may have been copied while held, switch the feature off.
void after_fork_in_child()
{
    new (&g_lock) std::mutex;
    new (&g_lanes) std::vector<Lane *>;   // the lanes are left behind: their threads and locks belong to the parent
    g_enabled.store(false, std::memory_order_release);
    nbh_queue_in_use.store(0, std::memory_order_release);
    g_generation.fetch_add(1, std::memory_order_release);
}

void register_fork_handler()
{
    static std::once_flag once;
    std::call_once(once, [] { pthread_atfork(nullptr, nullptr, after_fork_in_child); });
}

// Launch what is queued everywhere, then stop and join every thread.
void stop_all()
{
    std::vector<Lane *> lanes;
    {
        std::lock_guard<std::mutex> hold(g_lock);
        lanes.swap(g_lanes);
        g_generation.fetch_add(1, std::memory_order_release);
    }
    for (Lane *l : lanes) {
        wait_launched(l);
        retire(l);
    }
}

bool is_default_stream(nbh_stream_t s)
{
    return s == nullptr || (hipStream_t)s == hipStreamLegacy || (hipStream_t)s == hipStreamPerThread;
}

// Joins the threads when the library is unloaded or the process ends.  Launches still queued
// at that point are dropped (the runtime may be gone already); nothing here calls into it.
struct AtExit {
    ~AtExit()
    {
        std::vector<Lane *> lanes;
        {
            std::lock_guard<std::mutex> hold(g_lock);
            lanes.swap(g_lanes);
            g_generation.fetch_add(1, std::memory_order_release);
        }
        for (Lane *l : lanes)
            retire(l);
    }
} g_at_exit;

}  // namespace

// Waits until everything queued for `stream` has been launched; a default stream (or 0)
// stands for all streams.  Called by nbh_hip_stream() whenever a queue is in use.
void nbh_queue_drain(nbh_stream_t stream)
{
    if (t_is_launcher)
        return;  // the launching thread resolving its own stream
    if (!is_default_stream(stream)) {
        if (Lane *lane = lane_of(stream, false))
            wait_launched(lane);
        return;
    }
    // with the list locked: a lane leaves it (nbh_queue_forget) before it is deleted.  The
    // launching threads never take this lock.
    std::lock_guard<std::mutex> hold(g_lock);
    for (Lane *l : g_lanes)
        wait_launched(l);
}

// The stream is about to be destroyed: launch what is queued, stop its thread.
void nbh_queue_forget(nbh_stream_t stream)
{
    if (is_default_stream(stream))
        return;
    Lane *lane = nullptr;
    {
        std::lock_guard<std::mutex> hold(g_lock);
        for (size_t i = 0; i < g_lanes.size(); ++i)
            if (g_lanes[i]->stream == stream) {
                lane = g_lanes[i];
                g_lanes.erase(g_lanes.begin() + (long)i);
                break;
            }
        if (lane)
            g_generation.fetch_add(1, std::memory_order_release);
    }
    if (lane) {
        wait_launched(lane);
        retire(lane);
    }
}

// First failure of a queued launch on `stream` since the last call (0: none).
int nbh_queue_take_status(nbh_stream_t stream)
{
    if (is_default_stream(stream))
        return 0;
    Lane *lane = lane_of(stream, false);
    return lane ? lane->status.exchange(0) : 0;
}

extern "C" {

int nbh_launch_threads(int enable)
{
    if (enable < 0) {  // the process is about to end: nothing may be left to the threads
        g_enabled.store(false, std::memory_order_release);
        stop_all();
        return 0;
    }
    if (enable) {
        register_fork_handler();
        nbh_queue_in_use.store(1, std::memory_order_release);
        g_enabled.store(true, std::memory_order_release);
    } else {
        g_enabled.store(false, std::memory_order_release);
        // The threads stay (asleep) until their streams go, and nbh_queue_in_use stays up: a
        // call that read the switch just before it went off may still queue one launch, and
        // the entry points must go on looking for it.
        nbh_queue_drain(nullptr);
    }
    return 0;
}

// The stream's handle is about to be used by code outside the library, which cannot know
// about the queue: launch what is queued, and from now on launch on the calling thread.
int nbh_stream_pin_direct(nbh_stream_t stream)
{
    if (is_default_stream(stream))
        return 0;
    if (!nbh_queue_in_use.load(std::memory_order_acquire) && !g_enabled.load(std::memory_order_acquire)) {
        // nothing has ever been queued; remember the stream all the same, the mode may be switched on later
        register_fork_handler();
        nbh_queue_in_use.store(1, std::memory_order_release);
    }
    Lane *lane = lane_of(stream, true, false);
    if (!lane)
        return 0;
    {
        std::lock_guard<std::mutex> hold(lane->push_lock);
        lane->direct.store(true, std::memory_order_relaxed);
    }
    wait_launched(lane);
    return 0;
}

int nbh_launch_threads_wait(nbh_stream_t stream)
{
    if (nbh_queue_in_use.load(std::memory_order_relaxed))
        nbh_queue_drain(stream);
    return 0;
}

int nbh_reduce_queued(int op, int dtype, const void *in, int64_t n, int64_t in_stride, const void *init, void *out,
                      void *scratch, size_t scratch_bytes, nbh_stream_t stream)
{
    if (!g_enabled.load(std::memory_order_acquire) || is_default_stream(stream) || !in || !init || !out ||
        !scratch || n < 1 || item_bytes(dtype) == 0)
        return nbh_reduce(op, dtype, in, n, in_stride, init, out, scratch, scratch_bytes, stream);
    Lane *lane = lane_of(stream, true);
    if (!lane)
        return nbh_reduce(op, dtype, in, n, in_stride, init, out, scratch, scratch_bytes, stream);
    std::unique_lock<std::mutex> hold(lane->push_lock);
    if (lane->direct.load(std::memory_order_relaxed)) {
        hold.unlock();
        return nbh_reduce(op, dtype, in, n, in_stride, init, out, scratch, scratch_bytes, stream);
    }
    const uint64_t at = lane->pushed.load(std::memory_order_relaxed);
    if (at - lane->issued.load(std::memory_order_acquire) >= kRing) {
        rouse(lane);
        while (at - lane->issued.load(std::memory_order_acquire) >= kRing)
            cpu_relax();
    }
    Job &job = lane->ring[at % kRing];
    job.op = op;
    job.dtype = dtype;
    job.in = in;
    job.n = n;
    job.stride = in_stride;
    std::memcpy(job.init, init, item_bytes(dtype));
    job.out = out;
    job.scratch = scratch;
    job.scratch_bytes = scratch_bytes;
    lane->pushed.store(at + 1);  // sequentially consistent: see run()
    rouse(lane);
    return 0;
}

}  // extern "C"
