// Large copies between PAGEABLE host memory and the device.
//
// hipMemcpy moves pageable memory through one staging buffer with one host thread.
// Measured on an MI355X box (1 GiB): host-to-device 31 GB/s, device-to-host 17.7 GB/s,
// device-to-host into memory that has never been touched (np.empty, what
// copy_to_host() allocates) 10.4 GB/s, while page-locked memory moves at 57 GB/s
// either way and one host thread copies 15 GB/s.  The bus is not the limit, the single
// host thread is.  Here the copy is cut into chunks that travel through a ring of
// page-locked staging buffers: the DMA of one chunk overlaps the host-side copy of
// its neighbours, and the host-side copy (and with it the first touch of fresh
// pages) is shared by a few threads (NBH_HOST_COPY_THREADS, default 8; 0 switches the
// pipeline off).  Result, same box: host-to-device 53 GB/s, device-to-host 50 GB/s,
// also into untouched memory.  Chunks are a quarter of the copy (1 to 16 MiB), so copies
// from a few MiB on gain as well: device-to-host 4 MiB 17 -> 26 GB/s, 16 MiB 18 -> 39 GB/s.
//
// Ordering is hipMemcpy's / hipMemcpyAsync's: the DMA legs are issued on the stream the
// caller names (the legacy default stream when none is named, so that they wait for
// earlier work of every blocking stream), and the call returns when the whole copy is
// done - as HIP's own asynchronous copies of pageable memory do.  One pipelined copy
// runs at a time per process; a second caller waits for the first.
#include "common.h"

#include <algorithm>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <thread>
#include <vector>

#include <unistd.h>

namespace {

constexpr size_t kChunkMax = (size_t)16 << 20;  // bytes per staging buffer
constexpr int kRing = 4;                        // staging buffers in flight
// Smallest copies worth the pipeline (measured against hipMemcpy, GB/s: device-to-host 2 MiB
// 21.6 against 16.9, 16 MiB 39.6 against 17.7; host-to-device 8 MiB 36.8 against 33.9, below that
// hipMemcpy is as fast or faster).
constexpr size_t kMinD2H = (size_t)2 << 20;
constexpr size_t kMinH2D = (size_t)8 << 20;

// A quarter of the copy per chunk, so that four are in flight, between 1 and 16 MiB: chunks
// below 1 MiB spend their time waking the helpers (0.5 MiB chunks: 21 GB/s at any size).
size_t chunk_for(size_t nbytes)
{
    size_t c = (nbytes / kRing + ((size_t)1 << 20) - 1) & ~(((size_t)1 << 20) - 1);
    return std::max((size_t)1 << 20, std::min(c, kChunkMax));
}

// ---- a few helper threads that copy slices of a chunk --------------------------------
class CopyCrew {
public:
    explicit CopyCrew(int helpers)
    {
        for (int i = 0; i < helpers; ++i)
            threads_.emplace_back([this] { work(); });
    }
    ~CopyCrew()
    {
        {
            std::lock_guard<std::mutex> lock(mu_);
            quit_ = true;
        }
        wake_.notify_all();
        for (auto &t : threads_)
            t.join();
    }
    int size() const { return (int)threads_.size(); }

    // dst[0:n] = src[0:n], split between the helpers and the calling thread; returns
    // when every byte has been copied
    void copy(char *dst, const char *src, size_t n)
    {
        const int parts = size() + 1;
        const size_t step = ((n + parts - 1) / parts + 4095) & ~(size_t)4095;
        size_t mine = std::min(step, n);
        {
            std::lock_guard<std::mutex> lock(mu_);
            for (size_t off = mine; off < n; off += step) {
                jobs_.push_back({dst + off, src + off, std::min(step, n - off)});
                ++pending_;
            }
        }
        wake_.notify_all();
        std::memcpy(dst, src, mine);
        std::unique_lock<std::mutex> lock(mu_);
        done_.wait(lock, [this] { return pending_ == 0; });
    }

private:
    struct Job {
        char *dst;
        const char *src;
        size_t n;
    };
    void work()
    {
        std::unique_lock<std::mutex> lock(mu_);
        for (;;) {
            wake_.wait(lock, [this] { return quit_ || !jobs_.empty(); });
            if (quit_)
                return;
            Job j = jobs_.back();
            jobs_.pop_back();
            lock.unlock();
            std::memcpy(j.dst, j.src, j.n);
            lock.lock();
            if (--pending_ == 0)
                done_.notify_all();
        }
    }
    std::mutex mu_;
    std::condition_variable wake_, done_;
    std::vector<Job> jobs_;
    std::vector<std::thread> threads_;
    int pending_ = 0;
    bool quit_ = false;
};

// ---- staging ring of one device ----------------------------------------------------------
struct Ring {
    char *buf[kRing] = {};
    hipEvent_t landed[kRing] = {};  // the DMA that last used buf[k] has finished
    bool ready = false;
};

struct Pipeline {
    std::mutex mu;        // one pipelined copy at a time
    Ring rings[64];       // per device, made on first use, kept for the life of the process
    CopyCrew *crew = nullptr;
    int helpers = -1;     // -1: not read from the environment yet
};

// Never destroyed: no thread joins at exit.  A forked child inherits the object but
// neither the helper threads nor a usable lock (another thread may have held it): it
// starts over with a pipeline of its own.
Pipeline &pipeline()
{
    static Pipeline *p = nullptr;
    static pid_t owner = 0;
    const pid_t me = getpid();
    if (!p || owner != me) {
        p = new Pipeline;
        owner = me;
    }
    return *p;
}

int prepare(Pipeline &p, Ring **out)
{
    if (p.helpers < 0) {
        const char *env = std::getenv("NBH_HOST_COPY_THREADS");
        // 8 by default: first touch of fresh destination pages is what needs them
        // (1 GiB into np.empty: 2 threads 23 GB/s, 4 threads 33, 8 threads 50)
        const unsigned cores = std::thread::hardware_concurrency();
        int threads = env ? std::atoi(env) : (int)std::min(8u, cores ? cores : 8u);
        p.helpers = std::max(0, std::min(threads, 16) - 1);  // the caller is one of the threads
        if (env && std::atoi(env) <= 0)
            p.helpers = -2;  // switched off
    }
    if (p.helpers == -2)
        return -1;
    int dev = 0;
    NBH_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64)
        return -1;
    Ring &r = p.rings[dev];
    if (!r.ready) {
        // what an earlier, failed attempt already made is kept and not made again
        for (int k = 0; k < kRing; ++k) {
            if (!r.buf[k])
                NBH_TRY(hipHostMalloc((void **)&r.buf[k], kChunkMax, hipHostMallocDefault));
            if (!r.landed[k])
                NBH_TRY(hipEventCreateWithFlags(&r.landed[k], hipEventDisableTiming));
        }
        r.ready = true;
    }
    if (!p.crew)
        p.crew = new CopyCrew(p.helpers);
    *out = &r;
    return 0;
}

// Memory HIP knows nothing about is ordinary pageable memory.
bool pageable(const void *host)
{
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, host) != hipSuccess) {
        (void)hipGetLastError();
        return true;
    }
    return attr.type == hipMemoryTypeUnregistered;
}

}  // namespace

// Both return 0 on success, a hipError_t on failure, and -1 when the copy is not one
// for the pipeline (too small, page-locked host memory, switched off): the caller
// then uses hipMemcpy.

int nbh_staged_d2h(void *dst, const void *src, size_t nbytes, hipStream_t stream)
{
    if (nbytes < kMinD2H || !pageable(dst))
        return -1;
    const size_t kChunk = chunk_for(nbytes);
    Pipeline &p = pipeline();
    std::lock_guard<std::mutex> lock(p.mu);
    Ring *ring = nullptr;
    int rc = prepare(p, &ring);
    if (rc) {  // no staging buffers, or switched off: hipMemcpy can still do it
        (void)hipGetLastError();
        return -1;
    }
    const size_t chunks = (nbytes + kChunk - 1) / kChunk;
    auto span = [&](size_t i) { return std::min(kChunk, nbytes - i * kChunk); };
    auto fetch = [&](size_t i) -> int {  // device -> staging buffer i % kRing
        const int k = (int)(i % kRing);
        NBH_TRY(hipMemcpyAsync(ring->buf[k], (const char *)src + i * kChunk, span(i), hipMemcpyDeviceToHost, stream));
        NBH_TRY(hipEventRecord(ring->landed[k], stream));
        return 0;
    };
    auto run = [&]() -> int {
        for (size_t i = 0; i < std::min<size_t>(kRing, chunks); ++i)
            if (int e = fetch(i))
                return e;
        for (size_t i = 0; i < chunks; ++i) {
            const int k = (int)(i % kRing);
            NBH_TRY(hipEventSynchronize(ring->landed[k]));
            p.crew->copy((char *)dst + i * kChunk, ring->buf[k], span(i));
            if (i + kRing < chunks)  // the buffer is free again
                if (int e = fetch(i + kRing))
                    return e;
        }
        return 0;
    };
    rc = run();
    if (rc)  // chunks already issued still write into the ring: nobody may use it before they are done
        (void)hipStreamSynchronize(stream);
    return rc;
}

int nbh_staged_h2d(void *dst, const void *src, size_t nbytes, hipStream_t stream)
{
    if (nbytes < kMinH2D || !pageable(src))
        return -1;
    const size_t kChunk = chunk_for(nbytes);
    Pipeline &p = pipeline();
    std::lock_guard<std::mutex> lock(p.mu);
    Ring *ring = nullptr;
    int rc = prepare(p, &ring);
    if (rc) {  // no staging buffers, or switched off: hipMemcpy can still do it
        (void)hipGetLastError();
        return -1;
    }
    const size_t chunks = (nbytes + kChunk - 1) / kChunk;
    auto run = [&]() -> int {
        for (size_t i = 0; i < chunks; ++i) {
            const int k = (int)(i % kRing);
            const size_t n = std::min(kChunk, nbytes - i * kChunk);
            if (i >= (size_t)kRing)  // the DMA that read this buffer kRing chunks ago must be over
                NBH_TRY(hipEventSynchronize(ring->landed[k]));
            p.crew->copy(ring->buf[k], (const char *)src + i * kChunk, n);
            NBH_TRY(hipMemcpyAsync((char *)dst + i * kChunk, ring->buf[k], n, hipMemcpyHostToDevice, stream));
            NBH_TRY(hipEventRecord(ring->landed[k], stream));
        }
        return 0;
    };
    rc = run();
    // success or not, the ring is only handed to the next copy once every DMA that reads it is over
    const int drained = (int)hipStreamSynchronize(stream);
    return rc ? rc : drained;
}
