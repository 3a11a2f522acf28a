// Host-side check of numba_cuda_amd/csrc/launchq.hip (the launching threads), no device needed:
// a recording stand-in for nbh_reduce, six producers on six streams, waits for one queue and
// for all, the mode switched off and on meanwhile, a stream destroyed and made again 300 times,
// the error report.  Checks that every launch was made exactly once, in the order of the calls
// of its stream, with its own arguments.  BURSTS=1 pauses the producers now and then so that
// the launching threads fall asleep and have to be woken.  Built with the thread sanitizer and
// run by tests/test_launchq_host.py.
#include "common.h"
#include <atomic>
#include <chrono>
#include <cstdio>
#include <csignal>
#include <cstdlib>
#include <map>
#include <mutex>
#include <thread>
#include <vector>
#include <sys/wait.h>
#include <unistd.h>
extern "C" int nbh_launch_threads(int enable);
extern "C" int nbh_launch_threads_wait(nbh_stream_t stream);
extern "C" int nbh_stream_pin_direct(nbh_stream_t stream);
extern "C" int nbh_reduce_queued(int op, int dtype, const void *in, int64_t n, int64_t in_stride, const void *init, void *out,
                                 void *scratch, size_t scratch_bytes, nbh_stream_t stream);
static std::mutex g_m;
static std::map<void *, std::vector<int64_t>> g_seen;   // per stream: the n of each launch, in order
static std::atomic<long> g_calls{0};
static std::atomic<bool> g_block{false};   // holds the launching threads inside a launch
extern "C" int nbh_reduce(int op, int dtype, const void *in, int64_t n, int64_t in_stride, const void *init, void *out,
                          void *scratch, size_t scratch_bytes, nbh_stream_t stream)
{
    (void)nbh_hip_stream(stream);   // what the real one does first
    while (g_block.load()) std::this_thread::sleep_for(std::chrono::milliseconds(1));
    if (in_stride == 6) return 1;
    {
        std::lock_guard<std::mutex> h(g_m);
        g_seen[stream].push_back(n);
    }
    *(int64_t *)out = n + *(const int32_t *)init;
    g_calls++;
    return 0;
}
void nbh_pool_note_stream(hipStream_t) {}
void nbh_pool_forget_stream(hipStream_t) {}
int main()
{
    nbh_launch_threads(1);
    const int S = 6, N = 20000;
    std::vector<void *> streams;
    for (int s = 0; s < S; ++s) streams.push_back((void *)(uintptr_t)(0x1000 + 0x100 * s));
    std::vector<std::vector<int64_t>> outs(S, std::vector<int64_t>(N, -1));
    std::vector<std::thread> th;
    int dummy_in = 0, scratch = 0;
    for (int s = 0; s < S; ++s)
        th.emplace_back([&, s] {
            for (int i = 0; i < N; ++i) {
                int32_t init = 7;
                if (nbh_reduce_queued(0, 2, &dummy_in, i + 1, 4, &init, &outs[s][i], &scratch, 4, streams[s])) abort();
                if (getenv("BURSTS") && i % 64 == 0) std::this_thread::sleep_for(std::chrono::microseconds(700));
                if (i % 997 == 0) nbh_queue_drain(streams[s]);
                if (i % 4999 == 0) nbh_queue_drain(nullptr);
                if (s == 0 && i % 7001 == 0) { nbh_launch_threads(0); nbh_launch_threads(1); }
            }
        });
    // a thread that keeps destroying and re-making a stream of its own
    th.emplace_back([&] {
        int64_t out = 0; int32_t init = 1;
        for (int r = 0; r < 300; ++r) {
            void *st = (void *)(uintptr_t)(0x9000 + 0x10 * (r % 3));
            for (int i = 0; i < 20; ++i) nbh_reduce_queued(0, 2, &dummy_in, 5, 4, &init, &out, &scratch, 4, st);
            nbh_queue_forget(st);
            if (out != 6) { printf("bad out %ld\n", (long)out); abort(); }
        }
    });
    for (auto &t : th) t.join();
    nbh_queue_drain(nullptr);
    for (int s = 0; s < S; ++s) {
        for (int i = 0; i < N; ++i) if (outs[s][i] != i + 1 + 7) { printf("stream %d item %d: %ld\n", s, i, (long)outs[s][i]); return 1; }
        const auto &v = g_seen[streams[s]];
        if ((int)v.size() != N) { printf("stream %d saw %zu\n", s, v.size()); return 1; }
        for (int i = 0; i < N; ++i) if (v[i] != i + 1) { printf("stream %d out of order at %d\n", s, i); return 1; }
    }
    // error report
    int32_t init = 0; int64_t o = 0;
    nbh_reduce_queued(0, 2, &dummy_in, 3, 6, &init, &o, &scratch, 4, streams[0]);
    nbh_queue_drain(streams[0]);
    if (nbh_queue_take_status(streams[0]) != 1 || nbh_queue_take_status(streams[0]) != 0) { printf("status\n"); return 1; }
    // A stream whose handle leaves the library: what is queued is launched before the call returns,
    // later launches are made by the caller (their result is there when the call returns), also
    // for a stream that is pinned before it was ever used
    {
        void *st = (void *)(uintptr_t)0x5000, *fresh = (void *)(uintptr_t)0x5100;
        std::vector<int64_t> got(200, -1);
        for (int i = 0; i < 200; ++i) nbh_reduce_queued(0, 2, &dummy_in, i + 1, 4, &init, &got[i], &scratch, 4, st);
        nbh_stream_pin_direct(st);
        for (int i = 0; i < 200; ++i) if (got[i] != i + 1) { printf("pin returned before launch %d\n", i); return 1; }
        int64_t now = -1;
        nbh_reduce_queued(0, 2, &dummy_in, 77, 4, &init, &now, &scratch, 4, st);
        if (now != 77) { printf("pinned stream still queues\n"); return 1; }
        nbh_stream_pin_direct(fresh);
        now = -1;
        nbh_reduce_queued(0, 2, &dummy_in, 78, 4, &init, &now, &scratch, 4, fresh);
        if (now != 78) { printf("stream pinned before use still queues\n"); return 1; }
        nbh_queue_forget(st);
        nbh_queue_forget(fresh);
        // the handle value comes back for a new stream: queued again
        now = -1;
        g_block.store(true);
        nbh_reduce_queued(0, 2, &dummy_in, 79, 4, &init, &now, &scratch, 4, st);
        const bool was_queued = now == -1;
        g_block.store(false);
        nbh_queue_drain(st);
        if (!was_queued || now != 79) { printf("a new stream with an old handle value is not queued\n"); return 1; }
        nbh_queue_forget(st);
    }
    // A fork while launches are queued: the child has no launching threads; every call that waits
    // for queues must return there, and launches go straight through (feature off in the child).
    g_block.store(true);
    for (int i = 0; i < 50; ++i) nbh_reduce_queued(0, 2, &dummy_in, 9, 4, &init, &o, &scratch, 4, streams[1]);
    const pid_t child = fork();
    if (child == 0) {
        g_block.store(false);
        nbh_queue_drain(nullptr);
        nbh_queue_drain(streams[1]);
        nbh_launch_threads_wait(streams[1]);
        int64_t mine = 0;
        if (nbh_reduce_queued(0, 2, &dummy_in, 11, 4, &init, &mine, &scratch, 4, streams[1]) || mine != 11) _exit(3);
        nbh_queue_forget(streams[1]);
        nbh_launch_threads(-1);
        _exit(0);
    }
    int status = -1;
    for (int waited = 0; waited < 200; ++waited) {          // 20 s at most: a hang in the child is the failure
        if (waitpid(child, &status, WNOHANG) == child) break;
        std::this_thread::sleep_for(std::chrono::milliseconds(100));
        status = -1;
    }
    g_block.store(false);
    if (status == -1) { kill(child, SIGKILL); printf("child hung after fork\n"); return 1; }
    if (!WIFEXITED(status) || WEXITSTATUS(status) != 0) { printf("child failed: %d\n", status); return 1; }
    nbh_queue_drain(nullptr);
    for (void *st : streams) nbh_queue_forget(st);
    // explicit stop at the end of a process: queued work is launched, the threads are joined, and
    // the switch can be used again afterwards
    nbh_launch_threads(1);
    for (int i = 0; i < 100; ++i) nbh_reduce_queued(0, 2, &dummy_in, 4, 4, &init, &o, &scratch, 4, streams[2]);
    const long before = g_calls.load();
    nbh_launch_threads(-1);
    if (g_calls.load() < before || o != 4) { printf("stop lost launches\n"); return 1; }
    printf("ok, %ld launches\n", g_calls.load());
    return 0;
}
