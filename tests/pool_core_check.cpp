// Host-only check of the pool's stream bookkeeping (numba_cuda_amd/csrc/pool_core.h)
// against a scripted device: events complete when the test says so.
#include "pool_core.h"

#include <cstdio>
#include <cstdlib>
#include <set>

struct FakeBackend {
    using Event = int;
    static inline int next_event = 1;
    static inline std::set<int> pending;              // recorded, not completed
    static inline std::set<int> live;                 // created, not destroyed
    static inline std::vector<std::pair<int, int>> recorded;  // (event, stream)
    static inline int syncs = 0;
    static inline uint64_t current_thread = 1;
    static inline bool fail_record = false;
    static bool event_record(Event *out, int stream)
    {
        if (fail_record)
            return false;
        *out = next_event++;
        pending.insert(*out);
        live.insert(*out);
        recorded.push_back({*out, stream});
        return true;
    }
    static bool event_done(Event e) { return pending.count(e) == 0; }
    static void event_destroy(Event e) { live.erase(e); }
    static void device_synchronize()
    {
        ++syncs;
        pending.clear();
    }
    static bool is_per_thread(int s) { return s == 2; }
    static uint64_t thread_id() { return current_thread; }
};
using Tracker = nbh_pool::Tracker<FakeBackend, int>;

#define CHECK(cond)                                                        \
    do {                                                                   \
        if (!(cond)) {                                                     \
            std::printf("FAILED line %d: %s\n", __LINE__, #cond);          \
            std::exit(1);                                                  \
        }                                                                  \
    } while (0)

int main()
{
    using B = FakeBackend;
    {  // a block freed while a stream has work waits for an event recorded after that work
        Tracker t;
        t.note_stream(7);
        auto w = t.waits_for_a_free();
        CHECK(w.size() == 1 && B::recorded.back() == std::make_pair(1, 7));
        CHECK(!Tracker::ready(w));
        B::pending.erase(1);  // the stream got there
        CHECK(Tracker::ready(w) && w.empty());
        // nothing new on the stream: a second free has nothing to wait for, no new event
        const size_t before = B::recorded.size();
        auto w2 = t.waits_for_a_free();
        CHECK(w2.empty() && B::recorded.size() == before);
    }
    {  // the scenario the reports are ordered for.  Thread A is about to launch on stream 5
       // (nothing reported yet); thread B frees a block: no event, the block is reusable at
       // once - which is right, A's launch holds its own buffers.  A's launch is enqueued and
       // reported; a free that follows must record an event that covers it.
        Tracker t;
        auto early = t.waits_for_a_free();
        CHECK(early.empty());
        t.note_stream(5);  // after the enqueue
        auto later = t.waits_for_a_free();
        CHECK(later.size() == 1 && B::recorded.back().second == 5);
        // still running when yet another block is freed: it shares the same event
        auto third = t.waits_for_a_free();
        CHECK(third.size() == 1 && third[0] == later[0]);
        B::pending.clear();
    }
    {  // two streams, one idle for long: only unfinished events are waited for
        Tracker t;
        t.note_stream(3);
        t.note_stream(4);
        auto w = t.waits_for_a_free();
        CHECK(w.size() == 2);
        B::pending.erase(w[0]->ev);
        auto w2 = t.waits_for_a_free();
        CHECK(w2.size() == 1);
        B::pending.clear();
        t.forget_stream(3);
        CHECK(t.tracked_streams() == 1);
    }
    {  // the per-thread default stream is one handle but one stream per host thread
        Tracker t;
        B::current_thread = 1;
        t.note_stream(2);
        const size_t before = B::recorded.size();
        auto mine = t.waits_for_a_free();  // my own per-thread stream: an ordinary event
        CHECK(mine.size() == 1 && B::recorded.size() == before + 1 && B::syncs == 0);
        B::pending.clear();
        B::current_thread = 9;
        t.note_stream(2);                  // thread 9 used ITS per-thread stream
        B::current_thread = 1;
        const int syncs = B::syncs;
        auto other = t.waits_for_a_free();  // thread 1 cannot record there: device-wide wait instead
        CHECK(other.empty() && B::syncs == syncs + 1);
        CHECK(t.tracked_streams() == 2);
    }
    {  // an event that cannot be recorded degrades to a device-wide wait, never to "no wait"
        Tracker t;
        t.note_stream(11);
        B::fail_record = true;
        const int syncs = B::syncs;
        auto w = t.waits_for_a_free();
        CHECK(w.empty() && B::syncs == syncs + 1);
        B::fail_record = false;
    }
    CHECK(B::live.empty());  // every event created was destroyed with its last holder
    CHECK(nbh_pool::size_class(1) == 512 && nbh_pool::size_class(513) == 1024);
    CHECK(nbh_pool::size_class((size_t)1 << 20) == ((size_t)1 << 20));
    CHECK(nbh_pool::size_class(((size_t)1 << 20) + 1) == ((size_t)1 << 20) + ((size_t)1 << 17));
    CHECK(nbh_pool::size_class((size_t)3 << 20) == ((size_t)3 << 20));
    std::printf("pool core ok\n");
    return 0;
}
