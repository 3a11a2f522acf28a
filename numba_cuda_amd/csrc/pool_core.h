// The bookkeeping of the caching device-memory pool, independent of the HIP runtime:
// everything that touches the device goes through a Backend policy, so the same code
// runs against HIP in the library (pool.hip) and against a scripted stand-in in the
// host-only tests.
//
// When is a freed block safe to hand out?  The owner dropped it, but kernels that use
// it may still be queued.  hipFree answers by waiting for the device.  Here every entry
// point of the library that puts work on a stream reports the stream AFTER the work has
// been enqueued (note_stream); when a block is freed, an event is recorded on each
// stream used since its last such event, and the block waits in the pool until those
// events have completed (queried when an allocation looks at the block: no host-side
// wait, no device-wide synchronisation).  Reporting after the enqueue is what makes this
// sound with several host threads: a free that slips in between a report and the enqueue
// it announced would record its event too early and cover nothing; a report made after
// the enqueue can only be followed by events that cover the work.  (The buffers of the
// launch itself are held by its caller until the call returns, so a free that runs
// before the report cannot concern them.)
//
// The per-thread default stream is one handle but a different stream in every host
// thread, and an event can only be recorded on the calling thread's: its uses are kept
// per thread, and a free that finds uses by OTHER threads falls back to what hipFree
// would have done, a device-wide wait.
//
// Backend requirements:
//   using Event = ...;                          // copyable handle, default-constructible
//   static bool event_record(Event *out, Stream s);   // create + record; false on failure
//   static bool event_done(Event e);            // query
//   static void event_destroy(Event e);
//   static void device_synchronize();
//   static bool is_per_thread(Stream s);
//   static uint64_t thread_id();
#pragma once

#include <stddef.h>
#include <stdint.h>

#include <map>
#include <memory>
#include <unordered_map>
#include <utility>
#include <vector>

namespace nbh_pool {

inline size_t size_class(size_t n)
{
    if (n == 0)
        n = 1;
    if (n <= ((size_t)1 << 20))
        return (n + 511) & ~(size_t)511;
    size_t pow2 = (size_t)1 << 21;
    while (pow2 < n)
        pow2 <<= 1;
    const size_t step = pow2 >> 4;  // 1/8 of the power of two below pow2
    return (n + step - 1) / step * step;
}

template <typename Backend, typename Stream> class Tracker {
  public:
    using Event = typename Backend::Event;
    struct SharedEvent {
        Event ev{};
        bool done = false;
        bool owns = false;
        ~SharedEvent()
        {
            if (owns)
                Backend::event_destroy(ev);
        }
        bool finished()
        {
            if (!done && Backend::event_done(ev))
                done = true;
            return done;
        }
    };
    using EventRef = std::shared_ptr<SharedEvent>;

    // Work has just been put on `stream` by the calling thread.
    void note_stream(Stream stream)
    {
        const uint64_t who = Backend::is_per_thread(stream) ? Backend::thread_id() : 0;
        streams_[{stream, who}].used = true;
    }
    void forget_stream(Stream stream)
    {
        for (auto it = streams_.begin(); it != streams_.end();)
            it = (it->first.first == stream) ? streams_.erase(it) : std::next(it);
    }
    // The events a block freed NOW has to wait for.
    std::vector<EventRef> waits_for_a_free()
    {
        const uint64_t me = Backend::thread_id();
        bool foreign = false;  // per-thread stream used by another host thread since its last event
        for (auto &entry : streams_)
            if (entry.second.used && entry.first.second != 0 && entry.first.second != me)
                foreign = true;
        if (foreign) {
            Backend::device_synchronize();
            for (auto &entry : streams_) {
                entry.second.used = false;
                entry.second.last.reset();
            }
            return {};
        }
        std::vector<EventRef> waits;
        for (auto &entry : streams_) {
            State &st = entry.second;
            if (st.used) {
                auto ev = std::make_shared<SharedEvent>();
                if (Backend::event_record(&ev->ev, entry.first.first)) {
                    ev->owns = true;
                } else {
                    // cannot track this stream: fall back to what hipFree would have done
                    Backend::device_synchronize();
                    ev->done = true;
                }
                st.last = ev;
                st.used = false;
            }
            if (st.last && !st.last->finished())
                waits.push_back(st.last);
        }
        return waits;
    }
    static bool ready(std::vector<EventRef> &waits)
    {
        for (size_t i = 0; i < waits.size();) {
            if (waits[i]->finished()) {
                waits[i] = waits.back();
                waits.pop_back();
            } else {
                ++i;
            }
        }
        return waits.empty();
    }
    size_t tracked_streams() const { return streams_.size(); }

  private:
    struct State {
        bool used = false;  // work submitted since `last` was recorded
        EventRef last;      // covers everything submitted before it
    };
    std::map<std::pair<Stream, uint64_t>, State> streams_;
};

}  // namespace nbh_pool
