// CPU test of the split-K counter windows (decx_amd/csrc/split_counter_ring.hpp) against a simulated runtime:
// streams are FIFO queues of launches and event markers that the test advances by hand.  The property that matters:
// a window handed to a launch never overlaps the window of a launch still queued on ANOTHER stream, nor a window that
// was given to a graph launch (those come from the upper half of the array, which the ring never enters).  Prints "ok <name>" per scenario; any failure aborts with a message.
#include "../../decx_amd/csrc/split_counter_ring.hpp"

#include <cstdio>
#include <cstdlib>
#include <deque>
#include <map>
#include <random>
#include <vector>

using namespace decx_hip;

#define REQUIRE(c) do { if (!(c)) { std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #c); std::exit(1); } } while (0)

struct Item { bool is_event; uint32_t begin, end; int event_id; };
struct SimRuntime final : CounterRingRuntime {
    std::map<void*, std::deque<Item>> queues;       // per stream, oldest first
    std::map<int, bool> done;                       // event id -> completed
    int next_event = 1, live_events = 0;
    void* record_event(void* stream) override
    {
        const int id = next_event++;
        done[id] = queues[stream].empty();
        if (!done[id]) queues[stream].push_back({true, 0, 0, id});
        ++live_events;
        return (void*)(intptr_t)id;
    }
    bool event_done(void* e) override { return done.at((int)(intptr_t)e); }
    void release_event(void*) override { --live_events; }
    bool stream_idle_or_gone(void* stream) override { return queues[stream].empty(); }
    // the device finishes the oldest `n` items of a stream
    void advance(void* stream, size_t n)
    {
        std::deque<Item>& q = queues[stream];
        while (n-- && !q.empty()) {
            if (q.front().is_event) done[q.front().event_id] = true;
            q.pop_front();
        }
    }
    void launch(void* stream, uint32_t begin, uint32_t n) { queues[stream].push_back({false, begin, begin + n, 0}); }
    bool overlaps_other_stream(void* stream, uint32_t begin, uint32_t n) const
    {
        for (const auto& kv : queues)
            if (kv.first != stream)
                for (const Item& it : kv.second)
                    if (!it.is_event && it.begin < begin + n && it.end > begin) return true;
        return false;
    }
};

static void* S(int i) { return (void*)(intptr_t)(0x1000 + i); }

// take + launch + commit, as the library does it
static uint32_t submit(CounterRing& ring, SimRuntime& rt, int stream, uint32_t n)
{
    uint64_t ticket = 0;
    const uint32_t at = ring.take(rt, S(stream), (uint64_t)(intptr_t)S(stream), n, false, &ticket);
    if (at == CounterRing::kNone) return at;
    REQUIRE(at + n <= ring.ring_size());
    REQUIRE(!rt.overlaps_other_stream(S(stream), at, n));
    rt.launch(S(stream), at, n);
    ring.commit(rt, ticket);
    return at;
}

static void one_stream_wraps_freely()
{
    CounterRing ring(2 * 1024); SimRuntime rt;
    for (int i = 0; i < 100; ++i) REQUIRE(submit(ring, rt, 0, 100) != CounterRing::kNone);   // never advanced: all queued
    REQUIRE(ring.stats().wraps >= 9 && ring.stats().refused == 0 && ring.stats().events == 0);
    std::puts("ok one_stream_wraps_freely");
}

static void second_stream_waits_for_the_first()
{
    CounterRing ring(2 * 1024); SimRuntime rt;
    for (int i = 0; i < 8; ++i) REQUIRE(submit(ring, rt, 0, 128) == (uint32_t)(128 * i));   // the ring is full of stream 0
    REQUIRE(submit(ring, rt, 1, 128) == CounterRing::kNone);       // stream 0 is busy, its launches carry no events
    REQUIRE(ring.stats().refused == 1);
    rt.advance(S(0), 100);                                         // stream 0 drains
    REQUIRE(submit(ring, rt, 1, 128) == 0);
    REQUIRE(ring.stats().events == 1);                             // two streams seen: events from now on
    // stream 0 again, onto windows of stream 0 (in order: fine), then onto the one stream 1 holds
    for (int i = 1; i < 8; ++i) REQUIRE(submit(ring, rt, 0, 128) == (uint32_t)(128 * i));
    REQUIRE(submit(ring, rt, 0, 128) == CounterRing::kNone);       // stream 1's launch is still queued
    rt.advance(S(1), 1);                                           // the launch, not yet its event
    REQUIRE(submit(ring, rt, 0, 128) == CounterRing::kNone);
    rt.advance(S(1), 1);                                           // the event
    REQUIRE(submit(ring, rt, 0, 128) == 0);
    std::puts("ok second_stream_waits_for_the_first");
}

static void a_later_event_covers_earlier_launches()
{
    CounterRing ring(2 * 1000); SimRuntime rt;
    REQUIRE(submit(ring, rt, 0, 100) == 0);                        // no event: one stream so far
    REQUIRE(submit(ring, rt, 1, 100) == 100);                      // event
    REQUIRE(submit(ring, rt, 0, 100) == 200);                      // event, behind the first launch of stream 0
    for (int i = 3; i < 10; ++i) REQUIRE(submit(ring, rt, 1, 100) == (uint32_t)(100 * i));
    REQUIRE(submit(ring, rt, 1, 100) == CounterRing::kNone);       // window 0: stream 0, queued
    rt.advance(S(0), 2);                                           // first launch and second launch of stream 0 done, event pending
    REQUIRE(submit(ring, rt, 1, 100) == CounterRing::kNone);
    rt.advance(S(0), 1);                                           // the event of the second launch: covers the first
    REQUIRE(submit(ring, rt, 1, 100) == 0);
    std::puts("ok a_later_event_covers_earlier_launches");
}

static void graph_launches_keep_their_windows()
{
    CounterRing ring(2048); SimRuntime rt;                         // launches outside graphs go round in [0, 1024)
    REQUIRE(ring.ring_size() == 1024 && ring.graph_left() == 1024);
    REQUIRE(submit(ring, rt, 0, 1000) == 0);                       // queued, never advanced
    uint64_t ticket = 77;
    // a graph launch asks nothing of the queued one: its windows lie where the ring never goes
    REQUIRE(ring.take(rt, S(1), 1, 100, true, &ticket) == 1948);
    REQUIRE(ticket == 0 && ring.ring_size() == 1024 && ring.graph_left() == 924);
    REQUIRE(ring.take(rt, S(1), 1, 24, true) == 1924);
    REQUIRE(ring.take(rt, S(1), 1, 901, true) == CounterRing::kNone);            // more than is left up there
    REQUIRE(ring.take(rt, S(1), 1, 900, true) == 1024);
    REQUIRE(ring.take(rt, S(1), 1, 1, true) == CounterRing::kNone);
    REQUIRE(ring.stats().reserved == 1024 && ring.stats().refused == 2);
    for (int i = 0; i < 50; ++i) {
        const uint32_t at = submit(ring, rt, 0, 300);
        REQUIRE(at != CounterRing::kNone && at + 300 <= 1024);
    }
    REQUIRE(submit(ring, rt, 0, 1025) == CounterRing::kNone);
    ring.reset(rt);                                                // the graphs still exist: nothing comes back
    REQUIRE(ring.graph_left() == 0);
    std::puts("ok graph_launches_keep_their_windows");
}

static void reset_forgets()
{
    CounterRing ring(2 * 256); SimRuntime rt;
    REQUIRE(submit(ring, rt, 0, 256) == 0);
    REQUIRE(submit(ring, rt, 1, 256) == CounterRing::kNone);
    rt.queues.clear();                                             // "the caller has waited for the device"
    ring.reset(rt);
    REQUIRE(submit(ring, rt, 1, 256) == 0);
    std::puts("ok reset_forgets");
}

static void events_come_back_when_launches_finish()
{
    CounterRing ring(2 * 65536); SimRuntime rt;                    // far from wrapping: nothing is retired by the cursor
    int most = 0;
    for (int i = 0; i < 1000; ++i) {
        REQUIRE(submit(ring, rt, i & 1, 10) != CounterRing::kNone);
        if (i % 4 == 3) { rt.advance(S(0), 100); rt.advance(S(1), 100); }      // both streams drain every four launches
        most = rt.live_events > most ? rt.live_events : most;
    }
    REQUIRE(ring.stats().events >= 998);
    REQUIRE(most <= 8);                                            // as many events out as launches in flight, not as launches made
    std::puts("ok events_come_back_when_launches_finish");
}

static void random_traffic(unsigned seed, int streams, uint32_t capacity, uint32_t max_n)
{
    CounterRing ring(2 * capacity); SimRuntime rt;                  // `capacity` counters to go round in, as many for graphs
    std::mt19937 rng(seed);
    uint64_t handed = 0, refused = 0;
    std::vector<std::pair<uint32_t, uint32_t>> reserved;
    for (int step = 0; step < 20000; ++step) {
        const int what = (int)(rng() % 100);
        const int s = (int)(rng() % (unsigned)streams);
        if (what < 55) {
            const uint32_t n = 1 + rng() % max_n;
            const uint32_t at = submit(ring, rt, s, n);             // (checks the overlap itself)
            if (at == CounterRing::kNone) ++refused; else {
                ++handed;
                for (const auto& r : reserved) REQUIRE(!(at < r.second && at + n > r.first));
            }
        } else if (what < 97) {
            rt.advance(S(s), 1 + rng() % 6);
        } else if (what < 98) {
            const uint32_t n = 1 + rng() % 64;
            const uint32_t at = ring.take(rt, S(s), (uint64_t)(intptr_t)S(s), n, true);
            if (at != CounterRing::kNone) {
                for (const auto& kv : rt.queues)
                    for (const Item& it : kv.second) REQUIRE(it.is_event || !(it.begin < at + n && it.end > at));
                reserved.push_back({at, at + n});
            }
        } else {
            rt.advance(S(s), 1000);
        }
    }
    REQUIRE(handed > 1000);
    REQUIRE(rt.live_events < 20000);                               // events come back when their windows are retired
    std::printf("ok random_traffic seed %u streams %d: %llu handed out, %llu refused, %llu wraps, %llu events\n", seed, streams,
                (unsigned long long)handed, (unsigned long long)refused, (unsigned long long)ring.stats().wraps,
                (unsigned long long)ring.stats().events);
}

int main()
{
    one_stream_wraps_freely();
    second_stream_waits_for_the_first();
    a_later_event_covers_earlier_launches();
    graph_launches_keep_their_windows();
    reset_forgets();
    events_come_back_when_launches_finish();
    random_traffic(1, 1, 4096, 512);
    random_traffic(2, 2, 4096, 512);
    random_traffic(3, 5, 65536, 4096);
    random_traffic(4, 3, 512, 300);
    std::puts("all ok");
    return 0;
}
