// Who owns which window of the split-K counter array, on the host.  Plain C++ (no HIP types), so that the policy can
// be driven on a CPU with stand-ins for streams and events.
//
// The counters of a launch are all zero again when it has finished, so a window may go to a new launch as soon as
// every launch that owned a part of it is known to be over.  Three ways to know:
//   * the earlier launch went to the same stream as the new one: the stream runs them in order;
//   * the earlier launch carries an event (recorded right behind it) that has completed;
//   * its stream is idle, or no longer exists (a stream is only destroyed once its work is done).
// A window whose earlier owners cannot be shown to be over is NOT handed out: take() returns kNone and the caller runs
// the product unsplit.  Events are only recorded once launches have been seen on more than one stream; a caller with
// one stream pays nothing.  The oldest owners are let go as soon as they are over for every stream (one query per
// take()), so that no more events are out than launches are in flight.
// Launches recorded into a graph are replayed at times the host does not see: they get windows of their own from the
// upper half of the array, which the ring never enters and which are never handed out twice.  Nothing has to be proved
// over for them, so recording a graph asks the runtime nothing (a query made while a stream records can end the
// recording with an error).
#pragma once
#include <cstddef>
#include <cstdint>
#include <deque>
#include <vector>

namespace decx_hip {

// What the ring needs from the runtime.  `stream` is the caller's handle, passed through untouched.
struct CounterRingRuntime {
    virtual ~CounterRingRuntime() {}
    virtual void* record_event(void* stream) = 0;      // an event behind the stream's last launch; nullptr: none to be had
    virtual bool event_done(void* event) = 0;
    virtual void release_event(void* event) = 0;
    virtual bool stream_idle_or_gone(void* stream) = 0;
};

class CounterRing {
public:
    static constexpr uint32_t kNone = 0xffffffffu;
    struct Stats { uint64_t taken, wraps, refused, events, reserved; };

    explicit CounterRing(uint32_t capacity) : capacity_(capacity), top_(capacity / 2), graph_top_(capacity) {}

    // A window of `n` counters for a launch on `stream` (`key`: the stream's identity -- the handle, made unique per
    // thread where one handle names a stream per thread).  Returns its first index, or kNone.  `capturing`: the launch
    // is being recorded into a graph.  `ticket` names the window for commit(), which must follow the launch of every
    // window taken with capturing == false (0: nothing to commit).
    uint32_t take(CounterRingRuntime& rt, void* stream, uint64_t key, uint32_t n, bool capturing, uint64_t* ticket = nullptr)
    {
        if (ticket) *ticket = 0;
        if (capturing) return reserve(n);
        if (n == 0 || n > top_) { ++stats_.refused; return kNone; }
        if (have_last_ && key != last_key_) multi_stream_ = true;
        last_key_ = key; have_last_ = true;
        // the oldest owners whose events have completed are over for everybody: their events go back to the runtime now, so
        // that no more of them are out than launches are in flight
        while (multi_stream_ && !owners_.empty() && over(rt, 0, kNobody)) {
            if (owners_.front().event) rt.release_event(owners_.front().event);
            owners_.pop_front();
        }
        uint32_t begin = cursor_;
        const bool wrap = begin + n > top_;
        // the stretch the cursor passes over: up to the top when the window does not fit in front of it, then the window
        if (wrap) {
            if (!retire(rt, begin, top_, key)) { ++stats_.refused; return kNone; }
            begin = 0;
            ++stats_.wraps;
        }
        // The stretch passed over stays with this stream: launches of it that owned parts of the stretch were let go
        // unproven (the stream runs them before anything it is given now), and whoever comes by next must see that
        // they may still run.
        if (wrap && cursor_ < top_) owners_.push_back({cursor_, top_, stream, key, nullptr, ++seq_});
        if (!retire(rt, begin, begin + n, key)) {
            if (wrap) cursor_ = 0;                       // (stay in front of the refusal)
            ++stats_.refused;
            return kNone;
        }
        owners_.push_back({begin, begin + n, stream, key, nullptr, ++seq_});
        cursor_ = begin + n;
        if (ticket) *ticket = seq_;
        ++stats_.taken;
        return begin;
    }

    // Behind the launch that uses the window of `ticket`: records its event where events are needed.
    void commit(CounterRingRuntime& rt, uint64_t ticket)
    {
        if (!ticket || !multi_stream_) return;
        for (size_t i = owners_.size(); i-- > 0 && owners_[i].seq >= ticket;) {
            if (owners_[i].seq != ticket) continue;
            if (!owners_[i].event && (owners_[i].event = rt.record_event(owners_[i].stream))) ++stats_.events;
            return;
        }
    }

    // Forgets every owner (the caller has waited for the device, or has put the counters back to zero itself).  Windows
    // of graph launches stay theirs: the graphs still exist.
    void reset(CounterRingRuntime& rt)
    {
        for (Owner& o : owners_) if (o.event) rt.release_event(o.event);
        owners_.clear();
        cursor_ = 0;
    }

    uint32_t ring_size() const { return top_; }           // the lower half: what launches outside graphs go round in
    uint32_t graph_left() const { return graph_top_ - top_; }
    uint32_t capacity() const { return capacity_; }
    const Stats& stats() const { return stats_; }

private:
    struct Owner { uint32_t begin, end; void* stream; uint64_t key; void* event; uint64_t seq; };

    // Windows for graph launches come off the top of the upper half, each once.
    uint32_t reserve(uint32_t n)
    {
        if (n == 0 || n > graph_top_ - top_) { ++stats_.refused; return kNone; }
        graph_top_ -= n;
        stats_.reserved += n;
        return graph_top_;
    }

    // Is the launch of owner i over, as far as a new launch on the stream `key` is concerned?
    bool over(CounterRingRuntime& rt, size_t i, uint64_t key)
    {
        const Owner& o = owners_[i];
        if (key != kNobody && o.key == key) return true;             // same stream: in order
        if (o.event && rt.event_done(o.event)) return true;
        for (size_t j = i + 1; j < owners_.size(); ++j)              // a later launch on its stream whose event is done covers it
            if (owners_[j].key == o.key && owners_[j].event && rt.event_done(owners_[j].event)) return true;
        return rt.stream_idle_or_gone(o.stream);
    }

    // Drops the owners that overlap [begin, end) -- the oldest ones, at the front -- when all of them are over.  An owner
    // that reaches beyond `end` keeps what lies beyond: its launch may still be running for all that a launch on
    // another stream can tell.
    bool retire(CounterRingRuntime& rt, uint32_t begin, uint32_t end, uint64_t key)
    {
        size_t n = 0;
        while (n < owners_.size() && owners_[n].begin < end && owners_[n].end > begin) {
            if (!over(rt, n, key)) return false;
            ++n;
        }
        for (size_t i = 0; i < n; ++i) {
            Owner& o = owners_.front();
            if (o.end > end) { o.begin = end; break; }               // (the last of them: the deque is in ring order)
            if (o.event) rt.release_event(o.event);
            owners_.pop_front();
        }
        return true;
    }

    static constexpr uint64_t kNobody = ~0ull;      // over(): the launch is over for every stream, not only for its own
    uint32_t capacity_, top_, graph_top_;
    uint32_t cursor_ = 0;
    std::deque<Owner> owners_;          // in the order taken = ring order starting at the oldest
    bool multi_stream_ = false, have_last_ = false;
    uint64_t last_key_ = 0, seq_ = 0;
    Stats stats_ = {0, 0, 0, 0, 0};
};

}  // namespace decx_hip
