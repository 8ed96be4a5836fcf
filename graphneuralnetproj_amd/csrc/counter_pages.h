// Who counts where: hands out the pages of arrival counters that the in-launch split-K
// reduction of the main kernel needs.  Host only, no GPU calls of its own (the two questions it
// has about a stream are asked through function pointers, so the logic runs in a CPU test).
//
// A page is a row of device counters, all zero between launches (the last workgroup to arrive
// sets its counter back).  Two launches may share a page only if they cannot overlap in time:
//   * eager calls on one stream run in order            -> one page per stream handle;
//   * calls captured into one graph on one stream are   -> one page per (capture, stream),
//     ordered in every replay of that graph                held for as long as the process runs,
//                                                          because the graph may be replayed at any time.
// Eager pages are recycled: when none is free, the least recently used page whose stream is
// idle (or no longer exists) changes hands.  A stream that is still busy keeps its page.
// When nothing can be had the caller runs the reduction as a kernel of its own.
#pragma once

#include <cstdint>
#include <mutex>

namespace tcsl {

class CounterPages {
public:
    static constexpr int kEagerPages = 64;
    static constexpr int kCapturePages = 192;
    static constexpr int kPages = kEagerPages + kCapturePages;
    static constexpr int kEvictionTries = 8;  // least recently used pages looked at when none is free

    // true: everything enqueued on the stream has finished, or the handle names no stream any more
    using IdleFn = bool (*)(void* stream);

    // Page (0 .. kPages-1) for a call about to be enqueued on `stream`, or -1.  capturing: the
    // stream is recording into a graph, capture_id names the capture.  The caller holds mutex()
    // from before this call until its launch has been enqueued, so that a page cannot change
    // hands between being looked up and being used.
    int acquire(void* stream, bool capturing, unsigned long long capture_id, IdleFn idle);

    std::mutex& mutex() { return mu_; }

    // for tests
    int eager_in_use() const { return eager_used_; }
    int capture_in_use() const { return capture_used_; }

private:
    struct Eager {
        void* stream;
        uint64_t last_use;
    };
    struct Captured {
        void* stream;
        unsigned long long capture_id;
    };
    std::mutex mu_;
    Eager eager_[kEagerPages] = {};
    Captured captured_[kCapturePages] = {};
    int eager_used_ = 0, capture_used_ = 0;
    uint64_t clock_ = 0;
};

}  // namespace tcsl
