// Who counts where: hands out the pages of arrival counters that the in-launch split-K
// reduction of the main kernel needs.  Host only, no GPU calls of its own (the one question it
// has about the GPU is asked through a function pointer, so the logic runs in a CPU test).
//
// A page is a row of device counters, all zero between launches (the last workgroup to arrive
// sets its counter back).  Two launches may share a page only if they cannot overlap in time:
//   * eager calls on one stream run in order            -> one page per stream handle;
//   * calls captured into one graph on one stream are   -> one page per (capture, stream),
//     ordered in every replay of that graph                held for as long as the process runs,
//                                                          because the graph may be replayed at any time.
// The first kPermanentPages stream handles keep their page for good.  Later handles share
// kRecycledPages pages that change hands: when none is free, the least recently used one whose
// last launch has finished goes to the newcomer.  Whether it has finished is asked of an event
// that the caller records behind every launch on such a page; a stream handle is never handed
// back to the runtime by this class or on its behalf (the stream may long have been destroyed).
// When nothing can be had the caller runs the reduction as a kernel of its own.
//
// The per-thread default stream is one handle value for every host thread but a different stream
// in each: a call on it is keyed by (handle, calling thread), see stream_key().
// What the scheme cannot see: a stream destroyed while its last launch is still running, and
// another stream then created at the same handle address (a permanent page has no event to ask).
// Callers that destroy streams with work in flight must synchronise them first.
#pragma once

#include <cstdint>
#include <mutex>

namespace tcsl {

class CounterPages {
public:
    static constexpr int kPermanentPages = 32;
    static constexpr int kRecycledPages = 32;
    static constexpr int kEagerPages = kPermanentPages + kRecycledPages;
    static constexpr int kCapturePages = 192;
    static constexpr int kPages = kEagerPages + kCapturePages;
    static constexpr int kEvictionTries = 8;  // least recently used pages looked at when none is free

    // true: the last launch that counted on this (recycled) page has finished
    using IdleFn = bool (*)(int page);

    // Page (0 .. kPages-1) for a call about to be enqueued on `stream`, or -1.  capturing: the
    // stream is recording into a graph, capture_id names the capture.  The caller holds mutex()
    // from before this call until its launch has been enqueued and, if recycled(page), the
    // page's event recorded behind it, so that a page cannot change hands in between.
    int acquire(void* stream, bool capturing, unsigned long long capture_id, IdleFn idle);

    // What names the stream of a call for acquire(): the handle itself, except for the per-thread
    // default stream (handle value kPerThreadHandle in every host thread, a different stream in
    // each), for which it is an address private to the calling thread.  Two host threads that
    // launch on "the" per-thread stream at the same time therefore count on different pages.
    static constexpr uintptr_t kPerThreadHandle = 2;  // hipStreamPerThread
    static void* stream_key(void* stream);

    // Pages whose every launch must be followed by the event that `idle` looks at.
    static constexpr bool recycled(int page) { return page >= kPermanentPages && page < kEagerPages; }

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
