#include "counter_pages.h"

namespace tcsl {

void* CounterPages::stream_key(void* stream)
{
    if (reinterpret_cast<uintptr_t>(stream) != kPerThreadHandle)
        return stream;
    // thread-local storage is no address a stream handle (a heap object of the runtime) can have
    thread_local char token;
    return &token;
}

int CounterPages::acquire(void* stream, bool capturing, unsigned long long capture_id, IdleFn idle)
{
    if (capturing) {
        for (int i = 0; i < capture_used_; i++)
            if (captured_[i].stream == stream && captured_[i].capture_id == capture_id)
                return kEagerPages + i;
        if (capture_used_ == kCapturePages)
            return -1;
        captured_[capture_used_] = Captured{stream, capture_id};
        return kEagerPages + capture_used_++;
    }
    ++clock_;
    for (int i = 0; i < eager_used_; i++)
        if (eager_[i].stream == stream) {
            eager_[i].last_use = clock_;
            return i;
        }
    if (eager_used_ < kEagerPages) {
        eager_[eager_used_] = Eager{stream, clock_};
        return eager_used_++;
    }
    // All pages have an owner: look at the least recently used recycled ones, oldest first, and
    // take the first whose last launch has finished.
    uint64_t newer_than = 0;
    for (int t = 0; t < kEvictionTries; t++) {
        int oldest = -1;
        for (int i = kPermanentPages; i < kEagerPages; i++)
            if (eager_[i].last_use > newer_than && (oldest < 0 || eager_[i].last_use < eager_[oldest].last_use))
                oldest = i;
        if (oldest < 0)
            break;
        if (idle && idle(oldest)) {
            eager_[oldest] = Eager{stream, clock_};
            return oldest;
        }
        newer_than = eager_[oldest].last_use;
    }
    return -1;
}

}  // namespace tcsl
