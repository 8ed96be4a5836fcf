// tcsl::CounterPages hammered from many host threads, for a build with ThreadSanitizer: every thread
// launches "work" on its own stream handle, on the per-thread default stream handle and inside
// "captures", the way spmm_api.cpp does (page taken and marked under mutex(), work in flight outside
// it).  Checked: a page never goes to a caller while another caller's launch on it is still in flight.
#include <atomic>
#include <cstdio>
#include <thread>
#include <vector>

#include "counter_pages.h"

namespace {

using tcsl::CounterPages;
CounterPages pages;
std::atomic<int> in_flight[CounterPages::kPages];   // launches not yet finished on a page
void* owner[CounterPages::kPages];                   // key of the last launch (guarded by pages.mutex())
std::atomic<int> violations{0}, refused{0}, granted{0};

bool idle(int page) { return in_flight[page].load(std::memory_order_acquire) == 0; }

void worker(int id, int rounds)
{
    unsigned state = 12345u + 977u * id;
    auto rnd = [&]() { return (state = state * 1664525u + 1013904223u) >> 12; };  // the low bits of such a generator cycle
    for (int r = 0; r < rounds; r++) {
        const unsigned pick = rnd() % 8;
        void* handle;
        bool capturing = false;
        unsigned long long capture_id = 0;
        if (pick < 3)
            handle = reinterpret_cast<void*>(static_cast<uintptr_t>(0x10000 + 0x40 * id));  // this thread's own stream
        else if (pick < 5)
            handle = reinterpret_cast<void*>(CounterPages::kPerThreadHandle);              // "the" per-thread stream
        else if (pick < 7)
            handle = reinterpret_cast<void*>(static_cast<uintptr_t>(0x90000 + 0x40 * (id * 64 + rnd() % 48)));  // short-lived streams
        else {
            handle = reinterpret_cast<void*>(static_cast<uintptr_t>(0x10000 + 0x40 * id));
            capturing = true;
            capture_id = 1 + id * 4 + rnd() % 4;
        }
        int page;
        {
            std::lock_guard<std::mutex> lock(pages.mutex());
            void* key = CounterPages::stream_key(handle);
            page = pages.acquire(key, capturing, capture_id, idle);
            if (page >= 0) {
                // launches of one key are ordered on their stream; anyone else must find the page idle
                if (in_flight[page].load(std::memory_order_acquire) != 0 && owner[page] != key && !capturing)
                    violations++;
                owner[page] = key;
                if (!capturing)
                    in_flight[page].fetch_add(1, std::memory_order_acq_rel);
            }
        }
        if (page < 0) {
            refused++;
            continue;
        }
        granted++;
        if (!capturing) {
            for (volatile int spin = 0; spin < static_cast<int>(rnd() % 200); spin++) {
            }
            in_flight[page].fetch_sub(1, std::memory_order_acq_rel);  // the launch has finished
        }
    }
}

}  // namespace

int main()
{
    std::vector<std::thread> threads;
    for (int t = 0; t < 16; t++)
        threads.emplace_back(worker, t, 4000);
    for (auto& t : threads)
        t.join();
    std::printf("granted %d, refused %d, violations %d, eager pages in use %d, capture pages in use %d\n", granted.load(),
                refused.load(), violations.load(), pages.eager_in_use(), pages.capture_in_use());
    return violations.load() == 0 && granted.load() > 0 ? 0 : 1;
}
