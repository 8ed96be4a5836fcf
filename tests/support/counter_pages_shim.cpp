// C handle on tcsl::CounterPages for tests/test_counter_pages.py (built by the test with g++).
// "Streams" are arbitrary integers; the set of busy ones is what the test says it is, and a page
// counts as busy while the stream that last acquired it is.
#include <map>
#include <set>

#include "../../graphneuralnetproj_amd/csrc/counter_pages.h"

namespace {
std::set<void*> busy;
std::map<int, void*> last_user;
bool idle(int page) { return busy.count(last_user[page]) == 0; }
}  // namespace

extern "C" {
void* cp_new() { return new tcsl::CounterPages(); }
void cp_delete(void* p) { delete static_cast<tcsl::CounterPages*>(p); }
void cp_set_busy(unsigned long stream, int is_busy)
{
    if (is_busy)
        busy.insert(reinterpret_cast<void*>(stream));
    else
        busy.erase(reinterpret_cast<void*>(stream));
}
int cp_acquire(void* p, unsigned long stream, int capturing, unsigned long long capture_id)
{
    tcsl::CounterPages* pages = static_cast<tcsl::CounterPages*>(p);
    std::lock_guard<std::mutex> lock(pages->mutex());
    // the key the library derives from the handle (the per-thread default stream: one per calling thread)
    void* key = tcsl::CounterPages::stream_key(reinterpret_cast<void*>(stream));
    const int page = pages->acquire(key, capturing != 0, capture_id, idle);
    if (page >= 0)
        last_user[page] = reinterpret_cast<void*>(stream);
    return page;
}
int cp_eager_in_use(void* p) { return static_cast<tcsl::CounterPages*>(p)->eager_in_use(); }
int cp_capture_in_use(void* p) { return static_cast<tcsl::CounterPages*>(p)->capture_in_use(); }
int cp_eager_pages() { return tcsl::CounterPages::kEagerPages; }
int cp_permanent_pages() { return tcsl::CounterPages::kPermanentPages; }
int cp_recycled(int page) { return tcsl::CounterPages::recycled(page) ? 1 : 0; }
int cp_capture_pages() { return tcsl::CounterPages::kCapturePages; }
unsigned long cp_per_thread_handle() { return tcsl::CounterPages::kPerThreadHandle; }
int cp_eviction_tries() { return tcsl::CounterPages::kEvictionTries; }
}
