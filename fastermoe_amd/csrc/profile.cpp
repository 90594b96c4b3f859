#include "profile.hpp"

#include <atomic>
#include <mutex>
#include <vector>

namespace fmoe {
namespace {

struct Record {
    int cls;
    double work;
    hipEvent_t start, stop;
};

std::atomic<bool> g_enabled{false};
std::mutex g_mutex;
std::vector<Record> g_records;
std::vector<hipEvent_t> g_free_events;

hipEvent_t take_event() {
    if (!g_free_events.empty()) {
        hipEvent_t e = g_free_events.back();
        g_free_events.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) return nullptr;
    return e;
}

}  // namespace

bool profile_enabled() { return g_enabled.load(std::memory_order_relaxed); }

int profile_begin(int cls, double work, hipStream_t stream) {
    std::lock_guard<std::mutex> lock(g_mutex);
    Record r{cls, work, take_event(), take_event()};
    if (!r.start || !r.stop) return -1;
    if (hipEventRecord(r.start, stream) != hipSuccess) return -1;
    g_records.push_back(r);
    return (int)g_records.size() - 1;
}

void profile_end(int token, hipStream_t stream) {
    std::lock_guard<std::mutex> lock(g_mutex);
    if (token >= 0 && token < (int)g_records.size()) (void)hipEventRecord(g_records[token].stop, stream);
}

}  // namespace fmoe

using namespace fmoe;

extern "C" int fmoe_profile_enable(int on) {
    g_enabled.store(on != 0);
    return FMOE_OK;
}

extern "C" int fmoe_profile_classes(void) { return kProfClasses; }

extern "C" int fmoe_profile_collect(int64_t *launches, double *milliseconds, double *work, int n_classes) {
    FMOE_REQUIRE(launches && milliseconds && work && n_classes >= kProfClasses,
                 "fmoe_profile_collect: need arrays of at least %d entries", (int)kProfClasses);
    FMOE_HIP_CHECK(hipDeviceSynchronize());
    std::lock_guard<std::mutex> lock(g_mutex);
    for (int c = 0; c < n_classes; ++c) { launches[c] = 0; milliseconds[c] = 0; work[c] = 0; }
    for (Record &r : g_records) {
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, r.start, r.stop) == hipSuccess) {
            launches[r.cls] += 1;
            milliseconds[r.cls] += ms;
            work[r.cls] += r.work;
        }
        g_free_events.push_back(r.start);
        g_free_events.push_back(r.stop);
    }
    g_records.clear();
    return FMOE_OK;
}
