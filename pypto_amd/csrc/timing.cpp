#include "timing.h"

#include <mutex>
#include <utility>
#include <vector>

namespace pto {
namespace {
bool g_on = false;
std::mutex g_mu;
std::vector<std::pair<hipEvent_t, hipEvent_t>> g_recs[KID_COUNT];
hipEvent_t g_open[KID_COUNT];
} // namespace

bool timing_enabled() { return g_on; }
void timing_set(bool on) { g_on = on; }

void timing_begin(int kid, hipStream_t s)
{
    if (!g_on) return;
    hipEvent_t e;
    if (hipEventCreate(&e) != hipSuccess) return;
    (void)hipEventRecord(e, s);
    std::lock_guard<std::mutex> lk(g_mu);
    g_open[kid] = e;
}

void timing_end(int kid, hipStream_t s)
{
    if (!g_on) return;
    hipEvent_t e;
    if (hipEventCreate(&e) != hipSuccess) return;
    (void)hipEventRecord(e, s);
    std::lock_guard<std::mutex> lk(g_mu);
    g_recs[kid].emplace_back(g_open[kid], e);
}

hipError_t timing_collect(int kid, double* total_ms, uint64_t* launches)
{
    std::vector<std::pair<hipEvent_t, hipEvent_t>> recs;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        recs.swap(g_recs[kid]);
    }
    double total = 0.0;
    hipError_t rc = hipSuccess;
    for (auto& r : recs) {
        hipError_t e = hipEventSynchronize(r.second);
        float ms = 0.f;
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, r.first, r.second);
        if (e != hipSuccess) rc = e;
        total += ms;
        (void)hipEventDestroy(r.first);
        (void)hipEventDestroy(r.second);
    }
    *total_ms = total;
    *launches = recs.size();
    return rc;
}

} // namespace pto
