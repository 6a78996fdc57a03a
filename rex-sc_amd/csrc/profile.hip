#include "profile.h"

#include <mutex>
#include <string.h>
#include <vector>

namespace rexsc {
namespace {
struct Rec { const char *name; double work; hipEvent_t start, stop; };
std::mutex g_mu;
bool g_on = false;
std::vector<Rec> g_recs;
} // namespace

ProfScope::ProfScope(const char *name, double work, hipStream_t s) : slot(-1), stream(s)
{
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_on) return;
    Rec r{name, work, nullptr, nullptr};
    if (hipEventCreate(&r.start) != hipSuccess || hipEventCreate(&r.stop) != hipSuccess) return;
    (void)hipEventRecord(r.start, stream);
    g_recs.push_back(r);
    slot = (int)g_recs.size() - 1;
}

ProfScope::~ProfScope()
{
    if (slot < 0) return;
    std::lock_guard<std::mutex> lk(g_mu);
    if (slot < (int)g_recs.size()) (void)hipEventRecord(g_recs[slot].stop, stream);
}

} // namespace rexsc

using namespace rexsc;

extern "C" int rexsc_profile_begin(void)
{
    std::lock_guard<std::mutex> lk(g_mu);
    for (auto &r : g_recs) { (void)hipEventDestroy(r.start); (void)hipEventDestroy(r.stop); }
    g_recs.clear();
    g_on = true;
    return REXSC_OK;
}

extern "C" int rexsc_profile_end(rexsc_profile_record *out, int max_records)
{
    std::lock_guard<std::mutex> lk(g_mu);
    g_on = false;
    int n = 0;
    for (auto &r : g_recs) {
        float ms = 0.f;
        if (hipEventSynchronize(r.stop) == hipSuccess && hipEventElapsedTime(&ms, r.start, r.stop) == hipSuccess) {
            // aggregate by kernel name
            int k = 0;
            for (; k < n; k++) if (strcmp(out[k].name, r.name) == 0) break;
            if (k == n) {
                if (n >= max_records) continue;
                memset(&out[n], 0, sizeof(out[n]));
                strncpy(out[n].name, r.name, sizeof(out[n].name) - 1);
                n++;
            }
            out[k].calls += 1;
            out[k].total_ms += ms;
            out[k].total_work += r.work;
        }
        (void)hipEventDestroy(r.start);
        (void)hipEventDestroy(r.stop);
    }
    g_recs.clear();
    return n;
}
