// Optional per-kernel timing.  When enabled, a launch site brackets its kernel with two HIP events
// on the launch stream and tags it with a name and the algorithmic FLOPs (or bytes) of the operator
// it belongs to.  dh_profile_read() waits for the events and adds them up per tag.  The events see
// the stream the kernel runs on, whichever that is.
#include <cstdio>
#include <cstring>
#include <vector>

#include "dh_common.h"

namespace dh
{
namespace
{
struct ProfRecord
{
    hipEvent_t e0, e1;
    int tag;
    double work, issued;
};
struct ProfTotal
{
    char name[96];
    long launches;
    double ms, work, issued;
};
int g_level = 0;   // 0 off, 1 convolution kernels, 2 every tagged kernel
int g_paused = 0;  // > 0: launches are not recorded (the library's own measuring runs)
std::vector<ProfRecord> g_open;      // begun, not yet ended
std::vector<ProfRecord> g_pending;   // ended, not yet read
std::vector<hipEvent_t> g_pool;
std::vector<ProfTotal> g_totals;

int tag_of(const char* name)
{
    for (size_t i = 0; i < g_totals.size(); ++i)
        if (!strcmp(g_totals[i].name, name))
            return (int)i;
    ProfTotal t{};
    snprintf(t.name, sizeof(t.name), "%s", name);
    g_totals.push_back(t);
    return (int)g_totals.size() - 1;
}

hipEvent_t take_event()
{
    if (!g_pool.empty())
    {
        hipEvent_t e = g_pool.back();
        g_pool.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    (void)hipEventCreate(&e);
    return e;
}
}  // namespace

bool profiling(int level) { return g_paused == 0 && g_level >= level; }
void prof_pause(bool on) { g_paused += on ? 1 : -1; }

int prof_begin(const char* name, double work, hipStream_t st, int level, double issued)
{
    if (g_paused > 0 || g_level < level)
        return -1;
    ProfRecord r{};
    r.tag = tag_of(name);
    r.work = work;
    r.issued = issued;
    r.e0 = take_event();
    r.e1 = take_event();
    (void)hipEventRecord(r.e0, st);
    g_open.push_back(r);
    return (int)g_open.size() - 1;
}

void prof_end(int handle, hipStream_t st)
{
    if (handle < 0 || handle >= (int)g_open.size())
        return;
    ProfRecord r = g_open[handle];
    g_open.erase(g_open.begin() + handle);
    (void)hipEventRecord(r.e1, st);
    g_pending.push_back(r);
}

}  // namespace dh

using namespace dh;

extern "C" {

int dh_profile_enable(int on)
{
    DH_TRY(ensure_init());
    g_level = on < 0 ? 0 : on;
    return 0;
}

int dh_profile_reset(void)
{
    DH_TRY(ensure_init());
    DH_HIP(hipDeviceSynchronize());
    for (ProfRecord& r : g_pending)
    {
        g_pool.push_back(r.e0);
        g_pool.push_back(r.e1);
    }
    g_pending.clear();
    g_totals.clear();
    return 0;
}

int dh_profile_read(char* buf, size_t buf_len)
{
    DH_TRY(ensure_init());
    for (ProfRecord& r : g_pending)
    {
        float ms = 0.f;
        DH_HIP(hipEventSynchronize(r.e1));
        DH_HIP(hipEventElapsedTime(&ms, r.e0, r.e1));
        ProfTotal& t = g_totals[r.tag];
        t.launches += 1;
        t.ms += ms;
        t.work += r.work;
        t.issued += r.issued;
        g_pool.push_back(r.e0);
        g_pool.push_back(r.e1);
    }
    g_pending.clear();
    size_t used = 0;
    if (buf && buf_len)
        buf[0] = 0;
    for (const ProfTotal& t : g_totals)
    {
        if (!buf || used >= buf_len)
            break;
        const int w = snprintf(buf + used, buf_len - used, "%s\t%ld\t%.6f\t%.0f\t%.0f\n", t.name, t.launches, t.ms, t.work, t.issued);
        if (w < 0 || (size_t)w >= buf_len - used)
            return fail(DH_EINVAL, "dh_profile_read: buffer too small");
        used += (size_t)w;
    }
    return 0;
}

}
