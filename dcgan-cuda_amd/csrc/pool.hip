// Pooled device memory for operator outputs and variables: dh_pool_alloc / dh_pool_free behind the host
// layer's tensor_alloc / tensor_free.  The reference calls cudaMalloc / cudaFree once per tensor at every
// Op::compile (src/memory/alloc.cu:16-37, src/ops/conv2d.cu:49-79) and again whenever an input's shape
// changes and its consumers are lowered anew (src/ops/graph.cu:104-120); here the memory is carved from
// a few large slabs that the library keeps, so that the steady state and a recompile at another shape
// make no hipMalloc or hipFree at all.
//
// A slab is one hipMalloc; inside it, free ranges are kept by offset (neighbours merge when a block
// comes back) and a request takes the smallest free range that holds it, 256-byte aligned.  A new slab
// is as large as everything held so far (at least 64 MiB, at most 1 GiB, never less than the request),
// so the number of hipMalloc calls grows with the logarithm of the footprint.
//
// A freed block can be handed out again at once, without waiting for the GPU: work that used the old
// tensor and work that uses the new one are ordered by the stream they are queued on.  That holds for
// callers that queue all their work on ONE stream, as the host runner does; a caller using several
// streams must make them meet (dh_event_record + dh_stream_wait_event, or a synchronisation) before
// it frees a block that another stream may still touch.
#include "dh_common.h"

#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace
{
using namespace dh;

constexpr size_t ALIGN = 256;
constexpr size_t MIN_SLAB = size_t(64) << 20;
constexpr size_t MAX_SLAB = size_t(1) << 30;

struct Slab
{
    char* base = nullptr;
    size_t bytes = 0;
    std::map<size_t, size_t> free_ranges;   // offset -> length
};

struct Pool
{
    std::vector<Slab> slabs;
    std::unordered_map<void*, std::pair<int, size_t>> live;   // block -> (slab, length)
    size_t hipmallocs = 0, held = 0, in_use = 0, peak = 0;
};

std::mutex g_pool_mu;
Pool g_pool[16];

int current_device(int* dev)
{
    DH_TRY(ensure_init());
    DH_HIP(hipGetDevice(dev));
    if (*dev < 0 || *dev >= 16)
        return fail(DH_EINVAL, "dh_pool: device %d out of range", *dev);
    return 0;
}

int add_slab(Pool& p, size_t bytes)
{
    void* base = nullptr;
    DH_HIP(hipMalloc(&base, bytes));
    Slab s;
    s.base = static_cast<char*>(base);
    s.bytes = bytes;
    s.free_ranges[0] = bytes;
    p.slabs.push_back(std::move(s));
    p.hipmallocs += 1;
    p.held += bytes;
    return 0;
}

// Smallest free range of any slab that holds `need` bytes.
bool best_fit(Pool& p, size_t need, int* slab, size_t* offset)
{
    size_t best = ~size_t(0);
    for (int i = 0; i < (int)p.slabs.size(); ++i)
        for (const auto& r : p.slabs[i].free_ranges)
            if (r.second >= need && r.second < best)
            {
                best = r.second;
                *slab = i;
                *offset = r.first;
            }
    return best != ~size_t(0);
}
}  // namespace

extern "C" {

int dh_pool_alloc(void** ptr, size_t bytes)
{
    if (!ptr) return fail(DH_EINVAL, "dh_pool_alloc: null result pointer");
    *ptr = nullptr;
    int dev;
    DH_TRY(current_device(&dev));
    const size_t need = bytes == 0 ? ALIGN : (bytes + ALIGN - 1) / ALIGN * ALIGN;
    if (need < bytes) return fail(DH_EINVAL, "dh_pool_alloc: size overflows");
    std::lock_guard<std::mutex> lock(g_pool_mu);
    Pool& p = g_pool[dev];
    int slab = -1;
    size_t offset = 0;
    if (!best_fit(p, need, &slab, &offset))
    {
        size_t want = p.held < MIN_SLAB ? MIN_SLAB : (p.held > MAX_SLAB ? MAX_SLAB : p.held);
        if (want < need) want = need;
        if (add_slab(p, want) != 0)
        {
            // not enough memory for a slab with headroom: take what the request needs
            (void)hipGetLastError();
            if (want == need) return fail(DH_EINVAL, "dh_pool_alloc: out of device memory (%zu bytes asked for, %zu held)", need, p.held);
            DH_TRY(add_slab(p, need));
        }
        slab = (int)p.slabs.size() - 1;
        offset = 0;
    }
    Slab& s = p.slabs[slab];
    const size_t length = s.free_ranges[offset];
    s.free_ranges.erase(offset);
    if (length > need)
        s.free_ranges[offset + need] = length - need;
    *ptr = s.base + offset;
    p.live[*ptr] = {slab, need};
    p.in_use += need;
    if (p.in_use > p.peak) p.peak = p.in_use;
    return 0;
}

int dh_pool_free(void* ptr)
{
    if (!ptr) return 0;
    int dev;
    DH_TRY(current_device(&dev));
    std::lock_guard<std::mutex> lock(g_pool_mu);
    Pool& p = g_pool[dev];
    auto it = p.live.find(ptr);
    if (it == p.live.end())
        return fail(DH_EINVAL, "dh_pool_free: %p is not a live block of this device's pool", ptr);
    Slab& s = p.slabs[it->second.first];
    size_t offset = (size_t)(static_cast<char*>(ptr) - s.base), length = it->second.second;
    p.in_use -= length;
    p.live.erase(it);
    auto next = s.free_ranges.lower_bound(offset);
    if (next != s.free_ranges.end() && offset + length == next->first)
    {
        length += next->second;
        next = s.free_ranges.erase(next);
    }
    if (next != s.free_ranges.begin())
    {
        auto prev = std::prev(next);
        if (prev->first + prev->second == offset)
        {
            offset = prev->first;
            length += prev->second;
            s.free_ranges.erase(prev);
        }
    }
    s.free_ranges[offset] = length;
    return 0;
}

int dh_pool_reserve(size_t bytes)
{
    int dev;
    DH_TRY(current_device(&dev));
    std::lock_guard<std::mutex> lock(g_pool_mu);
    Pool& p = g_pool[dev];
    // one idle range of that size, not idle bytes in total: fragments do not serve a large request
    const size_t need = bytes == 0 ? ALIGN : (bytes + ALIGN - 1) / ALIGN * ALIGN;
    if (need < bytes) return fail(DH_EINVAL, "dh_pool_reserve: size overflows");
    int slab = -1;
    size_t offset = 0;
    if (best_fit(p, need, &slab, &offset)) return 0;
    return add_slab(p, need);
}

int dh_pool_trim(void)
{
    int dev;
    DH_TRY(current_device(&dev));
    DH_HIP(hipDeviceSynchronize());   // queued work may still touch blocks that were freed a moment ago
    std::lock_guard<std::mutex> lock(g_pool_mu);
    Pool& p = g_pool[dev];
    // slabs are addressed by index from the live blocks: release only from the end backwards, and
    // leave a hole (an empty record) for an idle slab in the middle
    for (int i = (int)p.slabs.size() - 1; i >= 0; --i)
    {
        Slab& s = p.slabs[i];
        const bool idle = s.base && s.free_ranges.size() == 1 && s.free_ranges.begin()->second == s.bytes;
        if (!idle) continue;
        DH_HIP(hipFree(s.base));
        p.held -= s.bytes;
        s = Slab{};
        if (i == (int)p.slabs.size() - 1) p.slabs.pop_back();
    }
    while (!p.slabs.empty() && !p.slabs.back().base) p.slabs.pop_back();
    return 0;
}

int dh_pool_stats(size_t* hipmalloc_calls, size_t* bytes_held, size_t* bytes_in_use, size_t* peak_in_use)
{
    int dev;
    DH_TRY(current_device(&dev));
    std::lock_guard<std::mutex> lock(g_pool_mu);
    const Pool& p = g_pool[dev];
    if (hipmalloc_calls) *hipmalloc_calls = p.hipmallocs;
    if (bytes_held) *bytes_held = p.held;
    if (bytes_in_use) *bytes_in_use = p.in_use;
    if (peak_in_use) *peak_in_use = p.peak;
    return 0;
}
}
