// Runtime half of the C ABI: device selection, memory, streams, events and the scratch arena.
// Stands in for the GPU branches of the reference's src/memory (alloc.cu, copy.hxx).
#include "dh_common.h"

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>

namespace dh
{
namespace
{
thread_local char g_err[512] = "";

// Scratch of the entry points that must not allocate (dh_bias_grad_static): a fixed array in the
// code object, one copy per GPU.  Host code never uses this name as an address: init_device asks
// the runtime where the current device keeps its copy and stores that pointer in the device state.
__attribute__((used)) static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

struct DeviceState
{
    bool ready = false;
    int device = 0;
    int cus = 0;
    // one scratch arena per stream that asked for one: launches on different streams may overlap
    struct Arena { hipStream_t stream; void* ptr; size_t bytes; };
    Arena arena[MAX_ARENAS] = {};
    int n_arenas = 0;
    // pinned staging slots of dh_memcpy_h2d_staged, used round-robin; `done` is recorded behind the
    // slot's copy and waited for before the slot is written again
    struct Stage { void* host; size_t bytes; hipEvent_t done; bool in_flight; };
    Stage stage[STAGE_SLOTS] = {};
    int next_stage = 0;
    void* static_scratch = nullptr;   // this device's copy of `scratch`
};

std::mutex g_mu;
DeviceState g_dev[16];
int g_cur = -1;

// Copies `bytes` (a multiple of 4) from pinned host memory, which the device reads across the bus, to device
// memory: for the small inputs of a run an ordinary kernel in the launch stream starts sooner than a copy
// command does.
__global__ __launch_bounds__(256) void copy_from_pinned(void* __restrict__ dst, const void* __restrict__ src, size_t bytes,
                                                        bool vec)
{
    const size_t stride = (size_t)gridDim.x * 256, tid = (size_t)blockIdx.x * 256 + threadIdx.x;
    size_t done = 0;
    if (vec)
    {
        const size_t n16 = bytes / 16;
        for (size_t i = tid; i < n16; i += stride)
            static_cast<float4*>(dst)[i] = static_cast<const float4*>(src)[i];
        done = n16 * 16;
    }
    for (size_t i = done / 4 + tid; i < bytes / 4; i += stride)
        static_cast<float*>(dst)[i] = static_cast<const float*>(src)[i];
}
}  // namespace

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int fail_hip(hipError_t err, const char* what)
{
    return fail((int)err, "%s: %s (%s)", what, hipGetErrorString(err), hipGetErrorName(err));
}

static int init_device(int device)
{
    if (device < 0 || device >= 16)
        return fail(DH_EINVAL, "dh_init: device %d out of range", device);
    std::lock_guard<std::mutex> lock(g_mu);
    DH_HIP(hipSetDevice(device));
    DeviceState& st = g_dev[device];
    if (!st.ready)
    {
        hipDeviceProp_t prop;
        DH_HIP(hipGetDeviceProperties(&prop, device));
        if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
            return fail(DH_EINVAL, "dh_init: device %d is %s; this library holds gfx950 code only",
                        device, prop.gcnArchName);
        void* fixed = nullptr;
        DH_HIP(hipGetSymbolAddress(&fixed, HIP_SYMBOL(scratch)));
        st.static_scratch = fixed;
        st.device = device;
        st.cus = prop.multiProcessorCount;
        st.ready = true;
    }
    g_cur = device;
    return 0;
}

int ensure_init()
{
    if (g_cur >= 0)
        return 0;
    return init_device(0);
}

int num_cus()
{
    return g_cur >= 0 ? g_dev[g_cur].cus : 256;
}

int static_scratch(void** ptr)
{
    DH_TRY(ensure_init());
    *ptr = g_dev[g_cur].static_scratch;
    if (!*ptr)
        return fail(DH_EINVAL, "the fixed scratch buffer of device %d has no address", g_cur);
    return 0;
}

int workspace(size_t bytes, void** ptr, hipStream_t stream)
{
    DH_TRY(ensure_init());
    std::lock_guard<std::mutex> lock(g_mu);
    DeviceState& st = g_dev[g_cur];
    DeviceState::Arena* a = nullptr;
    for (int i = 0; i < st.n_arenas; ++i)
        if (st.arena[i].stream == stream)
            a = &st.arena[i];
    if (!a)
    {
        if (st.n_arenas == MAX_ARENAS)
            return fail(DH_EINVAL, "scratch arenas exist for %d streams already; no room for another stream", MAX_ARENAS);
        a = &st.arena[st.n_arenas++];
        *a = DeviceState::Arena{stream, nullptr, 0};
    }
    if (bytes > a->bytes)
    {
        // Work queued on the old arena must drain before it is released.
        DH_HIP(hipDeviceSynchronize());
        if (a->ptr)
            DH_HIP(hipFree(a->ptr));
        a->ptr = nullptr;
        a->bytes = 0;
        size_t want = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
        DH_HIP(hipMalloc(&a->ptr, want));
        a->bytes = want;
    }
    *ptr = a->ptr;
    return 0;
}

bool g_force_generic = false;
int g_force_splitk = 0;
int g_force_tile_width = 0;

}  // namespace dh

using namespace dh;

extern "C" {

const char* dh_version(void) { return "dcgan_hip 0.1 (gfx950)"; }

const char* dh_last_error(void) { return g_err; }

int dh_init(int device) { return init_device(device); }

int dh_device_info(char* name, size_t name_len, int* compute_units, int* clock_khz,
                   size_t* memory_bytes)
{
    DH_TRY(ensure_init());
    hipDeviceProp_t prop;
    DH_HIP(hipGetDeviceProperties(&prop, g_cur));
    if (name && name_len)
    {
        snprintf(name, name_len, "%s (%s)", prop.name, prop.gcnArchName);
    }
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (clock_khz) *clock_khz = prop.clockRate;
    if (memory_bytes) *memory_bytes = prop.totalGlobalMem;
    return 0;
}

int dh_malloc(void** ptr, size_t bytes)
{
    DH_TRY(ensure_init());
    if (!ptr) return fail(DH_EINVAL, "dh_malloc: null result pointer");
    *ptr = nullptr;
    if (bytes == 0) bytes = 4;
    DH_HIP(hipMalloc(ptr, bytes));
    return 0;
}

int dh_free(void* ptr)
{
    if (!ptr) return 0;
    DH_TRY(ensure_init());
    DH_HIP(hipFree(ptr));
    return 0;
}

int dh_memcpy_h2d(void* dst, const void* src, size_t bytes)
{
    DH_TRY(ensure_init());
    if (bytes == 0) return 0;
    DH_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return 0;
}

int dh_memcpy_h2d_staged(void* dst, const void* src, size_t bytes, void* stream)
{
    DH_TRY(ensure_init());
    if (bytes == 0) return 0;
    if (!dst || !src) return fail(DH_EINVAL, "dh_memcpy_h2d_staged: null pointer");
    if (bytes > STAGE_MAX_BYTES)
    {
        // too large to stage: a blocking copy, ordered behind what `stream` holds by waiting for it
        // (streams made by dh_stream_create do not synchronise with the null stream by themselves)
        DH_HIP(hipStreamSynchronize(as_stream(stream)));
        DH_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
        return 0;
    }
    std::lock_guard<std::mutex> lock(g_mu);
    DeviceState& st = g_dev[g_cur];
    DeviceState::Stage& slot = st.stage[st.next_stage];
    st.next_stage = (st.next_stage + 1) % STAGE_SLOTS;
    if (slot.in_flight)
    {
        DH_HIP(hipEventSynchronize(slot.done));
        slot.in_flight = false;
    }
    if (!slot.done)
        DH_HIP(hipEventCreateWithFlags(&slot.done, hipEventDisableTiming));
    if (bytes > slot.bytes)
    {
        if (slot.host)
            DH_HIP(hipHostFree(slot.host));
        slot.host = nullptr;
        slot.bytes = 0;
        const size_t want = (bytes + 65535) & ~size_t(65535);
        DH_HIP(hipHostMalloc(&slot.host, want, hipHostMallocDefault));
        slot.bytes = want;
    }
    memcpy(slot.host, src, bytes);
    // From the staging buffer to the device with a kernel that reads the pinned memory across the bus: in the
    // launch stream a copy command costs ~20 us before the kernel behind it starts, whatever its size (measured
    // on the 25 KB latent batch of a training step: 43 us per iteration for two such copies, 11 us for two of
    // these launches); for megabytes the two are equally fast (the 3 MB image batch: 80 us either way).
    if (bytes % 4 == 0 && (reinterpret_cast<uintptr_t>(dst) & 3) == 0)
    {
        const bool vec = (reinterpret_cast<uintptr_t>(dst) & 15) == 0;
        size_t blocks = (bytes / 16 + 255) / 256;
        if (blocks < 1) blocks = 1;
        if (blocks > 1024) blocks = 1024;
        hipLaunchKernelGGL(copy_from_pinned, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), dst, slot.host, bytes, vec);
        DH_LAUNCH_CHECK("copy_from_pinned");
    }
    else
        DH_HIP(hipMemcpyAsync(dst, slot.host, bytes, hipMemcpyHostToDevice, as_stream(stream)));
    DH_HIP(hipEventRecord(slot.done, as_stream(stream)));
    slot.in_flight = true;
    return 0;
}

int dh_memcpy_d2h(void* dst, const void* src, size_t bytes)
{
    DH_TRY(ensure_init());
    if (bytes == 0) return 0;
    DH_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return 0;
}

int dh_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream)
{
    DH_TRY(ensure_init());
    if (bytes == 0) return 0;
    DH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
    return 0;
}

int dh_sync(void)
{
    DH_TRY(ensure_init());
    DH_HIP(hipDeviceSynchronize());
    return 0;
}

int dh_stream_create(void** stream)
{
    DH_TRY(ensure_init());
    hipStream_t s;
    DH_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream = s;
    return 0;
}

int dh_stream_destroy(void* stream)
{
    DH_TRY(ensure_init());
    hipStream_t s = as_stream(stream);
    DH_HIP(hipStreamSynchronize(s));
    {
        // the stream's scratch arena goes with it (the table holds at most MAX_ARENAS streams)
        std::lock_guard<std::mutex> lock(g_mu);
        DeviceState& st = g_dev[g_cur];
        for (int i = 0; i < st.n_arenas; ++i)
            if (st.arena[i].stream == s && s != nullptr)
            {
                if (st.arena[i].ptr)
                    DH_HIP(hipFree(st.arena[i].ptr));
                st.arena[i] = st.arena[st.n_arenas - 1];
                st.arena[--st.n_arenas] = DeviceState::Arena{nullptr, nullptr, 0};
                break;
            }
    }
    DH_HIP(hipStreamDestroy(s));
    return 0;
}

int dh_stream_sync(void* stream)
{
    DH_TRY(ensure_init());
    DH_HIP(hipStreamSynchronize(as_stream(stream)));
    return 0;
}

int dh_event_create(void** event)
{
    DH_TRY(ensure_init());
    hipEvent_t e;
    DH_HIP(hipEventCreate(&e));
    *event = e;
    return 0;
}

int dh_event_destroy(void* event)
{
    DH_HIP(hipEventDestroy(static_cast<hipEvent_t>(event)));
    return 0;
}

int dh_event_record(void* event, void* stream)
{
    DH_HIP(hipEventRecord(static_cast<hipEvent_t>(event), as_stream(stream)));
    return 0;
}

int dh_stream_wait_event(void* stream, void* event)
{
    DH_HIP(hipStreamWaitEvent(as_stream(stream), static_cast<hipEvent_t>(event), 0));
    return 0;
}

int dh_event_elapsed_ms(void* start, void* stop, float* ms)
{
    DH_HIP(hipEventSynchronize(static_cast<hipEvent_t>(stop)));
    DH_HIP(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
    return 0;
}

int dh_workspace_reserve(size_t bytes)
{
    void* p;
    return workspace(bytes, &p, nullptr);
}

size_t dh_workspace_bytes(void)
{
    size_t total = 0;
    if (g_cur >= 0)
        for (int i = 0; i < g_dev[g_cur].n_arenas; ++i)
            total += g_dev[g_cur].arena[i].bytes;
    return total;
}


int dh_debug_force_generic_conv(int on)
{
    g_force_generic = on != 0;
    return 0;
}

int dh_debug_force_splitk(int splits)
{
    if (splits < 0) return fail(DH_EINVAL, "dh_debug_force_splitk: negative split count");
    g_force_splitk = splits;
    return 0;
}

int dh_debug_force_tile_width(int width)
{
    if (width != 0 && width != 64 && width != 128)
        return fail(DH_EINVAL, "dh_debug_force_tile_width: width must be 0, 64 or 128");
    g_force_tile_width = width;
    return 0;
}

}
