// Internal helpers shared by the HIP translation units of libdcgan_hip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "dcgan_hip.h"

namespace dh
{

// Records `msg` as the calling thread's last error and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int fail_hip(hipError_t err, const char* what);
// Makes sure a device is selected and the library state exists (device 0 by default).
int ensure_init();
// Scratch arena of the current device for launches on `stream`, at least `bytes` large (grows, never
// shrinks).  Each stream has its own, so that split-K launches on different streams may overlap.
constexpr int MAX_ARENAS = 8;
constexpr int STAGE_SLOTS = 16;                       // pinned staging buffers of dh_memcpy_h2d_staged
constexpr size_t STAGE_MAX_BYTES = size_t(64) << 20;  // larger copies are plain blocking copies
int workspace(size_t bytes, void** ptr, hipStream_t stream);
// The current device's fixed scratch buffer (STATIC_SCRATCH_BYTES, part of the code object, never
// allocated or freed): for entry points that must not allocate.  Every call on a device shares it.
constexpr size_t STATIC_SCRATCH_BYTES = size_t(2) << 20;
int static_scratch(void** ptr);
int num_cus();

// Per-kernel timing (see dh_profile_enable): prof_begin records an event on `st` and returns a
// handle (-1 while timing is off), prof_end records the closing event.  `work` is the algorithmic
// FLOPs or bytes the launch stands for.
// Level 1 times the convolution kernels only (a few dozen launches per training iteration, so the
// events barely disturb it); level 2 also times the reductions, dense and element-wise kernels.
bool profiling(int level = 1);
// Launches between prof_pause(true) and prof_pause(false) are not recorded (calls nest).
void prof_pause(bool on);
// `issued` (convolution kernels): the FLOPs the matrix cores are issued for the launch, 0 = not known.
int prof_begin(const char* name, double work, hipStream_t st, int level = 1, double issued = 0.0);
void prof_end(int handle, hipStream_t st);
// Brackets the launches of one scope.  Memory-bound kernels report algorithmic BYTES as their work
// and carry the prefix "hbm:" in their name.
struct ProfScope
{
    int handle;
    hipStream_t st;
    ProfScope(const char* name, double work, hipStream_t s, int level = 2) : handle(prof_begin(name, work, s, level)), st(s) {}
    ~ProfScope() { prof_end(handle, st); }
    ProfScope(const ProfScope&) = delete;
    ProfScope& operator=(const ProfScope&) = delete;
};

// Input gradient onto at most 4 channels on the vector ALUs (conv_small.hip).  Returns 1 when the
// shape is not one it takes (the caller then runs the implicit GEMM), 0 after a launch, else an error.
int conv_dx_few_channels(const float* dy, const float* k, float* dx, int N, int Ho, int Wo, int O, int kh, int kw,
                         int C, int sh, int sw, int pt, int pl, int H, int W, const float* bias, int act,
                         float alpha, hipStream_t st);
// The same product for the DCGAN's image layer (5x5, stride 2, at most 3 result channels, 64 dy channels,
// dy rows of at most 32 pixels) as one dense product on the matrix cores followed by a scatter in LDS;
// same return convention.  Tried before conv_dx_few_channels.
int conv_dx_col2im(const float* dy, const float* k, float* dx, int N, int Ho, int Wo, int O, int kh, int kw, int C, int sh,
                   int sw, int pt, int pl, int H, int W, const float* bias, int act, float alpha, hipStream_t st);
// Forward convolution with a contraction of at most 80 (few input channels) and at most 64 output
// channels, MFMA operands loaded straight from global memory; same return convention.
int conv_fwd_thin(const float* x, const float* k, float* y, int N, int H, int W, int C, int kh, int kw, int O, int sh,
                  int sw, int pt, int pl, int Ho, int Wo, const float* bias, int act, float alpha, hipStream_t st);

// The image layer's forward product (5 filter rows of 15 values, at most 64 output channels) for two batches of N
// images that share the filter, in one launch; same return convention.  fwd_rows_takes answers for the geometry.
int conv_fwd_rows(const float* x, const float* x2, const float* k, float* y, float* y2, int N, int H, int W, int C, int kh,
                  int kw, int O, int sh, int sw, int pt, int pl, int Ho, int Wo, const float* bias, int act, float alpha,
                  hipStream_t st);
bool fwd_rows_takes(int N, int H, int W, int C, int kh, int kw, int O, int sh, int sw, int pt, int pl, int Ho, int Wo);

// Filter gradient of a thin input (at most 80 filter elements per output channel, at most 64 output
// channels): writes *splits slices of partial sums to the scratch arena and returns them in *part for
// the caller to add up; same return convention.
// x2 / dy2 (both null, or both set): a second pair of operands contracted into the same result.
int conv_dk_thin(const float* x, const float* dy, const float* x2, const float* dy2, float** part, int* splits, int N,
                 int H, int W, int C, int Ho, int Wo, int O, int kh, int kw, int sh, int sw, int pt, int pl, hipStream_t st);
// Whether conv_dk_thin takes this geometry (16-byte aligned operands assumed).
bool dk_thin_takes(int N, int H, int W, int C, int Ho, int Wo, int O, int kh, int kw, int sw);

// Test and tuning switches (dh_debug_force_generic_conv, dh_debug_force_splitk).
extern bool g_force_generic;  // route every convolution through the general kernel
extern int g_force_splitk;    // > 0: this many k splits (at most one per k-slab) instead of the automatic choice
extern int g_force_tile_width;  // 64 / 128: width of the 128-row tiles of wide forward / input-gradient launches

inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }

#define DH_TRY(expr)                                   \
    do {                                               \
        int dh_rc_ = (expr);                           \
        if (dh_rc_ != 0) return dh_rc_;                \
    } while (0)

#define DH_HIP(expr)                                                \
    do {                                                            \
        hipError_t dh_e_ = (expr);                                  \
        if (dh_e_ != hipSuccess) return ::dh::fail_hip(dh_e_, #expr); \
    } while (0)

// Call right after a kernel launch: reports launch-configuration errors.
#define DH_LAUNCH_CHECK(name)                                              \
    do {                                                                   \
        hipError_t dh_e_ = hipGetLastError();                              \
        if (dh_e_ != hipSuccess) return ::dh::fail_hip(dh_e_, name);       \
    } while (0)

// Division of a non-negative 31-bit integer by a runtime constant without the hardware's
// ~40-instruction integer divide (Granlund-Montgomery round-up method):
//   q = (umulhi(n, mul) + n) >> shift   for 0 <= n < 2^31, 1 <= d < 2^31.
struct FastDiv
{
    uint32_t mul;
    uint32_t shift;
    uint32_t d;

    FastDiv() : mul(0), shift(0), d(1) {}
    explicit FastDiv(uint32_t div) : d(div ? div : 1)
    {
        uint32_t l = 0;
        while ((1ull << l) < d) ++l;
        shift = l;
        mul = (uint32_t)(((1ull << 32) * ((1ull << l) - d)) / d + 1);
    }
    __host__ __device__ inline uint32_t div(uint32_t n) const
    {
#if defined(__HIP_DEVICE_COMPILE__)
        return (__umulhi(n, mul) + n) >> shift;
#else
        return (uint32_t)((((uint64_t)n * mul) >> 32) + n) >> shift;
#endif
    }
    __host__ __device__ inline void divmod(uint32_t n, uint32_t& q, uint32_t& r) const
    {
        q = div(n);
        r = n - q * d;
    }
};

}  // namespace dh
