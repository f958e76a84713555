// HBM-bound operators of the hot path: bias add / bias gradient, activations and their
// gradients, tensor add, the Adam kernels and the small loss reductions.
// Every kernel streams its operands once with 16-byte accesses where the sizes allow and has a
// scalar tail, so any length and any alignment is accepted.
//
// Reference counterparts: src/gpu/relu.cu, src/gpu/sigmoid.cu, src/gpu/sum.cu, src/gpu/update.cu,
// mvrow_add in src/gpu/matmul.cu; arithmetic as in src/cpu/ops.hxx.
#include "dh_common.h"

using namespace dh;

namespace
{

constexpr int TPB = 256;

inline bool aligned16(const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; }

// Workgroups of a grid-stride kernel over `work` threads' worth of accesses.  Mid-sized launches get
// 8 workgroups per compute unit and loop; from 8192 workgroups on (8 M floats in 16-byte accesses)
// every thread makes one access and the loop runs once.  Measured on 16-byte maps: the same speed
// at 8 M floats, 4-7 % faster without the cap at 16 M, 8 % at 32 M, 20 % at 128 M (the in-place Adam
// kernels 23-30 %); at 4 M the capped grid is 9 % faster on two-input maps.
inline unsigned grid_for(size_t work, int per_cu = 8)
{
    size_t blocks = (work + TPB - 1) / TPB;
    const size_t cap = (size_t)num_cus() * per_cu;
    if (blocks > cap && blocks < 8192) blocks = cap;
    if (blocks > 0x7fffffffu) blocks = 0x7fffffffu;
    return blocks == 0 ? 1u : (unsigned)blocks;
}

// ---- generic element-wise maps ----------------------------------------------------------------

struct OpRelu { __device__ float operator()(float x) const { return x < 0.f ? 0.f : x; } };
struct OpLeaky { float alpha; __device__ float operator()(float x) const { return x < 0.f ? alpha * x : x; } };
struct OpTanh { __device__ float operator()(float x) const { return tanhf(x); } };
struct OpSigmoid { __device__ float operator()(float x) const { return 1.f / (1.f + expf(-x)); } };

struct OpReluGrad { __device__ float operator()(float z, float d) const { return z > 0.f ? d : 0.f; } };
struct OpLeakyGrad { float alpha; __device__ float operator()(float z, float d) const { return z < 0.f ? alpha * d : d; } };
struct OpTanhGrad { __device__ float operator()(float t, float d) const { return (1.f - t * t) * d; } };
struct OpSigmoidGrad { __device__ float operator()(float s, float d) const { return s * (1.f - s) * d; } };
struct OpAdd { __device__ float operator()(float a, float b) const { return a + b; } };
struct OpSceGrad { float inv_n; __device__ float operator()(float y, float x) const { return (1.f / (1.f + expf(-x)) - y) * inv_n; } };
struct OpMseGrad { float coeff; __device__ float operator()(float y, float yh) const { return coeff * (yh - y); } };
// The optimiser's arithmetic with contraction into fused multiply-adds switched off: every product
// and sum is rounded on its own, as in the reference's CPU kernels (src/cpu/ops.hxx moment_update /
// adam_update compiled without FMA).  Left to itself the compiler fuses a*m + b*g into one FMA, and
// not the same one at every place the expression is inlined, so the separate kernels, the
// single-pass step and the multi-variable step would differ in the last bit.
__device__ __forceinline__ float moment1(float a, float m, float b, float g)
{
#pragma clang fp contract(off)
    const float am = a * m, bg = b * g;
    return am + bg;
}
__device__ __forceinline__ float moment2(float a, float v, float b, float g)
{
#pragma clang fp contract(off)
    const float av = a * v, bg = b * g;
    const float bgg = bg * g;
    return av + bgg;
}
__device__ __forceinline__ float adam_apply1(float p, float m, float v, float lrt, float eps)
{
#pragma clang fp contract(off)
    const float num = lrt * m, den = sqrtf(v) + eps;
    const float q = num / den;
    return p - q;
}
struct OpMoment { float a, b; __device__ float operator()(float m, float g) const { return moment1(a, m, b, g); } };
struct OpMoment2 { float a, b; __device__ float operator()(float v, float g) const { return moment2(a, v, b, g); } };

template <class F>
__global__ __launch_bounds__(TPB) void map1(const float* __restrict__ x, float* __restrict__ out, size_t n, bool vec, F f)
{
    const size_t stride = (size_t)gridDim.x * TPB;
    const size_t tid = (size_t)blockIdx.x * TPB + threadIdx.x;
    size_t done = 0;
    if (vec)
    {
        const size_t n4 = n / 4;
        for (size_t i = tid; i < n4; i += stride)
        {
            float4 v = reinterpret_cast<const float4*>(x)[i];
            v.x = f(v.x); v.y = f(v.y); v.z = f(v.z); v.w = f(v.w);
            reinterpret_cast<float4*>(out)[i] = v;
        }
        done = n4 * 4;
    }
    for (size_t i = done + tid; i < n; i += stride)
        out[i] = f(x[i]);
}

// out may alias a (in-place moment updates) -- no __restrict__ on those two.
template <class F>
__global__ __launch_bounds__(TPB) void map2(const float* a, const float* __restrict__ b, float* out, size_t n, bool vec, F f)
{
    const size_t stride = (size_t)gridDim.x * TPB;
    const size_t tid = (size_t)blockIdx.x * TPB + threadIdx.x;
    size_t done = 0;
    if (vec)
    {
        const size_t n4 = n / 4;
        for (size_t i = tid; i < n4; i += stride)
        {
            const float4 u = reinterpret_cast<const float4*>(a)[i];
            const float4 w = reinterpret_cast<const float4*>(b)[i];
            float4 v;
            v.x = f(u.x, w.x); v.y = f(u.y, w.y); v.z = f(u.z, w.z); v.w = f(u.w, w.w);
            reinterpret_cast<float4*>(out)[i] = v;
        }
        done = n4 * 4;
    }
    for (size_t i = done + tid; i < n; i += stride)
        out[i] = f(a[i], b[i]);
}

template <class F>
int run_map1(const char* who, const float* x, float* out, size_t n, void* stream, F f)
{
    DH_TRY(ensure_init());
    if (n == 0) return 0;
    if (!x || !out) return fail(DH_EINVAL, "%s: null tensor", who);
    const bool vec = aligned16(x) && aligned16(out);
    ProfScope prof("hbm:unary map (8 B/elem)", 8.0 * n, as_stream(stream));
    hipLaunchKernelGGL(map1<F>, dim3(grid_for(vec ? (n + 3) / 4 : n)), dim3(TPB), 0, as_stream(stream), x, out, n, vec, f);
    DH_LAUNCH_CHECK(who);
    return 0;
}

template <class F>
int run_map2(const char* who, const float* a, const float* b, float* out, size_t n, void* stream, F f)
{
    DH_TRY(ensure_init());
    if (n == 0) return 0;
    if (!a || !b || !out) return fail(DH_EINVAL, "%s: null tensor", who);
    const bool vec = aligned16(a) && aligned16(b) && aligned16(out);
    ProfScope prof("hbm:binary map (12 B/elem)", 12.0 * n, as_stream(stream));
    hipLaunchKernelGGL(map2<F>, dim3(grid_for(vec ? (n + 3) / 4 : n)), dim3(TPB), 0, as_stream(stream), a, b, out, n, vec, f);
    DH_LAUNCH_CHECK(who);
    return 0;
}

__global__ __launch_bounds__(TPB) void fill_zero(float* __restrict__ out, size_t n, bool vec)
{
    const size_t stride = (size_t)gridDim.x * TPB;
    const size_t tid = (size_t)blockIdx.x * TPB + threadIdx.x;
    size_t done = 0;
    if (vec)
    {
        const size_t n4 = n / 4;
        for (size_t i = tid; i < n4; i += stride)
            reinterpret_cast<float4*>(out)[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        done = n4 * 4;
    }
    for (size_t i = done + tid; i < n; i += stride)
        out[i] = 0.f;
}

// ---- bias add: out[r,c] = z[r,c] + b[c] ---------------------------------------------------------
// The flat index runs over the whole matrix; the column of a 4-chunk is (4*i) % cols.
template <bool VEC>
__global__ __launch_bounds__(TPB) void bias_add_kernel(const float* __restrict__ z, const float* __restrict__ b,
                                                       float* __restrict__ out, size_t n, FastDiv fd_cols)
{
    const size_t stride = (size_t)gridDim.x * TPB;
    const size_t tid = (size_t)blockIdx.x * TPB + threadIdx.x;
    const uint32_t cols = fd_cols.d;
    if (VEC)
    {
        const size_t n4 = n / 4;
        for (size_t i = tid; i < n4; i += stride)
        {
            const uint32_t e = (uint32_t)(i * 4);
            const uint32_t c = e - fd_cols.div(e) * cols;
            float4 v = reinterpret_cast<const float4*>(z)[i];
            const float4 w = *reinterpret_cast<const float4*>(b + c);
            v.x += w.x; v.y += w.y; v.z += w.z; v.w += w.w;
            reinterpret_cast<float4*>(out)[i] = v;
        }
    }
    else
    {
        for (size_t i = tid; i < n; i += stride)
        {
            const uint32_t e = (uint32_t)i;
            out[i] = z[i] + b[e - fd_cols.div(e) * cols];
        }
    }
}

// ---- column sums (bias gradient), optionally fused with the activation gradient ------------------
// Stage 1: the rows are cut into `chunks` contiguous ranges; a workgroup owns one range and one
// tile of 256 columns.  For narrow matrices (cols <= 256) G = 256/cols consecutive rows are laid
// side by side so that consecutive lanes still read consecutive addresses.  Each lane adds its
// column serially; lanes of the same column are then added in lane order.  Stage 2 adds the
// per-range sums in range order.  The result is therefore independent of scheduling.
struct ActGrad
{
    int act;
    float alpha;
    __device__ float operator()(float ref, float d) const
    {
        switch (act)
        {
        case DH_ACT_RELU: return ref > 0.f ? d : 0.f;
        case DH_ACT_LEAKY: return ref < 0.f ? alpha * d : d;
        case DH_ACT_TANH: return (1.f - ref * ref) * d;
        case DH_ACT_SIGMOID: return ref * (1.f - ref) * d;
        default: return d;
        }
    }
};

template <bool FUSED>
__global__ __launch_bounds__(TPB) void colsum_stage1(const float* __restrict__ a, const float* __restrict__ act_ref,
                                                     float* __restrict__ dz, float* __restrict__ partial,
                                                     size_t rows, uint32_t cols, uint32_t G, size_t rows_per_chunk,
                                                     ActGrad g)
{
    __shared__ float lds[TPB];
    const uint32_t t = threadIdx.x;
    const size_t r_begin = (size_t)blockIdx.y * rows_per_chunk;
    size_t r_end = r_begin + rows_per_chunk;
    if (r_end > rows) r_end = rows;
    float acc = 0.f;
    uint32_t col;
    bool live;
    if (G >= 1 && cols <= TPB)
    {
        live = t < G * cols;
        const uint32_t rsub = t / cols;
        col = t - rsub * cols;
        if (live)
            for (size_t r = r_begin + rsub; r < r_end; r += G)
            {
                const size_t idx = r * cols + col;
                float v = a[idx];
                if (FUSED)
                {
                    v = g(act_ref[idx], v);
                    dz[idx] = v;
                }
                acc += v;
            }
        lds[t] = acc;
        __syncthreads();
        if (t < cols)
        {
            float s = lds[t];
            for (uint32_t q = 1; q < G; ++q)
                s += lds[q * cols + t];
            if (partial)
                partial[(size_t)blockIdx.y * cols + t] = s;
        }
    }
    else
    {
        col = blockIdx.x * TPB + t;
        live = col < cols;
        if (live)
        {
            for (size_t r = r_begin; r < r_end; ++r)
            {
                const size_t idx = r * cols + col;
                float v = a[idx];
                if (FUSED)
                {
                    v = g(act_ref[idx], v);
                    dz[idx] = v;
                }
                acc += v;
            }
            if (partial)
                partial[(size_t)blockIdx.y * cols + col] = acc;
        }
    }
}

// Stage 1 for column counts divisible by 4: a lane owns 4 adjacent columns (one 16-byte access per
// tensor and row; ALIGNED says whether the tensors allow it, otherwise the same 4 elements are
// accessed one by one), G4 = 256 / (cols / 4) rows lie side by side for matrices of up to 1024
// columns, wider ones are cut into tiles of 1024 columns.  Same two-level order of additions as the
// scalar kernel: a lane adds its rows serially, lanes of the same columns are added in lane order.
template <bool FUSED, bool ALIGNED>
__global__ __launch_bounds__(TPB) void colsum_stage1_v4(const float* __restrict__ a, const float* __restrict__ act_ref,
                                                        float* __restrict__ dz, float* __restrict__ partial,
                                                        size_t rows, uint32_t cols, uint32_t G4, size_t rows_per_chunk,
                                                        ActGrad g)
{
    __shared__ float4 lds[TPB];
    const uint32_t t = threadIdx.x;
    const uint32_t c4n = cols / 4;
    const size_t r_begin = (size_t)blockIdx.y * rows_per_chunk;
    size_t r_end = r_begin + rows_per_chunk;
    if (r_end > rows) r_end = rows;
    uint32_t rsub = 0, col4, step = 1;
    bool live;
    if (G4 >= 1)
    {
        rsub = t / c4n;
        col4 = t - rsub * c4n;
        live = t < G4 * c4n;
        step = G4;
    }
    else
    {
        col4 = blockIdx.x * TPB + t;
        live = col4 < c4n;
    }
    auto load4 = [](const float* q) {
        if (ALIGNED)
            return *reinterpret_cast<const float4*>(q);
        return make_float4(q[0], q[1], q[2], q[3]);
    };
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (live)
    {
#pragma unroll 4
        for (size_t r = r_begin + rsub; r < r_end; r += step)
        {
            const size_t idx = r * cols + (size_t)col4 * 4;
            float4 v = load4(a + idx);
            if (FUSED)
            {
                const float4 ref = load4(act_ref + idx);
                v.x = g(ref.x, v.x); v.y = g(ref.y, v.y); v.z = g(ref.z, v.z); v.w = g(ref.w, v.w);
                if (ALIGNED)
                    *reinterpret_cast<float4*>(dz + idx) = v;
                else
                {
                    dz[idx] = v.x; dz[idx + 1] = v.y; dz[idx + 2] = v.z; dz[idx + 3] = v.w;
                }
            }
            acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
        }
    }
    if (G4 >= 1)
    {
        lds[t] = acc;
        __syncthreads();
        if (t < c4n)
        {
            float4 s = lds[t];
            for (uint32_t q = 1; q < G4; ++q)
            {
                const float4 o = lds[q * c4n + t];
                s.x += o.x; s.y += o.y; s.z += o.z; s.w += o.w;
            }
            if (partial)
            {
                float* dst = partial + (size_t)blockIdx.y * cols + (size_t)t * 4;
                dst[0] = s.x; dst[1] = s.y; dst[2] = s.z; dst[3] = s.w;
            }
        }
    }
    else if (live && partial)
    {
        float* dst = partial + (size_t)blockIdx.y * cols + (size_t)col4 * 4;
        dst[0] = acc.x; dst[1] = acc.y; dst[2] = acc.z; dst[3] = acc.w;
    }
}

// One wavefront per column: lane l adds the per-range sums l, l+64, ... in that order, then the 64
// lane sums are combined by a fixed shuffle tree.
__global__ __launch_bounds__(TPB) void colsum_stage2(const float* __restrict__ partial, float* __restrict__ out,
                                                     uint32_t cols, uint32_t chunks)
{
    const uint32_t c = blockIdx.x * (TPB / 64) + (threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63;
    if (c >= cols) return;
    float s = 0.f;
    for (uint32_t q = lane; q < chunks; q += 64)
        s += partial[(size_t)q * cols + c];
    for (int off = 32; off > 0; off >>= 1)
        s += __shfl_down(s, off, 64);
    if (lane == 0) out[c] = s;
}

// How run_colsum cuts the rows: `chunks` ranges of rows_per_chunk rows (G rows side by side for
// narrow matrices), col_tiles tiles of 256 lanes; with vec4 a lane holds 4 adjacent columns.
struct ColsumCut { bool vec4; uint32_t G; unsigned col_tiles; size_t chunks, rows_per_chunk; };

ColsumCut colsum_cut(size_t rows, size_t cols)
{
    ColsumCut c;
    c.vec4 = cols % 4 == 0;
    const size_t lanes = c.vec4 ? cols / 4 : cols;   // lanes that one row occupies
    c.G = lanes <= TPB ? (uint32_t)(TPB / lanes) : 0;
    c.col_tiles = lanes <= TPB ? 1u : (unsigned)((lanes + TPB - 1) / TPB);
    // aim at ~4 workgroups per compute unit, at least 4 row groups each
    size_t row_groups = c.G ? (rows + c.G - 1) / c.G : rows;
    size_t chunks = ((size_t)num_cus() * 4 + c.col_tiles - 1) / c.col_tiles;
    if (chunks > (row_groups + 3) / 4) chunks = (row_groups + 3) / 4;
    if (chunks < 1) chunks = 1;
    if (chunks > 65535) chunks = 65535;
    size_t rows_per_chunk = (rows + chunks - 1) / chunks;
    if (c.G) rows_per_chunk = (rows_per_chunk + c.G - 1) / c.G * c.G;
    c.rows_per_chunk = rows_per_chunk;
    c.chunks = (rows + rows_per_chunk - 1) / rows_per_chunk;
    return c;
}

// db: the column sums (both stages).  parts_out: the per-range sums of stage 1 only, left to the caller.
// fixed_scratch: the row-range sums go to the device's fixed buffer instead of the stream's arena (no
// allocation; the call is refused when they do not fit).
int run_colsum(const char* who, const float* a, const float* act_ref, float* dz, float* db, float* parts_out,
               size_t rows, size_t cols, ActGrad g, bool fused, void* stream, bool fixed_scratch = false)
{
    DH_TRY(ensure_init());
    if (cols == 0) return 0;
    if (!a || (fused && (!act_ref || !dz))) return fail(DH_EINVAL, "%s: null tensor", who);
    if (cols > 0x7fffffffu) return fail(DH_EINVAL, "%s: too many columns", who);
    hipStream_t st = as_stream(stream);
    if (rows == 0)
    {
        float* zero = parts_out ? parts_out : db;   // no rows: one range, whose sums are zero
        if (zero)
        {
            hipLaunchKernelGGL(fill_zero, dim3(grid_for(cols)), dim3(TPB), 0, st, zero, cols, false);
            DH_LAUNCH_CHECK(who);
        }
        return 0;
    }
    const ColsumCut cut = colsum_cut(rows, cols);
    float* partial = parts_out;
    // one range of rows: its sums are the column sums (the second stage would add zeros to them)
    const bool single = db && !parts_out && cut.chunks == 1;
    if (single)
        partial = db;
    else if (db && !partial)
    {
        void* ws;
        const size_t need = cut.chunks * cols * sizeof(float);
        if (fixed_scratch)
        {
            if (need > STATIC_SCRATCH_BYTES)
                return fail(DH_EINVAL, "%s: %zu x %zu needs %zu bytes of scratch, the fixed buffer holds %zu", who, rows,
                            cols, need, STATIC_SCRATCH_BYTES);
            DH_TRY(static_scratch(&ws));
        }
        else
            DH_TRY(workspace(need, &ws, st));
        partial = static_cast<float*>(ws);
    }
    dim3 grid(cut.col_tiles, (unsigned)cut.chunks);
    ProfScope prof(fused ? "hbm:activation gradient + column sums (12 B/elem)" : "hbm:column sums (4 B/elem)",
                   (fused ? 12.0 : 4.0) * rows * cols, st, fixed_scratch ? 1 << 20 : 2);   // no events without allocating
    const bool al = aligned16(a) && (!fused || (aligned16(act_ref) && aligned16(dz)));
#define DH_COLSUM_LAUNCH(KERNEL) \
    hipLaunchKernelGGL(KERNEL, grid, dim3(TPB), 0, st, a, act_ref, dz, partial, rows, (uint32_t)cols, cut.G, cut.rows_per_chunk, g)
    if (cut.vec4 && fused && al) DH_COLSUM_LAUNCH((colsum_stage1_v4<true, true>));
    else if (cut.vec4 && fused) DH_COLSUM_LAUNCH((colsum_stage1_v4<true, false>));
    else if (cut.vec4 && al) DH_COLSUM_LAUNCH((colsum_stage1_v4<false, true>));
    else if (cut.vec4) DH_COLSUM_LAUNCH((colsum_stage1_v4<false, false>));
    else if (fused) DH_COLSUM_LAUNCH(colsum_stage1<true>);
    else DH_COLSUM_LAUNCH(colsum_stage1<false>);
#undef DH_COLSUM_LAUNCH
    DH_LAUNCH_CHECK(who);
    if (db && !parts_out && !single)
    {
        hipLaunchKernelGGL(colsum_stage2, dim3((unsigned)((cols + TPB / 64 - 1) / (TPB / 64))), dim3(TPB), 0, st,
                           partial, db, (uint32_t)cols, (uint32_t)cut.chunks);
        DH_LAUNCH_CHECK(who);
    }
    return 0;
}

// ---- row sums: one wavefront per row -------------------------------------------------------------
__global__ __launch_bounds__(TPB) void rowsum_kernel(const float* __restrict__ a, float* __restrict__ out,
                                                     size_t rows, size_t cols)
{
    const size_t row = (size_t)blockIdx.x * (TPB / 64) + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= rows) return;
    float s = 0.f;
    for (size_t c = lane; c < cols; c += 64)
        s += a[row * cols + c];
    for (int off = 32; off > 0; off >>= 1)
        s += __shfl_down(s, off, 64);
    if (lane == 0) out[row] = s;
}

// ---- scalar reductions over short vectors (length = batch): one workgroup, fixed tree -------------
struct RedSce
{
    __device__ float operator()(float y, float x) const
    {
        return x >= 0.f ? x - x * y + logf(1.f + expf(-x)) : -x * y + logf(1.f + expf(x));
    }
};
struct RedMse
{
    __device__ float operator()(float y, float yh) const { return (y - yh) * (y - yh); }
};

template <class F>
__global__ __launch_bounds__(1024) void mean_reduce(const float* __restrict__ a, const float* __restrict__ b,
                                                    float* __restrict__ out, size_t n, F f)
{
    __shared__ float lds[1024];
    float s = 0.f;
    for (size_t i = threadIdx.x; i < n; i += 1024)
        s += f(a[i], b[i]);
    lds[threadIdx.x] = s;
    __syncthreads();
    for (int w = 512; w > 0; w >>= 1)
    {
        if ((int)threadIdx.x < w) lds[threadIdx.x] += lds[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) out[0] = lds[0] / (float)n;
}

// Sigmoid cross-entropy of one or two logit vectors in ONE launch: the loss (mean_reduce<RedSce>'s sums, tree
// and division), its gradient (map2<OpSceGrad>'s formula) and, for two, the sum of the two losses -- the
// values of the separate launches to the bit, where a training step otherwise issues up to five one-workgroup
// launches of ~4.5 us each (src/gpu/sigmoid.cu:61-111 and the vect_add that joins the discriminator's losses).
struct SceHead
{
    const float* y[2];
    const float* x[2];
    float* loss[2];      // may be null
    float* grad[2];      // may be null
    float* sum;          // loss[0] + loss[1], or null
    int count;
};

__global__ __launch_bounds__(1024) void sce_head_kernel(const SceHead h, size_t n)
{
    __shared__ float lds[1024];
    const RedSce value{};
    const OpSceGrad slope{1.f / (float)n};
    float losses[2] = {0.f, 0.f};
    for (int q = 0; q < h.count; ++q)
    {
        const float* __restrict__ y = h.y[q];
        const float* __restrict__ x = h.x[q];
        float* __restrict__ grad = h.grad[q];
        float s = 0.f;
        for (size_t i = threadIdx.x; i < n; i += 1024)
        {
            const float yi = y[i], xi = x[i];
            s += value(yi, xi);
            if (grad)
                grad[i] = slope(yi, xi);
        }
        lds[threadIdx.x] = s;
        __syncthreads();
        for (int w = 512; w > 0; w >>= 1)
        {
            if ((int)threadIdx.x < w) lds[threadIdx.x] += lds[threadIdx.x + w];
            __syncthreads();
        }
        losses[q] = lds[0] / (float)n;
        __syncthreads();
        if (threadIdx.x == 0 && h.loss[q])
            h.loss[q][0] = losses[q];
    }
    if (threadIdx.x == 0 && h.sum)
        h.sum[0] = losses[0] + losses[1];
}

// rows whose first-maximum column agrees in y and y_hat (strict '>' keeps the lowest index on ties)
__global__ __launch_bounds__(1024) void argmax_acc_kernel(const float* __restrict__ y, const float* __restrict__ yh,
                                                          float* __restrict__ out, size_t rows, size_t cols)
{
    __shared__ unsigned int lds[1024];
    unsigned int hits = 0;
    for (size_t r = threadIdx.x; r < rows; r += 1024)
    {
        size_t by = 0, bh = 0;
        for (size_t c = 1; c < cols; ++c)
        {
            if (y[r * cols + c] > y[r * cols + by]) by = c;
            if (yh[r * cols + c] > yh[r * cols + bh]) bh = c;
        }
        hits += by == bh;
    }
    lds[threadIdx.x] = hits;
    __syncthreads();
    for (int w = 512; w > 0; w >>= 1)
    {
        if ((int)threadIdx.x < w) lds[threadIdx.x] += lds[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) out[0] = (float)lds[0];
}

// ---- Adam ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(TPB) void adam_update_kernel(float* __restrict__ p, const float* __restrict__ m,
                                                          const float* __restrict__ v, float lrt, float eps, size_t n,
                                                          bool vec)
{
    const size_t stride = (size_t)gridDim.x * TPB;
    const size_t tid = (size_t)blockIdx.x * TPB + threadIdx.x;
    size_t done = 0;
    if (vec)
    {
        const size_t n4 = n / 4;
        for (size_t i = tid; i < n4; i += stride)
        {
            float4 pp = reinterpret_cast<float4*>(p)[i];
            const float4 mm = reinterpret_cast<const float4*>(m)[i];
            const float4 vv = reinterpret_cast<const float4*>(v)[i];
            pp.x = adam_apply1(pp.x, mm.x, vv.x, lrt, eps);
            pp.y = adam_apply1(pp.y, mm.y, vv.y, lrt, eps);
            pp.z = adam_apply1(pp.z, mm.z, vv.z, lrt, eps);
            pp.w = adam_apply1(pp.w, mm.w, vv.w, lrt, eps);
            reinterpret_cast<float4*>(p)[i] = pp;
        }
        done = n4 * 4;
    }
    for (size_t i = done + tid; i < n; i += stride)
        p[i] = adam_apply1(p[i], m[i], v[i], lrt, eps);
}

__device__ __forceinline__ void adam1(float& p, float& m, float& v, float g, float b1, float c1, float b2, float c2,
                                      float lrt, float eps)
{
    m = moment1(b1, m, c1, g);
    v = moment2(b2, v, c2, g);
    p = adam_apply1(p, m, v, lrt, eps);
}

__global__ __launch_bounds__(TPB) void adam_step_kernel(float* __restrict__ p, float* __restrict__ m, float* __restrict__ v,
                                                        const float* __restrict__ g, float b1, float c1, float b2, float c2,
                                                        float lrt, float eps, size_t n, bool vec)
{
    const size_t stride = (size_t)gridDim.x * TPB;
    const size_t tid = (size_t)blockIdx.x * TPB + threadIdx.x;
    size_t done = 0;
    if (vec)
    {
        const size_t n4 = n / 4;
        for (size_t i = tid; i < n4; i += stride)
        {
            float4 pp = reinterpret_cast<float4*>(p)[i];
            float4 mm = reinterpret_cast<float4*>(m)[i];
            float4 vv = reinterpret_cast<float4*>(v)[i];
            const float4 gg = reinterpret_cast<const float4*>(g)[i];
            adam1(pp.x, mm.x, vv.x, gg.x, b1, c1, b2, c2, lrt, eps);
            adam1(pp.y, mm.y, vv.y, gg.y, b1, c1, b2, c2, lrt, eps);
            adam1(pp.z, mm.z, vv.z, gg.z, b1, c1, b2, c2, lrt, eps);
            adam1(pp.w, mm.w, vv.w, gg.w, b1, c1, b2, c2, lrt, eps);
            reinterpret_cast<float4*>(p)[i] = pp;
            reinterpret_cast<float4*>(m)[i] = mm;
            reinterpret_cast<float4*>(v)[i] = vv;
        }
        done = n4 * 4;
    }
    for (size_t i = done + tid; i < n; i += stride)
        adam1(p[i], m[i], v[i], g[i], b1, c1, b2, c2, lrt, eps);
}

// Several variables in one launch.  Each workgroup owns ADAM_BLOCK consecutive elements of one
// variable; first_block[i] is the first workgroup of item i (a short scalar search finds the item).
constexpr int ADAM_MAX_ITEMS = 24;
constexpr int ADAM_BLOCK = TPB * 16;

struct AdamBatch
{
    float* p[ADAM_MAX_ITEMS];
    float* m[ADAM_MAX_ITEMS];
    float* v[ADAM_MAX_ITEMS];
    const float* g1[ADAM_MAX_ITEMS];
    const float* g2[ADAM_MAX_ITEMS];    // second gradient contribution, or null
    unsigned long long n[ADAM_MAX_ITEMS];
    float lrt[ADAM_MAX_ITEMS];
    unsigned first_block[ADAM_MAX_ITEMS + 1];
    unsigned char vec[ADAM_MAX_ITEMS];  // every pointer of the item 16-byte aligned
    // > 1: the gradient is the sum of that many vectors of n elements (row-range sums of a bias
    // gradient); such an item gives each of its elements to one wavefront
    unsigned parts1[ADAM_MAX_ITEMS], parts2[ADAM_MAX_ITEMS];
    int count;
};

// Sum of `parts` vectors at element e, one wavefront: lane l adds parts l, l + 64, ... in that order,
// the lane sums are combined by the shuffle tree of colsum_stage2 -- the same additions in the same
// order as the bias gradient's second stage, whose place this takes.  Valid in lane 0.
__device__ __forceinline__ float sum_of_parts(const float* __restrict__ g, unsigned parts, size_t n, size_t e, unsigned lane)
{
    // (sixteen loads are issued before the first add: the parts of a gradient that was written many launches ago
    // come from HBM, and one round trip per add made a 1024-part sum the longest thing in the optimiser launch;
    // a missing part adds +0, which leaves the running sum's bits alone)
    float s = 0.f;
    for (unsigned q0 = lane; q0 < parts; q0 += 64 * 16)
    {
        float val[16];
#pragma unroll
        for (int u = 0; u < 16; ++u)
        {
            const unsigned q = q0 + 64u * (unsigned)u;
            val[u] = q < parts ? g[(size_t)q * n + e] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 16; ++u)
            s += val[u];
    }
    for (int off = 32; off > 0; off >>= 1)
        s += __shfl_down(s, off, 64);
    return s;
}

__global__ __launch_bounds__(TPB) void adam_step_multi_kernel(const AdamBatch batch, float b1, float c1, float b2, float c2,
                                                              float eps)
{
    int item = 0;
    while (item + 1 < batch.count && blockIdx.x >= batch.first_block[item + 1])
        ++item;
    float* __restrict__ p = batch.p[item];
    float* __restrict__ m = batch.m[item];
    float* __restrict__ v = batch.v[item];
    const float* __restrict__ g1 = batch.g1[item];
    const float* __restrict__ g2 = batch.g2[item];
    const size_t n = batch.n[item];
    const float lrt = batch.lrt[item];
    if (batch.parts1[item] > 1 || batch.parts2[item] > 1)
    {
        const size_t e = (size_t)(blockIdx.x - batch.first_block[item]) * (TPB / 64) + (threadIdx.x >> 6);
        const unsigned lane = threadIdx.x & 63;
        if (e >= n)
            return;
        float ga = batch.parts1[item] > 1 ? sum_of_parts(g1, batch.parts1[item], n, e, lane) : g1[e];
        if (g2)
            ga += batch.parts2[item] > 1 ? sum_of_parts(g2, batch.parts2[item], n, e, lane) : g2[e];
        if (lane == 0)
            adam1(p[e], m[e], v[e], ga, b1, c1, b2, c2, lrt, eps);
        return;
    }
    const size_t base = (size_t)(blockIdx.x - batch.first_block[item]) * ADAM_BLOCK;
    if (batch.vec[item])
    {
#pragma unroll
        for (int it = 0; it < ADAM_BLOCK / (TPB * 4); ++it)
        {
            const size_t e = base + ((size_t)it * TPB + threadIdx.x) * 4;
            if (e + 3 < n)
            {
                float4 pp = *reinterpret_cast<float4*>(p + e);
                float4 mm = *reinterpret_cast<float4*>(m + e);
                float4 vv = *reinterpret_cast<float4*>(v + e);
                float4 gg = *reinterpret_cast<const float4*>(g1 + e);
                if (g2)
                {
                    const float4 hh = *reinterpret_cast<const float4*>(g2 + e);
                    gg.x += hh.x; gg.y += hh.y; gg.z += hh.z; gg.w += hh.w;
                }
                adam1(pp.x, mm.x, vv.x, gg.x, b1, c1, b2, c2, lrt, eps);
                adam1(pp.y, mm.y, vv.y, gg.y, b1, c1, b2, c2, lrt, eps);
                adam1(pp.z, mm.z, vv.z, gg.z, b1, c1, b2, c2, lrt, eps);
                adam1(pp.w, mm.w, vv.w, gg.w, b1, c1, b2, c2, lrt, eps);
                *reinterpret_cast<float4*>(p + e) = pp;
                *reinterpret_cast<float4*>(m + e) = mm;
                *reinterpret_cast<float4*>(v + e) = vv;
            }
            else
                for (size_t q = e; q < n && q < e + 4; ++q)
                    adam1(p[q], m[q], v[q], g2 ? g1[q] + g2[q] : g1[q], b1, c1, b2, c2, lrt, eps);
        }
    }
    else
    {
        const size_t end = base + ADAM_BLOCK < n ? base + ADAM_BLOCK : n;
        for (size_t q = base + threadIdx.x; q < end; q += TPB)
            adam1(p[q], m[q], v[q], g2 ? g1[q] + g2[q] : g1[q], b1, c1, b2, c2, lrt, eps);
    }
}

__global__ __launch_bounds__(TPB) void sgd_update_kernel(float* __restrict__ var, const float* __restrict__ dv,
                                                         const float* __restrict__ coeff, size_t n)
{
    const float c = coeff[0];
    const size_t stride = (size_t)gridDim.x * TPB;
    for (size_t i = (size_t)blockIdx.x * TPB + threadIdx.x; i < n; i += stride)
        var[i] += c * dv[i];
}

}  // namespace

extern "C" {

int dh_memset0(void* ptr, size_t bytes, void* stream)
{
    DH_TRY(ensure_init());
    if (bytes == 0) return 0;
    if (!ptr || (bytes & 3) || (reinterpret_cast<uintptr_t>(ptr) & 3))
        return fail(DH_EINVAL, "dh_memset0: pointer and size must be multiples of 4 bytes");
    const size_t n = bytes / 4;
    const bool vec = aligned16(ptr);
    // a fill kernel rather than hipMemsetAsync, so that callers may capture it in a HIP graph
    hipLaunchKernelGGL(fill_zero, dim3(grid_for(vec ? (n + 3) / 4 : n)), dim3(TPB), 0, as_stream(stream),
                       static_cast<float*>(ptr), n, vec);
    DH_LAUNCH_CHECK("dh_memset0");
    return 0;
}

int dh_bias_add(const float* z, const float* b, float* out, size_t rows, size_t cols, void* stream)
{
    DH_TRY(ensure_init());
    const size_t n = rows * cols;
    if (n == 0) return 0;
    if (!z || !b || !out) return fail(DH_EINVAL, "dh_bias_add: null tensor");
    if (n > 0x7fffffffu) return fail(DH_EINVAL, "dh_bias_add: more than 2^31-1 elements");
    const bool vec = cols % 4 == 0 && aligned16(z) && aligned16(b) && aligned16(out);
    const FastDiv fd((uint32_t)cols);
    if (vec)
        hipLaunchKernelGGL(bias_add_kernel<true>, dim3(grid_for(n / 4)), dim3(TPB), 0, as_stream(stream), z, b, out, n, fd);
    else
        hipLaunchKernelGGL(bias_add_kernel<false>, dim3(grid_for(n)), dim3(TPB), 0, as_stream(stream), z, b, out, n, fd);
    DH_LAUNCH_CHECK("dh_bias_add");
    return 0;
}

int dh_bias_grad(const float* dz, float* db, size_t rows, size_t cols, void* stream)
{
    if (!db && cols) return fail(DH_EINVAL, "dh_bias_grad: null result");
    return run_colsum("dh_bias_grad", dz, nullptr, nullptr, db, nullptr, rows, cols, ActGrad{DH_ACT_NONE, 0.f}, false, stream);
}

int dh_bias_grad_static(const float* dz, float* db, size_t rows, size_t cols, void* stream)
{
    if (!db && cols) return fail(DH_EINVAL, "dh_bias_grad_static: null result");
    return run_colsum("dh_bias_grad_static", dz, nullptr, nullptr, db, nullptr, rows, cols, ActGrad{DH_ACT_NONE, 0.f}, false,
                      stream, true);
}

size_t dh_bias_grad_static_max_bytes(void) { return STATIC_SCRATCH_BYTES; }

size_t dh_bias_grad_part_count(size_t rows, size_t cols)
{
    if (rows == 0 || cols == 0 || ensure_init() != 0) return rows == 0 && cols != 0 ? 1 : 0;
    return colsum_cut(rows, cols).chunks;
}

int dh_bias_grad_parts(const float* dz, float* parts, size_t rows, size_t cols, void* stream)
{
    if (!parts && cols) return fail(DH_EINVAL, "dh_bias_grad_parts: null result");
    return run_colsum("dh_bias_grad_parts", dz, nullptr, nullptr, nullptr, parts, rows, cols, ActGrad{DH_ACT_NONE, 0.f}, false,
                      stream);
}

int dh_act_bias_grad(const float* act_ref, const float* dout, float* dz, float* db, size_t rows, size_t cols,
                     int act, float alpha, void* stream)
{
    return run_colsum("dh_act_bias_grad", dout, act_ref, dz, db, nullptr, rows, cols, ActGrad{act, alpha}, true, stream);
}

int dh_act_bias_grad_parts(const float* act_ref, const float* dout, float* dz, float* parts, size_t rows, size_t cols,
                           int act, float alpha, void* stream)
{
    if (!parts && cols) return fail(DH_EINVAL, "dh_act_bias_grad_parts: null result");
    return run_colsum("dh_act_bias_grad_parts", dout, act_ref, dz, nullptr, parts, rows, cols, ActGrad{act, alpha}, true,
                      stream);
}

int dh_mat_sum_rows(const float* a, float* out, size_t rows, size_t cols, void* stream)
{
    DH_TRY(ensure_init());
    if (rows == 0) return 0;
    if (!a || !out) return fail(DH_EINVAL, "dh_mat_sum_rows: null tensor");
    hipLaunchKernelGGL(rowsum_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(TPB), 0, as_stream(stream), a, out, rows, cols);
    DH_LAUNCH_CHECK("dh_mat_sum_rows");
    return 0;
}

int dh_relu(const float* x, float* out, size_t n, void* stream) { return run_map1("dh_relu", x, out, n, stream, OpRelu{}); }
int dh_relu_leaky(const float* x, float* out, size_t n, float alpha, void* stream)
{ return run_map1("dh_relu_leaky", x, out, n, stream, OpLeaky{alpha}); }
int dh_tanh(const float* x, float* out, size_t n, void* stream) { return run_map1("dh_tanh", x, out, n, stream, OpTanh{}); }
int dh_sigmoid(const float* x, float* out, size_t n, void* stream) { return run_map1("dh_sigmoid", x, out, n, stream, OpSigmoid{}); }

int dh_relu_grad(const float* z, const float* dout, float* out, size_t n, void* stream)
{ return run_map2("dh_relu_grad", z, dout, out, n, stream, OpReluGrad{}); }
int dh_leaky_relu_grad(const float* z, const float* dout, float* out, float alpha, size_t n, void* stream)
{ return run_map2("dh_leaky_relu_grad", z, dout, out, n, stream, OpLeakyGrad{alpha}); }
int dh_tanh_grad(const float* t, const float* dout, float* out, size_t n, void* stream)
{ return run_map2("dh_tanh_grad", t, dout, out, n, stream, OpTanhGrad{}); }
int dh_sigmoid_grad(const float* s, const float* dout, float* out, size_t n, void* stream)
{ return run_map2("dh_sigmoid_grad", s, dout, out, n, stream, OpSigmoidGrad{}); }
int dh_add(const float* a, const float* b, float* out, size_t n, void* stream)
{ return run_map2("dh_add", a, b, out, n, stream, OpAdd{}); }

int dh_sigmoid_cross_entropy(const float* y, const float* logits, float* out, size_t n, void* stream)
{
    DH_TRY(ensure_init());
    if (!y || !logits || !out || n == 0) return fail(DH_EINVAL, "dh_sigmoid_cross_entropy: null tensor or n == 0");
    hipLaunchKernelGGL(mean_reduce<RedSce>, dim3(1), dim3(1024), 0, as_stream(stream), y, logits, out, n, RedSce{});
    DH_LAUNCH_CHECK("dh_sigmoid_cross_entropy");
    return 0;
}

int dh_sigmoid_cross_entropy_grad(const float* y, const float* logits, float* out, size_t n, void* stream)
{ return run_map2("dh_sigmoid_cross_entropy_grad", y, logits, out, n, stream, OpSceGrad{1.f / (float)n}); }

int dh_sigmoid_cross_entropy_head(const float* y1, const float* logits1, float* loss1, float* grad1, const float* y2,
                                  const float* logits2, float* loss2, float* grad2, float* loss_sum, size_t n, void* stream)
{
    DH_TRY(ensure_init());
    const bool two = y2 || logits2 || loss2 || grad2;
    if (!y1 || !logits1 || n == 0 || (two && (!y2 || !logits2)))
        return fail(DH_EINVAL, "dh_sigmoid_cross_entropy_head: null tensor or n == 0");
    if (loss_sum && !two)
        return fail(DH_EINVAL, "dh_sigmoid_cross_entropy_head: a sum of losses needs two logit vectors");
    SceHead h{};
    h.y[0] = y1; h.x[0] = logits1; h.loss[0] = loss1; h.grad[0] = grad1;
    h.y[1] = y2; h.x[1] = logits2; h.loss[1] = loss2; h.grad[1] = grad2;
    h.sum = loss_sum;
    h.count = two ? 2 : 1;
    hipLaunchKernelGGL(sce_head_kernel, dim3(1), dim3(1024), 0, as_stream(stream), h, n);
    DH_LAUNCH_CHECK("dh_sigmoid_cross_entropy_head");
    return 0;
}

int dh_mse(const float* y, const float* y_hat, float* out, size_t rows, size_t cols, void* stream)
{
    DH_TRY(ensure_init());
    if (!y || !y_hat || !out || rows * cols == 0) return fail(DH_EINVAL, "dh_mse: null tensor or empty");
    hipLaunchKernelGGL(mean_reduce<RedMse>, dim3(1), dim3(1024), 0, as_stream(stream), y, y_hat, out, rows * cols, RedMse{});
    DH_LAUNCH_CHECK("dh_mse");
    return 0;
}

int dh_mse_grad(const float* y, const float* y_hat, float* out, size_t n, void* stream)
{ return run_map2("dh_mse_grad", y, y_hat, out, n, stream, OpMseGrad{(float)(2. / (double)n)}); }

int dh_argmax_acc(const float* y, const float* y_hat, float* out, size_t rows, size_t cols, void* stream)
{
    DH_TRY(ensure_init());
    if (!y || !y_hat || !out || cols == 0) return fail(DH_EINVAL, "dh_argmax_acc: null tensor or no columns");
    hipLaunchKernelGGL(argmax_acc_kernel, dim3(1), dim3(1024), 0, as_stream(stream), y, y_hat, out, rows, cols);
    DH_LAUNCH_CHECK("dh_argmax_acc");
    return 0;
}

int dh_moment_update(float* m, const float* g, float a, float b, size_t n, void* stream)
{ return run_map2("dh_moment_update", m, g, m, n, stream, OpMoment{a, b}); }
int dh_moment_update2(float* v, const float* g, float a, float b, size_t n, void* stream)
{ return run_map2("dh_moment_update2", v, g, v, n, stream, OpMoment2{a, b}); }

int dh_adam_update(float* p, const float* m, const float* v, float lrt, float eps, size_t n, void* stream)
{
    DH_TRY(ensure_init());
    if (n == 0) return 0;
    if (!p || !m || !v) return fail(DH_EINVAL, "dh_adam_update: null tensor");
    const bool vec = aligned16(p) && aligned16(m) && aligned16(v);
    hipLaunchKernelGGL(adam_update_kernel, dim3(grid_for(vec ? (n + 3) / 4 : n)), dim3(TPB), 0, as_stream(stream), p, m, v,
                       lrt, eps, n, vec);
    DH_LAUNCH_CHECK("dh_adam_update");
    return 0;
}

int dh_adam_step(float* p, float* m, float* v, const float* g, float m_decay, float m_gain, float v_decay,
                 float v_gain, float lrt, float eps, size_t n, void* stream)
{
    DH_TRY(ensure_init());
    if (n == 0) return 0;
    if (!p || !m || !v || !g) return fail(DH_EINVAL, "dh_adam_step: null tensor");
    const bool vec = aligned16(p) && aligned16(m) && aligned16(v) && aligned16(g);
    ProfScope prof("hbm:adam_step (28 B/param)", 28.0 * n, as_stream(stream));
    hipLaunchKernelGGL(adam_step_kernel, dim3(grid_for(vec ? (n + 3) / 4 : n)), dim3(TPB), 0, as_stream(stream), p, m, v, g,
                       m_decay, m_gain, v_decay, v_gain, lrt, eps, n, vec);
    DH_LAUNCH_CHECK("dh_adam_step");
    return 0;
}

int dh_adam_step_multi(const dh_adam_item* items, int count, float m_decay, float m_gain, float v_decay,
                       float v_gain, float eps, void* stream)
{
    DH_TRY(ensure_init());
    if (count < 0 || (count > 0 && !items)) return fail(DH_EINVAL, "dh_adam_step_multi: bad item list");
    hipStream_t st = as_stream(stream);
    int at = 0;
    while (at < count)
    {
        AdamBatch batch{};
        unsigned blocks = 0;
        double bytes = 0.0;
        for (; at < count && batch.count < ADAM_MAX_ITEMS; ++at)
        {
            const dh_adam_item& it = items[at];
            if (it.n == 0)
                continue;
            if (!it.p || !it.m || !it.v || !it.g1) return fail(DH_EINVAL, "dh_adam_step_multi: null tensor in item %d", at);
            const bool in_parts = it.g1_parts > 1 || (it.g2 && it.g2_parts > 1);
            if (it.g1_parts > 0xffffffffu || it.g2_parts > 0xffffffffu)
                return fail(DH_EINVAL, "dh_adam_step_multi: too many gradient parts in item %d", at);
            const size_t nb = in_parts ? (it.n + TPB / 64 - 1) / (TPB / 64) : (it.n + ADAM_BLOCK - 1) / ADAM_BLOCK;
            if (nb > 0x7fffffffu - blocks) return fail(DH_EINVAL, "dh_adam_step_multi: too many elements");
            const int i = batch.count++;
            batch.p[i] = it.p; batch.m[i] = it.m; batch.v[i] = it.v; batch.g1[i] = it.g1; batch.g2[i] = it.g2;
            batch.n[i] = it.n; batch.lrt[i] = it.lrt;
            batch.parts1[i] = (unsigned)it.g1_parts; batch.parts2[i] = it.g2 ? (unsigned)it.g2_parts : 0;
            batch.vec[i] = aligned16(it.p) && aligned16(it.m) && aligned16(it.v) && aligned16(it.g1) &&
                           (!it.g2 || aligned16(it.g2));
            batch.first_block[i] = blocks;
            blocks += (unsigned)nb;
            bytes += (24.0 + 4.0 * (it.g1_parts > 1 ? it.g1_parts : 1) + (it.g2 ? 4.0 * (it.g2_parts > 1 ? it.g2_parts : 1) : 0.0)) * it.n;
        }
        if (batch.count == 0)
            continue;
        batch.first_block[batch.count] = blocks;
        ProfScope prof("hbm:adam_step_multi (28 B/param, 32 with a second gradient)", bytes, st);
        hipLaunchKernelGGL(adam_step_multi_kernel, dim3(blocks), dim3(TPB), 0, st, batch, m_decay, m_gain, v_decay, v_gain,
                           eps);
        DH_LAUNCH_CHECK("dh_adam_step_multi");
    }
    return 0;
}

int dh_sgd_update(float* var, const float* dv, const float* coeff_device, size_t n, void* stream)
{
    DH_TRY(ensure_init());
    if (n == 0) return 0;
    if (!var || !dv || !coeff_device) return fail(DH_EINVAL, "dh_sgd_update: null tensor");
    hipLaunchKernelGGL(sgd_update_kernel, dim3(grid_for(n)), dim3(TPB), 0, as_stream(stream), var, dv, coeff_device, n);
    DH_LAUNCH_CHECK("dh_sgd_update");
    return 0;
}

}
