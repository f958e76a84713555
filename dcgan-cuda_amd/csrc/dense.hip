// Dense-layer products of the DCGAN (z -> 4*4*512 and 8192 -> 1, and their gradients): well under
// 1 % of an iteration's FLOPs and all of them thin (a batch of 64 rows, a contraction of 1, 64 or
// 100, or a single output column), so what matters is latency, not arithmetic:
//   * gemm_skinny: B has unit stride along its columns and the contraction is short: the A operand
//     (at most 64 rows x 128) is staged in LDS once, every thread streams one column of B;
//   * gemm_block_per_output: few outputs and a long contraction (8192 -> 1): one workgroup per output;
//   * gemm_tiled: everything else, an LDS-tiled FMA kernel with strided operand views.
//
// Reference counterparts: src/gpu/matmul.cu:12-86 (one thread per output, no tiling).
#include "dh_common.h"

#include <type_traits>

using namespace dh;

namespace
{

constexpr int TS = 64;   // output tile
constexpr int KS = 16;   // k slab

// activation applied in the write-out (DH_ACT_NONE: none)
struct Act
{
    int code;
    float alpha;
    __device__ __forceinline__ float operator()(float v) const
    {
        switch (code)
        {
        case DH_ACT_RELU: return v < 0.f ? 0.f : v;
        case DH_ACT_LEAKY: return v < 0.f ? alpha * v : v;
        case DH_ACT_TANH: return tanhf(v);
        case DH_ACT_SIGMOID: return 1.f / (1.f + expf(-v));
        default: return v;
        }
    }
};

// C[i,j] = sum_k A(i,k) * B(k,j) (+ bias[j]),  A(i,k) = a[i*sai + k*sak],  B(k,j) = b[k*sbk + j*sbj]
__global__ __launch_bounds__(256) void gemm_tiled(const float* __restrict__ a, const float* __restrict__ b,
                                                  const float* __restrict__ bias, float* __restrict__ out,
                                                  int M, int K, int P, size_t sai, size_t sak, size_t sbk, size_t sbj, Act act)
{
    __shared__ float la[KS][TS + 1];
    __shared__ float lb[KS][TS + 1];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int i0 = blockIdx.y * TS, j0 = blockIdx.x * TS;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += KS)
    {
        for (int e = threadIdx.x; e < TS * KS; e += 256)
        {
            // pick the index that is contiguous in memory as the fast one
            int ia, ka, kb, jb;
            if (sak == 1) { ka = e % KS; ia = e / KS; } else { ia = e % TS; ka = e / TS; }
            if (sbj == 1) { jb = e % TS; kb = e / TS; } else { kb = e % KS; jb = e / KS; }
            la[ka][ia] = (i0 + ia < M && k0 + ka < K) ? a[(size_t)(i0 + ia) * sai + (size_t)(k0 + ka) * sak] : 0.f;
            lb[kb][jb] = (j0 + jb < P && k0 + kb < K) ? b[(size_t)(k0 + kb) * sbk + (size_t)(j0 + jb) * sbj] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < KS; ++k)
        {
            float ra[4], rb[4];
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                ra[q] = la[k][ty + 16 * q];
                rb[q] = lb[k][tx + 16 * q];
            }
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    acc[q][r] += ra[q] * rb[r];
        }
        __syncthreads();
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int r = 0; r < 4; ++r)
        {
            const int i = i0 + ty + 16 * q, j = j0 + tx + 16 * r;
            if (i < M && j < P)
                out[(size_t)i * P + j] = act(acc[q][r] + (bias ? bias[j] : 0.f));
        }
}

// C[i,j] = sum_k A(i,k) * B(k,j) (+ bias[j]) for K <= SK_MAXK and B(k,j) = b[k*sbk + j] (unit column
// stride).  A workgroup owns 64 columns and 4*RPT rows: wavefront ty accumulates rows
// ty*RPT .. ty*RPT+RPT-1 of column j0+tx; B[k][j0+tx] is one coalesced load per k shared by those rows
// (the loop is bound by latency, so loads and LDS reads of four k are issued before their FMAs), the
// A values are LDS broadcasts read RPT at a time.  RPT = 16 serves a batch of 64 rows, RPT = 1 the products with a
// single row (a vector times a matrix).
constexpr int SK_MAXK = 128;

template <int RPT>
__global__ __launch_bounds__(256) void gemm_skinny(const float* __restrict__ a, const float* __restrict__ b,
                                                   const float* __restrict__ bias, float* __restrict__ out,
                                                   int M, int K, int P, size_t sai, size_t sak, size_t sbk,
                                                   size_t out_si, size_t out_sj, Act act)
{
    constexpr int ROWS = 4 * RPT;
    constexpr int LD = ROWS + 4;   // keeps 16-byte alignment of a wavefront's rows
    __shared__ __attribute__((aligned(16))) float la[SK_MAXK * LD];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int i0 = blockIdx.y * ROWS, j = blockIdx.x * 64 + tx;
    // stage the A block: lanes run along whichever index is contiguous in memory; eight loads in flight
    // per thread (addresses are clamped into the matrix and the value discarded, so that nothing here
    // turns into a branch around a load)
    {
        const bool k_fast = sak == 1;
        const int fast_n = k_fast ? K : ROWS, slow_n = k_fast ? ROWS : K;
        const int fast_steps = (fast_n + 63) / 64;
        const int items = ((slow_n + 3) / 4) * fast_steps;   // (slow index, 64-wide fast segment) pairs of this wavefront
        for (int it0 = 0; it0 < items; it0 += 8)
        {
            float v[8];
            int dst[8];
#pragma unroll
            for (int u = 0; u < 8; ++u)
            {
                const int it = it0 + u;
                const int slow = ty + 4 * (it / fast_steps), fast = tx + 64 * (it % fast_steps);
                const int ia = k_fast ? slow : fast, ka = k_fast ? fast : slow;
                const bool in_tile = it < items && ia < ROWS && ka < K;
                const bool in_matrix = in_tile && i0 + ia < M;
                const size_t off = in_matrix ? (size_t)(i0 + ia) * sai + (size_t)ka * sak : 0;
                const float x = a[off];
                v[u] = in_matrix ? x : 0.f;
                dst[u] = in_tile ? ka * LD + ia : -1;
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (dst[u] >= 0)
                    la[dst[u]] = v[u];
        }
    }
    __syncthreads();
    float acc[RPT] = {};
    if (j < P)
    {
        const float* mine = la + ty * RPT;
        // KB k values at a time: their B loads, then their LDS reads, are all issued before the FMAs
        auto block = [&](int k, auto kb_tag) {
            constexpr int KB = decltype(kb_tag)::value;
            float w[KB];
#pragma unroll
            for (int u = 0; u < KB; ++u)
                w[u] = b[(size_t)(k + u) * sbk + j];
            float x[KB][RPT];
#pragma unroll
            for (int u = 0; u < KB; ++u)
            {
                if (RPT % 4 == 0)
                {
#pragma unroll
                    for (int r = 0; r < RPT; r += 4)
                    {
                        const float4 q = *reinterpret_cast<const float4*>(mine + (k + u) * LD + r);
                        x[u][r] = q.x; x[u][r + 1] = q.y; x[u][r + 2] = q.z; x[u][r + 3] = q.w;
                    }
                }
                else
                {
#pragma unroll
                    for (int r = 0; r < RPT; ++r)
                        x[u][r] = mine[(k + u) * LD + r];
                }
            }
#pragma unroll
            for (int u = 0; u < KB; ++u)
#pragma unroll
                for (int r = 0; r < RPT; ++r)
                    acc[r] = fmaf(x[u][r], w[u], acc[r]);
        };
        int k = 0;
        if (RPT <= 4)   // registers allow sixteen k in flight: a contraction of 64 or 100 is 4 or 7 round trips, not 16 or 25
            for (; k + 16 <= K; k += 16)
                block(k, std::integral_constant<int, 16>{});
        for (; k + 4 <= K; k += 4)
            block(k, std::integral_constant<int, 4>{});
        for (; k < K; ++k)
            block(k, std::integral_constant<int, 1>{});
        const float bj = bias ? bias[j] : 0.f;
#pragma unroll
        for (int r = 0; r < RPT; ++r)
        {
            const int i = i0 + ty * RPT + r;
            if (i < M)
                out[(size_t)i * out_si + (size_t)j * out_sj] = act(acc[r] + bj);
        }
    }
}

// out[j] = sum_k a[k*sak] * B[k*sbk + j] (+ bias[j]): a vector times a matrix with contiguous rows (the
// filter gradient of the 8192 -> 1 layer: 64 logit gradients times the [64 x 8192] activations).  A
// workgroup owns 64 columns; its four wavefronts take a quarter of the contraction each, sixteen loads in
// flight per lane, and wavefront 0 adds the four partial sums in a fixed order.  (gemm_skinny<1> walks
// the whole contraction in one wavefront, four loads at a time, while three wavefronts idle: 10 us
// against 5 for this shape.)
// With a second pair of operands (a2, b2 non-null) the contraction runs over both, K elements each: the
// first two wavefronts take the first pair, the other two the second.
__global__ __launch_bounds__(256) void gemv_rows(const float* __restrict__ a, const float* __restrict__ b,
                                                 const float* __restrict__ a2, const float* __restrict__ b2,
                                                 const float* __restrict__ bias, float* __restrict__ out, int K, int P,
                                                 size_t sak, size_t sbk, Act act)
{
    __shared__ float part[4][64];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int j = blockIdx.x * 64 + tx;
    const int jc = j < P ? j : P - 1;
    const bool two = a2 != nullptr;
    const int shares = two ? 2 : 4;          // wavefronts per pair of operands
    const int kq = (K + shares - 1) / shares;
    const int share = two ? (ty & 1) : ty;
    const float* __restrict__ av = two && ty >= 2 ? a2 : a;
    const float* __restrict__ bm = two && ty >= 2 ? b2 : b;
    const int k0 = share * kq, k1 = K < k0 + kq ? K : k0 + kq;
    float s = 0.f;
    for (int k = k0; k < k1; k += 16)
    {
        float w[16], x[16];
#pragma unroll
        for (int u = 0; u < 16; ++u)
        {
            const bool live = k + u < k1;
            const int kk = live ? k + u : k0;   // a valid row; its product is dropped
            w[u] = bm[(size_t)kk * sbk + jc];
            x[u] = live ? av[(size_t)kk * sak] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 16; ++u)
            s = fmaf(x[u], w[u], s);
    }
    part[ty][tx] = s;
    __syncthreads();
    if (ty == 0 && j < P)
        out[j] = act(((part[0][tx] + part[1][tx]) + part[2][tx]) + part[3][tx] + (bias ? bias[j] : 0.f));
}

// one workgroup per output element: 256 lanes stride over k, then a fixed LDS tree
__global__ __launch_bounds__(256) void gemm_block_per_output(const float* __restrict__ a, const float* __restrict__ b,
                                                             const float* __restrict__ bias, float* __restrict__ out,
                                                             int M, int K, int P, size_t sai, size_t sak, size_t sbk,
                                                             size_t sbj, Act act)
{
    __shared__ float lds[256];
    const size_t o = blockIdx.x;
    const int i = (int)(o / P), j = (int)(o % P);
    float s = 0.f;
    const float* ar = a + (size_t)i * sai;
    const float* bc = b + (size_t)j * sbj;
    if (sak == 1 && sbk == 1 && K % 4 == 0 && ((reinterpret_cast<uintptr_t>(ar) | reinterpret_cast<uintptr_t>(bc)) & 15) == 0)
    {
        // both operands contiguous along k: 16-byte loads
        for (int k = threadIdx.x * 4; k < K; k += 1024)
        {
            const float4 x = *reinterpret_cast<const float4*>(ar + k);
            const float4 y = *reinterpret_cast<const float4*>(bc + k);
            s += x.x * y.x + x.y * y.y + x.z * y.z + x.w * y.w;
        }
    }
    else
        for (int k = threadIdx.x; k < K; k += 256)
            s += ar[(size_t)k * sak] * bc[(size_t)k * sbk];
    lds[threadIdx.x] = s;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1)
    {
        if ((int)threadIdx.x < w) lds[threadIdx.x] += lds[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) out[o] = act(lds[0] + (bias ? bias[j] : 0.f));
    (void)M;
}

int run_gemm(const char* who, const float* a, const float* b, const float* bias, float* out, size_t m, size_t n,
             size_t p, size_t sai, size_t sak, size_t sbk, size_t sbj, void* stream, Act act = Act{DH_ACT_NONE, 0.f})
{
    DH_TRY(ensure_init());
    if (m == 0 || p == 0) return 0;
    if (!a || !b || !out) return fail(DH_EINVAL, "%s: null tensor", who);
    if (m > 0x7fffffff || n > 0x7fffffff || p > 0x7fffffff) return fail(DH_EINVAL, "%s: extent too large", who);
    hipStream_t st = as_stream(stream);
    ProfScope prof("dense gemm", 2.0 * m * n * p, st);
    if (n <= SK_MAXK && sbj == 1 && p >= 64 && m > 4 && ((p + 63) / 64) * ((m + 63) / 64) < 2 * (size_t)num_cus())
    {
        // too few workgroups of 64 rows to fill the device: 16 rows each
        hipLaunchKernelGGL(gemm_skinny<4>, dim3((unsigned)((p + 63) / 64), (unsigned)((m + 15) / 16)), dim3(256), 0, st, a, b,
                           bias, out, (int)m, (int)n, (int)p, sai, sak, sbk, p, (size_t)1, act);
    }
    else if (n <= SK_MAXK && sbj == 1 && p >= 64 && m > 4)
        hipLaunchKernelGGL(gemm_skinny<16>, dim3((unsigned)((p + 63) / 64), (unsigned)((m + 63) / 64)), dim3(256), 0, st, a, b,
                           bias, out, (int)m, (int)n, (int)p, sai, sak, sbk, p, (size_t)1, act);
    else if (n <= SK_MAXK && sbj == 1 && p >= 64 && m == 1)
        hipLaunchKernelGGL(gemv_rows, dim3((unsigned)((p + 63) / 64)), dim3(256), 0, st, a, b, (const float*)nullptr,
                           (const float*)nullptr, bias, out, (int)n, (int)p, sak, sbk, act);
    else if (n <= SK_MAXK && sbj == 1 && p >= 64)
        hipLaunchKernelGGL(gemm_skinny<1>, dim3((unsigned)((p + 63) / 64), 1u), dim3(256), 0, st, a, b, bias, out, (int)m,
                           (int)n, (int)p, sai, sak, sbk, p, (size_t)1, act);
    else if (n <= SK_MAXK && p == 1 && sai == 1 && !bias && m >= 64)
        // a single output column: out[i] = sum_k a[k*sak + i] * b[k*sbk] is the row vector b times the
        // matrix a, whose rows are contiguous -- the same kernel with the roles exchanged
        hipLaunchKernelGGL(gemv_rows, dim3((unsigned)((m + 63) / 64)), dim3(256), 0, st, b, a, (const float*)nullptr,
                           (const float*)nullptr, bias, out, (int)n, (int)m, sbk, sak, act);
    else if (m * p <= 16384 && n >= 512)
        hipLaunchKernelGGL(gemm_block_per_output, dim3((unsigned)(m * p)), dim3(256), 0, st, a, b, bias, out,
                           (int)m, (int)n, (int)p, sai, sak, sbk, sbj, act);
    else
        hipLaunchKernelGGL(gemm_tiled, dim3((unsigned)((p + TS - 1) / TS), (unsigned)((m + TS - 1) / TS)), dim3(256), 0,
                           st, a, b, bias, out, (int)m, (int)n, (int)p, sai, sak, sbk, sbj, act);
    DH_LAUNCH_CHECK(who);
    return 0;
}

}  // namespace

extern "C" {

int dh_gemm_nn(const float* a, const float* b, const float* bias, float* out, size_t m, size_t n, size_t p, void* stream)
{
    return run_gemm("dh_gemm_nn", a, b, bias, out, m, n, p, n, 1, p, 1, stream);
}

int dh_gemm_nn_act(const float* a, const float* b, const float* bias, float* out, size_t m, size_t n, size_t p, int act,
                   float alpha, void* stream)
{
    if (act < DH_ACT_NONE || act > DH_ACT_SIGMOID) return fail(DH_EINVAL, "dh_gemm_nn_act: unknown activation %d", act);
    return run_gemm("dh_gemm_nn_act", a, b, bias, out, m, n, p, n, 1, p, 1, stream, Act{act, alpha});
}

int dh_gemm_tn(const float* a, const float* b, float* out, size_t m, size_t n, size_t p, void* stream)
{
    return run_gemm("dh_gemm_tn", a, b, nullptr, out, m, n, p, 1, m, p, 1, stream);
}

int dh_gemm_tn_pair_supported(size_t m, size_t n, size_t p) { return p == 1 && m >= 64 && n >= 1 && n <= 64 ? 1 : 0; }

int dh_gemm_tn_pair(const float* a1, const float* b1, const float* a2, const float* b2, float* out, size_t m, size_t n,
                    size_t p, void* stream)
{
    DH_TRY(ensure_init());
    if (!a1 || !b1 || !a2 || !b2 || !out) return fail(DH_EINVAL, "dh_gemm_tn_pair: null tensor");
    if (!dh_gemm_tn_pair_supported(m, n, p))
        return fail(DH_ENOTSUP, "dh_gemm_tn_pair: takes a single output column (p == 1) with m >= 64 and n <= 64");
    if (m > 0x7fffffff) return fail(DH_EINVAL, "dh_gemm_tn_pair: extent too large");
    hipStream_t st = as_stream(stream);
    ProfScope prof("dense gemm", 2.0 * m * (2 * n) * p, st);
    // out[i] = sum_k b1[k] * a1[k*m + i] + sum_k b2[k] * a2[k*m + i]: the row vectors b times the matrices a,
    // whose rows are contiguous (see run_gemm's single-output-column case)
    hipLaunchKernelGGL(gemv_rows, dim3((unsigned)((m + 63) / 64)), dim3(256), 0, st, b1, a1, b2, a2, (const float*)nullptr, out,
                       (int)n, (int)m, (size_t)1, m, Act{DH_ACT_NONE, 0.f});
    DH_LAUNCH_CHECK("dh_gemm_tn_pair");
    return 0;
}

int dh_gemm_nt(const float* a, const float* b, float* out, size_t m, size_t n, size_t p, void* stream)
{
    return run_gemm("dh_gemm_nt", a, b, nullptr, out, m, n, p, n, 1, 1, n, stream);
}

}
