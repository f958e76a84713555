// Dense-layer products of the DCGAN (z -> 4*4*512 and 8192 -> 1, and their gradients): well under
// 1 % of an iteration's FLOPs, so a compact LDS-tiled FMA kernel with strided operand views covers
// A*B, tr(A)*B and A*tr(B); tall-skinny products with few outputs and a long contraction (8192 -> 1)
// use one workgroup per output instead.
//
// Reference counterparts: src/gpu/matmul.cu:12-86 (one thread per output, no tiling).
#include "dh_common.h"

using namespace dh;

namespace
{

constexpr int TS = 64;   // output tile
constexpr int KS = 16;   // k slab

// C[i,j] = sum_k A(i,k) * B(k,j) (+ bias[j]),  A(i,k) = a[i*sai + k*sak],  B(k,j) = b[k*sbk + j*sbj]
__global__ __launch_bounds__(256) void gemm_tiled(const float* __restrict__ a, const float* __restrict__ b,
                                                  const float* __restrict__ bias, float* __restrict__ out,
                                                  int M, int K, int P, size_t sai, size_t sak, size_t sbk, size_t sbj)
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
                out[(size_t)i * P + j] = acc[q][r] + (bias ? bias[j] : 0.f);
        }
}

// one workgroup per output element: 256 lanes stride over k, then a fixed LDS tree
__global__ __launch_bounds__(256) void gemm_block_per_output(const float* __restrict__ a, const float* __restrict__ b,
                                                             const float* __restrict__ bias, float* __restrict__ out,
                                                             int M, int K, int P, size_t sai, size_t sak, size_t sbk,
                                                             size_t sbj)
{
    __shared__ float lds[256];
    const size_t o = blockIdx.x;
    const int i = (int)(o / P), j = (int)(o % P);
    float s = 0.f;
    for (int k = threadIdx.x; k < K; k += 256)
        s += a[(size_t)i * sai + (size_t)k * sak] * b[(size_t)k * sbk + (size_t)j * sbj];
    lds[threadIdx.x] = s;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1)
    {
        if ((int)threadIdx.x < w) lds[threadIdx.x] += lds[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) out[o] = lds[0] + (bias ? bias[j] : 0.f);
    (void)M;
}

int run_gemm(const char* who, const float* a, const float* b, const float* bias, float* out, size_t m, size_t n,
             size_t p, size_t sai, size_t sak, size_t sbk, size_t sbj, void* stream)
{
    DH_TRY(ensure_init());
    if (m == 0 || p == 0) return 0;
    if (!a || !b || !out) return fail(DH_EINVAL, "%s: null tensor", who);
    if (m > 0x7fffffff || n > 0x7fffffff || p > 0x7fffffff) return fail(DH_EINVAL, "%s: extent too large", who);
    hipStream_t st = as_stream(stream);
    ProfScope prof("dense gemm", 2.0 * m * n * p, st);
    if (m * p <= 4096 && n >= 512)
        hipLaunchKernelGGL(gemm_block_per_output, dim3((unsigned)(m * p)), dim3(256), 0, st, a, b, bias, out,
                           (int)m, (int)n, (int)p, sai, sak, sbk, sbj);
    else
        hipLaunchKernelGGL(gemm_tiled, dim3((unsigned)((p + TS - 1) / TS), (unsigned)((m + TS - 1) / TS)), dim3(256), 0,
                           st, a, b, bias, out, (int)m, (int)n, (int)p, sai, sak, sbk, sbj);
    DH_LAUNCH_CHECK(who);
    return 0;
}

}  // namespace

extern "C" {

int dh_gemm_nn(const float* a, const float* b, const float* bias, float* out, size_t m, size_t n, size_t p, void* stream)
{
    return run_gemm("dh_gemm_nn", a, b, bias, out, m, n, p, n, 1, p, 1, stream);
}

int dh_gemm_tn(const float* a, const float* b, float* out, size_t m, size_t n, size_t p, void* stream)
{
    return run_gemm("dh_gemm_tn", a, b, nullptr, out, m, n, p, 1, m, p, 1, stream);
}

int dh_gemm_nt(const float* a, const float* b, float* out, size_t m, size_t n, size_t p, void* stream)
{
    return run_gemm("dh_gemm_nt", a, b, nullptr, out, m, n, p, n, 1, 1, n, stream);
}

}
