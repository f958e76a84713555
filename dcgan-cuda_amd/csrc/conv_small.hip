// Input gradient / transposed convolution onto FEW channels (the image end of the DCGAN: the
// generator's last layer [N,32,32,64] -> [N,64,64,3] and the gradient of the discriminator's first).
// As an implicit GEMM this product has an n extent of 3, which leaves a 32-wide MFMA tile 90 % empty
// and re-reads the dy operand once per filter tap; here it runs on the vector ALUs instead:
//
//   * a workgroup owns an (8*sh) x (8*sw) patch of output pixels of one image and first copies the
//     dy pixels that patch depends on (all channels of a 64-wide channel block) into LDS, once;
//   * each wavefront takes one output phase (h mod sh, w mod sw) of the patch, one output pixel per
//     lane: all 64 lanes then use the same filter taps, so the filter values are wave-uniform and
//     are fetched through the scalar path while the dy values come from LDS as 16-byte reads;
//   * bias and activation are applied before the single store of each output pixel.
//
// Reference counterpart: kernel_conv2d_input_grad / kernel_conv2d_transpose (src/gpu/conv2d.cu:70-117,
// 167-212), which dilate dy with zeros and run a dense im2col GEMM over it.
#include "dh_common.h"

using namespace dh;

namespace
{

constexpr int QUADS = 8;          // output pixels per phase along each axis of a patch
constexpr int OC = 64;            // dy channels staged per pass
constexpr int OCP = OC + 4;       // LDS pixel stride: 16-byte aligned, conflict-free for 8 neighbouring pixels
constexpr int MAX_PATCH = 12;     // dy rows / columns a patch may depend on

struct SmallDxParams
{
    const float* dy;
    const float* k;
    float* dx;
    const float* bias;
    int act;
    float alpha;
    int N, Ho, Wo, O, kh, kw, C, sh, sw, pt, pl, H, W;
    int lo_h, lo_w;       // first dy row / column of a patch, relative to (patch origin / stride)
    int pr, pc;           // dy rows / columns per patch
    int tiles_h, tiles_w;
};

// The filter is read-only for the whole launch and every lane of a wavefront reads the same
// element: a pointer into the constant address space makes these loads scalar (one fetch per
// wavefront into scalar registers, which then feed the FMAs directly).
typedef const float __attribute__((address_space(4))) * uniform_p;

__device__ __forceinline__ float act_apply(float v, int act, float alpha)
{
    switch (act)
    {
    case DH_ACT_RELU: return v < 0.f ? 0.f : v;
    case DH_ACT_LEAKY: return v < 0.f ? alpha * v : v;
    case DH_ACT_TANH: return tanhf(v);
    case DH_ACT_SIGMOID: return 1.f / (1.f + expf(-v));
    default: return v;
    }
}

template <int CC>
__global__ __launch_bounds__(256) void dx_few_channels(const SmallDxParams p)
{
    __shared__ __attribute__((aligned(16))) float patch[MAX_PATCH * MAX_PATCH * OCP];

    const int tile = blockIdx.x;
    const int b = tile / (p.tiles_h * p.tiles_w);
    const int trem = tile - b * (p.tiles_h * p.tiles_w);
    const int ty = trem / p.tiles_w, tx = trem - ty * p.tiles_w;
    // patch origin in units of stride-sized pixel blocks, and the first dy row/column it needs
    const int qh0 = ty * QUADS, qw0 = tx * QUADS;
    const int i0 = qh0 + p.lo_h, j0 = qw0 + p.lo_w;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int qy = lane >> 3, qx = lane & 7;
    const int nph = p.sh * p.sw;

    for (int phase0 = 0; phase0 < nph; phase0 += 4)
    {
        // wave-uniform description of this wavefront's phase (inactive when past the last phase)
        const int phase = phase0 + wave;
        const bool live = phase < nph;
        const int ph = live ? phase / p.sw : 0, pw = live ? phase - (phase / p.sw) * p.sw : 0;
        const int rh = (ph + p.pt) % p.sh, rw = (pw + p.pl) % p.sw;
        const int q0h = (ph + p.pt) / p.sh, q0w = (pw + p.pl) / p.sw;
        const int nth = live && rh < p.kh ? (p.kh - rh + p.sh - 1) / p.sh : 0;
        const int ntw = live && rw < p.kw ? (p.kw - rw + p.sw - 1) / p.sw : 0;

        float acc[CC];
#pragma unroll
        for (int c = 0; c < CC; ++c)
            acc[c] = 0.f;

        for (int o0 = 0; o0 < p.O; o0 += OC)
        {
            // ---- stage dy[b, i0.., j0.., o0..o0+OC) into LDS (zero outside the tensor) ----
            __syncthreads();
            const int chunks = p.pr * p.pc * (OC / 4);
            for (int e = threadIdx.x; e < chunks; e += 256)
            {
                const int pix = e / (OC / 4), o4 = (e - pix * (OC / 4)) * 4;
                const int li = pix / p.pc, lj = pix - li * p.pc;
                const int i = i0 + li, j = j0 + lj;
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if ((unsigned)i < (unsigned)p.Ho && (unsigned)j < (unsigned)p.Wo && o0 + o4 < p.O)
                    v = *reinterpret_cast<const float4*>(p.dy + (((size_t)b * p.Ho + i) * p.Wo + j) * p.O + o0 + o4);
                *reinterpret_cast<float4*>(&patch[pix * OCP + o4]) = v;
            }
            __syncthreads();

            // ---- every lane: its pixel's taps, all staged channels ----
            const int ocount = min(OC, p.O - o0);
            for (int th = 0; th < nth; ++th)
            {
                const int li = qy + q0h - th - p.lo_h;
                for (int tw = 0; tw < ntw; ++tw)
                {
                    const int lj = qx + q0w - tw - p.lo_w;
                    const float* src = &patch[(li * p.pc + lj) * OCP];
                    const int di = rh + p.sh * th, dj = rw + p.sw * tw;
                    const uniform_p wt =
                        (uniform_p)(p.k + ((size_t)(di * p.kw + dj) * p.C) * p.O + o0);   // wave-uniform
                    int o = 0;
                    for (; o + 16 <= ocount; o += 16)
                    {
                        float4 d[4];
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            d[q] = *reinterpret_cast<const float4*>(src + o + 4 * q);
#pragma unroll
                        for (int c = 0; c < CC; ++c)
                        {
                            const uniform_p wc = wt + (size_t)c * p.O + o;
#pragma unroll
                            for (int q = 0; q < 4; ++q)
                            {
                                acc[c] = fmaf(d[q].x, wc[4 * q + 0], acc[c]);
                                acc[c] = fmaf(d[q].y, wc[4 * q + 1], acc[c]);
                                acc[c] = fmaf(d[q].z, wc[4 * q + 2], acc[c]);
                                acc[c] = fmaf(d[q].w, wc[4 * q + 3], acc[c]);
                            }
                        }
                    }
                    for (; o < ocount; o += 4)
                    {
                        const float4 d = *reinterpret_cast<const float4*>(src + o);
#pragma unroll
                        for (int c = 0; c < CC; ++c)
                        {
                            const uniform_p wc = wt + (size_t)c * p.O + o;
                            acc[c] = fmaf(d.x, wc[0], acc[c]);
                            acc[c] = fmaf(d.y, wc[1], acc[c]);
                            acc[c] = fmaf(d.z, wc[2], acc[c]);
                            acc[c] = fmaf(d.w, wc[3], acc[c]);
                        }
                    }
                }
            }
        }

        const int h = (qh0 + qy) * p.sh + ph, w = (qw0 + qx) * p.sw + pw;
        if (live && h < p.H && w < p.W)
        {
            float* dst = p.dx + (((size_t)b * p.H + h) * p.W + w) * p.C;
#pragma unroll
            for (int c = 0; c < CC; ++c)
                dst[c] = act_apply(acc[c] + (p.bias ? p.bias[c] : 0.f), p.act, p.alpha);
        }
    }
}

// ---- forward from a thin input: contraction of at most 80 ----------------------------------------
// The discriminator's first layer, [N,64,64,3] -> [N,32,32,64] with a 5x5 filter: the contraction is
// only kh*kw*C = 75 long and a pixel is 12 bytes, so the tiled kernel spends its time on scalar
// gathers into LDS.  Here the MFMA operands never pass through LDS: lane (m, h) of a wavefront owns
// output pixel m of a 32-pixel tile and loads ITS patch values k = h*40 + j straight from global
// memory into the register that MFMA number j consumes; the filter (at most 80 x 64 values) is
// staged in LDS once per workgroup and read from there, one value per lane and MFMA.  A wavefront
// computes TF_TILES tiles.
typedef float f32x16 __attribute__((ext_vector_type(16)));
constexpr int TF_KH = 40;           // MFMAs per 32-output-channel block; the contraction is padded to 2 * TF_KH
constexpr int TF_NB = 2;            // 32-channel blocks: up to 64 output channels
constexpr int TF_TILES = 1;         // 32-pixel tiles per wavefront

struct ThinFwdParams
{
    const float* x;
    const float* k;
    float* y;
    const float* bias;
    int act;
    float alpha;
    int N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pt, pl;
    int K, row;             // kh*kw*C and kw*C (one filter row of taps)
    int pixels;             // N*Ho*Wo
    uint32_t x_bytes;
    FastDiv fd_HoWo, fd_Wo, fd_row, fd_C;
};

__global__ __launch_bounds__(256) void fwd_thin(const ThinFwdParams p)
{
    __shared__ float filt[2 * TF_KH * 32 * TF_NB];   // [k][n], zero beyond K and O
    {
        // all of a thread's filter loads in flight together (out-of-range elements read element 0 and
        // are replaced by zero: no branch around a load)
        constexpr int PER_THREAD = 2 * TF_KH * 32 * TF_NB / 256;
        float v[PER_THREAD];
#pragma unroll
        for (int u = 0; u < PER_THREAD; ++u)
        {
            const int e = threadIdx.x + u * 256;
            const int k = e / (32 * TF_NB), n = e - k * (32 * TF_NB);
            const bool ok = k < p.K && n < p.O;
            const float w = p.k[ok ? (size_t)k * p.O + n : 0];
            v[u] = ok ? w : 0.f;
        }
#pragma unroll
        for (int u = 0; u < PER_THREAD; ++u)
            filt[threadIdx.x + u * 256] = v[u];
    }
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const float* bw = filt + half * TF_KH * (32 * TF_NB) + l32;   // + q * 64 + nb * 32

    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.x), 0, (int)p.x_bytes, 0x00020000);
    const int tiles = (p.pixels + 31) / 32;
#pragma unroll 1
    for (int u = 0; u < TF_TILES; ++u)
    {
        const int tile = (blockIdx.x * 4 + wave) * TF_TILES + u;
        if (tile >= tiles)
            break;
        const int pix = tile * 32 + l32;
        const bool live = pix < p.pixels;
        uint32_t b, rem, i, j;
        p.fd_HoWo.divmod(live ? pix : 0, b, rem);
        p.fd_Wo.divmod(rem, i, j);
        const int h0 = (int)i * p.sh - p.pt, w0 = (int)j * p.sw - p.pl;
        const int base = (((int)b * p.H + h0) * p.W + w0) * p.C * 4;

        float a[TF_KH];
#pragma unroll
        for (int q = 0; q < TF_KH; ++q)
        {
            const int k = half * TF_KH + q;
            uint32_t di, t, dj, c;
            p.fd_row.divmod(k, di, t);
            p.fd_C.divmod(t, dj, c);
            const bool ok = (int)live & (int)(k < p.K) & (int)((unsigned)(h0 + (int)di) < (unsigned)p.H) &
                            (int)((unsigned)(w0 + (int)dj) < (unsigned)p.W);
            const int off = ok ? base + ((int)di * p.W * p.C + (int)t) * 4 : (int)0x80000000u;
            a[q] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xr, off, 0, 0));
        }
        f32x16 acc[TF_NB];
#pragma unroll
        for (int nb = 0; nb < TF_NB; ++nb)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[nb][r] = 0.f;
#pragma unroll
        for (int q = 0; q < TF_KH; ++q)
#pragma unroll
            for (int nb = 0; nb < TF_NB; ++nb)
                acc[nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(bw[q * (32 * TF_NB) + nb * 32], a[q], acc[nb], 0, 0, 0);

        // register r of lane (m, h) holds channel 32*nb + 8*(r/4) + 4*h + r%4 of pixel m
        if (live)
        {
            float* dst = p.y + (size_t)pix * p.O;
#pragma unroll
            for (int nb = 0; nb < TF_NB; ++nb)
#pragma unroll
                for (int g = 0; g < 4; ++g)
                {
                    const int n = nb * 32 + 8 * g + 4 * half;
                    if (n >= p.O)
                        continue;
                    float4 v = make_float4(acc[nb][4 * g], acc[nb][4 * g + 1], acc[nb][4 * g + 2], acc[nb][4 * g + 3]);
                    if (p.bias)
                    {
                        const float4 bb = *reinterpret_cast<const float4*>(p.bias + n);
                        v.x += bb.x; v.y += bb.y; v.z += bb.z; v.w += bb.w;
                    }
                    v.x = act_apply(v.x, p.act, p.alpha); v.y = act_apply(v.y, p.act, p.alpha);
                    v.z = act_apply(v.z, p.act, p.alpha); v.w = act_apply(v.w, p.act, p.alpha);
                    *reinterpret_cast<float4*>(dst + n) = v;
                }
        }
    }
}

}  // namespace

namespace dh
{

// Returns 1 when the shape is not one this kernel takes (the caller then uses the implicit GEMM),
// 0 after a launch, or an error code.
int conv_fwd_thin(const float* x, const float* k, float* y, int N, int H, int W, int C, int kh, int kw, int O, int sh,
                  int sw, int pt, int pl, int Ho, int Wo, const float* bias, int act, float alpha, hipStream_t st)
{
    const long K = (long)kh * kw * C;
    const size_t x_bytes = (size_t)N * H * W * C * 4;
    if (K > 2 * TF_KH || C > 4 || O > 32 * TF_NB || O % 4 != 0 || x_bytes >= (size_t(1) << 31) ||
        (reinterpret_cast<uintptr_t>(y) & 15) != 0 || (reinterpret_cast<uintptr_t>(bias) & 15) != 0)
        return 1;
    ThinFwdParams p{};
    p.x = x; p.k = k; p.y = y; p.bias = bias; p.act = act; p.alpha = alpha;
    p.N = N; p.H = H; p.W = W; p.C = C; p.Ho = Ho; p.Wo = Wo; p.O = O; p.kh = kh; p.kw = kw;
    p.sh = sh; p.sw = sw; p.pt = pt; p.pl = pl;
    p.K = (int)K; p.row = kw * C;
    p.pixels = N * Ho * Wo;
    p.x_bytes = (uint32_t)x_bytes;
    p.fd_HoWo = FastDiv((uint32_t)Ho * Wo); p.fd_Wo = FastDiv(Wo); p.fd_row = FastDiv(kw * C); p.fd_C = FastDiv(C);
    const long blocks = ((long)(p.pixels + 31) / 32 + 4 * TF_TILES - 1) / (4 * TF_TILES);
    if (blocks > 0x7fffffffL)
        return 1;
    const int prof = prof_begin("fwd_thin", 2.0 * N * Ho * Wo * O * kh * kw * C, st);
    hipLaunchKernelGGL(fwd_thin, dim3((unsigned)blocks), dim3(256), 0, st, p);
    prof_end(prof, st);
    DH_LAUNCH_CHECK("fwd_thin launch");
    return 0;
}



// Returns 1 when the shape is not one this kernel takes (the caller then uses the implicit GEMM),
// 0 after a launch, or an error code.
int conv_dx_few_channels(const float* dy, const float* k, float* dx, int N, int Ho, int Wo, int O, int kh, int kw,
                         int C, int sh, int sw, int pt, int pl, int H, int W, const float* bias, int act,
                         float alpha, hipStream_t st)
{
    if (C > 4 || O % 4 != 0 || sh * sw < 2 || (reinterpret_cast<uintptr_t>(dy) & 15) != 0)
        return 1;
    SmallDxParams p{};
    p.dy = dy; p.k = k; p.dx = dx; p.bias = bias; p.act = act; p.alpha = alpha;
    p.N = N; p.Ho = Ho; p.Wo = Wo; p.O = O; p.kh = kh; p.kw = kw; p.C = C; p.sh = sh; p.sw = sw;
    p.pt = pt; p.pl = pl; p.H = H; p.W = W;
    // dy rows a patch depends on: i = quad + q0 - t over all phases and taps
    int lo_h = 1 << 30, hi_h = -(1 << 30), lo_w = 1 << 30, hi_w = -(1 << 30);
    for (int ph = 0; ph < sh; ++ph)
    {
        const int rh = (ph + pt) % sh, q0 = (ph + pt) / sh;
        const int nt = rh < kh ? (kh - rh + sh - 1) / sh : 0;
        if (nt == 0) continue;
        if (q0 - (nt - 1) < lo_h) lo_h = q0 - (nt - 1);
        if (q0 + QUADS - 1 > hi_h) hi_h = q0 + QUADS - 1;
    }
    for (int pw = 0; pw < sw; ++pw)
    {
        const int rw = (pw + pl) % sw, q0 = (pw + pl) / sw;
        const int nt = rw < kw ? (kw - rw + sw - 1) / sw : 0;
        if (nt == 0) continue;
        if (q0 - (nt - 1) < lo_w) lo_w = q0 - (nt - 1);
        if (q0 + QUADS - 1 > hi_w) hi_w = q0 + QUADS - 1;
    }
    if (hi_h < lo_h || hi_w < lo_w)
        return 1;   // no tap at all: left to the general path
    p.lo_h = lo_h; p.lo_w = lo_w;
    p.pr = hi_h - lo_h + 1; p.pc = hi_w - lo_w + 1;
    if (p.pr > MAX_PATCH || p.pc > MAX_PATCH)
        return 1;
    p.tiles_h = (H + QUADS * sh - 1) / (QUADS * sh);
    p.tiles_w = (W + QUADS * sw - 1) / (QUADS * sw);
    const long tiles = (long)N * p.tiles_h * p.tiles_w;
    if (tiles > 0x7fffffffL)
        return 1;
    const int prof = prof_begin("dx_few_channels", 2.0 * N * Ho * Wo * O * kh * kw * C, st);
    switch (C)
    {
    case 1: hipLaunchKernelGGL(dx_few_channels<1>, dim3((unsigned)tiles), dim3(256), 0, st, p); break;
    case 2: hipLaunchKernelGGL(dx_few_channels<2>, dim3((unsigned)tiles), dim3(256), 0, st, p); break;
    case 3: hipLaunchKernelGGL(dx_few_channels<3>, dim3((unsigned)tiles), dim3(256), 0, st, p); break;
    default: hipLaunchKernelGGL(dx_few_channels<4>, dim3((unsigned)tiles), dim3(256), 0, st, p); break;
    }
    prof_end(prof, st);
    DH_LAUNCH_CHECK("dx_few_channels launch");
    return 0;
}

}  // namespace dh
