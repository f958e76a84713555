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
        // which of the four phases of this round the wavefront takes rotates with the workgroup: the
        // phases differ in length (9, 6, 6 and 4 taps for 5x5 stride 2) and wavefront w of every workgroup
        // tends to land on the same SIMD, which would otherwise get all the long ones (measured: 1 %)
        const int phase = phase0 + ((wave + (int)blockIdx.x) & 3);
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
// staged in LDS once per workgroup and read from there, one value per lane and MFMA.  Workgroups are
// persistent (two per compute unit, two wavefronts per SIMD): a wavefront walks over tiles with the
// loads of its next tile issued before the MFMAs of the current one, so that one wavefront of a SIMD
// multiplies while the other waits for memory or writes its tile out.
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4v __attribute__((ext_vector_type(4)));
constexpr int TF_KH = 40;           // MFMAs per 32-output-channel block; the contraction is padded to 2 * TF_KH
constexpr int TF_NB = 2;            // 32-channel blocks: up to 64 output channels

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
    int tiles;              // 32-pixel tiles
    uint32_t x_bytes;
    FastDiv fd_HoWo, fd_Wo, fd_row, fd_C;
};

// ROWS: the contraction index is laid out as filter row x 16 (k' = di*16 + dj*C + c; needs kw*C <= 16
// and kh*16 <= 2*TF_KH), so that a lane's 40 values are ten 16-byte loads of consecutive floats of its
// input rows instead of forty 4-byte loads -- a quarter of the load instructions for the same lines.
// Elements of a 16-byte load that belong to no tap (the 16th of a row, columns in the padding) are
// replaced by zero after the load; the buffer descriptor's range check is per dword, so a load that
// runs past the end of the tensor still delivers its in-range elements.
template <bool ROWS>
__global__ __launch_bounds__(256, 2) void fwd_thin(const ThinFwdParams p)
{
    __shared__ float filt[2 * TF_KH * 32 * TF_NB];   // [k][n], zero beyond K and O
    __shared__ __attribute__((aligned(16))) float lbias[32 * TF_NB];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const float* bw = filt + half * TF_KH * (32 * TF_NB) + l32;   // + q * 64 + nb * 32

    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.x), 0, (int)p.x_bytes, 0x00020000);

    // Patch of this lane's pixel of `tile`, in two halves so that the round trip to memory lies behind
    // the MFMAs of the tile before: issue() sends the loads (raw 16-byte pieces for ROWS, the values
    // themselves otherwise; nothing is in range for a tile past the last one), finish() -- called when
    // the values are needed -- replaces the elements that belong to no tap by zero.
    struct Pixel { int h0, w0, base; bool live, corner; };
    auto pixel_of = [&](int tile) {
        const int pix = tile * 32 + l32;
        Pixel px;
        px.live = tile < p.tiles && pix < p.pixels;
        uint32_t b, rem, i, j;
        p.fd_HoWo.divmod(px.live ? pix : 0, b, rem);
        p.fd_Wo.divmod(rem, i, j);
        px.h0 = (int)i * p.sh - p.pt;
        px.w0 = (int)j * p.sw - p.pl;
        px.base = (((int)b * p.H + px.h0) * p.W + px.w0) * p.C * 4;
        // Pixels of the first image whose patch has padding on its left and holds input row 0: the
        // 16-byte load of that row would begin before the tensor (a negative offset, which the range
        // check rejects as a whole, in-range elements included).  Those few pixels take 4-byte loads.
        px.corner = px.live && b == 0 && px.h0 <= 0 && px.w0 < 0;
        return px;
    };
    // per-lane constants of the ten 16-byte chunks: byte offset within the patch (far out of range for
    // a chunk whose filter row does not exist) and filter row
    constexpr int FAR = (int)0xC0000000u;     // + any patch offset stays above every tensor size (< 2 GiB)
    int chunk_off[TF_KH / 4], chunk_di[TF_KH / 4];
#pragma unroll
    for (int u = 0; u < TF_KH / 4; ++u)
    {
        const int k0 = half * TF_KH + 4 * u;        // first k' of the chunk
        const int di = k0 >> 4, t0 = k0 & 15;
        chunk_di[u] = di;
        chunk_off[u] = di < p.kh ? (di * p.W * p.C + t0) * 4 : FAR;
    }
    auto issue = [&](const Pixel& px, f32x4v (&raw)[TF_KH / 4], float (&a)[TF_KH]) {
        if (ROWS)
        {
            const int base = px.live ? px.base : FAR;
#pragma unroll
            for (int u = 0; u < TF_KH / 4; ++u)
            {
                const bool row_ok = (unsigned)(px.h0 + chunk_di[u]) < (unsigned)p.H;
                const int off = row_ok ? base + chunk_off[u] : FAR;
                raw[u] = __builtin_bit_cast(f32x4v, __builtin_amdgcn_raw_buffer_load_b128(xr, off, 0, 0));
            }
        }
        else
        {
#pragma unroll
            for (int q = 0; q < TF_KH; ++q)
            {
                const int k = half * TF_KH + q;
                uint32_t di, t, dj, c;
                p.fd_row.divmod(k, di, t);
                p.fd_C.divmod(t, dj, c);
                const bool ok = (int)px.live & (int)(k < p.K) & (int)((unsigned)(px.h0 + (int)di) < (unsigned)p.H) &
                                (int)((unsigned)(px.w0 + (int)dj) < (unsigned)p.W);
                const int off = ok ? px.base + ((int)di * p.W * p.C + (int)t) * 4 : (int)0x80000000u;
                a[q] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xr, off, 0, 0));
            }
        }
    };
    auto finish = [&](const Pixel& px, const f32x4v (&raw)[TF_KH / 4], float (&a)[TF_KH]) {
        if (!ROWS)
            return;
        // Element q of the lane is column t = (q + 8*half) mod 16 of its filter row; the columns that
        // meet the image are tlo <= t < thi.  As a 16-bit mask rotated by the lane's 8*half, the bit
        // of element q is bit q mod 16 -- a compile-time position: two ALU operations per element, no
        // branches, and a NaN in a dropped element does not propagate (bitwise and).
        const int tlo = max(0, -px.w0) * p.C, thi = min(p.row, (p.W - px.w0) * p.C);
        uint32_t cols = thi > tlo ? ((1u << thi) - 1u) & ~((1u << tlo) - 1u) : 0u;
        cols = half ? ((cols >> 8) | (cols << 8)) & 0xffffu : cols;
#pragma unroll
        for (int u = 0; u < TF_KH / 4; ++u)
#pragma unroll
            for (int e = 0; e < 4; ++e)
            {
                const int q = 4 * u + e;
                const uint32_t keep = (uint32_t)__builtin_amdgcn_sbfe((int)cols, q & 15, 1);   // 0 or all ones
                const float v = raw[u][e];   // (a copy: bit_cast of a vector-element lvalue reads element 0)
                a[q] = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v) & keep);
            }
        if (px.corner)
        {
#pragma unroll
            for (int q = 0; q < TF_KH; ++q)
            {
                const int kq = half * TF_KH + q;
                const int di = kq >> 4, t = kq & 15;
                const int dj = (int)p.fd_C.div((uint32_t)t);
                const bool ok = (int)(di < p.kh) & (int)(t < p.row) & (int)((unsigned)(px.h0 + di) < (unsigned)p.H) &
                                (int)((unsigned)(px.w0 + dj) < (unsigned)p.W);
                const int off = ok ? px.base + (di * p.W * p.C + t) * 4 : (int)0x80000000u;
                a[q] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xr, off, 0, 0));
            }
        }
    };

    // The wavefront's tiles: wave w of workgroup g takes tiles g*4 + w, + 4*gridDim.x, ...  The patch
    // loads of the first are issued before the filter is staged, so that the two round trips to memory
    // overlap; inside the loop the loads of the NEXT tile are issued before the MFMAs of the current
    // one, so that a wavefront always has a tile's loads in flight while it multiplies and stores.
    const int stride = (int)gridDim.x * 4;
    int tile = (int)blockIdx.x * 4 + wave;
    float a[TF_KH];
    f32x4v raw[TF_KH / 4];
    Pixel px = pixel_of(tile);
    issue(px, raw, a);
    {
        // all of a thread's filter loads in flight together (out-of-range elements read element 0 and
        // are replaced by zero: no branch around a load)
        constexpr int PER_THREAD = 2 * TF_KH * 32 * TF_NB / 256;
        float v[PER_THREAD];
#pragma unroll
        for (int u = 0; u < PER_THREAD; ++u)
        {
            const int e = threadIdx.x + u * 256;
            int k = e / (32 * TF_NB);
            const int n = e - k * (32 * TF_NB);
            bool ok = k < p.K && n < p.O;
            if (ROWS)
            {
                // k' = di*16 + t  ->  element (di*row + t) of the filter
                const int di = k >> 4, t = k & 15;
                ok = di < p.kh && t < p.row && n < p.O;
                k = di * p.row + t;
            }
            const float w = p.k[ok ? (size_t)k * p.O + n : 0];
            v[u] = ok ? w : 0.f;
        }
#pragma unroll
        for (int u = 0; u < PER_THREAD; ++u)
            filt[threadIdx.x + u * 256] = v[u];
    }
    if (threadIdx.x < 32 * TF_NB)
        lbias[threadIdx.x] = (p.bias && (int)threadIdx.x < p.O) ? p.bias[threadIdx.x] : 0.f;
    __syncthreads();

    for (; tile < p.tiles; tile += stride)
    {
        // (the filter values are read from LDS in every round: kept in registers across the loop they
        // would take 160 of them and halve the wavefronts a SIMD holds)
        asm volatile("" ::: "memory");
        finish(px, raw, a);
        px = pixel_of(tile + stride);
        float a_next[TF_KH];
        issue(px, raw, a_next);
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
        const int pix = tile * 32 + l32;
        if (pix < p.pixels)
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
                    const float4 bb = *reinterpret_cast<const float4*>(lbias + n);
                    float4 v = make_float4(acc[nb][4 * g], acc[nb][4 * g + 1], acc[nb][4 * g + 2], acc[nb][4 * g + 3]);
                    v.x += bb.x; v.y += bb.y; v.z += bb.z; v.w += bb.w;
                    v.x = act_apply(v.x, p.act, p.alpha); v.y = act_apply(v.y, p.act, p.alpha);
                    v.z = act_apply(v.z, p.act, p.alpha); v.w = act_apply(v.w, p.act, p.alpha);
                    *reinterpret_cast<float4*>(dst + n) = v;
                }
        }
        if (!ROWS)
        {
#pragma unroll
            for (int q = 0; q < TF_KH; ++q)
                a[q] = a_next[q];
        }
    }
}



// ---- filter gradient of a thin input ------------------------------------------------------------
// dk[(di,dj,c), o] = sum over pixels of x[b, i*sh+di-pt, j*sw+dj-pl, c] * dy[b,i,j,o] for a filter
// with at most 80 elements per output channel and at most 64 output channels (the discriminator's
// first layer: 75 x 64).  As an implicit GEMM it is a 75-row product whose "im2col" operand has to
// be gathered element by element (3 channels); here a wavefront takes segments of 16 neighbouring
// output pixels of one image row and stages, per segment, the kh input rows they touch and their
// 16 dy pixels in LDS.  Element ((di, dj, c), j) of the gathered operand is then
//     patch[di][(dj*C + c) + j*sw*C]
// -- a strided view of the staged rows, read straight into the MFMA registers with no gather at all.
// The result is tiled 5 x 4 by 16x16x4 MFMAs (80 x 64: 6 % padding for the 75-row filter, where 32-wide
// tiles would waste 22 %).  Each wavefront has staging memory of its own and LDS operations of one
// wavefront execute in order, so the segment loop needs no barrier: a wavefront writes segment s+1 over
// segment s as soon as its own fragment reads of s are issued, and the global loads of the segment after
// are in flight meanwhile.  Two wavefronts share a SIMD.  The eight wavefronts of a workgroup add their
// accumulators through LDS in wavefront order; each workgroup writes one slice of partial sums, which
// the caller adds up (fixed order, so the result is repeatable to the bit).
typedef float dt_f32x4 __attribute__((ext_vector_type(4)));
constexpr int DT_SEG = 16;                    // output pixels per segment
constexpr int DT_XMAX = 640;                  // floats of one staged input patch (kh rows)
constexpr int DT_OMAX = 64;                   // output channels
constexpr int DT_OSTRIDE = 80;                // LDS stride of a dy pixel: the 4 pixels of a fragment read fall into disjoint banks
constexpr int DT_XPL = DT_XMAX / 64;          // patch elements a lane loads
constexpr int DT_WAVES = 8;
constexpr int DT_MT = 5, DT_NT = 4;           // 16x16 MFMA tiles of the result
// floats per wavefront (the last 64: zeros); eight of them also hold the four regions in which the
// accumulators of a workgroup are added up
constexpr int DT_WAVE_LDS = 4 * DT_MT * 16 * DT_OMAX / DT_WAVES;
constexpr int DT_DUMP = DT_XMAX + DT_SEG * DT_OSTRIDE + 64;   // 64 + 256 floats that nothing reads
static_assert(DT_WAVE_LDS >= DT_DUMP + 64 + 256, "staging memory of a wavefront");

struct ThinDkParams
{
    const float* x;
    const float* dy;
    const float* x2;      // a second pair of operands, contracted into the same result (images N .. 2N-1), or null
    const float* dy2;
    float* part;          // [workgroup][M][O]
    int N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pt, pl;
    int M;                // kh * kw * C
    int row;              // kw * C
    int rsw;              // floats of a staged input row: (DT_SEG - 1) * sw * C + kw * C
    int rs;               // its LDS stride (bank-conflict-free fragment reads)
    int segs_per_row, total_segs, segs_per_wave;
    uint32_t x_bytes, dy_bytes;
    FastDiv fd_segs_per_row, fd_Ho, fd_rsw, fd_row, fd_O4;
};

__global__ __launch_bounds__(64 * DT_WAVES, 2) void dk_thin(const ThinDkParams p)
{
    __shared__ __attribute__((aligned(16))) float lds[DT_WAVES * DT_WAVE_LDS];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // (scalar: segment arithmetic runs on the scalar unit)
    float* lx = lds + wave * DT_WAVE_LDS;
    float* ld = lx + DT_XMAX;
    float* lzero = ld + DT_SEG * DT_OSTRIDE;
    lzero[lane] = 0.f;
    const int s_begin = ((int)blockIdx.x * DT_WAVES + wave) * p.segs_per_wave;
    const int s_end = min(p.total_segs, s_begin + p.segs_per_wave);

    // patch elements of this lane: e = lane + 64 q -> (row r, column col) of the staged rows
    // (row and column packed into one register: r << 16 | col; r = 0x7fff for a lane without element)
    int x_rc[DT_XPL];
#pragma unroll
    for (int q = 0; q < DT_XPL; ++q)
    {
        const int e = lane + 64 * q;
        uint32_t r, col;
        p.fd_rsw.divmod(e, r, col);
        x_rc[q] = (int)(((int)r < p.kh ? r : 0x7fffu) << 16 | col);
    }
    // dy elements of this lane: 16-byte pieces f = lane + 64 q -> (pixel, channel quad)
    int d_pix[4], d_o4[4];
#pragma unroll
    for (int q = 0; q < 4; ++q)
    {
        uint32_t pix, o4;
        p.fd_O4.divmod(lane + 64 * q, pix, o4);
        d_pix[q] = (int)pix < DT_SEG ? (int)pix : (1 << 28);
        d_o4[q] = (int)o4;
    }
    // MFMA fragments (16x16x4): A[m = (di, dj*C + c)][k = pixel], B[k = pixel][n = o]; lane (l16, kq)
    // supplies row / column l16 for pixel kq of each group of four
    const int l16 = lane & 15, kq = lane >> 4;
    // (rows and columns past the result's extents read a zero word, with a step of zero)
    int a_ptr[DT_MT], b_ptr[DT_NT];   // offsets into this wavefront's LDS
    int a_step[DT_MT], b_step[DT_NT]; // per group of four pixels
    const int zero_at = DT_XMAX + DT_SEG * DT_OSTRIDE + lane;
#pragma unroll
    for (int mt = 0; mt < DT_MT; ++mt)
    {
        const int m = mt * 16 + l16;
        uint32_t di, mp;
        p.fd_row.divmod(m, di, mp);
        a_ptr[mt] = m < p.M ? (int)di * p.rs + (int)mp + kq * p.sw * p.C : zero_at;
        a_step[mt] = m < p.M ? 4 * p.sw * p.C : 0;
    }
#pragma unroll
    for (int nt = 0; nt < DT_NT; ++nt)
    {
        const int n = nt * 16 + l16;
        b_ptr[nt] = n < p.O ? DT_XMAX + kq * DT_OSTRIDE + n : zero_at;
        b_step[nt] = n < p.O ? 4 * DT_OSTRIDE : 0;
    }
    dt_f32x4 acc[DT_MT][DT_NT];
#pragma unroll
    for (int mt = 0; mt < DT_MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < DT_NT; ++nt)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                acc[mt][nt][r] = 0.f;

    // two register sets: the loads of a segment are issued two segments ahead of its use
    float xv0[DT_XPL], xv1[DT_XPL];
    float4 dv0[4], dv1[4];
    // Loads go through buffer descriptors: an element that does not exist (outside the image, past the
    // row's end, a segment past the wavefront's last) gets an out-of-range offset and reads as zero, so
    // that the loop body is one basic block and the loads of a segment are issued back to back.
    const __amdgpu_buffer_rsrc_t xr1 = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.x), 0, (int)p.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t xr2 = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.x2 ? p.x2 : p.x), 0, (int)p.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t dr1 = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.dy), 0, (int)p.dy_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t dr2 = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.dy2 ? p.dy2 : p.dy), 0, (int)p.dy_bytes, 0x00020000);
    constexpr uint32_t FAR = 0xffffff00u;     // beyond any tensor the kernel takes (below 4 GiB - 256 bytes)
    auto load = [&](int s, float (&xv)[DT_XPL], float4 (&dv)[4]) {
        const bool live = s < s_end;
        uint32_t bi, js, b, i;
        p.fd_segs_per_row.divmod(live ? s : 0, bi, js);
        p.fd_Ho.divmod(bi, b, i);
        const int j0 = (int)js * DT_SEG;
        const int ih0 = (int)i * p.sh - p.pt;
        const int g0 = (j0 * p.sw - p.pl) * p.C;      // first staged column, in floats from the row start
        const bool second = (int)b >= p.N;       // only with a second pair of operands
        b -= second ? (uint32_t)p.N : 0u;
        const __amdgpu_buffer_rsrc_t xr = second ? xr2 : xr1;
        const __amdgpu_buffer_rsrc_t dr = second ? dr2 : dr1;
        // byte offset of the staged patch's origin, modulo 2^32 (exact for every element that exists:
        // the tensors are below 4 GiB)
        const uint32_t origin = ((b * (uint32_t)p.H + (uint32_t)ih0) * (uint32_t)(p.W * p.C) + (uint32_t)g0) * 4u;
        const uint32_t row_bytes = (uint32_t)(p.W * p.C) * 4u;
#pragma unroll
        for (int q = 0; q < DT_XPL; ++q)
        {
            const int r = x_rc[q] >> 16, col = x_rc[q] & 0xffff;
            const int ih = ih0 + r, g = g0 + col;
            const bool ok = (int)live & (int)((unsigned)ih < (unsigned)p.H) & (int)((unsigned)g < (unsigned)(p.W * p.C));
            const uint32_t off = ok ? origin + (uint32_t)r * row_bytes + (uint32_t)col * 4u : FAR;
            xv[q] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xr, (int)off, 0, 0));
        }
        const uint32_t drow = ((b * (uint32_t)p.Ho + i) * (uint32_t)p.Wo + (uint32_t)j0) * (uint32_t)p.O * 4u;
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            const bool ok = (int)live & (int)(d_pix[q] < DT_SEG) & (int)(j0 + d_pix[q] < p.Wo);
            const uint32_t off = ok ? drow + ((uint32_t)d_pix[q] * (uint32_t)p.O + (uint32_t)d_o4[q] * 4u) * 4u : FAR;
            const dt_f32x4 t = __builtin_bit_cast(dt_f32x4, __builtin_amdgcn_raw_buffer_load_b128(dr, (int)off, 0, 0));
            dv[q] = make_float4(t[0], t[1], t[2], t[3]);
        }
    };
    // where this lane's elements go in the staging memory (an element that does not exist goes to a
    // dump word of the lane's own: no branch around a write)
    int x_lds[DT_XPL], d_lds[4];
#pragma unroll
    for (int q = 0; q < DT_XPL; ++q)
        x_lds[q] = (x_rc[q] >> 16) != 0x7fff ? (x_rc[q] >> 16) * p.rs + (x_rc[q] & 0xffff) : DT_DUMP + lane;
#pragma unroll
    for (int q = 0; q < 4; ++q)
        d_lds[q] = d_pix[q] < DT_SEG ? DT_XMAX + d_pix[q] * DT_OSTRIDE + d_o4[q] * 4 : DT_DUMP + 64 + 4 * lane;
    auto stash = [&](const float (&xv)[DT_XPL], const float4 (&dv)[4]) {
#pragma unroll
        for (int q = 0; q < DT_XPL; ++q)
            lx[x_lds[q]] = xv[q];
#pragma unroll
        for (int q = 0; q < 4; ++q)
            *reinterpret_cast<float4*>(lx + d_lds[q]) = dv[q];
    };

    auto multiply = [&]() {
        // the fragments of a group of four pixels are read while the MFMAs of the group before run
        float a[2][DT_MT], b[2][DT_NT];
#pragma unroll
        for (int mt = 0; mt < DT_MT; ++mt)
            a[0][mt] = lx[a_ptr[mt]];
#pragma unroll
        for (int nt = 0; nt < DT_NT; ++nt)
            b[0][nt] = lx[b_ptr[nt]];
#pragma unroll
        for (int jj = 0; jj < DT_SEG / 4; ++jj)
        {
            const int cur = jj & 1, nxt = cur ^ 1;
            if (jj + 1 < DT_SEG / 4)
            {
#pragma unroll
                for (int mt = 0; mt < DT_MT; ++mt)
                    a[nxt][mt] = lx[a_ptr[mt] + (jj + 1) * a_step[mt]];
#pragma unroll
                for (int nt = 0; nt < DT_NT; ++nt)
                    b[nxt][nt] = lx[b_ptr[nt] + (jj + 1) * b_step[nt]];
            }
#pragma unroll
            for (int mt = 0; mt < DT_MT; ++mt)
#pragma unroll
                for (int nt = 0; nt < DT_NT; ++nt)
                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[cur][mt], b[cur][nt], acc[mt][nt], 0, 0, 0);
        }
    };
    // LDS operations of one wavefront execute in program order: the writes of a segment come after the
    // fragment reads of the segment before, the reads after them see the new segment.  The fences keep
    // the compiler from moving them across each other; no instruction results from them.
    auto step = [&](int s, float (&xv)[DT_XPL], float4 (&dv)[4]) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        stash(xv, dv);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        load(s + 2, xv, dv);
        multiply();
    };

    // (an odd last segment runs as a segment of zeros: every load of it is out of range)
    load(s_begin, xv0, dv0);
    load(s_begin + 1, xv1, dv1);
    for (int s = s_begin; s < s_end; s += 2)
    {
        step(s, xv0, dv0);
        step(s + 1, xv1, dv1);
    }

    // Add the eight accumulators in a fixed order: wavefronts 0-3 put theirs into four regions of the
    // staging memory, wavefronts 4-7 add theirs on top (region w - 4), then every thread adds the four
    // regions of its elements in region order and writes them to the workgroup's slice.  Register r of
    // lane (l16, kq) holds element (m = 4 * kq + r, n = l16) of its 16x16 tile.
    constexpr int REGION = DT_MT * 16 * DT_OMAX;
    __syncthreads();
    for (int round = 0; round < 2; ++round)
    {
        if ((wave >> 2) == round)
        {
            float* reg = lds + (wave & 3) * REGION;
#pragma unroll
            for (int mt = 0; mt < DT_MT; ++mt)
#pragma unroll
                for (int nt = 0; nt < DT_NT; ++nt)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                    {
                        float* dst = reg + (mt * 16 + 4 * kq + r) * DT_OMAX + nt * 16 + l16;
                        *dst = round == 0 ? acc[mt][nt][r] : *dst + acc[mt][nt][r];
                    }
        }
        __syncthreads();
    }
    const int total = p.M * p.O;
    float* out = p.part + (size_t)blockIdx.x * total;
    for (int idx = threadIdx.x * 4; idx < total; idx += 64 * DT_WAVES * 4)
    {
        const int m = idx / p.O, n = idx - m * p.O;   // O is a multiple of 4: a quad stays in its row
        const float* src = lds + m * DT_OMAX + n;
        float4 v = *reinterpret_cast<const float4*>(src);
#pragma unroll
        for (int g = 1; g < 4; ++g)
        {
            const float4 t = *reinterpret_cast<const float4*>(src + g * REGION);
            v.x += t.x; v.y += t.y; v.z += t.z; v.w += t.w;
        }
        *reinterpret_cast<float4*>(out + idx) = v;
    }
}

// ---- forward from three channels, a row of output pixels per step ---------------------------------
// The same product as fwd_thin, [N,64,64,3] -> [N,32,32,64] with a 5x5 filter, organised so that next
// to the MFMAs almost no vector instruction is left (fp32 MFMAs and vector instructions share the
// SIMD's ALU: fwd_thin issues ~470 of them per 32 pixels for offsets, masks and selects).
//   * y^T = K^T * patches: the filter is the A operand (80 registers per lane for the whole kernel:
//     four tiles of 16 output channels x the contraction 5 filter rows x 16), the patches are B, so
//     that result lane (pixel, q) holds 4 consecutive channels of its pixel: 16-byte stores.
//   * The contraction index is (di, e) with e = dj*C + c = 0 .. 14: the 15 values of a filter row's
//     taps are 15 CONSECUTIVE floats of input row i*sh + di - pad, starting at ((j*sw - pad)*C).  A
//     wavefront parks the input rows of its task (4 output rows: 11 input rows, 8.4 KB that are
//     contiguous in memory and are loaded as such, 16 bytes per lane) in LDS of its own, every row
//     with zeros to its left and right and rows outside the image as zeros, and each lane reads its
//     operand values from there with an address that is a per-lane constant plus the row's base:
//     20 LDS reads per 16 pixels, no masks, no bounds checks.
//   * The sixteenth slot of filter row 0 carries the bias (operand value 1), of the other rows zero.
//   * No wavefront depends on another: no barrier.  Tasks are strided over persistent wavefronts, the
//     loads of the next task are issued before the MFMAs of this one and waited for after the first
//     row's MFMAs, before any store of this task is issued (the counter of outstanding memory
//     operations is in order and counts stores).
// Takes kh = 5, kw*C = 15, at most 64 output channels in multiples of 16, rows of at most 32 output
// pixels; other shapes keep fwd_thin.
// Reference counterpart: kernel_conv2d (src/gpu/conv2d.cu:13-62) with kernel_mat_rvect_add and the
// activation that follow it.
typedef unsigned int fr_u32x4 __attribute__((__vector_size__(16)));
constexpr int FR_WAVES = 8;
constexpr int FR_STAGED = 11;           // input rows of a task: (4 - 1) * 2 + 5
constexpr int FR_RS = 208;              // floats per parked row: 8 of zeros, up to 192 of data, zeros
constexpr int FR_LEFT = 8;
constexpr int FR_LOADS = 9;             // 16-byte loads per lane and task: 11 rows x 48 <= 9 x 64
constexpr int FR_HEAD = 4;              // the first of them hold input rows 0 .. 4: 5 x 48 <= 4 x 64
constexpr int FR_ACT_LEAKY01 = 5;       // leaky relu with a slope in [0, 1]: max(v, slope * v), the same value in two instructions

struct FwdRowsParams
{
    const float* x;
    const float* k;
    const float* bias;
    float* y;
    const float* x2;                    // a second batch of N images with the same filter (images N .. 2N-1 of the
    float* y2;                          // launch), or null
    float alpha;
    int N, H, W, C, Ho, Wo, O, sh, sw, pt, pl;
    int rows_per_task, tasks_per_image, tasks;
    int staged, chunks_per_row;         // input rows of a task; 16-byte chunks of an input row
    uint32_t x_bytes, y_bytes;
};

template <int ACT>
__global__ __launch_bounds__(64 * FR_WAVES, 2) void fwd_rows(const FwdRowsParams p)
{
    __shared__ __attribute__((aligned(16))) float parked[FR_WAVES][(FR_STAGED + 1) * FR_RS];   // (+1: where surplus lanes write)
    __shared__ __attribute__((aligned(16))) float filt[77 * 64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l16 = lane & 15, kq = lane >> 4;
    float* const my = &parked[wave][0];
    for (int e = 4 * lane; e < (FR_STAGED + 1) * FR_RS; e += 256)
        *reinterpret_cast<float4*>(my + e) = make_float4(0.f, 0.f, 0.f, 0.f);

    // The filter goes through LDS once per workgroup: 16-byte loads of the [75][O] matrix as it lies in
    // memory (row 75: the bias, row 76 and the columns from O on: zeros -- what does not exist is out of
    // the descriptors' range and reads as zero), then every lane picks its 80 values (fetched by each
    // lane itself they would be 84 four-byte loads per lane of every wavefront).
    constexpr uint32_t FAR = 0xffffff00u;
    {
        const __amdgpu_buffer_rsrc_t kr = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.k), 0, 75 * p.O * 4, 0x00020000);
        const __amdgpu_buffer_rsrc_t br = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.bias), 0, p.bias ? p.O * 4 : 0, 0x00020000);
        for (int slot = threadIdx.x; slot < 77 * 16; slot += 64 * FR_WAVES)
        {
            const int row = slot >> 4, col = 4 * (slot & 15);
            const bool in_k = (int)(row < 75) & (int)(col < p.O), in_b = (int)(row == 75) & (int)(col < p.O);
            const dt_f32x4 kv = __builtin_bit_cast(dt_f32x4, __builtin_amdgcn_raw_buffer_load_b128(kr, (int)(in_k ? (uint32_t)(row * p.O + col) * 4u : FAR), 0, 0));
            const dt_f32x4 bv = __builtin_bit_cast(dt_f32x4, __builtin_amdgcn_raw_buffer_load_b128(br, (int)(in_b ? (uint32_t)col * 4u : FAR), 0, 0));
            *reinterpret_cast<dt_f32x4*>(&filt[row * 64 + col]) = row == 75 ? bv : kv;
        }
    }
    __syncthreads();
    // A[m = channel 16 mt + l16][k = 16 di + 4 u + kq] of MFMA step 4 di + u
    float aq[4][20];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int s = 0; s < 20; ++s)
        {
            const int di = s >> 2, e = 4 * (s & 3) + kq;
            const int row = e < 15 ? di * 15 + e : (di == 0 ? 75 : 76);
            aq[mt][s] = filt[row * 64 + 16 * mt + l16];
        }
    // (a task's image is the same for the whole wavefront: picking the first or the second batch's descriptor is
    // scalar work)
    const __amdgpu_buffer_rsrc_t xr1 = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.x), 0, (int)p.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t yr1 = __builtin_amdgcn_make_buffer_rsrc(p.y, 0, (int)p.y_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t xr2 = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.x2 ? p.x2 : p.x), 0, (int)p.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t yr2 = __builtin_amdgcn_make_buffer_rsrc(p.y2 ? p.y2 : p.y, 0, (int)p.y_bytes, 0x00020000);
    // chunk t*64 + lane of a task's rows: its row and where it is parked
    int put[FR_LOADS], chunk_row[FR_LOADS];
#pragma unroll
    for (int t = 0; t < FR_LOADS; ++t)
    {
        const int q = t * 64 + lane;
        const int r = q / p.chunks_per_row;
        chunk_row[t] = r < p.staged ? r : -0x10000;         // surplus chunks: loaded as zeros ...
        put[t] = r < p.staged ? r * FR_RS + FR_LEFT + 4 * (q - r * p.chunks_per_row)
                              : FR_STAGED * FR_RS + 4 * (lane & 31);                 // ... and parked out of the way
    }
    // this lane's operand values of pixel 16 t + l16: floats 4u + kq from here in the parked row
    int take[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
        take[t] = FR_LEFT + ((16 * t + l16) * p.sw - p.pl) * p.C + kq;
    const float slot15_row0 = p.bias ? 1.f : 0.f;
    const uint32_t row_bytes = (uint32_t)p.W * p.C * 4u;

    auto issue = [&](int task, dt_f32x4 (&raw)[FR_LOADS]) {
        const int bb = task / p.tasks_per_image;
        const int h0 = (task - bb * p.tasks_per_image) * p.rows_per_task * p.sh - p.pt;
        const bool second = bb >= p.N;
        const int b = second ? bb - p.N : bb;
        const __amdgpu_buffer_rsrc_t xr = second ? xr2 : xr1;
        const uint32_t base = ((uint32_t)b * p.H + (uint32_t)h0) * row_bytes;        // (wraps for h0 < 0; such rows are not loaded)
#pragma unroll
        for (int t = 0; t < FR_LOADS; ++t)
        {
            const int h = h0 + chunk_row[t];
            const bool ok = (int)(task < p.tasks) & (int)(h >= 0) & (int)(h < p.H);
            raw[t] = __builtin_bit_cast(dt_f32x4, __builtin_amdgcn_raw_buffer_load_b128(xr, (int)(ok ? base + (uint32_t)(t * 64 + lane) * 16u : FAR), 0, 0));
        }
    };
    auto park = [&](const dt_f32x4 (&raw)[FR_LOADS], int from, int to) {
#pragma unroll
        for (int t = 0; t < FR_LOADS; ++t)
            if (t >= from && t < to)
                *reinterpret_cast<dt_f32x4*>(my + put[t]) = raw[t];
    };

    const int stride = gridDim.x * FR_WAVES;
    int task = blockIdx.x * FR_WAVES + wave;
    dt_f32x4 raw[FR_LOADS];
    // The first task: every wavefront of the device asks for its rows at the same moment, and until they
    // arrive there is nothing to multiply.  Output row 0 needs input rows 0 .. 4 only, which the first
    // FR_HEAD loads hold (5 rows of at most 48 chunks); they are parked as soon as THEY are there, and the
    // rest of the task's rows after the first row's MFMAs.
    issue(task, raw);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    park(raw, 0, FR_HEAD);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    bool first_task = true;
    for (; task < p.tasks; task += stride)
    {
        if (!first_task)
            issue(task + stride, raw);
        __builtin_amdgcn_sched_barrier(0);      // (the scheduler would sink the loads to where they are used)
        const int bb = task / p.tasks_per_image;
        const int i0 = (task - bb * p.tasks_per_image) * p.rows_per_task;
        const bool second = bb >= p.N;
        const int b = second ? bb - p.N : bb;
        const __amdgpu_buffer_rsrc_t yr = second ? yr2 : yr1;
#pragma unroll
        for (int ii = 0; ii < 4; ++ii)
        {
            if (ii < p.rows_per_task && i0 + ii < p.Ho)
            {
                dt_f32x4 acc[2][4];
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            acc[t][mt][r] = 0.f;
                // operand values of filter row di: 4 floats per pixel tile, read one filter row ahead of
                // the MFMAs that consume them (left to itself the scheduler puts every read right in front
                // of its first use and the wavefront waits out the LDS latency twenty times per row)
                auto fetch = [&](int di, float (&v)[2][4]) {
                    const float* row = my + (ii * p.sh + di) * FR_RS;
#pragma unroll
                    for (int t = 0; t < 2; ++t)
                    {
#pragma unroll
                        for (int u = 0; u < 4; ++u)
                            v[t][u] = row[take[t] + 4 * u];
                    }
                };
                float bv[5][2][4];
                fetch(0, bv[0]);
#pragma unroll
                for (int di = 0; di < 5; ++di)
                {
                    if (di + 1 < 5)
                        fetch(di + 1, bv[di + 1]);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int t = 0; t < 2; ++t)
                    {
                        if (kq == 3)
                            bv[di][t][3] = di == 0 ? slot15_row0 : 0.f;
#pragma unroll
                        for (int u = 0; u < 4; ++u)
#pragma unroll
                            for (int mt = 0; mt < 4; ++mt)
                                acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x4f32(aq[mt][4 * di + u], bv[di][t][u], acc[t][mt], 0, 0, 0);
                    }
                }
                if (ii == 0)
                {
                    __builtin_amdgcn_sched_barrier(0);
                    if (first_task)
                    {
                        // the rest of this task's rows, then the request for the next task's
                        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                        park(raw, FR_HEAD, FR_LOADS);
                        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                        __builtin_amdgcn_wave_barrier();
                        issue(task + stride, raw);
                        first_task = false;
                    }
                    else
                    {
                        // the next task's rows have had these MFMAs to arrive; no store of this task is out yet
#pragma unroll
                        for (int t = 0; t < FR_LOADS; ++t)
                            asm volatile("" : "+v"(raw[t]));
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                // lane (pixel, q) holds channels 16 mt + 4 q .. + 3 of its pixel
                const uint32_t row_off = (((uint32_t)b * p.Ho + (uint32_t)(i0 + ii)) * p.Wo) * (uint32_t)p.O * 4u;
#pragma unroll
                for (int t = 0; t < 2; ++t)
                {
                    const int j = 16 * t + l16;
#pragma unroll
                    for (int mt = 0; mt < 4; ++mt)
                    {
                        dt_f32x4 v = acc[t][mt];
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                        {
                            if (ACT == DH_ACT_RELU) v[r] = v[r] < 0.f ? 0.f : v[r];
                            else if (ACT == DH_ACT_LEAKY) v[r] = v[r] < 0.f ? p.alpha * v[r] : v[r];
                            else if (ACT == FR_ACT_LEAKY01) v[r] = fmaxf(v[r], p.alpha * v[r]);
                            else if (ACT == DH_ACT_TANH) v[r] = tanhf(v[r]);
                            else if (ACT == DH_ACT_SIGMOID) v[r] = 1.f / (1.f + expf(-v[r]));
                        }
                        const bool ok = (int)(j < p.Wo) & (int)(16 * mt + 4 * kq < p.O);
                        const uint32_t off = row_off + ((uint32_t)j * p.O + 16u * mt + 4u * kq) * 4u;
                        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(fr_u32x4, v), yr, (int)(ok ? off : FAR), 0, 0);
                    }
                }
            }
        }
        // the rows of this task have been read: the next task's take their place
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        park(raw, 0, FR_LOADS);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
}

// ---- transposed convolution onto few channels as a product followed by in-register sums ----------
// The generator's image layer, [N,32,32,64] -> [N,64,64,3] (5x5, stride 2), and the gradient of the
// discriminator's first layer.  Written as dx[b, 2i+di-1, 2j+dj-1, c] += Z[(b,i,j), (di,dj,c)] with
//     Z[pixel, (di,dj,c)] = sum_o dy[pixel, o] * k[(di,dj,c), o]
// the arithmetic is ONE dense product, 75 x pixels x 64, with no product against an inserted zero and
// no tap enumeration: it runs on the matrix cores (16x16x4 tiles), and what remains is to add up, for
// every output element, the 4 to 9 entries of Z that land on it.
//   * The filter is the MFMA's A operand, 80 values per lane for the whole kernel: tile dj holds, in
//     row 3 di + c, the filter row (di, dj, c) (row 15 is zero).  A row of 32 dy pixels is the B operand
//     of two tiles: tile t holds pixel 2 n + t in column n, lane (n, q) loading channels 16q .. 16q+15
//     of its pixel straight from global memory into the registers the MFMAs consume.  A wavefront
//     multiplies one dy row per step (160 MFMAs); the loads of the next row are issued before them.
//   * ACROSS a row: the result lane (n, q) holds Z[pixel 2n+t][(di,c) = 4q+r][dj] in register r of
//     accumulator (t, dj) -- all five dj of a pixel in ONE lane, and the neighbouring pixels 2n-1 and
//     2n+2 one lane to the left and right.  The sums over dj for the output columns 4n .. 4n+3 are
//     therefore register adds, three of them through a one-lane row shift (DPP): 28 adds give
//     R[(di,c)][w], the row of Z summed over dj, 16 x 64 values, which the wavefront writes to a ring
//     of three rows in LDS that only it reads (4 KB a row; LDS operations of one wavefront execute in
//     order, so no barrier).
//   * DOWN the rows: lane w then adds, for the row before, the two output rows it completes from R of
//     three consecutive dy rows (5 reads per channel), applies bias and activation and stores them.
//   * Eight wavefronts share a strip of rows of one image, each taking consecutive rows.  Wavefronts
//     w and w + 4 run on one SIMD: their MFMA bursts alternate (timestamps show one burst of 160 at a
//     time, 5440 cycles each, 200 to 600 cycles apart), and the sums and stores of one proceed while
//     the other multiplies.  fp32 MFMAs and vector instructions share the SIMD's ALU here -- a loop
//     of MFMAs and one of FMAs in two wavefronts of a SIMD take the sum of their times -- so every
//     vector instruction saved is matrix time gained; that is why the sums run across lanes in
//     registers instead of gathering from LDS.
//   * The first and the last row of a wavefront also need R of the neighbouring wavefront's last and
//     first row: those parts (9 x 64 values) are published in LDS, and after ONE barrier per strip
//     every wavefront finishes its two edge rows.  Strips that are not whole images compute one row
//     above and below what they own.
// Takes 5x5 filters, stride 2, one pixel of padding before, at most 3 result channels, 64 dy channels,
// dy rows of at most 32 pixels; other shapes keep dx_few_channels.
// Reference counterpart: kernel_conv2d_transpose / kernel_conv2d_input_grad (src/gpu/conv2d.cu:70-117,
// 167-212).
constexpr int CT_PIX = 32;          // pixels of a dy row (two 16-pixel MFMA tiles)
constexpr int CT_WAVES = 8;         // wavefronts per workgroup
constexpr int CT_RING = 3;          // rows of R a wavefront keeps
constexpr int CT_ROWF = 16 * 64;    // floats in a row of R: 16 (di,c) slots x 64 output columns
constexpr int CT_KS = 16;           // MFMA steps: 64 dy channels, 4 per step

struct Col2imParams
{
    const float* dy;
    const float* k;
    float* dx;
    const float* bias;
    int act;
    float alpha;
    int N, Ho, Wo, C, H, W;
    int rows_per_strip, strips_per_image, strips;
    uint32_t dy_bytes;
};

// value of lane n-1 (n+1) of the same 16-lane row, zero at the row's end
__device__ __forceinline__ float ct_from_left(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x111, 0xf, 0xf, true));
}
__device__ __forceinline__ float ct_from_right(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x101, 0xf, 0xf, true));
}

__global__ __launch_bounds__(64 * CT_WAVES, 2) void dx_col2im(const Col2imParams p)
{
    __shared__ __attribute__((aligned(16))) float ring[CT_WAVES][CT_RING][CT_ROWF];
    __shared__ float xfirst[CT_WAVES][3 * 64];   // R[(0,c)] of a wavefront's first row
    __shared__ float xlast[CT_WAVES][6 * 64];    // R[(3,c)], R[(4,c)] of its last row
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l16 = lane & 15, kq = lane >> 4;

    // the filter as MFMA operand A[m = (di,c)][k = o] of tile dj: lane (m, q) holds o = 16q .. 16q+15
    // (rows that do not exist are out of the descriptor's range and read as zero: no select, and no wait
    // for the filter before the first row's loads go out)
    constexpr uint32_t FAR = 0xffffff00u;
    float aq[5][CT_KS];
    {
        const __amdgpu_buffer_rsrc_t kr = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.k), 0, 25 * p.C * 64 * 4, 0x00020000);
        const int di = l16 / 3, c = l16 - 3 * di;
        const bool ok = (int)(l16 < 15) & (int)(c < p.C);
#pragma unroll
        for (int dj = 0; dj < 5; ++dj)
        {
            const uint32_t off = (uint32_t)(((di * 5 + dj) * p.C + c) * 64 + kq * 16) * 4u;
#pragma unroll
            for (int g = 0; g < 4; ++g)
            {
                const dt_f32x4 v = __builtin_bit_cast(dt_f32x4, __builtin_amdgcn_raw_buffer_load_b128(kr, (int)(ok ? off + 16u * g : FAR), 0, 0));
                aq[dj][4 * g + 0] = v[0]; aq[dj][4 * g + 1] = v[1]; aq[dj][4 * g + 2] = v[2]; aq[dj][4 * g + 3] = v[3];
            }
        }
    }
    const float bias_c[3] = {p.bias && p.C > 0 ? p.bias[0] : 0.f, p.bias && p.C > 1 ? p.bias[1] : 0.f,
                             p.bias && p.C > 2 ? p.bias[2] : 0.f};
    const __amdgpu_buffer_rsrc_t dr = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.dy), 0, (int)p.dy_bytes, 0x00020000);
    float* const my_ring = &ring[wave][0][0];

    for (int strip = blockIdx.x; strip < p.strips; strip += gridDim.x)
    {
        const int b = strip / p.strips_per_image;
        const int own0 = (strip - b * p.strips_per_image) * p.rows_per_strip;
        const int own1 = min(p.Ho, own0 + p.rows_per_strip);
        const int c0 = max(0, own0 - 1), c1 = min(p.Ho, own1 + 1);      // rows of Z the strip computes
        const int row_a = c0 + wave * (c1 - c0) / CT_WAVES, row_b = c0 + (wave + 1) * (c1 - c0) / CT_WAVES;

        // dy[b, i, 2 n + t, 16 q ..] for both tiles of row i: zeros past the wavefront's rows or the row's end
        auto issue = [&](int i, dt_f32x4 (&raw)[2][4]) {
#pragma unroll
            for (int t = 0; t < 2; ++t)
            {
                const int jpix = 2 * l16 + t;
                const bool ok = (int)(i < row_b) & (int)(jpix < p.Wo);
                const uint32_t off = ((((uint32_t)b * p.Ho + (uint32_t)i) * p.Wo + (uint32_t)jpix) * 64u + (uint32_t)kq * 16u) * 4u;
#pragma unroll
                for (int g = 0; g < 4; ++g)
                    raw[t][g] = __builtin_bit_cast(dt_f32x4, __builtin_amdgcn_raw_buffer_load_b128(dr, (int)(ok ? off + 16u * g : FAR), 0, 0));
            }
        };
        // the parts of output rows 2i and 2i+1, column `lane`, that come from R of row i / i-1 / i+1
        auto add_mid = [&](const float* r, float (&o)[6]) {
#pragma unroll
            for (int c = 0; c < 3; ++c) { o[c] += r[(3 + c) * 64 + lane]; o[3 + c] += r[(6 + c) * 64 + lane]; }
        };
        auto add_up = [&](const float* r3, const float* r4, float (&o)[6]) {
#pragma unroll
            for (int c = 0; c < 3; ++c) { o[c] += r3[c * 64 + lane]; o[3 + c] += r4[c * 64 + lane]; }
        };
        auto add_down = [&](const float* r0, float (&o)[6]) {
#pragma unroll
            for (int c = 0; c < 3; ++c) o[3 + c] += r0[c * 64 + lane];
        };
        auto store = [&](int i, const float (&o)[6]) {
            if (i < own0 || i >= own1 || lane >= p.W)
                return;
            float* dst = p.dx + (((size_t)b * p.H + 2 * i) * p.W + lane) * p.C;
#pragma unroll
            for (int c = 0; c < 3; ++c)
                if (c < p.C)
                {
                    dst[c] = act_apply(o[c] + bias_c[c], p.act, p.alpha);
                    dst[(size_t)p.W * p.C + c] = act_apply(o[3 + c] + bias_c[c], p.act, p.alpha);
                }
        };

        float edge_first[6], edge_last[6];      // the wavefront's first and last row, still without the neighbours' parts
        dt_f32x4 b_cur[2][4], b_next[2][4];
        if (row_a < row_b)
            issue(row_a, b_cur);
        for (int i = row_a; i < row_b; ++i)
        {
            issue(i + 1, b_next);
            dt_f32x4 acc[2][5];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int dj = 0; dj < 5; ++dj)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        acc[t][dj][r] = 0.f;
#pragma unroll
            for (int s = 0; s < CT_KS; ++s)
#pragma unroll
                for (int t = 0; t < 2; ++t)
                {
                    const float bv = b_cur[t][s >> 2][s & 3];
#pragma unroll
                    for (int dj = 0; dj < 5; ++dj)
                        acc[t][dj] = __builtin_amdgcn_mfma_f32_16x16x4f32(aq[dj][s], bv, acc[t][dj], 0, 0, 0);
                }
            // sums over dj: output column 2 j + dj - 1 of pixel j; this lane's pixels are 2n (tile 0) and
            // 2n+1 (tile 1), pixel 2n-1 is tile 1 of the lane to the left, pixel 2n+2 tile 0 of the lane to the right
            float* rr = my_ring + (i % CT_RING) * CT_ROWF;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
#pragma unroll
            for (int r = 0; r < 4; ++r)
            {
                float4 v;
                v.x = acc[0][1][r] + ct_from_left(acc[1][3][r]);                       // column 4n
                v.y = acc[0][2][r] + ct_from_left(acc[1][4][r]) + acc[1][0][r];        // column 4n+1
                v.z = acc[1][1][r] + acc[0][3][r];                                     // column 4n+2
                v.w = acc[1][2][r] + acc[0][4][r] + ct_from_right(acc[0][0][r]);       // column 4n+3
                *reinterpret_cast<float4*>(rr + (4 * kq + r) * 64 + 4 * l16) = v;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            if (i == row_a)
            {
#pragma unroll
                for (int c = 0; c < 3; ++c) xfirst[wave][c * 64 + lane] = rr[c * 64 + lane];
            }
            if (i == row_b - 1)
            {
#pragma unroll
                for (int c = 0; c < 6; ++c) xlast[wave][c * 64 + lane] = rr[(9 + c) * 64 + lane];
            }
            if (i > row_a)
            {
                // row i-1 is complete but for what a neighbouring wavefront holds
                const float* rm = my_ring + ((i - 1) % CT_RING) * CT_ROWF;
                float o[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                add_mid(rm, o);
                if (i - 1 > row_a)
                {
                    const float* ru = my_ring + ((i - 2) % CT_RING) * CT_ROWF;
                    add_up(ru + 9 * 64, ru + 12 * 64, o);
                    add_down(rr, o);
                    store(i - 1, o);
                }
                else
                {
                    add_down(rr, o);
#pragma unroll
                    for (int e = 0; e < 6; ++e) edge_first[e] = o[e];
                }
            }
            if (i == row_b - 1)
            {
                float o[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                add_mid(rr, o);
                if (i > row_a)
                {
                    const float* ru = my_ring + ((i - 1) % CT_RING) * CT_ROWF;
                    add_up(ru + 9 * 64, ru + 12 * 64, o);
                }
#pragma unroll
                for (int e = 0; e < 6; ++e) edge_last[e] = o[e];
            }
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int g = 0; g < 4; ++g)
                    b_cur[t][g] = b_next[t][g];
        }
        __syncthreads();
        if (row_a < row_b)
        {
            // the wavefronts holding rows row_a - 1 and row_b (rows are dealt out in order, some wavefronts
            // of a short strip get none)
            int above = -1, below = -1;
            for (int v = 0; v < CT_WAVES; ++v)
            {
                const int va = c0 + v * (c1 - c0) / CT_WAVES, vb = c0 + (v + 1) * (c1 - c0) / CT_WAVES;
                if (va < vb && vb == row_a) above = v;
                if (va < vb && va == row_b) below = v;
            }
            if (row_b - 1 > row_a)
            {
                if (above >= 0)
                    add_up(&xlast[above][0], &xlast[above][3 * 64], edge_first);
                store(row_a, edge_first);
            }
            else if (above >= 0)
                add_up(&xlast[above][0], &xlast[above][3 * 64], edge_last);
            if (below >= 0)
                add_down(&xfirst[below][0], edge_last);
            store(row_b - 1, edge_last);
        }
        __syncthreads();   // the next strip overwrites what the neighbours published
    }
}

}  // namespace

namespace dh
{

// Whether the geometry is one fwd_rows takes (see the kernel's header; the tensors must be 16-byte aligned besides).
bool fwd_rows_takes(int N, int H, int W, int C, int kh, int kw, int O, int sh, int sw, int pt, int pl, int Ho, int Wo)
{
    const double x_bytes = (double)N * H * W * C * 4.0, y_bytes = (double)N * Ho * Wo * O * 4.0;
    const int rows = 4;   // (the launcher may take fewer rows per task; four must fit)
    return !(kh != 5 || kw * C != 15 || O > 64 || O % 16 != 0 || Wo > 32 || sh < 1 || sh > 2 || sw < 1 || sw > 2 || pt < 0 ||
             pl < 0 || pl * C > FR_LEFT || (W * C) % 4 != 0 || W * C > FR_RS - FR_LEFT - 8 ||
             FR_LEFT + (31 * sw - pl) * C + 16 > FR_RS || x_bytes >= 4294967040.0 || y_bytes >= 4294967040.0 ||
             (rows - 1) * sh + 5 > FR_STAGED || ((rows - 1) * sh + 5) * (W * C / 4) > FR_LOADS * 64 ||
             2L * N * ((Ho + rows - 1) / rows) > 0x3fffffffL);
}

// Returns 1 when the shape is not one fwd_rows takes, 0 after a launch.  x2 / y2 (both null, or both set): a
// second batch of N images through the same filter in the same launch.
int conv_fwd_rows(const float* x, const float* x2, const float* k, float* y, float* y2, int N, int H, int W, int C, int kh,
                  int kw, int O, int sh, int sw, int pt, int pl, int Ho, int Wo, const float* bias, int act, float alpha,
                  hipStream_t st)
{
    const double x_bytes = (double)N * H * W * C * 4.0, y_bytes = (double)N * Ho * Wo * O * 4.0;
    const int images = x2 ? 2 * N : N;
    if (!fwd_rows_takes(N, H, W, C, kh, kw, O, sh, sw, pt, pl, Ho, Wo) || act < DH_ACT_NONE || act > DH_ACT_SIGMOID ||
        ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(x2) |
          reinterpret_cast<uintptr_t>(y2)) & 15) != 0)
        return 1;
    FwdRowsParams p{};
    p.x = x; p.k = k; p.bias = bias; p.y = y; p.x2 = x2; p.y2 = y2; p.alpha = alpha;
    p.N = N; p.H = H; p.W = W; p.C = C; p.Ho = Ho; p.Wo = Wo; p.O = O; p.sh = sh; p.sw = sw; p.pt = pt; p.pl = pl;
    p.x_bytes = (uint32_t)x_bytes; p.y_bytes = (uint32_t)y_bytes;
    p.chunks_per_row = W * C / 4;
    // output rows per task: four (they share input rows) when that still gives every wavefront slot a task
    const long slots = (long)num_cus() * FR_WAVES;
    int rows = 4;
    while (rows > 1 && (long)images * ((Ho + rows - 1) / rows) < slots)
        rows /= 2;
    p.rows_per_task = rows;
    p.staged = (rows - 1) * sh + 5;
    if (p.staged > FR_STAGED || p.staged * p.chunks_per_row > FR_LOADS * 64)
        return 1;
    p.tasks_per_image = (Ho + rows - 1) / rows;
    const long tasks = (long)images * p.tasks_per_image;
    if (tasks > 0x3fffffffL)
        return 1;
    p.tasks = (int)tasks;
    long wgs = (tasks + FR_WAVES - 1) / FR_WAVES;
    if (wgs > num_cus())
        wgs = num_cus();
    const int prof = prof_begin("fwd_rows", 2.0 * images * Ho * Wo * O * kh * kw * C, st, 1, (double)images * Ho * 160.0 * 2048.0);
    const dim3 grid((unsigned)wgs), block(64 * FR_WAVES);
    switch (act)
    {
    case DH_ACT_NONE: hipLaunchKernelGGL(fwd_rows<DH_ACT_NONE>, grid, block, 0, st, p); break;
    case DH_ACT_RELU: hipLaunchKernelGGL(fwd_rows<DH_ACT_RELU>, grid, block, 0, st, p); break;
    case DH_ACT_LEAKY:
        if (alpha >= 0.f && alpha <= 1.f)
            hipLaunchKernelGGL(fwd_rows<FR_ACT_LEAKY01>, grid, block, 0, st, p);
        else
            hipLaunchKernelGGL(fwd_rows<DH_ACT_LEAKY>, grid, block, 0, st, p);
        break;
    case DH_ACT_TANH: hipLaunchKernelGGL(fwd_rows<DH_ACT_TANH>, grid, block, 0, st, p); break;
    default: hipLaunchKernelGGL(fwd_rows<DH_ACT_SIGMOID>, grid, block, 0, st, p); break;
    }
    prof_end(prof, st);
    DH_LAUNCH_CHECK("fwd_rows launch");
    return 0;
}

// Returns 1 when the shape is not one this kernel takes (the caller then uses the implicit GEMM),
// 0 after a launch, or an error code.
int conv_fwd_thin(const float* x, const float* k, float* y, int N, int H, int W, int C, int kh, int kw, int O, int sh,
                  int sw, int pt, int pl, int Ho, int Wo, const float* bias, int act, float alpha, hipStream_t st)
{
    if (conv_fwd_rows(x, nullptr, k, y, nullptr, N, H, W, C, kh, kw, O, sh, sw, pt, pl, Ho, Wo, bias, act, alpha, st) == 0)
        return 0;
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
    // four wavefronts per workgroup, each walking over 32-pixel tiles; at most two workgroups per compute
    // unit (two wavefronts per SIMD: one multiplies while the other waits for its loads or drains its stores)
    const long tiles = ((long)p.pixels + 31) / 32;
    if (tiles > 0x3fffffffL)
        return 1;
    p.tiles = (int)tiles;
    long blocks = (tiles + 3) / 4;
    const long resident = 2L * num_cus();
    if (blocks > resident)
        blocks = resident;
    const int prof = prof_begin("fwd_thin", 2.0 * N * Ho * Wo * O * kh * kw * C, st, 1,
                                (double)tiles * TF_KH * TF_NB * 4096.0);   // 32x32x2 MFMAs issued, padding included
    if (kw * C <= 16 && kh * 16 <= 2 * TF_KH)
        hipLaunchKernelGGL(fwd_thin<true>, dim3((unsigned)blocks), dim3(256), 0, st, p);
    else
        hipLaunchKernelGGL(fwd_thin<false>, dim3((unsigned)blocks), dim3(256), 0, st, p);
    prof_end(prof, st);
    DH_LAUNCH_CHECK("fwd_thin launch");
    return 0;
}




// Returns 1 when the shape is not one dx_col2im takes (see the kernel's header), 0 after a launch.
int conv_dx_col2im(const float* dy, const float* k, float* dx, int N, int Ho, int Wo, int O, int kh, int kw, int C, int sh,
                   int sw, int pt, int pl, int H, int W, const float* bias, int act, float alpha, hipStream_t st)
{
    const double dy_bytes = (double)N * Ho * Wo * O * 4.0;
    if (sh != 2 || sw != 2 || kh != 5 || kw != 5 || pt != 1 || pl != 1 || C > 3 || O != 64 || Wo > CT_PIX || W != 2 * Wo ||
        H != 2 * Ho || W > 64 || dy_bytes >= 4294967040.0 || (reinterpret_cast<uintptr_t>(dy) & 15) != 0 ||
        (reinterpret_cast<uintptr_t>(k) & 15) != 0)
        return 1;
    Col2imParams p{};
    p.dy = dy; p.k = k; p.dx = dx; p.bias = bias; p.act = act; p.alpha = alpha;
    p.N = N; p.Ho = Ho; p.Wo = Wo; p.C = C; p.H = H; p.W = W;
    p.dy_bytes = (uint32_t)dy_bytes;
    // rows per strip: whole images when those give every compute unit a workgroup, else the largest
    // power of two that does (a strip computes two rows more than it owns)
    int rows = 32;
    while (rows > 4 && (long)N * ((Ho + rows - 1) / rows) < 1L * num_cus())
        rows /= 2;
    p.rows_per_strip = rows;
    p.strips_per_image = (Ho + rows - 1) / rows;
    const long strips = (long)N * p.strips_per_image;
    if (strips > 0x7fffffffL)
        return 1;
    p.strips = (int)strips;
    const long wgs = strips < num_cus() ? strips : num_cus();
    // rows of Z computed, the strips' extra rows included: 160 MFMAs of 16x16x4 each
    long z_rows = 0;
    for (int r0 = 0; r0 < Ho; r0 += rows)
        z_rows += (r0 + rows + 1 < Ho ? r0 + rows + 1 : Ho) - (r0 > 0 ? r0 - 1 : 0);
    const int prof = prof_begin("dx_col2im", 2.0 * N * Ho * Wo * O * kh * kw * C, st, 1, (double)N * z_rows * 160.0 * 2048.0);
    hipLaunchKernelGGL(dx_col2im, dim3((unsigned)wgs), dim3(64 * CT_WAVES), 0, st, p);
    prof_end(prof, st);
    DH_LAUNCH_CHECK("dx_col2im launch");
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


// Returns 1 when the shape is not one this kernel takes, 0 after a launch (the caller then adds the
// *splits slices of M x O partial sums at *part), or an error code.
// Whether the geometry is one dk_thin takes (the operands must be 16-byte aligned besides).
bool dk_thin_takes(int N, int H, int W, int C, int Ho, int Wo, int O, int kh, int kw, int sw)
{
    const int M = kh * kw * C, row = kw * C;
    const int rsw = (DT_SEG - 1) * sw * C + row;
    const int rs = rsw + ((row - rsw) % 32 + 32) % 32;
    // (both operand tensors below 4 GiB - 256 bytes: 32-bit byte offsets into buffer descriptors)
    return !(M > DT_MT * 16 || O > DT_OMAX || O % 4 != 0 || kh * rs > DT_XMAX || kh * rsw > 64 * DT_XPL ||
             (long)N * Ho * Wo < 2048 || (double)N * H * W * C * 4.0 >= 4294967040.0 ||
             (double)N * Ho * Wo * O * 4.0 >= 4294967040.0);
}

// x2 / dy2: a second pair of operands whose filter gradient is added to the first's (both null: one pair).
int conv_dk_thin(const float* x, const float* dy, const float* x2, const float* dy2, float** part, int* splits, int N,
                 int H, int W, int C, int Ho, int Wo, int O, int kh, int kw, int sh, int sw, int pt, int pl, hipStream_t st)
{
    const int M = kh * kw * C, row = kw * C;
    const int rsw = (DT_SEG - 1) * sw * C + row;
    const int rs = rsw + ((row - rsw) % 32 + 32) % 32;   // rs = row (mod 32): the 32 lanes of a fragment read hit 32 banks
    const int images = x2 ? 2 * N : N;
    if (!dk_thin_takes(N, H, W, C, Ho, Wo, O, kh, kw, sw) || (reinterpret_cast<uintptr_t>(dy) & 15) != 0 ||
        (reinterpret_cast<uintptr_t>(dy2) & 15) != 0)
        return 1;
    ThinDkParams p{};
    p.x = x; p.dy = dy; p.x2 = x2; p.dy2 = dy2;
    p.N = N; p.H = H; p.W = W; p.C = C; p.Ho = Ho; p.Wo = Wo; p.O = O; p.kh = kh; p.kw = kw;
    p.sh = sh; p.sw = sw; p.pt = pt; p.pl = pl;
    p.M = M; p.row = row; p.rsw = rsw; p.rs = rs;
    p.x_bytes = (uint32_t)((size_t)N * H * W * C * 4); p.dy_bytes = (uint32_t)((size_t)N * Ho * Wo * O * 4);
    p.segs_per_row = (Wo + DT_SEG - 1) / DT_SEG;
    const long total = (long)images * Ho * p.segs_per_row;
    if (total > 0x7fffffffL)
        return 1;
    p.total_segs = (int)total;
    // one workgroup of eight wavefronts per compute unit (two wavefronts per SIMD: one multiplies while
    // the other stages its next segment), at least two segments per wavefront
    long wgs = 1L * num_cus();
    long per_wave = (total + wgs * DT_WAVES - 1) / (wgs * DT_WAVES);
    if (per_wave < 2) per_wave = 2;
    wgs = (total + per_wave * DT_WAVES - 1) / (per_wave * DT_WAVES);
    p.segs_per_wave = (int)per_wave;
    p.fd_segs_per_row = FastDiv(p.segs_per_row); p.fd_Ho = FastDiv(Ho); p.fd_rsw = FastDiv(rsw);
    p.fd_row = FastDiv(row); p.fd_O4 = FastDiv(O / 4);
    void* ws;
    DH_TRY(workspace((size_t)wgs * M * O * sizeof(float), &ws, st));
    p.part = static_cast<float*>(ws);
    const int prof = prof_begin("dk_thin", 2.0 * images * Ho * Wo * O * kh * kw * C, st, 1,
                                2.0 * images * Ho * Wo * (DT_MT * 16.0) * (DT_NT * 16.0));   // the 80 x 64 tile per pixel
    hipLaunchKernelGGL(dk_thin, dim3((unsigned)wgs), dim3(64 * DT_WAVES), 0, st, p);
    prof_end(prof, st);
    DH_LAUNCH_CHECK("dk_thin launch");
    *part = p.part;
    *splits = (int)wgs;
    return 0;
}

}  // namespace dh
