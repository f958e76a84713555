// fp32 implicit-GEMM convolutions on the CDNA4 matrix cores (v_mfma_f32_32x32x2_f32).
//
// One kernel template serves the three contractions of the convolution hot path:
//
//   FWD  y[m, o]  = sum_k  X(m, k)  * Kf[k, o]    m = (b,i,j)      k = (di,dj,c)
//   DX   dx[m, c] = sum_k  DY(m, k) * Kt(k, c)    m = (b,hh,ww) of one stride phase, k = (tap,o)
//   DK   dk[m, o] = sum_k  Xt(k, m) * DY[k, o]    m = (di,dj,c)    k = (b,i,j)
//
// Nothing is materialised: the "im2col" operand is gathered straight from the NHWC tensor into an
// LDS tile (zero where a tap falls into the padding), the other operand tile is staged next to it,
// and each of the four wavefronts of a workgroup multiplies its share of the tiles with MFMA.
// DX is split into the sh*sw output phases (h mod sh, w mod sw): within a phase every output pixel
// uses the same subset of filter taps, so each phase is a dense GEMM and no product with an
// inserted zero is ever formed (for 5x5/stride 2 the phases use 2x2, 2x3, 3x2 and 3x3 taps).
//
// Reference counterparts: src/gpu/conv2d.cu:13-307 (dispatch) and src/gpu/conv2d_gemm.hh (the
// im2col + GEMM + re-layout pipeline this replaces).
#include "dh_common.h"

#include <cstdio>
#include <cstring>
#include <vector>

using namespace dh;

namespace
{

typedef float f32x16 __attribute__((ext_vector_type(16)));

enum { MODE_FWD = 0, MODE_DX = 1, MODE_DK = 2 };

constexpr int BK = 16;        // k extent of one LDS stage
constexpr int NTHREADS = 256;  // 4 wavefronts
constexpr int MAX_PHASES = 4;  // stride phases handled by one launch (grid.z)

struct Phase
{
    int M, K;            // GEMM extents of this phase
    int ph, pw;          // DX: output phase (h mod sh, w mod sw)
    int Hp, Wp;          // DX: output rows/cols in this phase
    int rh, rw;          // DX: first filter tap of the phase
    int q0h, q0w;        // DX: i = hh + q0h - th
    int nth, ntw;        // DX: taps along h and w
    FastDiv fd_HpWp, fd_Wp, fd_ntw;
};

struct ConvParams
{
    const float* a_src;   // FWD: x    DX: dy   DK: x
    const float* b_src;   // FWD: k    DX: k    DK: dy
    float* out;           // result (splitk == 1) ...
    float* part;          // ... or split-K partial sums [splitk][out_elems]
    const float* bias;
    int act;
    float alpha;
    int N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pt, pl;
    int ncols;            // GEMM n extent: O (FWD, DK) or C (DX)
    int splitk;
    int vec_out;          // 16-byte stores allowed (n extent divisible by 4, aligned destination and bias)
    size_t out_elems;
    FastDiv fd_HoWo, fd_Wo, fd_C, fd_O, fd_kw;
    Phase phase[MAX_PHASES];
};

__device__ __forceinline__ float apply_act(float v, int act, float alpha)
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

// ---- gathers: element (m,k) of the A operand, element (k,n) of the B operand -------------------
// Each returns the address of the element and whether it exists (false = contributes zero).
// With VEC the caller loads 4 consecutive elements from the address; this is legal because the
// 4-chunk runs along the channel axis, never crosses a tap (channel count divisible by 4) and
// is 16-byte aligned.

template <int MODE>
__device__ __forceinline__ bool addr_a(const ConvParams& p, const Phase& ph, int m, int k, size_t& off)
{
    if (m >= ph.M || k >= ph.K)
        return false;
    if (MODE == MODE_FWD)
    {
        uint32_t b, rem, i, j, tap, c, di, dj;
        p.fd_HoWo.divmod(m, b, rem);
        p.fd_Wo.divmod(rem, i, j);
        p.fd_C.divmod(k, tap, c);
        p.fd_kw.divmod(tap, di, dj);
        const int ih = (int)i * p.sh + (int)di - p.pt;
        const int iw = (int)j * p.sw + (int)dj - p.pl;
        if ((unsigned)ih >= (unsigned)p.H || (unsigned)iw >= (unsigned)p.W)
            return false;
        off = (((size_t)b * p.H + ih) * p.W + iw) * p.C + c;
        return true;
    }
    else if (MODE == MODE_DX)
    {
        uint32_t b, rem, hh, ww, tap, o, th, tw;
        ph.fd_HpWp.divmod(m, b, rem);
        ph.fd_Wp.divmod(rem, hh, ww);
        p.fd_O.divmod(k, tap, o);
        ph.fd_ntw.divmod(tap, th, tw);
        const int i = (int)hh + ph.q0h - (int)th;
        const int j = (int)ww + ph.q0w - (int)tw;
        if ((unsigned)i >= (unsigned)p.Ho || (unsigned)j >= (unsigned)p.Wo)
            return false;
        off = (((size_t)b * p.Ho + i) * p.Wo + j) * p.O + o;
        return true;
    }
    else
    {
        uint32_t tap, c, di, dj, b, rem, i, j;
        p.fd_C.divmod(m, tap, c);
        p.fd_kw.divmod(tap, di, dj);
        p.fd_HoWo.divmod(k, b, rem);
        p.fd_Wo.divmod(rem, i, j);
        const int ih = (int)i * p.sh + (int)di - p.pt;
        const int iw = (int)j * p.sw + (int)dj - p.pl;
        if ((unsigned)ih >= (unsigned)p.H || (unsigned)iw >= (unsigned)p.W)
            return false;
        off = (((size_t)b * p.H + ih) * p.W + iw) * p.C + c;
        return true;
    }
}

template <int MODE>
__device__ __forceinline__ bool addr_b(const ConvParams& p, const Phase& ph, int k, int n, size_t& off)
{
    if (n >= p.ncols || k >= ph.K)
        return false;
    if (MODE == MODE_DX)
    {
        uint32_t tap, o, th, tw;
        p.fd_O.divmod(k, tap, o);
        ph.fd_ntw.divmod(tap, th, tw);
        const int di = ph.rh + p.sh * (int)th;
        const int dj = ph.rw + p.sw * (int)tw;
        off = (((size_t)di * p.kw + dj) * p.C + n) * p.O + o;
        return true;
    }
    else
    {
        off = (size_t)k * p.ncols + n;  // FWD: k[(di,dj,c)][o]   DK: dy[(b,i,j)][o]
        return true;
    }
}

template <int MODE, bool VEC>
__device__ __forceinline__ float4 fetch_a(const ConvParams& p, const Phase& ph, int m, int k)
{
    constexpr bool KC = MODE != MODE_DK;  // chunk runs along k, else along m
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    size_t off;
    if (VEC)
    {
        if (addr_a<MODE>(p, ph, m, k, off))
            v = *reinterpret_cast<const float4*>(p.a_src + off);
    }
    else
    {
        float* e = reinterpret_cast<float*>(&v);
#pragma unroll
        for (int q = 0; q < 4; ++q)
            if (addr_a<MODE>(p, ph, KC ? m : m + q, KC ? k + q : k, off))
                e[q] = p.a_src[off];
    }
    return v;
}

template <int MODE, bool VEC>
__device__ __forceinline__ float4 fetch_b(const ConvParams& p, const Phase& ph, int k, int n)
{
    constexpr bool KC = MODE == MODE_DX;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    size_t off;
    if (VEC)
    {
        if (addr_b<MODE>(p, ph, k, n, off))
            v = *reinterpret_cast<const float4*>(p.b_src + off);
    }
    else
    {
        float* e = reinterpret_cast<float*>(&v);
#pragma unroll
        for (int q = 0; q < 4; ++q)
            if (addr_b<MODE>(p, ph, KC ? k + q : k, KC ? n : n + q, off))
                e[q] = p.b_src[off];
    }
    return v;
}

// ---- LDS tiles -----------------------------------------------------------------------------------
// KCONTIG: [row][BK + 4]  (rows = m or n, a lane reads 4 consecutive k with one ds_read_b128)
// else   : [BK][R + 4]    (rows = k, a lane reads its row's element of 4 k with ds_read_b32)
// A lane of an MFMA needs, per group of 8 k, the values k = 4*half + {0,1,2,3} of its row
// (half = lane / 32); the j-th of the 4 MFMAs of the group then contracts k = j and k = 4 + j.
template <bool KCONTIG, int R>
struct Tile
{
    static constexpr int STRIDE = KCONTIG ? BK + 4 : R + 4;
    static constexpr int SIZE = KCONTIG ? R * STRIDE : BK * STRIDE;
    static constexpr int CHUNKS = R * BK / 4;                       // float4 chunks per stage
    static constexpr int PER_THREAD = (CHUNKS + NTHREADS - 1) / NTHREADS;

    // chunk index -> (row, k) of its first element
    __device__ static __forceinline__ void chunk(int idx, int& row, int& k)
    {
        if (KCONTIG)
        {
            row = idx / (BK / 4);
            k = (idx % (BK / 4)) * 4;
        }
        else
        {
            k = idx / (R / 4);
            row = (idx % (R / 4)) * 4;
        }
    }
    __device__ static __forceinline__ void store(float* t, int row, int k, float4 v)
    {
        if (KCONTIG)
            *reinterpret_cast<float4*>(t + row * STRIDE + k) = v;
        else
            *reinterpret_cast<float4*>(t + k * STRIDE + row) = v;
    }
    __device__ static __forceinline__ float4 frag(const float* t, int row, int kgroup, int half)
    {
        const int k0 = kgroup * 8 + half * 4;
        if (KCONTIG)
            return *reinterpret_cast<const float4*>(t + row * STRIDE + k0);
        return make_float4(t[(k0 + 0) * STRIDE + row], t[(k0 + 1) * STRIDE + row],
                           t[(k0 + 2) * STRIDE + row], t[(k0 + 3) * STRIDE + row]);
    }
};

// Write-out of a wavefront's accumulators.  The MFMAs are issued with the operands exchanged
// (filter-side fragment first), so that register r of lane l holds
//     C[m = l % 32][n = 8*(r/4) + 4*(l/32) + r%4]
// i.e. every group of 4 registers is 4 consecutive output channels of one row: one 16-byte store.
// With split-K the raw partial sums go to the scratch arena; otherwise bias and activation are
// applied here.
template <int MODE, int TM, int TN>
__device__ __forceinline__ void write_tile(const ConvParams& p, const Phase& ph, f32x16 (&acc)[TM][TN], int m_base,
                                           int n_base, int l32, int half)
{
    const bool direct = p.splitk == 1;
    float* dst = direct ? p.out : p.part + (size_t)blockIdx.y * p.out_elems;
#pragma unroll
    for (int a = 0; a < TM; ++a)
    {
        const int m = m_base + a * 32 + l32;
        if (m >= ph.M)
            continue;
        size_t row_off;
        if (MODE == MODE_DX)
        {
            uint32_t b, rem, hh, ww;
            ph.fd_HpWp.divmod(m, b, rem);
            ph.fd_Wp.divmod(rem, hh, ww);
            row_off = (((size_t)b * p.H + hh * p.sh + ph.ph) * p.W + ww * p.sw + ph.pw) * p.C;
        }
        else
            row_off = (size_t)m * p.ncols;
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int g = 0; g < 4; ++g)
            {
                const int n = n_base + b * 32 + 8 * g + 4 * half;
                float4 v = make_float4(acc[a][b][4 * g], acc[a][b][4 * g + 1], acc[a][b][4 * g + 2], acc[a][b][4 * g + 3]);
                if (p.vec_out)
                {
                    if (n >= p.ncols)
                        continue;
                    if (direct)
                    {
                        if (p.bias)
                        {
                            const float4 bb = *reinterpret_cast<const float4*>(p.bias + n);
                            v.x += bb.x; v.y += bb.y; v.z += bb.z; v.w += bb.w;
                        }
                        v.x = apply_act(v.x, p.act, p.alpha); v.y = apply_act(v.y, p.act, p.alpha);
                        v.z = apply_act(v.z, p.act, p.alpha); v.w = apply_act(v.w, p.act, p.alpha);
                    }
                    *reinterpret_cast<float4*>(dst + row_off + n) = v;
                }
                else
                {
                    const float* e = reinterpret_cast<const float*>(&v);
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                    {
                        if (n + q >= p.ncols)
                            continue;
                        float w = e[q];
                        if (direct)
                        {
                            if (p.bias)
                                w += p.bias[n + q];
                            w = apply_act(w, p.act, p.alpha);
                        }
                        dst[row_off + n + q] = w;
                    }
                }
            }
    }
}

// BM x BN output tile per workgroup, WGM x WGN wavefronts, each owning (BM/WGM) x (BN/WGN).
template <int MODE, int BM, int BN, int WGM, int WGN, bool VECA, bool VECB>
__global__ __launch_bounds__(NTHREADS) void conv_igemm(const ConvParams p)
{
    static_assert(WGM * WGN == 4, "four wavefronts per workgroup");
    constexpr bool A_KC = MODE != MODE_DK;
    constexpr bool B_KC = MODE == MODE_DX;
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int TM = WM / 32, TN = WN / 32;
    static_assert(TM >= 1 && TN >= 1, "wave tile is a multiple of the 32x32 MFMA tile");
    using TA = Tile<A_KC, BM>;
    using TB = Tile<B_KC, BN>;

    __shared__ __attribute__((aligned(16))) float lds_a[2][TA::SIZE];
    __shared__ __attribute__((aligned(16))) float lds_b[2][TB::SIZE];

    const Phase& ph = p.phase[blockIdx.z];
    const int tiles_n = (p.ncols + BN - 1) / BN;
    const int tile_m = blockIdx.x / tiles_n;
    const int tile_n = blockIdx.x - tile_m * tiles_n;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    if (m0 >= ph.M)
        return;  // this phase has fewer row tiles than the largest one

    const int nslabs = (ph.K + BK - 1) / BK;
    const int per_split = (nslabs + p.splitk - 1) / p.splitk;
    const int s_begin = blockIdx.y * per_split;
    const int s_end = min(nslabs, s_begin + per_split);

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int half = lane >> 5, l32 = lane & 31;
    const int wm0 = (wave / WGN) * WM, wn0 = (wave % WGN) * WN;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[a][b][r] = 0.f;

    float4 ra[TA::PER_THREAD], rb[TB::PER_THREAD];

    auto load_global = [&](int slab) {
        const int k0 = slab * BK;
#pragma unroll
        for (int q = 0; q < TA::PER_THREAD; ++q)
        {
            const int idx = tid + q * NTHREADS;
            if (TA::CHUNKS % NTHREADS == 0 || idx < TA::CHUNKS)
            {
                int row, k;
                TA::chunk(idx, row, k);
                ra[q] = fetch_a<MODE, VECA>(p, ph, m0 + row, k0 + k);
            }
        }
#pragma unroll
        for (int q = 0; q < TB::PER_THREAD; ++q)
        {
            const int idx = tid + q * NTHREADS;
            if (TB::CHUNKS % NTHREADS == 0 || idx < TB::CHUNKS)
            {
                int row, k;
                TB::chunk(idx, row, k);
                rb[q] = fetch_b<MODE, VECB>(p, ph, k0 + k, n0 + row);
            }
        }
    };
    auto store_lds = [&](int stage) {
#pragma unroll
        for (int q = 0; q < TA::PER_THREAD; ++q)
        {
            const int idx = tid + q * NTHREADS;
            if (TA::CHUNKS % NTHREADS == 0 || idx < TA::CHUNKS)
            {
                int row, k;
                TA::chunk(idx, row, k);
                TA::store(lds_a[stage], row, k, ra[q]);
            }
        }
#pragma unroll
        for (int q = 0; q < TB::PER_THREAD; ++q)
        {
            const int idx = tid + q * NTHREADS;
            if (TB::CHUNKS % NTHREADS == 0 || idx < TB::CHUNKS)
            {
                int row, k;
                TB::chunk(idx, row, k);
                TB::store(lds_b[stage], row, k, rb[q]);
            }
        }
    };

    if (s_begin < s_end)
    {
        load_global(s_begin);
        store_lds(0);
        __syncthreads();
        for (int s = s_begin; s < s_end; ++s)
        {
            const int stage = (s - s_begin) & 1;
            if (s + 1 < s_end)
                load_global(s + 1);  // in flight while the matrix cores work on this stage
#pragma unroll
            for (int kg = 0; kg < BK / 8; ++kg)
            {
                float4 fa[TM], fb[TN];
#pragma unroll
                for (int a = 0; a < TM; ++a)
                    fa[a] = TA::frag(lds_a[stage], wm0 + a * 32 + l32, kg, half);
#pragma unroll
                for (int b = 0; b < TN; ++b)
                    fb[b] = TB::frag(lds_b[stage], wn0 + b * 32 + l32, kg, half);
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int a = 0; a < TM; ++a)
#pragma unroll
                        for (int b = 0; b < TN; ++b)
                            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                                reinterpret_cast<const float*>(&fb[b])[j],
                                reinterpret_cast<const float*>(&fa[a])[j], acc[a][b], 0, 0, 0);
            }
            if (s + 1 < s_end)
                store_lds(stage ^ 1);
            __syncthreads();
        }
    }

    write_tile<MODE, TM, TN>(p, ph, acc, m0 + wm0, n0 + wn0, l32, half);
}

// ---- fast path -------------------------------------------------------------------------------------
// Same tiling and arithmetic as conv_igemm, for the common case where every 4-chunk can be loaded as
// one 16-byte access (channel counts divisible by 4, 16-byte aligned tensors of less than 2^31
// bytes).  What changes is how operands are fetched:
//   * the part of an address that depends on the tile row (image, output pixel) is decoded ONCE per
//     thread before the k loop; per k-slab only the filter tap is decoded, once per thread;
//   * loads go through buffer descriptors: an element that falls into the padding, past the end of
//     the contraction or outside the tile gets an out-of-range offset and the hardware returns 0,
//     so the loop body has no branches and the compiler can interleave address arithmetic, LDS
//     traffic and MFMA in one basic block.
typedef float f32x4 __attribute__((ext_vector_type(4)));
constexpr int32_t OOB = (int32_t)0x80000000u;  // any offset >= num_records reads as zero

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const float* ptr, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(ptr), 0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ f32x4 buf_load4(__amdgpu_buffer_rsrc_t r, int32_t byte_off)
{
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, 0));
}

template <int MODE, int BM, int BN, int WGM, int WGN>
__global__ __launch_bounds__(NTHREADS) void conv_igemm_fast(const ConvParams p, uint32_t a_bytes, uint32_t b_bytes)
{
    static_assert(WGM * WGN == 4, "four wavefronts per workgroup");
    constexpr bool A_KC = MODE != MODE_DK;
    constexpr bool B_KC = MODE == MODE_DX;
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int TM = WM / 32, TN = WN / 32;
    using TA = Tile<A_KC, BM>;
    using TB = Tile<B_KC, BN>;
    constexpr int NA = TA::PER_THREAD, NB = TB::PER_THREAD;

    __shared__ __attribute__((aligned(16))) float lds_a[2][TA::SIZE];
    __shared__ __attribute__((aligned(16))) float lds_b[2][TB::SIZE];

    const Phase& ph = p.phase[blockIdx.z];
    const int tiles_n = (p.ncols + BN - 1) / BN;
    const int tile_m = blockIdx.x / tiles_n;
    const int tile_n = blockIdx.x - tile_m * tiles_n;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    if (m0 >= ph.M)
        return;

    const int nslabs = (ph.K + BK - 1) / BK;
    const int per_split = (nslabs + p.splitk - 1) / p.splitk;
    const int s_begin = blockIdx.y * per_split;
    const int s_end = min(nslabs, s_begin + per_split);

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int half = lane >> 5, l32 = lane & 31;
    const int wm0 = (wave / WGN) * WM, wn0 = (wave % WGN) * WN;

    const __amdgpu_buffer_rsrc_t ra_src = make_rsrc(p.a_src, a_bytes);
    const __amdgpu_buffer_rsrc_t rb_src = make_rsrc(p.b_src, b_bytes);

    // ---- per-thread state that does not depend on k -------------------------------------------------
    // K-contiguous operand tiles: chunk q of this thread is row (tid + q*256) / 4, k offset (tid % 4) * 4.
    // Other tiles: chunk q is k row tid / (R/4) + q * 256/(R/4), row offset (tid % (R/4)) * 4.
    const int kloc = (tid % (BK / 4)) * 4;
    int a_base[NA], a_h[NA], a_w[NA];   // FWD/DX: byte offset of the row's origin, its (h, w) origin
    int a_krow[NA];                      // DK: k row of the chunk inside the slab
    int a_moff = 0, a_dh = 0, a_dw = 0;  // DK: per-thread filter tap (byte offset, h and w shifts)
    bool a_mvalid = true;
#pragma unroll
    for (int q = 0; q < NA; ++q)
    {
        const int idx = tid + q * NTHREADS;
        a_base[q] = 0; a_h[q] = 0; a_w[q] = 0; a_krow[q] = 0;
        if (A_KC)
        {
            const int m = m0 + idx / (BK / 4);
            const bool live = m < ph.M && idx < TA::CHUNKS;
            uint32_t b = 0, rem = 0, r1 = 0, r2 = 0;
            if (MODE == MODE_FWD)
            {
                p.fd_HoWo.divmod(m, b, rem);
                p.fd_Wo.divmod(rem, r1, r2);
                a_h[q] = (int)r1 * p.sh - p.pt;
                a_w[q] = (int)r2 * p.sw - p.pl;
                a_base[q] = (((int)b * p.H + a_h[q]) * p.W + a_w[q]) * p.C * 4;
            }
            else
            {
                ph.fd_HpWp.divmod(m, b, rem);
                ph.fd_Wp.divmod(rem, r1, r2);
                a_h[q] = (int)r1 + ph.q0h;
                a_w[q] = (int)r2 + ph.q0w;
                a_base[q] = (((int)b * p.Ho + a_h[q]) * p.Wo + a_w[q]) * p.O * 4;
            }
            if (!live)
                a_h[q] = -(1 << 28);  // fails every bounds check
        }
        else
            a_krow[q] = idx / (BM / 4);
    }
    if (!A_KC)
    {
        const int mc = m0 + (tid % (BM / 4)) * 4;
        a_mvalid = mc < ph.M;
        uint32_t tap, c, di, dj;
        p.fd_C.divmod(mc, tap, c);
        p.fd_kw.divmod(tap, di, dj);
        a_dh = (int)di - p.pt;
        a_dw = (int)dj - p.pl;
        a_moff = ((a_dh * p.W + a_dw) * p.C + (int)c) * 4;
    }

    int b_off[NB];  // FWD/DK: running byte offset; DX: byte offset of the row (output channel)
#pragma unroll
    for (int q = 0; q < NB; ++q)
    {
        const int idx = tid + q * NTHREADS;
        if (B_KC)
        {
            const int n = n0 + idx / (BK / 4);
            b_off[q] = (n < p.ncols && idx < TB::CHUNKS) ? n * p.O * 4 : OOB;
        }
        else
        {
            const int n = n0 + (tid % (BN / 4)) * 4;
            const int krow = idx / (BN / 4);
            b_off[q] = (n < p.ncols && idx < TB::CHUNKS) ? ((s_begin * BK + krow) * p.ncols + n) * 4 : OOB;
        }
    }

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[a][b][r] = 0.f;

    // Two register sets: a slab's loads are issued one slab time before its data is needed in LDS.
    f32x4 ra0[NA], rb0[NB], ra1[NA], rb1[NB];

    // Issues the loads of one k-slab into a register set.  Nothing in here may turn into a branch
    // (the compiler counts outstanding loads exactly only in straight-line code): validity tests use
    // the decoded tap rather than k itself and are combined with bitwise AND, divisions run
    // unconditionally (dh::FastDiv is total on [0, 2^31)), slabs past s_end get out-of-range offsets.
    auto load_global = [&](f32x4* ra, f32x4* rb, int slab) {
        const int k0 = slab * BK;
        // decode of the k coordinate shared by all chunks of this thread
        int ka_off = 0, ka_d0 = 0, ka_d1 = 0, kb_off = 0;
        bool kvalid = true;
        if (MODE == MODE_FWD)
        {
            const int kk = k0 + kloc;
            uint32_t tap, c, di, dj;
            p.fd_C.divmod(kk, tap, c);
            p.fd_kw.divmod(tap, di, dj);
            kvalid = (int)di < p.kh;
            ka_d0 = (int)di; ka_d1 = (int)dj;
            ka_off = (((int)di * p.W + (int)dj) * p.C + (int)c) * 4;
        }
        else if (MODE == MODE_DX)
        {
            const int kk = k0 + kloc;
            uint32_t tap, o, th, tw;
            p.fd_O.divmod(kk, tap, o);
            ph.fd_ntw.divmod(tap, th, tw);
            kvalid = (int)th < ph.nth;
            ka_d0 = -(int)th; ka_d1 = -(int)tw;
            ka_off = ((int)o - ((int)th * p.Wo + (int)tw) * p.O) * 4;
            kb_off = ((((ph.rh + p.sh * (int)th) * p.kw + ph.rw + p.sw * (int)tw) * p.C) * p.O + (int)o) * 4;
        }
#pragma unroll
        for (int q = 0; q < NA; ++q)
        {
            int off;
            if (A_KC)
            {
                const int lim_h = MODE == MODE_FWD ? p.H : p.Ho, lim_w = MODE == MODE_FWD ? p.W : p.Wo;
                const bool ok = (int)kvalid & (int)((unsigned)(a_h[q] + ka_d0) < (unsigned)lim_h) &
                                (int)((unsigned)(a_w[q] + ka_d1) < (unsigned)lim_w) & (int)(slab < s_end);
                off = ok ? a_base[q] + ka_off : OOB;
            }
            else
            {
                const int kk = k0 + a_krow[q];
                uint32_t b, rem, i, j;
                p.fd_HoWo.divmod(kk, b, rem);
                p.fd_Wo.divmod(rem, i, j);
                const int h = (int)i * p.sh, w = (int)j * p.sw;
                const bool ok = (int)((int)b < p.N) & (int)a_mvalid & (int)((unsigned)(h + a_dh) < (unsigned)p.H) &
                                (int)((unsigned)(w + a_dw) < (unsigned)p.W) & (int)((tid + q * NTHREADS) < TA::CHUNKS) &
                                (int)(slab < s_end);
                off = ok ? (((int)b * p.H + h) * p.W + w) * p.C * 4 + a_moff : OOB;
            }
            ra[q] = buf_load4(ra_src, off);
        }
#pragma unroll
        for (int q = 0; q < NB; ++q)
        {
            int off;
            if (B_KC)
                off = ((int)kvalid & (int)(b_off[q] != OOB) & (int)(slab < s_end)) ? b_off[q] + kb_off : OOB;
            else
            {
                // rows past the end of the contraction lie past the end of the buffer
                off = slab < s_end ? b_off[q] : OOB;
                b_off[q] = b_off[q] != OOB ? b_off[q] + BK * p.ncols * 4 : OOB;
            }
            rb[q] = buf_load4(rb_src, off);
        }
    };
    auto store_lds = [&](const f32x4* ra, const f32x4* rb, int stage) {
#pragma unroll
        for (int q = 0; q < NA; ++q)
        {
            const int idx = tid + q * NTHREADS;
            if (TA::CHUNKS % NTHREADS == 0 || idx < TA::CHUNKS)
            {
                int row, k;
                TA::chunk(idx, row, k);
                TA::store(lds_a[stage], row, k, make_float4(ra[q].x, ra[q].y, ra[q].z, ra[q].w));
            }
        }
#pragma unroll
        for (int q = 0; q < NB; ++q)
        {
            const int idx = tid + q * NTHREADS;
            if (TB::CHUNKS % NTHREADS == 0 || idx < TB::CHUNKS)
            {
                int row, k;
                TB::chunk(idx, row, k);
                TB::store(lds_b[stage], row, k, make_float4(rb[q].x, rb[q].y, rb[q].z, rb[q].w));
            }
        }
    };

    auto multiply = [&](int stage) {
        float4 fa[2][TM], fb[2][TN];
#pragma unroll
        for (int a = 0; a < TM; ++a)
            fa[0][a] = TA::frag(lds_a[stage], wm0 + a * 32 + l32, 0, half);
#pragma unroll
        for (int b = 0; b < TN; ++b)
            fb[0][b] = TB::frag(lds_b[stage], wn0 + b * 32 + l32, 0, half);
#pragma unroll
        for (int kg = 0; kg < BK / 8; ++kg)
        {
            const int cur = kg & 1;
            if (kg + 1 < BK / 8)
            {
#pragma unroll
                for (int a = 0; a < TM; ++a)
                    fa[cur ^ 1][a] = TA::frag(lds_a[stage], wm0 + a * 32 + l32, kg + 1, half);
#pragma unroll
                for (int b = 0; b < TN; ++b)
                    fb[cur ^ 1][b] = TB::frag(lds_b[stage], wn0 + b * 32 + l32, kg + 1, half);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int a = 0; a < TM; ++a)
#pragma unroll
                    for (int b = 0; b < TN; ++b)
                        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                            reinterpret_cast<const float*>(&fb[cur][b])[j],
                            reinterpret_cast<const float*>(&fa[cur][a])[j], acc[a][b], 0, 0, 0);
        }
    };

    // Software pipeline over pairs of slabs; every load and LDS store inside the loop is
    // unconditional, which keeps the loop body free of branches.
    const int nmine = s_end - s_begin;
    if (nmine > 0)
    {
        load_global(ra0, rb0, s_begin);
        load_global(ra1, rb1, s_begin + 1);
        store_lds(ra0, rb0, 0);
        __syncthreads();
        int s = s_begin;
        for (int pair = 0; pair < nmine / 2; ++pair, s += 2)
        {
            // slab s is in LDS stage 0, slab s+1 in flight in register set 1
            load_global(ra0, rb0, s + 2);
            multiply(0);
            store_lds(ra1, rb1, 1);
            __syncthreads();
            // slab s+1 is in LDS stage 1, slab s+2 in flight in register set 0
            load_global(ra1, rb1, s + 3);
            multiply(1);
            store_lds(ra0, rb0, 0);
            __syncthreads();
        }
        if (nmine & 1)
            multiply(0);
    }

    write_tile<MODE, TM, TN>(p, ph, acc, m0 + wm0, n0 + wn0, l32, half);
}

// out[i] = act(bias[i % cols] + sum_s part[s][i]) -- the partial sums are added in split order, so
// the result does not depend on which workgroup finished first.
template <bool VEC>
__global__ __launch_bounds__(256) void splitk_reduce(const float* __restrict__ part, float* __restrict__ out,
                                                     const float* __restrict__ bias, size_t n, int cols,
                                                     int splitk, int act, float alpha)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    if (VEC)
    {
        const size_t n4 = n / 4;
        for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride)
        {
            float4 s = reinterpret_cast<const float4*>(part)[i];
            for (int k = 1; k < splitk; ++k)
            {
                const float4 t = reinterpret_cast<const float4*>(part + (size_t)k * n)[i];
                s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
            }
            if (bias)
            {
                const float4 b = *reinterpret_cast<const float4*>(bias + (i * 4) % cols);
                s.x += b.x; s.y += b.y; s.z += b.z; s.w += b.w;
            }
            s.x = apply_act(s.x, act, alpha); s.y = apply_act(s.y, act, alpha);
            s.z = apply_act(s.z, act, alpha); s.w = apply_act(s.w, act, alpha);
            reinterpret_cast<float4*>(out)[i] = s;
        }
    }
    else
    {
        for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        {
            float s = part[i];
            for (int k = 1; k < splitk; ++k)
                s += part[(size_t)k * n + i];
            if (bias)
                s += bias[i % cols];
            out[i] = apply_act(s, act, alpha);
        }
    }
}

// The same for many splits and a small output (filter gradients of thin layers): 16 lanes share one
// 16-byte piece of the output; lane g adds the splits g, g+16, g+32, ... in that order and the 16
// sums are then combined by a fixed butterfly, so the result is again independent of timing.
__global__ __launch_bounds__(256) void splitk_reduce_wide(const float* __restrict__ part, float* __restrict__ out,
                                                          const float* __restrict__ bias, size_t n, int cols,
                                                          int splitk, int act, float alpha)
{
    const size_t n4 = n / 4;
    const int g = threadIdx.x & 15;
    const size_t stride = (size_t)gridDim.x * (blockDim.x / 16);
    for (size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) / 16; i < n4; i += stride)
    {
        float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 4
        for (int k = g; k < splitk; k += 16)
        {
            const float4 t = reinterpret_cast<const float4*>(part + (size_t)k * n)[i];
            s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
        }
#pragma unroll
        for (int w = 8; w > 0; w >>= 1)
        {
            s.x += __shfl_xor(s.x, w, 16); s.y += __shfl_xor(s.y, w, 16);
            s.z += __shfl_xor(s.z, w, 16); s.w += __shfl_xor(s.w, w, 16);
        }
        if (g == 0)
        {
            if (bias)
            {
                const float4 b = *reinterpret_cast<const float4*>(bias + (i * 4) % cols);
                s.x += b.x; s.y += b.y; s.z += b.z; s.w += b.w;
            }
            s.x = apply_act(s.x, act, alpha); s.y = apply_act(s.y, act, alpha);
            s.z = apply_act(s.z, act, alpha); s.w = apply_act(s.w, act, alpha);
            reinterpret_cast<float4*>(out)[i] = s;
        }
    }
}

// ---- host side -----------------------------------------------------------------------------------

struct TileCfg { int bm, bn; };

double g_prof_flops = 0.0;  // algorithmic FLOPs of the operator being launched

// Bytes of the two operand tensors, for the buffer descriptors of the fast path (0 = too large).
struct OperandBytes { size_t a, b; };
OperandBytes g_operand_bytes = {0, 0};
bool g_force_generic = false;  // tests: exercise the general kernel on shapes the fast one would take

template <int MODE, int BM, int BN, int WGM, int WGN>
int launch_cfg(const ConvParams& p, dim3 grid, bool veca, bool vecb, hipStream_t st)
{
    const bool fast = veca && vecb && !g_force_generic && g_operand_bytes.a > 0 && g_operand_bytes.b > 0 &&
                      g_operand_bytes.a < (size_t(1) << 31) && g_operand_bytes.b < (size_t(1) << 31);
    int prof = -1;
    if (profiling())
    {
        char name[96];
        snprintf(name, sizeof(name), "conv_igemm<%s,%dx%d,%s%s>", MODE == MODE_FWD ? "fwd" : MODE == MODE_DX ? "dx" : "dk",
                 BM, BN, veca ? "v" : "s", vecb ? "v" : "s");
        if (fast)
            snprintf(name, sizeof(name), "conv_igemm_fast<%s,%dx%d>", MODE == MODE_FWD ? "fwd" : MODE == MODE_DX ? "dx" : "dk", BM, BN);
        prof = prof_begin(name, g_prof_flops, st);
    }
    if (fast)
        hipLaunchKernelGGL((conv_igemm_fast<MODE, BM, BN, WGM, WGN>), grid, dim3(NTHREADS), 0, st, p,
                           (uint32_t)g_operand_bytes.a, (uint32_t)g_operand_bytes.b);
    else if (veca && vecb)
        hipLaunchKernelGGL((conv_igemm<MODE, BM, BN, WGM, WGN, true, true>), grid, dim3(NTHREADS), 0, st, p);
    else if (veca)
        hipLaunchKernelGGL((conv_igemm<MODE, BM, BN, WGM, WGN, true, false>), grid, dim3(NTHREADS), 0, st, p);
    else if (vecb)
        hipLaunchKernelGGL((conv_igemm<MODE, BM, BN, WGM, WGN, false, true>), grid, dim3(NTHREADS), 0, st, p);
    else
        hipLaunchKernelGGL((conv_igemm<MODE, BM, BN, WGM, WGN, false, false>), grid, dim3(NTHREADS), 0, st, p);
    prof_end(prof, st);
    DH_LAUNCH_CHECK("conv_igemm launch");
    return 0;
}

inline bool aligned16(const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; }

// Runs the phases [z0, z0+nz) held in p.phase[0..nz).
template <int MODE>
int run_igemm(ConvParams& p, int nz, int max_m, bool veca, bool vecb, hipStream_t st, TileCfg cfg)
{
    p.vec_out = p.ncols % 4 == 0 && aligned16(p.out) && (!p.part || aligned16(p.part)) && p.out_elems % 4 == 0 &&
                (!p.bias || aligned16(p.bias));
    const int tiles_m = (max_m + cfg.bm - 1) / cfg.bm;
    const int tiles_n = (p.ncols + cfg.bn - 1) / cfg.bn;
    dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)p.splitk, (unsigned)nz);
    if (cfg.bm == 128 && cfg.bn == 128) return launch_cfg<MODE, 128, 128, 2, 2>(p, grid, veca, vecb, st);
    if (cfg.bm == 128 && cfg.bn == 64) return launch_cfg<MODE, 128, 64, 2, 2>(p, grid, veca, vecb, st);
    if (cfg.bm == 64 && cfg.bn == 64) return launch_cfg<MODE, 64, 64, 2, 2>(p, grid, veca, vecb, st);
    if (cfg.bm == 128 && cfg.bn == 32) return launch_cfg<MODE, 128, 32, 4, 1>(p, grid, veca, vecb, st);
    return fail(DH_EINVAL, "conv_igemm: no kernel for tile %dx%d", cfg.bm, cfg.bn);
}

TileCfg pick_tile(long M, long N)
{
    if (N <= 32) return {128, 32};
    if (N <= 64) return M <= 64 ? TileCfg{64, 64} : TileCfg{128, 64};
    if (M <= 64) return {64, 64};
    return {128, 128};
}

// Enough workgroups to give every compute unit two, as long as each split keeps >= 8 k-slabs.
int g_force_splitk = 0;  // tests and tuning: > 0 overrides the choice (still at most one split per k-slab)

int pick_splitk(long wgs, long min_slabs)
{
    if (g_force_splitk > 0)
        return (int)(g_force_splitk < min_slabs ? g_force_splitk : (min_slabs > 0 ? min_slabs : 1));
    const long target = 2L * num_cus();
    if (wgs >= target || min_slabs < 16)
        return 1;
    long s = (target + wgs - 1) / wgs;
    if (s > min_slabs / 8) s = min_slabs / 8;
    if (s > 256) s = 256;
    return s < 1 ? 1 : (int)s;
}

int check_geom(const char* who, int N, int H, int W, int C, int Ho, int Wo, int O, int kh, int kw,
               int sh, int sw, int pt, int pl)
{
    if (N <= 0 || H <= 0 || W <= 0 || C <= 0 || Ho <= 0 || Wo <= 0 || O <= 0 || kh <= 0 || kw <= 0 ||
        sh <= 0 || sw <= 0 || pt < 0 || pl < 0)
        return fail(DH_EINVAL, "%s: non-positive extent", who);
    if (pt >= kh || pl >= kw)
        return fail(DH_EINVAL, "%s: pad before (%d,%d) must be smaller than the filter (%d,%d)", who, pt, pl, kh, kw);
    const double lim = 2147483647.0;
    if ((double)N * H * W * C > lim || (double)N * Ho * Wo * O > lim || (double)kh * kw * C * O > lim)
        return fail(DH_EINVAL, "%s: tensor with more than 2^31-1 elements", who);
    // every output pixel must have its first tap at or before the last input pixel
    if ((long)(Ho - 1) * sh - pt >= H || (long)(Wo - 1) * sw - pl >= W)
        return fail(DH_EINVAL, "%s: output extent %dx%d does not fit input %dx%d", who, Ho, Wo, H, W);
    return 0;
}

void fill_common(ConvParams& p, int N, int H, int W, int C, int Ho, int Wo, int O, int kh, int kw,
                 int sh, int sw, int pt, int pl)
{
    p.N = N; p.H = H; p.W = W; p.C = C; p.Ho = Ho; p.Wo = Wo; p.O = O;
    p.kh = kh; p.kw = kw; p.sh = sh; p.sw = sw; p.pt = pt; p.pl = pl;
    p.fd_HoWo = FastDiv((uint32_t)Ho * Wo);
    p.fd_Wo = FastDiv(Wo);
    p.fd_C = FastDiv(C);
    p.fd_O = FastDiv(O);
    p.fd_kw = FastDiv(kw);
}

int finish_splitk(const ConvParams& p, hipStream_t st)
{
    if (p.splitk == 1)
        return 0;
    const size_t n = p.out_elems;
    const bool vec = n % 4 == 0 && p.ncols % 4 == 0 && aligned16(p.out) && (!p.bias || aligned16(p.bias));
    const size_t work = vec ? n / 4 : n;
    unsigned blocks = (unsigned)((work + 255) / 256);
    if (blocks > 4096) blocks = 4096;
    if (blocks == 0) blocks = 1;
    ProfScope prof("hbm:splitk_reduce (4 B x (splits + 1) per output)", 4.0 * n * (p.splitk + 1), st);
    if (vec && p.splitk >= 32)
    {
        // few outputs per split: spread the splits of one output over 16 lanes
        size_t wide = (n / 4 * 16 + 255) / 256;
        if (wide > 4096) wide = 4096;
        hipLaunchKernelGGL(splitk_reduce_wide, dim3((unsigned)wide), dim3(256), 0, st, p.part, p.out, p.bias, n,
                           p.ncols, p.splitk, p.act, p.alpha);
    }
    else if (vec)
        hipLaunchKernelGGL(splitk_reduce<true>, dim3(blocks), dim3(256), 0, st, p.part, p.out, p.bias, n,
                           p.ncols, p.splitk, p.act, p.alpha);
    else
        hipLaunchKernelGGL(splitk_reduce<false>, dim3(blocks), dim3(256), 0, st, p.part, p.out, p.bias, n,
                           p.ncols, p.splitk, p.act, p.alpha);
    DH_LAUNCH_CHECK("splitk_reduce launch");
    return 0;
}

}  // namespace

extern "C" {

int dh_conv2d_fwd(const float* x, const float* k, float* y, int N, int H, int W, int C, int kh, int kw,
                  int O, int sh, int sw, int pad_top, int pad_left, int Ho, int Wo, const float* bias,
                  int act, float alpha, void* stream)
{
    DH_TRY(ensure_init());
    DH_TRY(check_geom("dh_conv2d_fwd", N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pad_top, pad_left));
    if (!x || !k || !y) return fail(DH_EINVAL, "dh_conv2d_fwd: null tensor");
    ConvParams p{};
    fill_common(p, N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pad_top, pad_left);
    p.a_src = x; p.b_src = k; p.out = y; p.bias = bias; p.act = act; p.alpha = alpha;
    p.ncols = O;
    p.out_elems = (size_t)N * Ho * Wo * O;
    p.phase[0].M = N * Ho * Wo;
    p.phase[0].K = kh * kw * C;
    const TileCfg cfg = pick_tile(p.phase[0].M, O);
    const long wgs = (long)((p.phase[0].M + cfg.bm - 1) / cfg.bm) * ((O + cfg.bn - 1) / cfg.bn);
    p.splitk = pick_splitk(wgs, (p.phase[0].K + BK - 1) / BK);
    if (p.splitk > 1)
    {
        void* ws;
        DH_TRY(workspace(p.out_elems * sizeof(float) * p.splitk, &ws));
        p.part = static_cast<float*>(ws);
    }
    const bool veca = C % 4 == 0 && aligned16(x);
    const bool vecb = O % 4 == 0 && aligned16(k);
    g_prof_flops = 2.0 * N * Ho * Wo * O * kh * kw * C;
    g_operand_bytes = {(size_t)N * H * W * C * 4, (size_t)kh * kw * C * O * 4};
    DH_TRY(run_igemm<MODE_FWD>(p, 1, p.phase[0].M, veca, vecb, as_stream(stream), cfg));
    return finish_splitk(p, as_stream(stream));
}

int dh_conv2d_dx(const float* dy, const float* k, float* dx, int N, int Ho, int Wo, int O, int kh, int kw,
                 int C, int sh, int sw, int pad_top, int pad_left, int H, int W, const float* bias, int act,
                 float alpha, void* stream)
{
    DH_TRY(ensure_init());
    DH_TRY(check_geom("dh_conv2d_dx", N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pad_top, pad_left));
    if (!dy || !k || !dx) return fail(DH_EINVAL, "dh_conv2d_dx: null tensor");
    if (!g_force_generic)
    {
        const int rc = conv_dx_few_channels(dy, k, dx, N, Ho, Wo, O, kh, kw, C, sh, sw, pad_top, pad_left, H, W, bias,
                                            act, alpha, as_stream(stream));
        if (rc != 1)
            return rc;
    }
    ConvParams p{};
    fill_common(p, N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pad_top, pad_left);
    p.a_src = dy; p.b_src = k; p.out = dx; p.bias = bias; p.act = act; p.alpha = alpha;
    p.ncols = C;
    p.out_elems = (size_t)N * H * W * C;

    // one dense GEMM per output phase (h mod sh, w mod sw)
    Phase all[64];
    const int nph = sh * sw;
    if (nph > 64) return fail(DH_EINVAL, "dh_conv2d_dx: stride %dx%d not supported", sh, sw);
    long max_m = 0, min_slabs = 1L << 40, total_tiles_m = 0;
    int n_live = 0;
    for (int q = 0; q < nph; ++q)
    {
        Phase f{};
        f.ph = q / sw; f.pw = q % sw;
        f.Hp = f.ph < H ? (H - f.ph + sh - 1) / sh : 0;
        f.Wp = f.pw < W ? (W - f.pw + sw - 1) / sw : 0;
        if (f.Hp == 0 || f.Wp == 0)
            continue;  // no output pixel in this phase
        f.rh = (f.ph + pad_top) % sh; f.rw = (f.pw + pad_left) % sw;
        f.q0h = (f.ph + pad_top) / sh; f.q0w = (f.pw + pad_left) / sw;
        const int nth = f.rh < kh ? (kh - f.rh + sh - 1) / sh : 0;
        f.nth = nth;
        f.ntw = f.rw < kw ? (kw - f.rw + sw - 1) / sw : 0;
        f.M = N * f.Hp * f.Wp;
        f.K = nth * f.ntw * O;  // 0 taps: the phase is bias/activation of zero
        f.fd_HpWp = FastDiv((uint32_t)f.Hp * f.Wp);
        f.fd_Wp = FastDiv(f.Wp);
        f.fd_ntw = FastDiv(f.ntw > 0 ? f.ntw : 1);
        all[n_live++] = f;
        if (f.M > max_m) max_m = f.M;
        const long slabs = (f.K + BK - 1) / BK;
        if (slabs < min_slabs) min_slabs = slabs;
    }
    const TileCfg cfg = pick_tile(max_m, C);
    for (int q = 0; q < n_live; ++q)
        total_tiles_m += (all[q].M + cfg.bm - 1) / cfg.bm;
    p.splitk = pick_splitk(total_tiles_m * ((C + cfg.bn - 1) / cfg.bn), min_slabs);
    if (p.splitk > 1)
    {
        void* ws;
        DH_TRY(workspace(p.out_elems * sizeof(float) * p.splitk, &ws));
        p.part = static_cast<float*>(ws);
    }
    const bool veca = O % 4 == 0 && aligned16(dy);
    const bool vecb = O % 4 == 0 && aligned16(k);
    // one launch covers up to MAX_PHASES phases; the operator's FLOPs are split evenly over launches
    g_prof_flops = 2.0 * N * Ho * Wo * O * kh * kw * C / ((n_live + MAX_PHASES - 1) / MAX_PHASES > 0 ? (n_live + MAX_PHASES - 1) / MAX_PHASES : 1);
    g_operand_bytes = {(size_t)N * Ho * Wo * O * 4, (size_t)kh * kw * C * O * 4};
    for (int z0 = 0; z0 < n_live; z0 += MAX_PHASES)
    {
        const int nz = n_live - z0 < MAX_PHASES ? n_live - z0 : MAX_PHASES;
        long mm = 0;
        for (int q = 0; q < nz; ++q)
        {
            p.phase[q] = all[z0 + q];
            if (p.phase[q].M > mm) mm = p.phase[q].M;
        }
        DH_TRY(run_igemm<MODE_DX>(p, nz, (int)mm, veca, vecb, as_stream(stream), cfg));
    }
    return finish_splitk(p, as_stream(stream));
}

int dh_conv2d_dk(const float* x, const float* dy, float* dk, int N, int H, int W, int C, int Ho, int Wo,
                 int O, int kh, int kw, int sh, int sw, int pad_top, int pad_left, void* stream)
{
    DH_TRY(ensure_init());
    DH_TRY(check_geom("dh_conv2d_dk", N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pad_top, pad_left));
    if (!x || !dy || !dk) return fail(DH_EINVAL, "dh_conv2d_dk: null tensor");
    ConvParams p{};
    fill_common(p, N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pad_top, pad_left);
    p.a_src = x; p.b_src = dy; p.out = dk; p.bias = nullptr; p.act = DH_ACT_NONE; p.alpha = 0.f;
    p.ncols = O;
    p.out_elems = (size_t)kh * kw * C * O;
    p.phase[0].M = kh * kw * C;
    p.phase[0].K = N * Ho * Wo;
    const TileCfg cfg = pick_tile(p.phase[0].M, O);
    const long wgs = (long)((p.phase[0].M + cfg.bm - 1) / cfg.bm) * ((O + cfg.bn - 1) / cfg.bn);
    p.splitk = pick_splitk(wgs, (p.phase[0].K + BK - 1) / BK);
    if (p.splitk > 1)
    {
        void* ws;
        DH_TRY(workspace(p.out_elems * sizeof(float) * p.splitk, &ws));
        p.part = static_cast<float*>(ws);
    }
    const bool veca = C % 4 == 0 && aligned16(x);
    const bool vecb = O % 4 == 0 && aligned16(dy);
    g_prof_flops = 2.0 * N * Ho * Wo * O * kh * kw * C;
    g_operand_bytes = {(size_t)N * H * W * C * 4, (size_t)N * Ho * Wo * O * 4};
    DH_TRY(run_igemm<MODE_DK>(p, 1, p.phase[0].M, veca, vecb, as_stream(stream), cfg));
    return finish_splitk(p, as_stream(stream));
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

}
