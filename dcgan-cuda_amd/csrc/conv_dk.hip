// Filter-gradient entry points: dh_conv2d_dk, dh_conv2d_dk_pair (see conv_igemm.inc for the kernels).
#include "conv_igemm.inc"

namespace
{
// dk(x, dy), or dk(x, dy) + dk(x2, dy2) in one contraction over both.
int conv_dk(const char* who, const float* x, const float* dy, const float* x2, const float* dy2, float* dk, int N, int H,
            int W, int C, int Ho, int Wo, int O, int kh, int kw, int sh, int sw, int pad_top, int pad_left, void* stream)
{
    DH_TRY(ensure_init());
    DH_TRY(check_geom(who, N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pad_top, pad_left));
    const bool pair = x2 != nullptr || dy2 != nullptr;
    if (!x || !dy || !dk || (pair && (!x2 || !dy2))) return fail(DH_EINVAL, "%s: null tensor", who);
    if (!g_force_generic && aligned16(dk))
    {
        float* part = nullptr;
        int splits = 0;
        const int rc = conv_dk_thin(x, dy, x2, dy2, &part, &splits, N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pad_top, pad_left,
                                    as_stream(stream));
        if (rc == 0)
        {
            // the slices are added in slice order, 16 lanes per output
            const size_t n = (size_t)kh * kw * C * O;
            size_t blocks = (n / 4 * 16 + 255) / 256;
            if (blocks > 4096) blocks = 4096;
            ProfScope prof("hbm:splitk_reduce (4 B x (splits + 1) per output)", 4.0 * n * (splits + 1), as_stream(stream));
            hipLaunchKernelGGL(splitk_reduce_wide, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), part, dk,
                               (float*)nullptr, (const float*)nullptr, n, n, O, splits, (int)DH_ACT_NONE, 0.f);
            DH_LAUNCH_CHECK("splitk_reduce_wide launch");
            return 0;
        }
        if (rc != 1)
            return rc;
    }
    ConvParams p{};
    fill_common(p, N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pad_top, pad_left);
    p.a_src = x; p.b_src = dy; p.out = dk; p.bias = nullptr; p.act = DH_ACT_NONE; p.alpha = 0.f;
    p.a_src2 = x2; p.b_src2 = dy2;
    p.ncols = O;
    p.out_elems = (size_t)kh * kw * C * O;
    p.phase[0].M = kh * kw * C;
    p.phase[0].K = N * Ho * Wo;
    const bool veca = C % 4 == 0 && aligned16(x) && aligned16(x2);
    const bool vecb = O % 4 == 0 && aligned16(dy) && aligned16(dy2);
    g_operand_bytes = {(size_t)N * H * W * C * 4, (size_t)N * Ho * Wo * O * 4, true};
    if (pair && !takes_fast_path(veca, vecb))
        return fail(DH_ENOTSUP, "%s: the paired launch needs channel counts divisible by 4, 16-byte aligned tensors below 2 GiB", who);
    const long slabs_one = (p.phase[0].K + BK - 1) / BK;
    const TileCfg cfg = pick_tile(p.phase[0].M, O);
    if (takes_fast_path(veca, vecb))
    {
        p.skip = N % BK == 0;
        g_prof_issued = 0.0;
        plan_launch<MODE_DK>(p, p.phase, 1, cfg, pair);
    }
    else
    {
        const long wgs = (long)((p.phase[0].M + cfg.bm - 1) / cfg.bm) * ((O + cfg.bn - 1) / cfg.bn);
        p.splitk = pick_splitk(wgs, slabs_one * (pair ? 2 : 1));
    }
    if (p.splitk > 1)
    {
        void* ws;
        DH_TRY(workspace(p.out_elems * sizeof(float) * p.splitk, &ws, as_stream(stream)));
        p.part = static_cast<float*>(ws);
    }
    g_prof_flops = 2.0 * N * Ho * Wo * O * kh * kw * C * (pair ? 2 : 1);
    DH_TRY(run_igemm<MODE_DK>(p, 1, p.phase[0].M, veca, vecb, as_stream(stream), cfg));
    return finish_splitk(p, as_stream(stream));
}
}  // namespace

extern "C" {

int dh_conv2d_dk_pair_supported(int N, int H, int W, int C, int Ho, int Wo, int O, int kh, int kw, int sh, int sw)
{
    (void)sh;
    if (ensure_init() != 0) return 0;
    const double lim = 2147483648.0;
    if (4.0 * N * H * W * C >= lim || 4.0 * N * Ho * Wo * O >= lim || 4.0 * kh * kw * C * O >= lim) return 0;
    if (g_force_generic) return 0;
    return (C % 4 == 0 && O % 4 == 0) || dk_thin_takes(N, H, W, C, Ho, Wo, O, kh, kw, sw) ? 1 : 0;
}

int dh_conv2d_dk(const float* x, const float* dy, float* dk, int N, int H, int W, int C, int Ho, int Wo,
                 int O, int kh, int kw, int sh, int sw, int pad_top, int pad_left, void* stream)
{
    return conv_dk("dh_conv2d_dk", x, dy, nullptr, nullptr, dk, N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pad_top, pad_left,
                   stream);
}

int dh_conv2d_dk_pair(const float* x1, const float* dy1, const float* x2, const float* dy2, float* dk, int N, int H,
                      int W, int C, int Ho, int Wo, int O, int kh, int kw, int sh, int sw, int pad_top, int pad_left,
                      void* stream)
{
    if (!x2 || !dy2) return fail(DH_EINVAL, "dh_conv2d_dk_pair: null tensor");
    return conv_dk("dh_conv2d_dk_pair", x1, dy1, x2, dy2, dk, N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pad_top, pad_left,
                   stream);
}

}
