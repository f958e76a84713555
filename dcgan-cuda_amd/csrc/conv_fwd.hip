// Forward convolution entry points: dh_conv2d_fwd, dh_conv2d_fwd_pair (see conv_igemm.inc for the kernels).
#include "conv_igemm.inc"

namespace
{
// One instance (x2 == y2 == nullptr) or two instances that share the filter.
int conv_fwd(const char* who, const float* x, const float* x2, const float* k, float* y, float* y2, int N, int H, int W,
             int C, int kh, int kw, int O, int sh, int sw, int pad_top, int pad_left, int Ho, int Wo, const float* bias,
             int act, float alpha, void* stream)
{
    DH_TRY(ensure_init());
    DH_TRY(check_geom(who, N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pad_top, pad_left));
    const bool pair = x2 != nullptr || y2 != nullptr;
    if (!x || !k || !y || (pair && (!x2 || !y2))) return fail(DH_EINVAL, "%s: null tensor", who);
    if (pair && !g_force_generic)
    {
        // the image layer of two towers: one launch over both batches
        const int rc = conv_fwd_rows(x, x2, k, y, y2, N, H, W, C, kh, kw, O, sh, sw, pad_top, pad_left, Ho, Wo, bias, act, alpha,
                                     as_stream(stream));
        if (rc != 1)
            return rc;
    }
    if (!pair && !g_force_generic)
    {
        const int rc = conv_fwd_thin(x, k, y, N, H, W, C, kh, kw, O, sh, sw, pad_top, pad_left, Ho, Wo, bias, act, alpha,
                                     as_stream(stream));
        if (rc != 1)
            return rc;
    }
    ConvParams p{};
    fill_common(p, N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pad_top, pad_left);
    p.a_src = x; p.b_src = k; p.out = y; p.bias = bias; p.act = act; p.alpha = alpha;
    p.a_src2 = x2; p.out2 = y2;
    p.ncols = O;
    p.out_elems = (size_t)N * Ho * Wo * O;
    p.phase[0].M = N * Ho * Wo;
    p.phase[0].K = kh * kw * C;
    const bool veca = C % 4 == 0 && aligned16(x) && aligned16(x2);
    const bool vecb = O % 4 == 0 && aligned16(k);
    g_operand_bytes = {(size_t)N * H * W * C * 4, (size_t)kh * kw * C * O * 4, C % BK == 0};
    if (pair && !takes_fast_path(veca, vecb))
        return fail(DH_ENOTSUP, "%s: the paired launch needs input channels divisible by 16, output channels divisible by 4, 16-byte aligned tensors below 2 GiB", who);
    TileCfg cfg = pick_tile(p.phase[0].M, O);
    const int instances = pair ? 2 : 1;
    if (takes_fast_path(veca, vecb))
    {
        const long tiles = (long)((p.phase[0].M + cfg.bm - 1) / cfg.bm) * ((O + cfg.bn - 1) / cfg.bn) * instances;
        cfg = narrower_if_split(cfg, tiles, tiles * ((p.phase[0].K + BK - 1) / BK));
        if (g_force_tile_width && cfg.bm == 128 && O > 64) cfg.bn = g_force_tile_width;
        if (g_tuning_width && cfg.bm == 128 && O > 64) cfg.bn = g_tuning_width;
        if (width_is_measured(cfg, tiles))
        {
            TuneKey key{MODE_FWD, N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pad_top, pad_left, pair ? 1 : 0, num_cus()};
            int width = 128;
            DH_TRY(measured_width(key, as_stream(stream), [&] {
                return conv_fwd(who, x, x2, k, y, y2, N, H, W, C, kh, kw, O, sh, sw, pad_top, pad_left, Ho, Wo, bias, act, alpha, stream);
            }, &width));
            cfg.bn = width;
        }
    }
    const long wgs = (long)((p.phase[0].M + cfg.bm - 1) / cfg.bm) * ((O + cfg.bn - 1) / cfg.bn) * instances;
    if (takes_fast_path(veca, vecb))
    {
        p.skip = p.posmajor = skipping_pays(wgs);
        g_prof_issued = 0.0;
        plan_launch<MODE_FWD>(p, p.phase, 1, cfg, pair);
    }
    else
        p.splitk = pick_splitk(wgs, (p.phase[0].K + BK - 1) / BK);
    if (p.splitk > 1)
    {
        void* ws;
        DH_TRY(workspace(p.out_elems * sizeof(float) * p.splitk * instances, &ws, as_stream(stream)));
        p.part = static_cast<float*>(ws);
    }
    g_prof_flops = 2.0 * N * Ho * Wo * O * kh * kw * C * instances;
    DH_TRY(run_igemm<MODE_FWD>(p, 1, p.phase[0].M, veca, vecb, as_stream(stream), cfg));
    return finish_splitk(p, as_stream(stream));
}
}  // namespace

extern "C" {

int dh_conv2d_fwd(const float* x, const float* k, float* y, int N, int H, int W, int C, int kh, int kw,
                  int O, int sh, int sw, int pad_top, int pad_left, int Ho, int Wo, const float* bias,
                  int act, float alpha, void* stream)
{
    return conv_fwd("dh_conv2d_fwd", x, nullptr, k, y, nullptr, N, H, W, C, kh, kw, O, sh, sw, pad_top, pad_left, Ho, Wo,
                    bias, act, alpha, stream);
}

int dh_conv2d_fwd_pair_supported(int N, int H, int W, int C, int kh, int kw, int O, int sh, int sw, int pad_top, int pad_left,
                                 int Ho, int Wo)
{
    if (N <= 0 || H <= 0 || W <= 0 || C <= 0 || O <= 0 || Ho <= 0 || Wo <= 0)
        return 0;
    if (fwd_rows_takes(N, H, W, C, kh, kw, O, sh, sw, pad_top, pad_left, Ho, Wo))
        return 1;
    const double lim = 2147483648.0;
    return C % BK == 0 && O % 4 == 0 && 4.0 * N * H * W * C < lim && 4.0 * N * Ho * Wo * O < lim && 4.0 * kh * kw * C * O < lim;
}

int dh_conv2d_fwd_pair(const float* x1, const float* x2, const float* k, float* y1, float* y2, int N, int H, int W,
                       int C, int kh, int kw, int O, int sh, int sw, int pad_top, int pad_left, int Ho, int Wo,
                       const float* bias, int act, float alpha, void* stream)
{
    if (!x2 || !y2) return fail(DH_EINVAL, "dh_conv2d_fwd_pair: null tensor");
    return conv_fwd("dh_conv2d_fwd_pair", x1, x2, k, y1, y2, N, H, W, C, kh, kw, O, sh, sw, pad_top, pad_left, Ho, Wo, bias,
                    act, alpha, stream);
}

}
