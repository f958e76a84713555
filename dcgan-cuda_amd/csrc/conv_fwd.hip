// Forward convolution entry point: dh_conv2d_fwd (see conv_igemm.inc for the kernels).
#include "conv_igemm.inc"

extern "C" {

int dh_conv2d_fwd(const float* x, const float* k, float* y, int N, int H, int W, int C, int kh, int kw,
                  int O, int sh, int sw, int pad_top, int pad_left, int Ho, int Wo, const float* bias,
                  int act, float alpha, void* stream)
{
    DH_TRY(ensure_init());
    DH_TRY(check_geom("dh_conv2d_fwd", N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pad_top, pad_left));
    if (!x || !k || !y) return fail(DH_EINVAL, "dh_conv2d_fwd: null tensor");
    if (!g_force_generic)
    {
        const int rc = conv_fwd_thin(x, k, y, N, H, W, C, kh, kw, O, sh, sw, pad_top, pad_left, Ho, Wo, bias, act, alpha,
                                     as_stream(stream));
        if (rc != 1)
            return rc;
    }
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
        DH_TRY(workspace(p.out_elems * sizeof(float) * p.splitk, &ws, as_stream(stream)));
        p.part = static_cast<float*>(ws);
    }
    const bool veca = C % 4 == 0 && aligned16(x);
    const bool vecb = O % 4 == 0 && aligned16(k);
    g_prof_flops = 2.0 * N * Ho * Wo * O * kh * kw * C;
    g_operand_bytes = {(size_t)N * H * W * C * 4, (size_t)kh * kw * C * O * 4};
    DH_TRY(run_igemm<MODE_FWD>(p, 1, p.phase[0].M, veca, vecb, as_stream(stream), cfg));
    return finish_splitk(p, as_stream(stream));
}

}
