// Filter-gradient entry point: dh_conv2d_dk (see conv_igemm.inc for the kernels).
#include "conv_igemm.inc"

extern "C" {

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
        DH_TRY(workspace(p.out_elems * sizeof(float) * p.splitk, &ws, as_stream(stream)));
        p.part = static_cast<float*>(ws);
    }
    const bool veca = C % 4 == 0 && aligned16(x);
    const bool vecb = O % 4 == 0 && aligned16(dy);
    g_prof_flops = 2.0 * N * Ho * Wo * O * kh * kw * C;
    g_operand_bytes = {(size_t)N * H * W * C * 4, (size_t)N * Ho * Wo * O * 4};
    DH_TRY(run_igemm<MODE_DK>(p, 1, p.phase[0].M, veca, vecb, as_stream(stream), cfg));
    return finish_splitk(p, as_stream(stream));
}

}
