// Input-gradient / transposed-convolution entry points: dh_conv2d_dx, dh_conv2d_dx_pair (see
// conv_igemm.inc for the kernels).
#include "conv_igemm.inc"

#include <algorithm>

namespace
{
// One instance (dy2 == dx2 == nullptr) or two instances that share the filter.
int conv_dx(const char* who, const float* dy, const float* dy2, const float* k, float* dx, float* dx2, int N, int Ho,
            int Wo, int O, int kh, int kw, int C, int sh, int sw, int pad_top, int pad_left, int H, int W,
            const float* bias, int act, float alpha, void* stream)
{
    DH_TRY(ensure_init());
    DH_TRY(check_geom(who, N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pad_top, pad_left));
    const bool pair = dy2 != nullptr || dx2 != nullptr;
    if (!dy || !k || !dx || (pair && (!dy2 || !dx2))) return fail(DH_EINVAL, "%s: null tensor", who);
    if (!pair && !g_force_generic)
    {
        const int rc0 = conv_dx_col2im(dy, k, dx, N, Ho, Wo, O, kh, kw, C, sh, sw, pad_top, pad_left, H, W, bias, act, alpha,
                                       as_stream(stream));
        if (rc0 != 1)
            return rc0;
        const int rc = conv_dx_few_channels(dy, k, dx, N, Ho, Wo, O, kh, kw, C, sh, sw, pad_top, pad_left, H, W, bias,
                                            act, alpha, as_stream(stream));
        if (rc != 1)
            return rc;
    }
    ConvParams p{};
    fill_common(p, N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pad_top, pad_left);
    p.a_src = dy; p.b_src = k; p.out = dx; p.bias = bias; p.act = act; p.alpha = alpha;
    p.a_src2 = dy2; p.out2 = dx2;
    p.ncols = C;
    p.out_elems = (size_t)N * H * W * C;

    // one dense GEMM per output phase (h mod sh, w mod sw)
    Phase all[64];
    const int nph = sh * sw;
    if (nph > 64) return fail(DH_EINVAL, "%s: stride %dx%d not supported", who, sh, sw);
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
    // Launch order of the phases.  Their contractions differ in length (9, 6, 6 and 4 taps for 5x5
    // stride 2) and the workgroups of one launch are handed to the compute units in grid order, a
    // second round joining the first on each unit.  Longest first, then the short half in reverse
    // (9, 6, 4, 6) makes the workgroups that share a unit add up to about the same work; in plain
    // order (9, 6, 6, 4) the units that got 9 + 6 finish long after those with 6 + 4 (measured: +5
    // to +9 points of MFMA peak at batch 64 and 256).
    std::sort(all, all + n_live, [](const Phase& a, const Phase& b) { return a.K > b.K; });
    std::reverse(all + (n_live + 1) / 2, all + n_live);
    const bool veca = O % 4 == 0 && aligned16(dy) && aligned16(dy2);
    const bool vecb = O % 4 == 0 && aligned16(k);
    g_operand_bytes = {(size_t)N * Ho * Wo * O * 4, (size_t)kh * kw * C * O * 4, O % BK == 0};
    if (pair && (!takes_fast_path(veca, vecb) || C % 4 != 0))
        return fail(DH_ENOTSUP, "%s: the paired launch needs dy channels divisible by 16, result channels divisible by 4, 16-byte aligned tensors below 2 GiB", who);
    const int instances = pair ? 2 : 1;
    TileCfg cfg = pick_tile(max_m, C);
    if (takes_fast_path(veca, vecb))
    {
        long tiles = 0, slabs = 0;
        for (int q = 0; q < n_live; ++q)
        {
            const long t = (all[q].M + cfg.bm - 1) / cfg.bm * ((C + cfg.bn - 1) / cfg.bn) * instances;
            tiles += t;
            slabs += t * ((all[q].K + BK - 1) / BK);
        }
        cfg = narrower_if_split(cfg, tiles, slabs);
        if (g_force_tile_width && cfg.bm == 128 && C > 64) cfg.bn = g_force_tile_width;
        if (g_tuning_width && cfg.bm == 128 && C > 64) cfg.bn = g_tuning_width;
        if (width_is_measured(cfg, tiles))
        {
            TuneKey key{MODE_DX, N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pad_top, pad_left, pair ? 1 : 0, num_cus()};
            int width = 128;
            DH_TRY(measured_width(key, as_stream(stream), [&] {
                return conv_dx(who, dy, dy2, k, dx, dx2, N, Ho, Wo, O, kh, kw, C, sh, sw, pad_top, pad_left, H, W, bias, act, alpha, stream);
            }, &width));
            cfg.bn = width;
        }
    }
    for (int q = 0; q < n_live; ++q)
        total_tiles_m += (all[q].M + cfg.bm - 1) / cfg.bm;
    if (takes_fast_path(veca, vecb))
    {
        p.skip = p.posmajor = skipping_pays(total_tiles_m * ((C + cfg.bn - 1) / cfg.bn) * instances);
        g_prof_issued = 0.0;
        plan_launch<MODE_DX>(p, all, n_live, cfg, pair);
    }
    else
        p.splitk = pick_splitk(total_tiles_m * ((C + cfg.bn - 1) / cfg.bn) * instances, min_slabs);
    if (p.splitk > 1)
    {
        void* ws;
        DH_TRY(workspace(p.out_elems * sizeof(float) * p.splitk * instances, &ws, as_stream(stream)));
        p.part = static_cast<float*>(ws);
    }
    // one launch covers up to MAX_PHASES phases; the operator's FLOPs are split evenly over launches
    const int launches = (n_live + MAX_PHASES - 1) / MAX_PHASES > 0 ? (n_live + MAX_PHASES - 1) / MAX_PHASES : 1;
    g_prof_flops = 2.0 * N * Ho * Wo * O * kh * kw * C * instances / launches;
    g_prof_issued /= launches;
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
}  // namespace

extern "C" {

int dh_conv2d_dx(const float* dy, const float* k, float* dx, int N, int Ho, int Wo, int O, int kh, int kw,
                 int C, int sh, int sw, int pad_top, int pad_left, int H, int W, const float* bias, int act,
                 float alpha, void* stream)
{
    return conv_dx("dh_conv2d_dx", dy, nullptr, k, dx, nullptr, N, Ho, Wo, O, kh, kw, C, sh, sw, pad_top, pad_left, H, W,
                   bias, act, alpha, stream);
}

int dh_conv2d_dx_pair(const float* dy1, const float* dy2, const float* k, float* dx1, float* dx2, int N, int Ho,
                      int Wo, int O, int kh, int kw, int C, int sh, int sw, int pad_top, int pad_left, int H, int W,
                      const float* bias, int act, float alpha, void* stream)
{
    if (!dy2 || !dx2) return fail(DH_EINVAL, "dh_conv2d_dx_pair: null tensor");
    return conv_dx("dh_conv2d_dx_pair", dy1, dy2, k, dx1, dx2, N, Ho, Wo, O, kh, kw, C, sh, sw, pad_top, pad_left, H, W,
                   bias, act, alpha, stream);
}

}
