// Host-side brute-force check of the convolution kernel's slab box (slab_set, SlabIter in
// csrc/conv_igemm.inc): for every tile of a set of shapes and the three products, every element that
// is inside the image must lie in a slab the iterator lists, the iterator must list each slab of the
// box once, and seek() must agree with next().  Compiled for the host only by tests/test_slab_box.py.
#include "conv_igemm.inc"
#include <set>
#include <cstdlib>
namespace dh { int fail(int c, const char*, ...) { return c; } int fail_hip(hipError_t, const char*) { return 1; } int ensure_init() { return 0; }
int workspace(size_t, void**, hipStream_t) { return 0; } int num_cus() { return 256; } bool profiling(int) { return false; }
int prof_begin(const char*, double, hipStream_t, int) { return -1; } void prof_end(int, hipStream_t) {} bool g_force_generic = false; int g_force_splitk = 0; }

static int same_pad(int n, int k, int s) { int p = n % s == 0 ? k - s : k - n % s; return p > 0 ? p : 0; }
static long checked = 0;

template <int MODE>
static bool run(ConvParams& p, const Phase& ph, int bm, int z = 0)
{
    for (int m0 = 0; m0 < ph.M; m0 += bm)
    {
        SlabSet s = slab_set<MODE>(p, ph, m0, bm, z);
        std::set<long> listed;
        SlabIter it; it.seek(s, 0);
        for (int t = 0; t < s.count(); ++t)
        {
            if (it.inst != 0) { printf("inst != 0 at t=%d\n", t); return false; }
            long key = ((long)it.o1 * 100000 + it.o2) * 100000 + it.cs;
            if (!listed.insert(key).second) { printf("duplicate slab\n"); return false; }
            // seek agrees with next
            SlabIter j; j.seek(s, t);
            if (j.o1 != it.o1 || j.o2 != it.o2 || j.cs != it.cs) { printf("seek != next at %d\n", t); return false; }
            it.next(s);
        }
        if (it.inst != 1) { printf("iterator did not wrap to instance 1\n"); return false; }
        const int m1 = imin(m0 + bm, ph.M);
        for (int m = m0; m < m1; ++m)
            for (int k = 0; k < ph.K; ++k)
            {
                bool valid; long key;
                if (MODE == MODE_FWD)
                {
                    int pos = p.posmajor ? pixel_of<MODE_FWD>(p, z, m / p.N) : m % (p.Ho * p.Wo), i = pos / p.Wo, j = pos % p.Wo;
                    int tap = k / p.C, c = k % p.C, di = tap / p.kw, dj = tap % p.kw;
                    int ih = i * p.sh + di - p.pt, iw = j * p.sw + dj - p.pl;
                    valid = ih >= 0 && ih < p.H && iw >= 0 && iw < p.W;
                    key = ((long)di * 100000 + dj) * 100000 + c / BK;   // the kernel's slabs never straddle taps
                }
                else if (MODE == MODE_DX)
                {
                    int pos = p.posmajor ? pixel_of<MODE_DX>(p, z, m / p.N) : m % (ph.Hp * ph.Wp), hh = pos / ph.Wp, ww = pos % ph.Wp;
                    int tap = k / p.O, o = k % p.O, th = tap / ph.ntw, tw = tap % ph.ntw;
                    int i = hh + ph.q0h - th, j = ww + ph.q0w - tw;
                    valid = i >= 0 && i < p.Ho && j >= 0 && j < p.Wo;
                    key = ((long)th * 100000 + tw) * 100000 + o / BK;
                }
                else
                {
                    // contraction index k in position-major order when skipping
                    int b, i, j;
                    if (p.skip) { int pos = k / p.N; b = k % p.N; i = pos / p.Wo; j = pos % p.Wo; }
                    else { b = k / (p.Ho * p.Wo); int r = k % (p.Ho * p.Wo); i = r / p.Wo; j = r % p.Wo; }
                    int tap = m / p.C, di = tap / p.kw, dj = tap % p.kw;
                    int ih = i * p.sh + di - p.pt, iw = j * p.sw + dj - p.pl;
                    valid = ih >= 0 && ih < p.H && iw >= 0 && iw < p.W;
                    key = p.skip ? ((long)i * 100000 + j) * 100000 + b / BK : k / BK;
                }
                ++checked;
                if (valid && !listed.count(key)) { printf("mode %d: live element m=%d k=%d outside the box (tile m0=%d)\n", MODE, m, k, m0); return false; }
            }
    }
    return true;
}

int main()
{
    int fails = 0, permuted = 0; long saved = 0, nominal = 0, saved_perm = 0;
    const int shapes[][8] = { // N H W C O kh sh
        {64, 16, 16, 16, 16, 5, 2}, {32, 9, 7, 16, 16, 5, 2}, {64, 5, 5, 16, 16, 5, 2}, {32, 6, 6, 16, 16, 3, 1},
        {16, 8, 8, 16, 32, 5, 2}, {32, 8, 8, 32, 16, 5, 2}, {16, 9, 7, 16, 16, 5, 2}, {16, 4, 4, 16, 16, 5, 2}, {16, 6, 6, 16, 16, 3, 1},
        {16, 7, 7, 16, 16, 4, 3}, {64, 8, 8, 32, 16, 5, 2}, {48, 5, 5, 16, 32, 5, 2}, {16, 3, 3, 16, 16, 5, 2}, {16, 2, 2, 16, 16, 5, 2},
        {16, 1, 1, 16, 16, 5, 2}, {3, 8, 8, 16, 16, 5, 2}, {16, 8, 8, 4, 8, 5, 2}, {20, 6, 8, 24, 40, 5, 2}, {16, 16, 16, 16, 16, 5, 2}, {128, 4, 4, 16, 16, 5, 2}};
    for (auto& sh : shapes)
        for (int bm : {64, 128})
        {
            int N = sh[0], H = sh[1], W = sh[2], C = sh[3], O = sh[4], kh = sh[5], s = sh[6], kw = kh;
            int Ho = (H + s - 1) / s, Wo = (W + s - 1) / s, pt = same_pad(H, kh, s) / 2, pl = same_pad(W, kw, s) / 2;
            ConvParams p{};
            fill_common(p, N, H, W, C, Ho, Wo, O, kh, kw, s, s, pt, pl);
            // FWD
            p.ncols = O; p.phase[0] = Phase{}; p.phase[0].M = N * Ho * Wo; p.phase[0].K = kh * kw * C; p.skip = p.posmajor = 0;
            p.use_perm = 0;
            if (C % BK == 0 && !run<MODE_FWD>(p, p.phase[0], bm)) { ++fails; printf("  FWD (nothing skipped) shape N%d H%d W%d C%d O%d k%d s%d bm%d\n", N, H, W, C, O, kh, s, bm); }
            p.skip = p.posmajor = C % BK == 0;
            if (p.skip && !run<MODE_FWD>(p, p.phase[0], bm)) { ++fails; printf("  FWD shape N%d H%d W%d C%d O%d k%d s%d bm%d\n", N, H, W, C, O, kh, s, bm); }
            order_pixels<MODE_FWD>(p, p.phase, 1, TileCfg{bm, 128});
            if (p.use_perm)
            {
                ++permuted;
                if (!run<MODE_FWD>(p, p.phase[0], bm)) { ++fails; printf("  FWD (permuted pixels) shape N%d H%d W%d C%d O%d k%d s%d bm%d\n", N, H, W, C, O, kh, s, bm); }
                for (int m0 = 0; m0 < p.phase[0].M; m0 += bm) saved_perm += slab_set<MODE_FWD>(p, p.phase[0], m0, bm, 0).count();
            }
            p.use_perm = 0;
            if (p.skip) for (int m0 = 0; m0 < p.phase[0].M; m0 += bm) { saved += slab_set<MODE_FWD>(p, p.phase[0], m0, bm, 0).count(); nominal += (p.phase[0].K + BK - 1) / BK; }
            // DK
            p.phase[0].M = kh * kw * C; p.phase[0].K = N * Ho * Wo; p.skip = N % BK == 0;
            if (!run<MODE_DK>(p, p.phase[0], bm)) { ++fails; printf("  DK shape N%d H%d W%d C%d O%d k%d s%d bm%d\n", N, H, W, C, O, kh, s, bm); }
            // DX phases
            p.ncols = C; p.skip = p.posmajor = O % BK == 0;
            Phase live[MAX_PHASES]; int nlive = 0;
            for (int q = 0; q < s * s; ++q)
            {
                Phase f{};
                f.ph = q / s; f.pw = q % s;
                f.Hp = f.ph < H ? (H - f.ph + s - 1) / s : 0; f.Wp = f.pw < W ? (W - f.pw + s - 1) / s : 0;
                if (!f.Hp || !f.Wp) continue;
                f.rh = (f.ph + pt) % s; f.rw = (f.pw + pl) % s; f.q0h = (f.ph + pt) / s; f.q0w = (f.pw + pl) / s;
                f.nth = f.rh < kh ? (kh - f.rh + s - 1) / s : 0; f.ntw = f.rw < kw ? (kw - f.rw + s - 1) / s : 0;
                f.M = N * f.Hp * f.Wp; f.K = f.nth * f.ntw * O;
                f.fd_HpWp = FastDiv(f.Hp * f.Wp); f.fd_Wp = FastDiv(f.Wp); f.fd_ntw = FastDiv(f.ntw > 0 ? f.ntw : 1);
                if (f.K == 0) continue;
                p.use_perm = 0;
                if (O % BK != 0) continue;
                p.skip = p.posmajor = 0;
                if (!run<MODE_DX>(p, f, bm)) { ++fails; printf("  DX (nothing skipped) shape N%d H%d W%d C%d O%d k%d s%d bm%d phase %d\n", N, H, W, C, O, kh, s, bm, q); }
                p.skip = p.posmajor = 1;
                if (!run<MODE_DX>(p, f, bm)) { ++fails; printf("  DX shape N%d H%d W%d C%d O%d k%d s%d bm%d phase %d\n", N, H, W, C, O, kh, s, bm, q); }
                if (nlive < MAX_PHASES) live[nlive++] = f;
            }
            order_pixels<MODE_DX>(p, live, nlive, TileCfg{bm, 128});
            if (p.use_perm)
            {
                ++permuted;
                for (int z = 0; z < nlive; ++z)
                    if (!run<MODE_DX>(p, live[z], bm, z)) { ++fails; printf("  DX (permuted pixels) shape N%d H%d W%d C%d O%d k%d s%d bm%d slot %d\n", N, H, W, C, O, kh, s, bm, z); }
            }
            p.use_perm = 0;
        }
    printf("%ld element checks, %d failures; FWD slabs kept %ld of %ld; %d launches with permuted pixels (FWD slabs kept %ld)\n",
           checked, fails, saved, nominal, permuted, saved_perm);
    if (permuted == 0) { printf("no shape exercised the permuted pixel order\n"); return 1; }
    return fails != 0;
}
