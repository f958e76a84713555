/*
 * dcgan_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C, CPU-only restatement of the arithmetic of obs145628/dcgan-cuda's
 * convolution hot path.  It exists so that the HIP kernels can be compared with
 * the reference's operators on identical inputs.  Only tests, the smoke check and
 * the CPU-baseline leg of the benchmark may link or load this file; the shipped
 * library never does.
 *
 * Every function cites the reference file:line (relative to the reference tree)
 * whose arithmetic -- including the ORDER of the fp32 additions -- it follows.
 * All sums are accumulated in `acc_t`: build with -DORC_ACC_DOUBLE to get a
 * float64-accumulating twin (symbols get the suffix `_f64`), which the tests use
 * to tell rounding noise from real errors.  Build with -ffp-contract=off: the
 * reference is built without fused multiply-add on the host.
 *
 * Layouts are the reference's: activations NHWC, filters HWIO, row-major matrices.
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   conv2d                   reference literals (tests/test_conv2d.cu, test_conv2d_padding.cu)
 *                            + bit-exact vs the reference header built in oracle/_ref
 *                            + torch float64 conv2d
 *   conv2d_input_grad        adjoint identity, torch float64 autograd, bit-exact vs oracle/_ref
 *   conv2d_kernel_grad       adjoint identity, torch float64 autograd, bit-exact vs oracle/_ref
 *   conv2d_transpose         reference literal (tests/test_conv2d_transpose.cu) + torch conv_transpose2d
 *   conv2d_transpose_*_grad  torch float64 autograd of conv_transpose2d; reference literal
 *                            (tests/test_conv2d_transpose_grad.cu, VALID-equivalent shape) vs oracle/_ref
 *   element-wise / Adam / CE closed forms + reference literals + bit-exact vs oracle/_ref
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef ORC_ACC_DOUBLE
typedef double acc_t;
#define ORC(name) orc_##name##_f64
#else
typedef float acc_t;
#define ORC(name) orc_##name
#endif

#ifdef _OPENMP
#include <omp.h>
#endif

/* Number of host threads the loops below may use (1 = the reference's RT_MODE=CPU). */
void ORC(set_threads)(int n)
{
#ifdef _OPENMP
    omp_set_num_threads(n < 1 ? 1 : n);
#else
    (void)n;
#endif
}

int ORC(max_threads)(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------------------------
 * SAME-padding rule.  src/ops/conv2d.cu:26-46 (total pad) and :16-18 (output = ceil(in/s)).
 * pad_before = pad_total / 2 is applied inside the kernels (src/cpu/ops.hxx:204-205).
 * ---------------------------------------------------------------------------------------- */
void ORC(same_pad)(int in, int k, int s, int* pad_total, int* out)
{
    int p;
    if (in % s == 0)
        p = k - s;
    else
        p = k - (in % s);
    if (p < 0)
        p = 0;
    *pad_total = p;
    *out = (in + s - 1) / s;
}

/* ------------------------------------------------------------------------------------------
 * conv2d forward.  src/cpu/ops.hxx:189-254 with valid = 0 (the only mode the kernel table
 * uses, src/cpu/kernels.cu:12-18): output extent ceil(H/s), pad_before = pad_total / 2,
 * taps outside the image are skipped, the sum runs channel -> kernel row -> kernel column.
 *   x [N,H,W,C]  k [kh,kw,C,O]  y [N,Ho,Wo,O]
 * ---------------------------------------------------------------------------------------- */
void ORC(conv2d)(const float* x, const float* k, float* y,
                 int N, int H, int W, int C, int kh, int kw, int O,
                 int sh, int sw, int pad_h_total, int pad_w_total)
{
    const int pt = pad_h_total / 2;
    const int pl = pad_w_total / 2;
    const int Ho = (H + sh - 1) / sh;
    const int Wo = (W + sw - 1) / sw;
    const long rows = (long)N * Ho * Wo;
#pragma omp parallel for schedule(static)
    for (long r = 0; r < rows; ++r)
    {
        const int j = (int)(r % Wo);
        const int i = (int)((r / Wo) % Ho);
        const int b = (int)(r / ((long)Wo * Ho));
        /* The sums of the O output channels do not touch each other: they advance side by side
         * (o innermost, where filter and output are contiguous), each in the reference's order. */
        acc_t val[O > 0 ? O : 1];
        for (int o = 0; o < O; ++o)
            val[o] = 0;
        for (int c = 0; c < C; ++c)
            for (int di = 0; di < kh; ++di)
                for (int dj = 0; dj < kw; ++dj)
                {
                    const int h = sh * i + di - pt;
                    const int w = sw * j + dj - pl;
                    if (h >= 0 && w >= 0 && h < H && w < W)
                    {
                        const float xv = x[(((size_t)b * H + h) * W + w) * C + c];
                        const float* kr = k + (((size_t)di * kw + dj) * C + c) * O;
                        for (int o = 0; o < O; ++o)
                            val[o] += xv * kr[o];
                    }
                }
        for (int o = 0; o < O; ++o)
            y[(size_t)r * O + o] = (float)val[o];
    }
}

/* ------------------------------------------------------------------------------------------
 * conv2d input gradient.  src/cpu/ops.hxx:597-698.
 * The reference dilates dy by the stride, pads it by pad_h = H - (Hs - kh + 1) split as
 * (pad_h - pad_h/2) before and pad_h/2 after (:609-625), then for every (input channel,
 * filter) pair runs a stride-1 VALID correlation with the 180-degree rotated filter plane
 * (:651-657, accessor src/cpu/ops.hh:357-381) and adds the per-filter planes in filter order
 * (:667-672).  Products with the inserted zeros do not change an fp32 sum, so only the taps
 * that meet a real dy element are visited here; the order of the remaining additions (kernel
 * row, kernel column, then filters) is the reference's.
 *   dy [N,Ho,Wo,O]  k [kh,kw,C,O]  dx [N,H,W,C]
 * ---------------------------------------------------------------------------------------- */
void ORC(conv2d_input_grad)(const float* dy, const float* k, float* dx,
                            int N, int Ho, int Wo, int O, int kh, int kw, int C,
                            int stride, int H, int W)
{
    const int Hs = (Ho - 1) * (stride - 1) + Ho;
    const int Ws = (Wo - 1) * (stride - 1) + Wo;
    const int pad_h = H - (Hs - kh + 1);
    const int pad_w = W - (Ws - kw + 1);
    const int pad_top = pad_h - pad_h / 2;
    const int pad_left = pad_w - pad_w / 2;
    const long rows = (long)N * H * W;
#pragma omp parallel for schedule(static)
    for (long r = 0; r < rows; ++r)
    {
        const int w = (int)(r % W);
        const int h = (int)((r / W) % H);
        const int b = (int)(r / ((long)W * H));
        for (int c = 0; c < C; ++c)
        {
            /* one sum per filter, advanced side by side (f innermost: dy and k are contiguous in
             * f), each over (kernel row, kernel column) in the reference's order; then the sums are
             * added in filter order */
            acc_t val[O > 0 ? O : 1];
            for (int f = 0; f < O; ++f)
                val[f] = 0;
            for (int a = 0; a < kh; ++a)
            {
                const int th = h + a - pad_top;
                if (th < 0 || th % stride != 0 || th / stride >= Ho)
                    continue;
                for (int e = 0; e < kw; ++e)
                {
                    const int tw = w + e - pad_left;
                    if (tw < 0 || tw % stride != 0 || tw / stride >= Wo)
                        continue;
                    const float* dr = dy + (((size_t)b * Ho + th / stride) * Wo + tw / stride) * O;
                    const float* kr = k + (((size_t)(kh - 1 - a) * kw + (kw - 1 - e)) * C + c) * O;
                    for (int f = 0; f < O; ++f)
                        val[f] += dr[f] * kr[f];
                }
            }
            acc_t total = 0;
            for (int f = 0; f < O; ++f)
                total = (f == 0) ? val[f] : total + val[f];
            dx[(size_t)r * C + c] = (float)total;
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * conv2d kernel (filter) gradient.  src/cpu/ops.hxx:700-799.
 * Per (input channel, image) the reference correlates the image plane, padded like the
 * forward pass, with dy dilated by the stride and used as a (Hs x Ws) filter (:716-767),
 * adds the per-image results in image order (:776-781) and re-lays the result out as HWIO
 * (:793, formatDw :521-541).  Filter extent is derived: kh = H + pad_total - (Hs - 1)
 * (:753-756).  Only taps that meet a real dy element are visited (see above).
 *   dy [N,Ho,Wo,O]  x [N,H,W,C]  dk [kh,kw,C,O]
 * ---------------------------------------------------------------------------------------- */
void ORC(conv2d_kernel_grad)(const float* dy, const float* x, float* dk,
                             int N, int Ho, int Wo, int O, int H, int W, int C,
                             int stride, int pad_h_total, int pad_w_total)
{
    const int Hs = (Ho - 1) * (stride - 1) + Ho;
    const int Ws = (Wo - 1) * (stride - 1) + Wo;
    const int kh = H + pad_h_total - Hs + 1;
    const int kw = W + pad_w_total - Ws + 1;
    const int pt = pad_h_total / 2;
    const int pl = pad_w_total / 2;
    const long rows = (long)kh * kw * C;
#pragma omp parallel for schedule(static)
    for (long r = 0; r < rows; ++r)
    {
        const int c = (int)(r % C);
        const int dj = (int)((r / C) % kw);
        const int di = (int)(r / ((long)C * kw));
        /* one sum per output channel, advanced side by side (o innermost: dy and dk are contiguous
         * in o), each over (output row, output column) of one image in the reference's order; the
         * per-image sums are added in image order */
        acc_t total[O > 0 ? O : 1], val[O > 0 ? O : 1];
        for (int o = 0; o < O; ++o)
            total[o] = 0;
        for (int b = 0; b < N; ++b)
        {
            for (int o = 0; o < O; ++o)
                val[o] = 0;
            for (int i = 0; i < Ho; ++i)
            {
                const int h = di + stride * i - pt;
                if (h < 0 || h >= H)
                    continue;
                for (int j = 0; j < Wo; ++j)
                {
                    const int w = dj + stride * j - pl;
                    if (w < 0 || w >= W)
                        continue;
                    const float xv = x[(((size_t)b * H + h) * W + w) * C + c];
                    const float* dr = dy + (((size_t)b * Ho + i) * Wo + j) * O;
                    for (int o = 0; o < O; ++o)
                        val[o] += xv * dr[o];
                }
            }
            for (int o = 0; o < O; ++o)
                total[o] = (b == 0) ? val[o] : total[o] + val[o];
        }
        for (int o = 0; o < O; ++o)
            dk[(size_t)r * O + o] = (float)total[o];
    }
}

/* ------------------------------------------------------------------------------------------
 * conv2d_transpose forward = conv2d_input_grad with the caller's output extent.
 * src/cpu/ops.hxx:801-806.   x [N,Hi,Wi,Ci]  k [kh,kw,Co,Ci]  y [N,Hout,Wout,Co]
 * ---------------------------------------------------------------------------------------- */
void ORC(conv2d_transpose)(const float* x, const float* k, float* y,
                           int N, int Hi, int Wi, int Ci, int kh, int kw, int Co,
                           int stride, int Hout, int Wout)
{
    ORC(conv2d_input_grad)(x, k, y, N, Hi, Wi, Ci, kh, kw, Co, stride, Hout, Wout);
}

/* ------------------------------------------------------------------------------------------
 * conv2d_transpose input gradient = forward conv2d of dy with the pad re-derived from the
 * extents, pad_total = (Hi - 1) * s + kh - Hy.  src/gpu/conv2d.cu:214-259.  (The CPU function
 * src/cpu/ops.hxx:808-820 handles pad_total = 0 only and is not followed.)
 *   dy [N,Hy,Wy,Co]  k [kh,kw,Co,Ci]  dx [N,Hi,Wi,Ci]
 * The extent of the result is Hi = ceil(Hy / s) for every shape the operator API can build.
 * ---------------------------------------------------------------------------------------- */
void ORC(conv2d_transpose_input_grad)(const float* dy, const float* k, float* dx,
                                      int N, int Hy, int Wy, int Co, int kh, int kw, int Ci,
                                      int stride, int Hi, int Wi)
{
    const int pad_h = (Hi - 1) * stride + kh - Hy;
    const int pad_w = (Wi - 1) * stride + kw - Wy;
    ORC(conv2d)(dy, k, dx, N, Hy, Wy, Co, kh, kw, Ci, stride, stride, pad_h, pad_w);
}

/* ------------------------------------------------------------------------------------------
 * conv2d_transpose kernel gradient = conv2d kernel gradient with the roles of the two
 * activations exchanged: the transpose's output-side gradient plays "x", the transpose's
 * input plays "dy".  src/gpu/conv2d.cu:264-307.  (src/cpu/ops.hxx:822-902 handles
 * pad_total = 0 only and is not followed.)
 *   dy [N,Hy,Wy,Co]  x [N,Hi,Wi,Ci]  dk [kh,kw,Co,Ci]
 * ---------------------------------------------------------------------------------------- */
void ORC(conv2d_transpose_kernel_grad)(const float* dy, const float* x, float* dk,
                                       int N, int Hy, int Wy, int Co, int Hi, int Wi, int Ci,
                                       int stride, int kh, int kw)
{
    const int pad_h = (Hi - 1) * stride + kh - Hy;
    const int pad_w = (Wi - 1) * stride + kw - Wy;
    ORC(conv2d_kernel_grad)(x, dy, dk, N, Hi, Wi, Ci, Hy, Wy, Co, stride, pad_h, pad_w);
}

/* ------------------------------------------------------------------------------------------
 * Bias add (lowered to mat_rvect_add, src/ops/conv2d-bias-add.cu:35-38) and its gradient
 * (lowered to mat_sum_cols, src/ops/conv2d-bias-add-grad.cu:29-31).
 * src/cpu/ops.hxx:107-117 and :405-416 (serial sum down each column).
 * ---------------------------------------------------------------------------------------- */
void ORC(mvrow_add)(const float* a, const float* b, float* out, size_t rows, size_t cols)
{
    for (size_t i = 0; i < rows; ++i)
        for (size_t j = 0; j < cols; ++j)
            out[i * cols + j] = a[i * cols + j] + b[j];
}

void ORC(mat_sum_cols)(const float* a, float* out, size_t rows, size_t cols)
{
    for (size_t j = 0; j < cols; ++j)
    {
        acc_t s = 0;
        for (size_t i = 0; i < rows; ++i)
            s += a[i * cols + j];
        out[j] = (float)s;
    }
}

/* src/cpu/ops.hxx:391-403 */
void ORC(mat_sum_rows)(const float* a, float* out, size_t rows, size_t cols)
{
    for (size_t i = 0; i < rows; ++i)
    {
        acc_t s = 0;
        for (size_t j = 0; j < cols; ++j)
            s += a[i * cols + j];
        out[i] = (float)s;
    }
}

/* ------------------------------------------------------------------------------------------
 * Activations and their gradients.
 * relu  src/cpu/ops.hxx:302-326   relu_grad (z > 0)            :425-431
 * leaky :328-343                  leaky_relu_grad (z < 0)      :926-931
 * tanh = 2/(1+exp(-2x)) - 1 with the exp in float and the rest in double   :345-359
 * tanh_grad = (1 - pow(t,2.0)) * dout, the pow in double                    :461-466
 * sigmoid = 1/(1+exp(-x)), exp in float, add and divide in double           :13-17, :119-123
 * sigmoid_grad = s * (1 - s) * dout in float                                :368-373
 * ---------------------------------------------------------------------------------------- */
void ORC(relu)(const float* a, float* out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = a[i] < 0 ? 0 : a[i];
}

void ORC(relu_grad)(const float* z, const float* dout, float* out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = z[i] > 0 ? dout[i] : 0;
}

void ORC(relu_leaky)(const float* a, float* out, size_t n, float alpha)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = a[i] < 0 ? alpha * a[i] : a[i];
}

void ORC(leaky_relu_grad)(const float* z, const float* dout, float* out, float alpha, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = z[i] < 0 ? alpha * dout[i] : dout[i];
}

static float orc_tanh1(float x)
{
    return (float)((2.0 / (1.0 + (double)expf(-2 * x))) - 1.0);
}

static float orc_sigmoid1(float x)
{
    return (float)(1.0 / (1.0 + (double)expf(-x)));
}

void ORC(tanh)(const float* a, float* out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = orc_tanh1(a[i]);
}

void ORC(tanh_grad)(const float* t, const float* dout, float* out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = (float)((1 - pow((double)t[i], 2.0)) * (double)dout[i]);
}

void ORC(sigmoid)(const float* a, float* out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = orc_sigmoid1(a[i]);
}

void ORC(sigmoid_grad)(const float* s, const float* dout, float* out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = s[i] * (1 - s[i]) * dout[i];
}

/* src/cpu/ops.hxx:933-938 */
void ORC(add)(const float* a, const float* b, float* out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = a[i] + b[i];
}

/* ------------------------------------------------------------------------------------------
 * Sigmoid cross-entropy (mean over n) and its gradient.  src/cpu/ops.hxx:440-459.
 * (y = labels, x = logits; the reference's float `1 + exp` is an int + float = float sum.)
 * ---------------------------------------------------------------------------------------- */
float ORC(sigmoid_cross_entropy)(const float* y, const float* x, size_t n)
{
    acc_t res = 0;
    for (size_t i = 0; i < n; ++i)
    {
        if (x[i] >= 0)
            res += x[i] - x[i] * y[i] + logf(1 + expf(-x[i]));
        else
            res += -x[i] * y[i] + logf(1 + expf(x[i]));
    }
    return (float)(res / n);
}

void ORC(sigmoid_cross_entropy_grad)(const float* y, const float* x, float* out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = (orc_sigmoid1(x[i]) - y[i]) / n;
}

/* src/cpu/ops.hxx:129-136 and src/cpu/kernels.cu:110-113 (coeff = 2/len as double -> float) */
float ORC(mse)(const float* y, const float* y_hat, size_t rows, size_t cols)
{
    const size_t len = rows * cols;
    acc_t res = 0;
    for (size_t i = 0; i < len; ++i)
        res += (y[i] - y_hat[i]) * (y[i] - y_hat[i]);
    return (float)(res / len);
}

void ORC(mse_grad)(const float* y, const float* y_hat, float* out, size_t len)
{
    const float coeff = (float)(2. / len);
    for (size_t i = 0; i < len; ++i)
        out[i] = coeff * (y_hat[i] - y[i]);
}

/* ------------------------------------------------------------------------------------------
 * Dense-layer matrix products (serial dot products).  src/cpu/ops.hxx:56-105, :375-390.
 * ---------------------------------------------------------------------------------------- */
void ORC(mm_mul)(const float* a, const float* b, float* out, size_t m, size_t n, size_t p)
{
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)m; ++i)
        for (size_t j = 0; j < p; ++j)
        {
            acc_t x = 0;
            for (size_t k = 0; k < n; ++k)
                x += a[i * n + k] * b[k * p + j];
            out[i * p + j] = (float)x;
        }
}

/* out (m x p) = tr(a) * b, a is (n x m), b is (n x p) */
void ORC(tmm_mul)(const float* a, const float* b, float* out, size_t m, size_t n, size_t p)
{
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)m; ++i)
        for (size_t j = 0; j < p; ++j)
        {
            acc_t x = 0;
            for (size_t k = 0; k < n; ++k)
                x += a[k * m + i] * b[k * p + j];
            out[i * p + j] = (float)x;
        }
}

/* out (m x p) = a * tr(b), a is (m x n), b is (p x n) */
void ORC(mtm_mul)(const float* a, const float* b, float* out, size_t m, size_t n, size_t p)
{
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)m; ++i)
        for (size_t j = 0; j < p; ++j)
        {
            acc_t x = 0;
            for (size_t k = 0; k < n; ++k)
                x += a[i * n + k] * b[j * n + k];
            out[i * p + j] = (float)x;
        }
}

void ORC(mat_mul_add)(const float* x, const float* w, const float* b, float* out,
                      size_t m, size_t n, size_t p)
{
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)m; ++i)
        for (size_t j = 0; j < p; ++j)
        {
            acc_t s = 0;
            for (size_t k = 0; k < n; ++k)
                s += x[i * n + k] * w[k * p + j];
            out[i * p + j] = (float)s + b[j];
        }
}

/* ------------------------------------------------------------------------------------------
 * argmax accuracy: rows whose first-maximum indices agree.  src/cpu/ops.hxx:38-46, :468-476.
 * ---------------------------------------------------------------------------------------- */
static size_t orc_argmax1(const float* v, size_t n)
{
    size_t best = 0;
    for (size_t i = 1; i < n; ++i)
        if (v[i] > v[best])
            best = i;
    return best;
}

size_t ORC(argmax_acc)(const float* y, const float* y_hat, size_t rows, size_t cols)
{
    size_t res = 0;
    for (size_t i = 0; i < rows; ++i)
        res += orc_argmax1(y + i * cols, cols) == orc_argmax1(y_hat + i * cols, cols);
    return res;
}

/* ------------------------------------------------------------------------------------------
 * Adam.  Moments: src/cpu/ops.hxx:905-917 (`b * dv * dv` groups as (b*dv)*dv).
 * Step: src/cpu/kernels.cu:193-206 -- t is a float counter incremented first, the corrected
 * rate lr * sqrt(1 - beta2^t) / (1 - beta1^t) is formed with float pow/sqrt on the host --
 * then src/cpu/ops.hxx:919-924.
 * ---------------------------------------------------------------------------------------- */
void ORC(moment_update)(const float* dv, float* out, float a, float b, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = a * out[i] + b * dv[i];
}

void ORC(moment_update2)(const float* dv, float* out, float a, float b, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = a * out[i] + b * dv[i] * dv[i];
}

float ORC(adam_lrt)(float* t, float lr, float beta1, float beta2)
{
    ++*t;
    return lr * sqrtf(1 - powf(beta2, *t)) / (1 - powf(beta1, *t));
}

void ORC(adam_apply)(const float* m, const float* v, float* out, float lrt, float eps, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = out[i] - lrt * m[i] / (sqrtf(v[i]) + eps);
}

/* src/cpu/ops.hxx:432-438 (SGD step; not on the DCGAN path, kept for the operator table) */
void ORC(vect_update)(const float* dv, float* out, float coeff, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] += coeff * dv[i];
}

#ifndef ORC_ACC_DOUBLE
/* ------------------------------------------------------------------------------------------
 * xorshift generator used by the reference's seeded layer tests.
 * src/utils/xorshift.cu:13-40 (mirrored by tests/xorshift.py:5-24).
 * ---------------------------------------------------------------------------------------- */
typedef struct { uint64_t s[4]; } orc_rng;

void orc_xorshift_seed(orc_rng* r, uint64_t x)
{
    r->s[0] = 1000 * x;
    r->s[1] = 2000 * x;
    r->s[2] = 3000 * x;
    r->s[3] = 4000 * x;
}

uint64_t orc_xorshift_next_u64(orc_rng* r)
{
    uint64_t t = r->s[0] ^ (r->s[0] << 11);
    r->s[0] = r->s[1];
    r->s[1] = r->s[2];
    r->s[2] = r->s[3];
    r->s[3] = r->s[3] ^ (r->s[3] >> 19) ^ t ^ (t >> 8);
    return r->s[3];
}

void orc_xorshift_fill(orc_rng* r, float* out, size_t n)
{
    const float div = (float)0xFFFFFFFFFFFFFFFFull;
    for (size_t i = 0; i < n; ++i)
        out[i] = (float)orc_xorshift_next_u64(r) / div;
}
#endif
