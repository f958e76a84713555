// ref_shim.cc -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// A thin extern "C" harness around the reference's own header-only CPU operators
// (src/cpu/ops.hh + ops.hxx of obs145628/dcgan-cuda), compiled from the sources where
// they lie (never copied into this repository) by oracle/Makefile into
// oracle/_ref/libdcgan_ref.so.  It is used (a) to check that oracle/dcgan_oracle.c restates
// the reference bit for bit and (b) as the "reference" CPU baseline of the benchmark.
// The argument order of each wrapper equals the matching orc_* function so that tests can
// call both through one table.
#include <cstddef>
#include <cstdint>
#include <map>
#include <vector>

#include "cpu/ops.hh"
#include "runtime/node.hh"
#include "runtime/graph.hh"
#include "runtime/nodes-list.hh"
#include "runtime/optimizer.hh"
#include "cpu/kernels.hh"
#include "cpu/runner.hh"
#include "cpu/thread-pool-runner.hh"

extern "C" {

// cpu::conv2d through the kernel-table signature (src/cpu/kernels.cu:12-18)
void ref_conv2d(const float* x, const float* k, float* y,
                int N, int H, int W, int C, int kh, int kw, int O,
                int sh, int sw, int pad_h_total, int pad_w_total)
{
    int strides[2] = {sh, sw};
    int xs[4] = {N, H, W, C};
    int ks[4] = {kh, kw, C, O};
    cpu::conv2d(x, k, y, strides, pad_h_total, pad_w_total, xs, ks, 0);
}

// src/cpu/kernels.cu:32-35
void ref_conv2d_input_grad(const float* dy, const float* k, float* dx,
                           int N, int Ho, int Wo, int O, int kh, int kw, int C,
                           int stride, int H, int W)
{
    int ys[4] = {N, Ho, Wo, O};
    int ks[4] = {kh, kw, C, O};
    int in_hw[2] = {H, W};
    cpu::conv2d_input_grad(dy, k, stride, ys, ks, dx, in_hw);
}

// src/cpu/kernels.cu:37-40
void ref_conv2d_kernel_grad(const float* dy, const float* x, float* dk,
                            int N, int Ho, int Wo, int O, int H, int W, int C,
                            int stride, int pad_h_total, int pad_w_total)
{
    int ys[4] = {N, Ho, Wo, O};
    int xs[4] = {N, H, W, C};
    int pads[2] = {pad_h_total, pad_w_total};
    cpu::conv2d_kernel_grad(dy, x, stride, ys, xs, dk, pads);
}

// src/cpu/kernels.cu:42-45
void ref_conv2d_transpose(const float* x, const float* k, float* y,
                          int N, int Hi, int Wi, int Ci, int kh, int kw, int Co,
                          int stride, int Hout, int Wout)
{
    int out_size[4] = {N, Hout, Wout, Co};
    int xs[4] = {N, Hi, Wi, Ci};
    int ks[4] = {kh, kw, Co, Ci};
    cpu::conv2d_transpose(x, k, out_size, stride, y, xs, ks);
}

// src/cpu/kernels.cu:47-50.  VALID-equivalent shapes only (pad_total == 0).
void ref_conv2d_transpose_input_grad(const float* dy, const float* k, float* dx,
                                     int N, int Hy, int Wy, int Co, int kh, int kw, int Ci,
                                     int stride, int Hi, int Wi)
{
    int ys[4] = {N, Hy, Wy, Co};
    int ks[4] = {kh, kw, Co, Ci};
    int in_hw[2] = {Hi, Wi};
    cpu::conv2d_transpose_input_grad(dy, k, stride, ys, ks, dx, in_hw);
}

// src/cpu/kernels.cu:52-55.  VALID-equivalent shapes only (pad_total == 0).
void ref_conv2d_transpose_kernel_grad(const float* dy, const float* x, float* dk,
                                      int N, int Hy, int Wy, int Co, int Hi, int Wi, int Ci,
                                      int stride, int kh, int kw)
{
    (void)kh; (void)kw;
    int ys[4] = {N, Hy, Wy, Co};
    int xs[4] = {N, Hi, Wi, Ci};
    cpu::conv2d_transpose_kernel_grad(dy, x, stride, ys, xs, dk);
}

void ref_mvrow_add(const float* a, const float* b, float* out, size_t rows, size_t cols)
{ cpu::mvrow_add(a, b, out, rows, cols); }
void ref_mat_sum_cols(const float* a, float* out, size_t rows, size_t cols)
{ cpu::mat_sum_cols(a, out, rows, cols); }
void ref_mat_sum_rows(const float* a, float* out, size_t rows, size_t cols)
{ cpu::mat_sum_rows(a, out, rows, cols); }
void ref_relu(const float* a, float* out, size_t n) { cpu::vect_relu(a, out, n); }
void ref_relu_grad(const float* z, const float* dout, float* out, size_t n)
{ cpu::relu_grad(z, dout, out, n); }
void ref_relu_leaky(const float* a, float* out, size_t n, float alpha)
{ cpu::vect_relu_leaky(a, out, n, alpha); }
void ref_leaky_relu_grad(const float* z, const float* dout, float* out, float alpha, size_t n)
{ cpu::leaky_relu_grad(z, dout, out, alpha, n); }
void ref_tanh(const float* a, float* out, size_t n) { cpu::vect_tanh(a, out, n); }
void ref_tanh_grad(const float* t, const float* dout, float* out, size_t n)
{ cpu::tanh_grad(t, dout, out, n); }
void ref_sigmoid(const float* a, float* out, size_t n) { cpu::vect_sigmoid(a, out, n); }
void ref_sigmoid_grad(const float* s, const float* dout, float* out, size_t n)
{ cpu::sigmoid_grad(s, dout, out, n); }
void ref_add(const float* a, const float* b, float* out, size_t n) { cpu::vect_add(a, b, out, n); }
float ref_sigmoid_cross_entropy(const float* y, const float* x, size_t n)
{ return cpu::sigmoid_cross_entropy(y, x, n); }
void ref_sigmoid_cross_entropy_grad(const float* y, const float* x, float* out, size_t n)
{ cpu::sigmoid_cross_entropy_grad(y, x, out, n); }
float ref_mse(const float* y, const float* y_hat, size_t rows, size_t cols)
{ return cpu::mse(y, y_hat, rows, cols); }
// src/cpu/kernels.cu:110-113
void ref_mse_grad(const float* y, const float* y_hat, float* out, size_t len)
{ cpu::vect_sub_coeff(y_hat, y, 2. / len, out, len); }
void ref_mm_mul(const float* a, const float* b, float* out, size_t m, size_t n, size_t p)
{ cpu::mm_mul(a, b, out, m, n, p); }
void ref_tmm_mul(const float* a, const float* b, float* out, size_t m, size_t n, size_t p)
{ cpu::tmm_mul(a, b, out, m, n, p); }
void ref_mtm_mul(const float* a, const float* b, float* out, size_t m, size_t n, size_t p)
{ cpu::mtm_mul(a, b, out, m, n, p); }
void ref_mat_mul_add(const float* x, const float* w, const float* b, float* out,
                     size_t m, size_t n, size_t p)
{ cpu::mat_mul_add(x, w, b, out, m, n, p); }
size_t ref_argmax_acc(const float* y, const float* y_hat, size_t rows, size_t cols)
{ return cpu::argmax_acc(y, y_hat, rows, cols); }
void ref_moment_update(const float* dv, float* out, float a, float b, size_t n)
{ cpu::moment_update(dv, out, a, b, n); }
void ref_moment_update2(const float* dv, float* out, float a, float b, size_t n)
{ cpu::moment_update2(dv, out, a, b, n); }
void ref_adam_apply(const float* m, const float* v, float* out, float lrt, float eps, size_t n)
{ cpu::adam_update(m, v, out, lrt, eps, n); }
void ref_vect_update(const float* dv, float* out, float coeff, size_t n)
{ cpu::vect_update(dv, out, coeff, n); }

// ---------------------------------------------------------------------------------------
// The reference's runtime: rt::Node lists executed by RT_MODE=CPU (cpu::run_sequential,
// src/cpu/runner.cu:10-14) or RT_MODE=MCPU (rt::optimize + cpu::ThreadPoolRunner,
// src/ops/graph.cu:180-192).  Nodes are built with the reference's own factory functions
// and kept in a reference rt::Graph which owns them.
// ---------------------------------------------------------------------------------------
struct RefProgram
{
    rt::Graph graph;
    std::vector<rt::Node*> nodes;
};

void* ref_program_new() { return new RefProgram; }
void ref_program_free(void* p) { delete static_cast<RefProgram*>(p); }

static int ref_push(void* p, rt::Node* n)
{
    auto prog = static_cast<RefProgram*>(p);
    prog->graph.add(n);
    prog->nodes.push_back(n);
    return int(prog->nodes.size()) - 1;
}

static std::vector<rt::Node*> ref_preds(void* p, const int* preds, int npreds)
{
    auto prog = static_cast<RefProgram*>(p);
    std::vector<rt::Node*> res;
    for (int i = 0; i < npreds; ++i)
        if (preds[i] >= 0)
            res.push_back(prog->nodes[preds[i]]);
    return res;
}

int ref_node_conv2d(void* p, const float* x, const float* k, float* y, const int* strides,
                    int pad_h_total, int pad_w_total, const int* xs, const int* ks,
                    const int* preds, int npreds)
{
    return ref_push(p, rt::Node::op_conv2d(x, k, strides, pad_h_total, pad_w_total, y, xs, ks,
                                           ref_preds(p, preds, npreds)));
}

int ref_node_conv2d_input_grad(void* p, const float* dy, const float* k, float* dx,
                               const int* strides, const int* ys, const int* ks, const int* xs,
                               const int* preds, int npreds)
{
    return ref_push(p, rt::Node::op_conv2d_input_grad(dy, k, strides, dx, ys, ks, xs,
                                                      ref_preds(p, preds, npreds)));
}

int ref_node_conv2d_kernel_grad(void* p, const float* dy, const float* x, float* dk,
                                const int* strides, const int* ys, const int* xs,
                                const int* pads, const int* preds, int npreds)
{
    return ref_push(p, rt::Node::op_conv2d_kernel_grad(dy, x, strides, dk, ys, xs, pads,
                                                       ref_preds(p, preds, npreds)));
}

int ref_node_conv2d_transpose(void* p, const float* x, const float* k, float* y,
                              const int* out_size, const int* strides, const int* xs,
                              const int* ks, const int* preds, int npreds)
{
    return ref_push(p, rt::Node::op_conv2d_transpose(x, k, out_size, strides, y, xs, ks,
                                                     ref_preds(p, preds, npreds)));
}

int ref_node_mat_rvect_add(void* p, const float* a, const float* b, float* out,
                           size_t rows, size_t cols, const int* preds, int npreds)
{
    return ref_push(p, rt::Node::op_mat_rvect_add(a, b, out, rows, cols,
                                                  ref_preds(p, preds, npreds)));
}

int ref_node_mat_sum_cols(void* p, const float* a, float* out, size_t rows, size_t cols,
                          const int* preds, int npreds)
{
    return ref_push(p, rt::Node::op_mat_sum_cols(a, out, rows, cols, ref_preds(p, preds, npreds)));
}

int ref_node_relu(void* p, const float* a, float* out, size_t n, const int* preds, int npreds)
{
    return ref_push(p, rt::Node::op_relu(a, out, n, ref_preds(p, preds, npreds)));
}

int ref_node_relu_leaky(void* p, const float* a, float* out, size_t n, float alpha,
                        const int* preds, int npreds)
{
    return ref_push(p, rt::Node::op_relu_leaky(a, out, n, alpha, ref_preds(p, preds, npreds)));
}

int ref_node_tanh(void* p, const float* a, float* out, size_t n, const int* preds, int npreds)
{
    return ref_push(p, rt::Node::op_tanh(a, out, n, ref_preds(p, preds, npreds)));
}

int ref_node_leaky_relu_grad(void* p, const float* z, const float* dout, float* out, float alpha,
                             size_t n, const int* preds, int npreds)
{
    return ref_push(p, rt::Node::op_leaky_relu_grad(z, dout, out, alpha, n,
                                                    ref_preds(p, preds, npreds)));
}

int ref_node_relu_grad(void* p, const float* z, const float* dout, float* out, size_t n,
                       const int* preds, int npreds)
{
    return ref_push(p, rt::Node::op_relu_grad(z, dout, out, n, ref_preds(p, preds, npreds)));
}

int ref_node_tanh_grad(void* p, const float* t, const float* dout, float* out, size_t n,
                       const int* preds, int npreds)
{
    return ref_push(p, rt::Node::op_tanh_grad(t, dout, out, n, ref_preds(p, preds, npreds)));
}

int ref_node_moment_update(void* p, float* var, const float* dt, float c1, float c2, size_t n,
                           const int* preds, int npreds)
{
    return ref_push(p, rt::Node::op_moment_update(var, dt, c1, c2, n, ref_preds(p, preds, npreds)));
}

int ref_node_moment_update2(void* p, float* var, const float* dt, float c1, float c2, size_t n,
                            const int* preds, int npreds)
{
    return ref_push(p, rt::Node::op_moment_update2(var, dt, c1, c2, n, ref_preds(p, preds, npreds)));
}

int ref_node_adam_update(void* p, float* var, float* t, const float* m, const float* v,
                         float lr, float beta1, float beta2, float eps, size_t n,
                         const int* preds, int npreds)
{
    return ref_push(p, rt::Node::op_adam_update(var, t, m, v, lr, beta1, beta2, eps, n,
                                                ref_preds(p, preds, npreds)));
}

int ref_node_add(void* p, const float* a, const float* b, float* out, size_t n,
                 const int* preds, int npreds)
{
    return ref_push(p, rt::Node::op_add(a, b, out, n, ref_preds(p, preds, npreds)));
}

// Run the nodes `outs` depend on.  mode 0 = RT_MODE=CPU, mode 1 = RT_MODE=MCPU with
// `nthreads` workers (the reference hard-codes 4, src/ops/graph.cu:32).
void ref_program_run(void* p, const int* outs, int nouts, int mode, int nthreads)
{
    auto prog = static_cast<RefProgram*>(p);
    std::vector<rt::Node*> targets;
    for (int i = 0; i < nouts; ++i)
        targets.push_back(prog->nodes[outs[i]]);
    auto sorted = prog->graph.topological_sort(targets);
    if (mode == 0)
    {
        rt::NodesList list(sorted);
        cpu::run_sequential(list);
    }
    else
    {
        cpu::ThreadPoolRunner pool(nthreads);
        std::map<rt::Node*, rt::Node*> opti_map;
        rt::Graph* opti = rt::optimize(prog->graph, opti_map);
        auto opti_targets = rt::convert_nodes(targets, opti_map);
        rt::NodesList list(opti->topological_sort(opti_targets));
        pool.run(list);
        delete opti;
    }
}

}
