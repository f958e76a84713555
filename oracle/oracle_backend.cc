// oracle_backend.cc -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// Plugs the CPU oracle (dcgan_oracle.c) into the host library's backend registry as the
// RT_MODE=CPU runner, so that the operator graph, the differentiation and the rt::Node packing can
// be exercised without a GPU and a whole DCGAN iteration can be evaluated on the CPU as the
// reference for the HIP backend.  Node decoding follows the reference's CPU kernel table
// (src/cpu/kernels.cu:12-216), except for the two conv2d_transpose gradients, which follow the
// reference's GPU entries (src/gpu/conv2d.cu:214-307) because its CPU functions handle
// VALID-equivalent shapes only.  Instructions run in list order on the calling thread
// (src/cpu/runner.cu:10-14).
#include <cmath>
#include <cstddef>
#include <stdexcept>
#include <string>

#include "backend.hh"

extern "C" {
void orc_conv2d(const float*, const float*, float*, int, int, int, int, int, int, int, int, int, int, int);
void orc_conv2d_input_grad(const float*, const float*, float*, int, int, int, int, int, int, int, int, int, int);
void orc_conv2d_kernel_grad(const float*, const float*, float*, int, int, int, int, int, int, int, int, int, int);
void orc_conv2d_transpose(const float*, const float*, float*, int, int, int, int, int, int, int, int, int, int);
void orc_conv2d_transpose_input_grad(const float*, const float*, float*, int, int, int, int, int, int, int, int, int, int);
void orc_conv2d_transpose_kernel_grad(const float*, const float*, float*, int, int, int, int, int, int, int, int, int, int);
void orc_mvrow_add(const float*, const float*, float*, size_t, size_t);
void orc_mat_sum_cols(const float*, float*, size_t, size_t);
void orc_mat_sum_rows(const float*, float*, size_t, size_t);
void orc_relu(const float*, float*, size_t);
void orc_relu_grad(const float*, const float*, float*, size_t);
void orc_relu_leaky(const float*, float*, size_t, float);
void orc_leaky_relu_grad(const float*, const float*, float*, float, size_t);
void orc_tanh(const float*, float*, size_t);
void orc_tanh_grad(const float*, const float*, float*, size_t);
void orc_sigmoid(const float*, float*, size_t);
void orc_sigmoid_grad(const float*, const float*, float*, size_t);
void orc_add(const float*, const float*, float*, size_t);
float orc_sigmoid_cross_entropy(const float*, const float*, size_t);
void orc_sigmoid_cross_entropy_grad(const float*, const float*, float*, size_t);
float orc_mse(const float*, const float*, size_t, size_t);
void orc_mse_grad(const float*, const float*, float*, size_t);
void orc_mm_mul(const float*, const float*, float*, size_t, size_t, size_t);
void orc_tmm_mul(const float*, const float*, float*, size_t, size_t, size_t);
void orc_mtm_mul(const float*, const float*, float*, size_t, size_t, size_t);
void orc_mat_mul_add(const float*, const float*, const float*, float*, size_t, size_t, size_t);
size_t orc_argmax_acc(const float*, const float*, size_t, size_t);
void orc_moment_update(const float*, float*, float, float, size_t);
void orc_moment_update2(const float*, float*, float, float, size_t);
float orc_adam_lrt(float*, float, float, float);
void orc_adam_apply(const float*, const float*, float*, float, float, size_t);
void orc_vect_update(const float*, float*, float, size_t);
}

namespace
{
using rt::Node;

void run_node(Node* n)
{
    switch (n->type)
    {
    case Node::OP_CONV2D:
        orc_conv2d(n->in1, n->in2, n->out1, n->sizes1[0], n->sizes1[1], n->sizes1[2], n->sizes1[3], n->sizes2[0],
                   n->sizes2[1], n->sizes2[3], n->intconst[0], n->intconst[1], n->int_cons1, n->int_cons2);
        break;
    case Node::OP_CONV2D_INPUT_GRAD:
        orc_conv2d_input_grad(n->in1, n->in2, n->out1, n->sizes1[0], n->sizes1[1], n->sizes1[2], n->sizes1[3],
                              n->sizes2[0], n->sizes2[1], n->sizes2[2], n->intconst[0], n->intconst2[0], n->intconst2[1]);
        break;
    case Node::OP_CONV2D_KERNEL_GRAD:
        orc_conv2d_kernel_grad(n->in1, n->in2, n->out1, n->sizes1[0], n->sizes1[1], n->sizes1[2], n->sizes1[3],
                               n->sizes2[1], n->sizes2[2], n->sizes2[3], n->intconst[0], n->intconst2[0], n->intconst2[1]);
        break;
    case Node::OP_CONV2D_TRANSPOSE:
        orc_conv2d_transpose(n->in1, n->in2, n->out1, n->sizes2[0], n->sizes2[1], n->sizes2[2], n->sizes2[3],
                             n->sizes3[0], n->sizes3[1], n->sizes3[2], n->intconst[0], n->sizes1[1], n->sizes1[2]);
        break;
    case Node::OP_CONV2D_TRANSPOSE_INPUT_GRAD:
        orc_conv2d_transpose_input_grad(n->in1, n->in2, n->out1, n->sizes1[0], n->sizes1[1], n->sizes1[2], n->sizes1[3],
                                        n->sizes2[0], n->sizes2[1], n->sizes2[3], n->intconst[0], n->intconst2[0],
                                        n->intconst2[1]);
        break;
    case Node::OP_CONV2D_TRANSPOSE_KERNEL_GRAD:
        orc_conv2d_transpose_kernel_grad(n->in1, n->in2, n->out1, n->sizes1[0], n->sizes1[1], n->sizes1[2], n->sizes1[3],
                                         n->sizes2[1], n->sizes2[2], n->sizes2[3], n->intconst[0], n->sizes3[0],
                                         n->sizes3[1]);
        break;
    case Node::OP_MAT_MAT_MUL: orc_mm_mul(n->in1, n->in2, n->out1, n->len1, n->len2, n->len3); break;
    case Node::OP_MAT_RVECT_ADD: orc_mvrow_add(n->in1, n->in2, n->out1, n->len1, n->len2); break;
    case Node::OP_MAT_MUL_ADD: orc_mat_mul_add(n->in1, n->in2, n->in3, n->out1, n->len1, n->len2, n->len3); break;
    case Node::OP_TMAT_MAT_MUL: orc_tmm_mul(n->in1, n->in2, n->out1, n->len1, n->len2, n->len3); break;
    case Node::OP_MAT_TMAT_MUL: orc_mtm_mul(n->in1, n->in2, n->out1, n->len1, n->len2, n->len3); break;
    case Node::OP_MAT_SUM_ROWS: orc_mat_sum_rows(n->in1, n->out1, n->len1, n->len2); break;
    case Node::OP_MAT_SUM_COLS: orc_mat_sum_cols(n->in1, n->out1, n->len1, n->len2); break;
    case Node::OP_RELU: orc_relu(n->in1, n->out1, n->len1); break;
    case Node::OP_RELU_LEAKY: orc_relu_leaky(n->in1, n->out1, n->len1, n->alpha_leaky); break;
    case Node::OP_TANH: orc_tanh(n->in1, n->out1, n->len1); break;
    case Node::OP_SIGMOID: orc_sigmoid(n->in1, n->out1, n->len1); break;
    case Node::OP_RELU_GRAD: orc_relu_grad(n->in1, n->in2, n->out1, n->len1); break;
    case Node::OP_LEAKY_RELU_GRAD: orc_leaky_relu_grad(n->in1, n->in2, n->out1, n->cons1, n->len1); break;
    case Node::OP_TANH_GRAD: orc_tanh_grad(n->in1, n->in2, n->out1, n->len1); break;
    case Node::OP_SIGMOID_GRAD: orc_sigmoid_grad(n->in1, n->in2, n->out1, n->len1); break;
    case Node::OP_ADD: orc_add(n->in1, n->in2, n->out1, n->len1); break;
    case Node::OP_SIGMOID_CROSS_ENTROPY: *n->out1 = orc_sigmoid_cross_entropy(n->in1, n->in2, n->len1); break;
    case Node::OP_SIGMOID_CROSS_ENTROPY_GRAD: orc_sigmoid_cross_entropy_grad(n->in1, n->in2, n->out1, n->len1); break;
    case Node::OP_MSE: *n->out1 = orc_mse(n->in1, n->in2, n->len1, n->len2); break;
    case Node::OP_MSE_GRAD: orc_mse_grad(n->in1, n->in2, n->out1, n->len1); break;
    case Node::OP_ARGMAX_ACC: *n->out1 = (float)orc_argmax_acc(n->in1, n->in2, n->len1, n->len2); break;
    case Node::OP_UPDATE: orc_vect_update(n->in1, n->out1, *n->in2, n->len1); break;
    case Node::OP_MOMENT_UPDATE: orc_moment_update(n->in1, n->out1, n->cons1, n->cons2, n->len1); break;
    case Node::OP_MOMENT_UPDATE2: orc_moment_update2(n->in1, n->out1, n->cons1, n->cons2, n->len1); break;
    case Node::OP_ADAM_UPDATE:
    {
        const float lrt = orc_adam_lrt(n->out2, n->cons1, n->cons2, n->cons3);
        orc_adam_apply(n->in1, n->in2, n->out1, lrt, n->cons4, n->len1);
        break;
    }
    default:
        throw std::runtime_error(std::string("oracle backend: operator '") + Node::name_of(n->type) + "' not restated");
    }
}

void run_sequential(rt::NodesList& tasks)
{
    for (Node* n : tasks.nodes())
        run_node(n);
}
}  // namespace

extern "C" void orc_register_backend(void)
{
    rt::register_cpu_backend(ProgramMode::MONOTHREAD, run_sequential);
    rt::register_cpu_backend(ProgramMode::MULTITHREAD, run_sequential);
}
