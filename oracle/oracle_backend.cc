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

// -DORC_BACKEND_F64 binds the float64-accumulating twin of every function (and registers as
// orc_register_backend_f64): the yardstick that tells rounding noise from real errors.
#ifdef ORC_BACKEND_F64
#define O(name) orc_##name##_f64
#define ORC_REGISTER orc_register_backend_f64
#else
#define O(name) orc_##name
#define ORC_REGISTER orc_register_backend
#endif

extern "C" {
void O(conv2d)(const float*, const float*, float*, int, int, int, int, int, int, int, int, int, int, int);
void O(conv2d_input_grad)(const float*, const float*, float*, int, int, int, int, int, int, int, int, int, int);
void O(conv2d_kernel_grad)(const float*, const float*, float*, int, int, int, int, int, int, int, int, int, int);
void O(conv2d_transpose)(const float*, const float*, float*, int, int, int, int, int, int, int, int, int, int);
void O(conv2d_transpose_input_grad)(const float*, const float*, float*, int, int, int, int, int, int, int, int, int, int);
void O(conv2d_transpose_kernel_grad)(const float*, const float*, float*, int, int, int, int, int, int, int, int, int, int);
void O(mvrow_add)(const float*, const float*, float*, size_t, size_t);
void O(mat_sum_cols)(const float*, float*, size_t, size_t);
void O(mat_sum_rows)(const float*, float*, size_t, size_t);
void O(relu)(const float*, float*, size_t);
void O(relu_grad)(const float*, const float*, float*, size_t);
void O(relu_leaky)(const float*, float*, size_t, float);
void O(leaky_relu_grad)(const float*, const float*, float*, float, size_t);
void O(tanh)(const float*, float*, size_t);
void O(tanh_grad)(const float*, const float*, float*, size_t);
void O(sigmoid)(const float*, float*, size_t);
void O(sigmoid_grad)(const float*, const float*, float*, size_t);
void O(add)(const float*, const float*, float*, size_t);
float O(sigmoid_cross_entropy)(const float*, const float*, size_t);
void O(sigmoid_cross_entropy_grad)(const float*, const float*, float*, size_t);
float O(mse)(const float*, const float*, size_t, size_t);
void O(mse_grad)(const float*, const float*, float*, size_t);
void O(mm_mul)(const float*, const float*, float*, size_t, size_t, size_t);
void O(tmm_mul)(const float*, const float*, float*, size_t, size_t, size_t);
void O(mtm_mul)(const float*, const float*, float*, size_t, size_t, size_t);
void O(mat_mul_add)(const float*, const float*, const float*, float*, size_t, size_t, size_t);
size_t O(argmax_acc)(const float*, const float*, size_t, size_t);
void O(moment_update)(const float*, float*, float, float, size_t);
void O(moment_update2)(const float*, float*, float, float, size_t);
float O(adam_lrt)(float*, float, float, float);
void O(adam_apply)(const float*, const float*, float*, float, float, size_t);
void O(vect_update)(const float*, float*, float, size_t);
}

namespace
{
using rt::Node;

void run_node(Node* n)
{
    switch (n->type)
    {
    case Node::OP_CONV2D:
        O(conv2d)(n->in1, n->in2, n->out1, n->sizes1[0], n->sizes1[1], n->sizes1[2], n->sizes1[3], n->sizes2[0],
                   n->sizes2[1], n->sizes2[3], n->intconst[0], n->intconst[1], n->int_cons1, n->int_cons2);
        break;
    case Node::OP_CONV2D_INPUT_GRAD:
        O(conv2d_input_grad)(n->in1, n->in2, n->out1, n->sizes1[0], n->sizes1[1], n->sizes1[2], n->sizes1[3],
                              n->sizes2[0], n->sizes2[1], n->sizes2[2], n->intconst[0], n->intconst2[0], n->intconst2[1]);
        break;
    case Node::OP_CONV2D_KERNEL_GRAD:
        O(conv2d_kernel_grad)(n->in1, n->in2, n->out1, n->sizes1[0], n->sizes1[1], n->sizes1[2], n->sizes1[3],
                               n->sizes2[1], n->sizes2[2], n->sizes2[3], n->intconst[0], n->intconst2[0], n->intconst2[1]);
        break;
    case Node::OP_CONV2D_TRANSPOSE:
        O(conv2d_transpose)(n->in1, n->in2, n->out1, n->sizes2[0], n->sizes2[1], n->sizes2[2], n->sizes2[3],
                             n->sizes3[0], n->sizes3[1], n->sizes3[2], n->intconst[0], n->sizes1[1], n->sizes1[2]);
        break;
    case Node::OP_CONV2D_TRANSPOSE_INPUT_GRAD:
        O(conv2d_transpose_input_grad)(n->in1, n->in2, n->out1, n->sizes1[0], n->sizes1[1], n->sizes1[2], n->sizes1[3],
                                        n->sizes2[0], n->sizes2[1], n->sizes2[3], n->intconst[0], n->intconst2[0],
                                        n->intconst2[1]);
        break;
    case Node::OP_CONV2D_TRANSPOSE_KERNEL_GRAD:
        O(conv2d_transpose_kernel_grad)(n->in1, n->in2, n->out1, n->sizes1[0], n->sizes1[1], n->sizes1[2], n->sizes1[3],
                                         n->sizes2[1], n->sizes2[2], n->sizes2[3], n->intconst[0], n->sizes3[0],
                                         n->sizes3[1]);
        break;
    case Node::OP_MAT_MAT_MUL: O(mm_mul)(n->in1, n->in2, n->out1, n->len1, n->len2, n->len3); break;
    case Node::OP_MAT_RVECT_ADD: O(mvrow_add)(n->in1, n->in2, n->out1, n->len1, n->len2); break;
    case Node::OP_MAT_MUL_ADD: O(mat_mul_add)(n->in1, n->in2, n->in3, n->out1, n->len1, n->len2, n->len3); break;
    case Node::OP_TMAT_MAT_MUL: O(tmm_mul)(n->in1, n->in2, n->out1, n->len1, n->len2, n->len3); break;
    case Node::OP_MAT_TMAT_MUL: O(mtm_mul)(n->in1, n->in2, n->out1, n->len1, n->len2, n->len3); break;
    case Node::OP_MAT_SUM_ROWS: O(mat_sum_rows)(n->in1, n->out1, n->len1, n->len2); break;
    case Node::OP_MAT_SUM_COLS: O(mat_sum_cols)(n->in1, n->out1, n->len1, n->len2); break;
    case Node::OP_RELU: O(relu)(n->in1, n->out1, n->len1); break;
    case Node::OP_RELU_LEAKY: O(relu_leaky)(n->in1, n->out1, n->len1, n->alpha_leaky); break;
    case Node::OP_TANH: O(tanh)(n->in1, n->out1, n->len1); break;
    case Node::OP_SIGMOID: O(sigmoid)(n->in1, n->out1, n->len1); break;
    case Node::OP_RELU_GRAD: O(relu_grad)(n->in1, n->in2, n->out1, n->len1); break;
    case Node::OP_LEAKY_RELU_GRAD: O(leaky_relu_grad)(n->in1, n->in2, n->out1, n->cons1, n->len1); break;
    case Node::OP_TANH_GRAD: O(tanh_grad)(n->in1, n->in2, n->out1, n->len1); break;
    case Node::OP_SIGMOID_GRAD: O(sigmoid_grad)(n->in1, n->in2, n->out1, n->len1); break;
    case Node::OP_ADD: O(add)(n->in1, n->in2, n->out1, n->len1); break;
    case Node::OP_SIGMOID_CROSS_ENTROPY: *n->out1 = O(sigmoid_cross_entropy)(n->in1, n->in2, n->len1); break;
    case Node::OP_SIGMOID_CROSS_ENTROPY_GRAD: O(sigmoid_cross_entropy_grad)(n->in1, n->in2, n->out1, n->len1); break;
    case Node::OP_MSE: *n->out1 = O(mse)(n->in1, n->in2, n->len1, n->len2); break;
    case Node::OP_MSE_GRAD: O(mse_grad)(n->in1, n->in2, n->out1, n->len1); break;
    case Node::OP_ARGMAX_ACC: *n->out1 = (float)O(argmax_acc)(n->in1, n->in2, n->len1, n->len2); break;
    case Node::OP_UPDATE: O(vect_update)(n->in1, n->out1, *n->in2, n->len1); break;
    case Node::OP_MOMENT_UPDATE: O(moment_update)(n->in1, n->out1, n->cons1, n->cons2, n->len1); break;
    case Node::OP_MOMENT_UPDATE2: O(moment_update2)(n->in1, n->out1, n->cons1, n->cons2, n->len1); break;
    case Node::OP_ADAM_UPDATE:
    {
        const float lrt = O(adam_lrt)(n->out2, n->cons1, n->cons2, n->cons3);
        O(adam_apply)(n->in1, n->in2, n->out1, lrt, n->cons4, n->len1);
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

extern "C" void ORC_REGISTER(void)
{
    rt::register_cpu_backend(ProgramMode::MONOTHREAD, run_sequential);
    rt::register_cpu_backend(ProgramMode::MULTITHREAD, run_sequential);
}
