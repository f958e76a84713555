// The kernel table of the HIP backend and its plain runner: the drop-in for gpu::kernels_list /
// gpu::run (src/gpu/kernels.cu:23-61, src/gpu/runner.cu:10-18).  Each table entry decodes the node
// exactly as the reference's GPU entry does (citations per function) and makes one C-ABI call;
// nothing else happens here.  This file depends on rt::Node and the C ABI only (see hip_table.hh).
#include "hip_table.hh"

#include <cmath>
#include <stdexcept>
#include <string>

#include "dcgan_hip.h"

namespace hip
{

void check(int rc, const char* what)
{
    if (rc != 0)
        throw std::runtime_error(std::string(what) + ": " + dh_last_error());
}

#define CK(call) check((call), #call)

const char* op_name(int type)
{
    if (type == rt::Node::OP_NOP)
        return "nop";
    return type >= 0 && type <= rt::Node::OP_ADD ? rt::Node::OP_NAMES[type] : "?";
}


// conv2d forward.  Node fields: src/runtime/node.cu:118-141; decode: src/gpu/conv2d.cu:13-40.
ConvGeom geom_conv2d(const rt::Node* n)
{
    ConvGeom g;
    g.N = n->sizes1[0]; g.H = n->sizes1[1]; g.W = n->sizes1[2]; g.C = n->sizes1[3];
    g.kh = n->sizes2[0]; g.kw = n->sizes2[1]; g.O = n->sizes2[3];
    g.sh = n->intconst[0]; g.sw = n->intconst[1];
    const int pad_h = n->int_cons1, pad_w = n->int_cons2;  // totals; the part before is half, rounded down
    g.pt = pad_h / 2; g.pl = pad_w / 2;
    g.Ho = (g.H + pad_h - g.kh) / g.sh + 1;
    g.Wo = (g.W + pad_w - g.kw) / g.sw + 1;
    return g;
}

// conv2d input gradient.  Fields: src/runtime/node.cu:171-193; decode: src/gpu/conv2d.cu:70-98
// (one stride for both axes, pads re-derived from the extents).
ConvGeom geom_input_grad(const rt::Node* n)
{
    ConvGeom g;
    g.N = n->sizes1[0]; g.Ho = n->sizes1[1]; g.Wo = n->sizes1[2]; g.O = n->sizes1[3];
    g.kh = n->sizes2[0]; g.kw = n->sizes2[1]; g.C = n->sizes2[2];
    g.sh = g.sw = n->intconst[0];
    g.H = n->intconst2[0]; g.W = n->intconst2[1];
    g.pt = ((g.Ho - 1) * g.sh - g.H + g.kh) / 2;
    g.pl = ((g.Wo - 1) * g.sw - g.W + g.kw) / 2;
    return g;
}

// conv2d filter gradient.  Fields: src/runtime/node.cu:195-217; decode: src/gpu/conv2d.cu:119-146
// (filter extent derived as H + pad - s*(Ho-1)).
ConvGeom geom_kernel_grad(const rt::Node* n)
{
    ConvGeom g;
    g.N = n->sizes2[0]; g.H = n->sizes2[1]; g.W = n->sizes2[2]; g.C = n->sizes2[3];
    g.Ho = n->sizes1[1]; g.Wo = n->sizes1[2]; g.O = n->sizes1[3];
    g.sh = n->intconst[0]; g.sw = n->intconst[1];
    const int pad_h = n->intconst2[0], pad_w = n->intconst2[1];
    g.pt = pad_h / 2; g.pl = pad_w / 2;
    g.kh = g.H + pad_h - g.sh * (g.Ho - 1);
    g.kw = g.W + pad_w - g.sw * (g.Wo - 1);
    return g;
}

// conv2d_transpose forward = input gradient of the conv whose "y" is this op's input.
// Fields: src/runtime/node.cu:219-243; decode: src/gpu/conv2d.cu:167-196.
ConvGeom geom_transpose(const rt::Node* n)
{
    ConvGeom g;
    g.N = n->sizes2[0]; g.Ho = n->sizes2[1]; g.Wo = n->sizes2[2]; g.O = n->sizes2[3];
    g.kh = n->sizes3[0]; g.kw = n->sizes3[1]; g.C = n->sizes3[2];
    g.sh = n->intconst[0]; g.sw = n->intconst[1];
    g.H = n->sizes1[1]; g.W = n->sizes1[2];
    g.pt = ((g.Ho - 1) * g.sh - g.H + g.kh) / 2;
    g.pl = ((g.Wo - 1) * g.sw - g.W + g.kw) / 2;
    return g;
}

// conv2d_transpose input gradient = forward conv of dy.  Fields: src/runtime/node.cu:245-267;
// decode: src/gpu/conv2d.cu:214-241.
ConvGeom geom_transpose_input_grad(const rt::Node* n)
{
    ConvGeom g;
    g.N = n->sizes1[0]; g.H = n->sizes1[1]; g.W = n->sizes1[2]; g.C = n->sizes2[2];
    g.kh = n->sizes2[0]; g.kw = n->sizes2[1]; g.O = n->sizes2[3];
    g.sh = g.sw = n->intconst[0];
    g.Ho = n->intconst2[0]; g.Wo = n->intconst2[1];
    g.pt = ((g.Ho - 1) * g.sh + g.kh - g.H) / 2;
    g.pl = ((g.Wo - 1) * g.sw + g.kw - g.W) / 2;
    return g;
}

// conv2d_transpose filter gradient = conv2d filter gradient with dy in the role of the image and
// the transpose's input in the role of the output gradient.  Fields: src/runtime/node.cu:269-294;
// decode: src/gpu/conv2d.cu:264-289.
ConvGeom geom_transpose_kernel_grad(const rt::Node* n)
{
    ConvGeom g;
    g.N = n->sizes2[0]; g.Ho = n->sizes2[1]; g.Wo = n->sizes2[2]; g.O = n->sizes2[3];  // transpose input
    g.H = n->sizes1[1]; g.W = n->sizes1[2]; g.C = n->sizes1[3];                        // dy
    g.kh = n->sizes3[0]; g.kw = n->sizes3[1];
    g.sh = n->intconst[0]; g.sw = n->intconst[1];
    g.pt = ((g.Ho - 1) * g.sh + g.kh - g.H) / 2;
    g.pl = ((g.Wo - 1) * g.sw + g.kw - g.W) / 2;
    return g;
}

namespace
{

void conv_fwd(const ConvGeom& g, const dbl_t* x, const dbl_t* k, dbl_t* y, const dbl_t* bias, int act, float alpha)
{
    CK(dh_conv2d_fwd(x, k, y, g.N, g.H, g.W, g.C, g.kh, g.kw, g.O, g.sh, g.sw, g.pt, g.pl, g.Ho, g.Wo, bias, act,
                     alpha, g_stream));
}

void conv_dx(const ConvGeom& g, const dbl_t* dy, const dbl_t* k, dbl_t* dx, const dbl_t* bias, int act, float alpha)
{
    CK(dh_conv2d_dx(dy, k, dx, g.N, g.Ho, g.Wo, g.O, g.kh, g.kw, g.C, g.sh, g.sw, g.pt, g.pl, g.H, g.W, bias, act,
                    alpha, g_stream));
}

void conv_dk(const ConvGeom& g, const dbl_t* x, const dbl_t* dy, dbl_t* dk)
{
    CK(dh_conv2d_dk(x, dy, dk, g.N, g.H, g.W, g.C, g.Ho, g.Wo, g.O, g.kh, g.kw, g.sh, g.sw, g.pt, g.pl, g_stream));
}

// ---- table entries -----------------------------------------------------------------------------
void k_conv2d(rt::Node* n) { conv_fwd(geom_conv2d(n), n->in1, n->in2, n->out1, nullptr, DH_ACT_NONE, 0.f); }
void k_conv2d_input_grad(rt::Node* n) { conv_dx(geom_input_grad(n), n->in1, n->in2, n->out1, nullptr, DH_ACT_NONE, 0.f); }
void k_conv2d_kernel_grad(rt::Node* n) { conv_dk(geom_kernel_grad(n), n->in2, n->in1, n->out1); }
void k_conv2d_transpose(rt::Node* n) { conv_dx(geom_transpose(n), n->in1, n->in2, n->out1, nullptr, DH_ACT_NONE, 0.f); }
void k_conv2d_transpose_input_grad(rt::Node* n)
{
    conv_fwd(geom_transpose_input_grad(n), n->in1, n->in2, n->out1, nullptr, DH_ACT_NONE, 0.f);
}
void k_conv2d_transpose_kernel_grad(rt::Node* n) { conv_dk(geom_transpose_kernel_grad(n), n->in1, n->in2, n->out1); }

// src/gpu/matmul.cu:88-150 (matmul, mvrow_add, matmul_add, tmat_mat_mul, mat_tmat_mul hosts)
void k_mat_mat_mul(rt::Node* n) { CK(dh_gemm_nn(n->in1, n->in2, nullptr, n->out1, n->len1, n->len2, n->len3, g_stream)); }
void k_mat_rvect_add(rt::Node* n) { CK(dh_bias_add(n->in1, n->in2, n->out1, n->len1, n->len2, g_stream)); }
void k_mat_mul_add(rt::Node* n) { CK(dh_gemm_nn(n->in1, n->in2, n->in3, n->out1, n->len1, n->len2, n->len3, g_stream)); }
void k_tmat_mat_mul(rt::Node* n) { CK(dh_gemm_tn(n->in1, n->in2, n->out1, n->len1, n->len2, n->len3, g_stream)); }
void k_mat_tmat_mul(rt::Node* n) { CK(dh_gemm_nt(n->in1, n->in2, n->out1, n->len1, n->len2, n->len3, g_stream)); }
// src/gpu/sum.cu:216-243
void k_mat_sum_rows(rt::Node* n) { CK(dh_mat_sum_rows(n->in1, n->out1, n->len1, n->len2, g_stream)); }
void k_mat_sum_cols(rt::Node* n) { CK(dh_bias_grad(n->in1, n->out1, n->len1, n->len2, g_stream)); }
void k_mse(rt::Node* n) { CK(dh_mse(n->in1, n->in2, n->out1, n->len1, n->len2, g_stream)); }
void k_mse_grad(rt::Node* n) { CK(dh_mse_grad(n->in1, n->in2, n->out1, n->len1, g_stream)); }
void k_argmax_acc(rt::Node* n) { CK(dh_argmax_acc(n->in1, n->in2, n->out1, n->len1, n->len2, g_stream)); }
void k_add(rt::Node* n) { CK(dh_add(n->in1, n->in2, n->out1, n->len1, g_stream)); }
// src/gpu/relu.cu:68-104
void k_relu(rt::Node* n) { CK(dh_relu(n->in1, n->out1, n->len1, g_stream)); }
void k_relu_leaky(rt::Node* n) { CK(dh_relu_leaky(n->in1, n->out1, n->len1, n->alpha_leaky, g_stream)); }
void k_relu_grad(rt::Node* n) { CK(dh_relu_grad(n->in1, n->in2, n->out1, n->len1, g_stream)); }
void k_leaky_relu_grad(rt::Node* n) { CK(dh_leaky_relu_grad(n->in1, n->in2, n->out1, n->cons1, n->len1, g_stream)); }
// src/gpu/sigmoid.cu:124-180
void k_sigmoid(rt::Node* n) { CK(dh_sigmoid(n->in1, n->out1, n->len1, g_stream)); }
void k_tanh(rt::Node* n) { CK(dh_tanh(n->in1, n->out1, n->len1, g_stream)); }
void k_sigmoid_grad(rt::Node* n) { CK(dh_sigmoid_grad(n->in1, n->in2, n->out1, n->len1, g_stream)); }
void k_tanh_grad(rt::Node* n) { CK(dh_tanh_grad(n->in1, n->in2, n->out1, n->len1, g_stream)); }
void k_sigmoid_cross_entropy(rt::Node* n) { CK(dh_sigmoid_cross_entropy(n->in1, n->in2, n->out1, n->len1, g_stream)); }
void k_sigmoid_cross_entropy_grad(rt::Node* n)
{
    CK(dh_sigmoid_cross_entropy_grad(n->in1, n->in2, n->out1, n->len1, g_stream));
}
// src/gpu/update.cu:56-96
void k_update(rt::Node* n) { CK(dh_sgd_update(n->out1, n->in1, n->in2, n->len1, g_stream)); }
void k_moment_update(rt::Node* n) { CK(dh_moment_update(n->out1, n->in1, n->cons1, n->cons2, n->len1, g_stream)); }
void k_moment_update2(rt::Node* n) { CK(dh_moment_update2(n->out1, n->in1, n->cons1, n->cons2, n->len1, g_stream)); }

// The step counter lives on the host (node->out2) and is advanced at issue time; the corrected
// rate is formed in float exactly as src/gpu/update.cu:81-93 does.
}  // namespace

float adam_advance(rt::Node* n)
{
    dbl_t* t = n->out2;
    const dbl_t lr = n->cons1, beta1 = n->cons2, beta2 = n->cons3;
    ++*t;
    return lr * std::sqrt(1 - std::pow(beta2, *t)) / (1 - std::pow(beta1, *t));
}

namespace
{

void k_adam_update(rt::Node* n)
{
    const float lrt = adam_advance(n);
    CK(dh_adam_update(n->out1, n->in1, n->in2, lrt, n->cons4, n->len1, g_stream));
}

}  // namespace

kernel_f kernels_list[512] = {
    k_mat_mat_mul,                   // 0
    k_mat_rvect_add,                 // 1
    k_sigmoid,                       // 2
    k_mse,                           // 3
    nullptr,                         // 4  softmax                (not on the convolution path)
    nullptr,                         // 5  log_softmax            (")
    nullptr,                         // 6  softmax_cross_entropy  (")
    k_conv2d,                        // 7
    k_relu,                          // 8
    k_relu_leaky,                    // 9
    k_tanh,                          // 10
    k_mse_grad,                      // 11
    k_sigmoid_grad,                  // 12
    k_mat_mul_add,                   // 13
    k_tmat_mat_mul,                  // 14
    k_mat_tmat_mul,                  // 15
    k_mat_sum_rows,                  // 16
    k_mat_sum_cols,                  // 17
    nullptr,                         // 18 softmax_cross_entropy_grad (")
    k_relu_grad,                     // 19
    nullptr,                         // 20 conv2d_bias_add: lowered to mat_rvect_add by the operator
    k_update,                        // 21
    k_sigmoid_cross_entropy,         // 22
    k_sigmoid_cross_entropy_grad,    // 23
    k_conv2d_input_grad,             // 24
    k_conv2d_kernel_grad,            // 25
    k_argmax_acc,                    // 26
    k_moment_update,                 // 27
    k_moment_update2,                // 28
    k_adam_update,                   // 29
    k_leaky_relu_grad,               // 30
    nullptr,                         // 31 conv2d_bias_add_grad: lowered to mat_sum_cols
    k_tanh_grad,                     // 32
    k_conv2d_transpose,              // 33
    k_conv2d_transpose_input_grad,   // 34
    k_conv2d_transpose_kernel_grad,  // 35
    k_add,                           // 36
};

void run_table(const std::vector<rt::Node*>& nodes)
{
    for (rt::Node* n : nodes)
    {
        kernel_f f = n->type >= 0 && n->type < 512 ? kernels_list[n->type] : nullptr;
        if (!f)
            throw std::runtime_error("hip backend: no kernel for op code " + std::to_string(n->type));
        f(n);
    }
    CK(dh_stream_sync(g_stream));
}

}  // namespace hip
