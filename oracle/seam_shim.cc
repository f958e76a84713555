// seam_shim.cc -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// Proves the kernel-table seam with the reference's own record: oracle/Makefile compiles this file
// together with dcgan-cuda_amd/host/hip_table.cc -- unchanged, but with the REFERENCE's
// src/runtime/node.hh on its include path -- and with the reference's src/runtime/node.cu (the
// rt::Node::op_* factories) and src/cpu/kernels.cu (its CPU kernel table), from where they lie, into
// oracle/_ref/libseam_ref.so.  A test then builds instructions with the reference's factories,
// runs them through hip::kernels_list[node->type] on device buffers and through
// cpu::kernels_list[node->type] on host buffers, and compares (src/gpu/kernels.cu:23-61,
// src/gpu/runner.cu:10-18 are what hip_table.cc replaces).
#include <cstddef>
#include <cstring>
#include <exception>
#include <string>
#include <vector>

#include "cpu/kernels.hh"
#include "runtime/node.hh"

#include "hip_table.hh"

namespace
{
std::string g_error;
}

extern "C" {

const char* seam_last_error(void) { return g_error.c_str(); }

// The reference's record, for a layout check against the host mirror (dg_node_layout).
// sizeof(rt::Node) followed by the offset of every field a kernel-table entry reads, in declaration
// order: type, in1, in2, in3, out1, out2, cons1..4, len1..3, intconst, intconst2, sizes1..3,
// int_cons1, int_cons2, alpha_leaky.  Returns the number of values written (at most n).
#pragma GCC diagnostic push
#pragma GCC diagnostic ignored "-Winvalid-offsetof"
int seam_node_layout(unsigned long* out, int n)
{
    using N = rt::Node;
    const unsigned long v[] = {sizeof(N), offsetof(N, type), offsetof(N, in1), offsetof(N, in2), offsetof(N, in3),
                               offsetof(N, out1), offsetof(N, out2), offsetof(N, cons1), offsetof(N, cons2),
                               offsetof(N, cons3), offsetof(N, cons4), offsetof(N, len1), offsetof(N, len2),
                               offsetof(N, len3), offsetof(N, intconst), offsetof(N, intconst2), offsetof(N, sizes1),
                               offsetof(N, sizes2), offsetof(N, sizes3), offsetof(N, int_cons1), offsetof(N, int_cons2),
                               offsetof(N, alpha_leaky)};
    const int count = (int)(sizeof(v) / sizeof(v[0]));
    for (int i = 0; i < count && i < n; ++i)
        out[i] = v[i];
    return count < n ? count : n;
}
#pragma GCC diagnostic pop

// One instruction made by the reference's factory of that name.  t[0..4]: in1, in2, in3, out1, out2
// in the factory's own argument roles; i[]: the integer arguments in the factory's order (arrays
// flattened); f[]: the float arguments in the factory's order.  Returns NULL for an unknown name.
void* seam_node_new(const char* op, float** t, const int* i, const float* f)
{
    const std::string o(op);
    const std::vector<rt::Node*> none;
    using N = rt::Node;
    if (o == "conv2d") return N::op_conv2d(t[0], t[1], i, i[2], i[3], t[3], i + 4, i + 8, none);
    if (o == "conv2d_input_grad") return N::op_conv2d_input_grad(t[0], t[1], i, t[3], i + 2, i + 6, i + 10, none);
    if (o == "conv2d_kernel_grad") return N::op_conv2d_kernel_grad(t[0], t[1], i, t[3], i + 2, i + 6, i + 10, none);
    if (o == "conv2d_transpose") return N::op_conv2d_transpose(t[0], t[1], i, i + 4, t[3], i + 6, i + 10, none);
    if (o == "conv2d_transpose_input_grad")
        return N::op_conv2d_transpose_input_grad(t[0], t[1], i, t[3], i + 2, i + 6, i + 10, none);
    if (o == "conv2d_transpose_kernel_grad")
        return N::op_conv2d_transpose_kernel_grad(t[0], t[1], i, t[3], i + 2, i + 6, i + 10, none);
    if (o == "mat_rvect_add") return N::op_mat_rvect_add(t[0], t[1], t[3], i[0], i[1], none);
    if (o == "mat_sum_cols") return N::op_mat_sum_cols(t[0], t[3], i[0], i[1], none);
    if (o == "mat_sum_rows") return N::op_mat_sum_rows(t[0], t[3], i[0], i[1], none);
    if (o == "mat_mat_mul") return N::op_mat_mat_mul(t[0], t[1], t[3], i[0], i[1], i[2], none);
    if (o == "mat_mul_add") return N::op_mat_mul_add(t[0], t[1], t[2], t[3], i[0], i[1], i[2], none);
    if (o == "tmat_mat_mul") return N::op_tmat_mat_mul(t[0], t[1], t[3], i[0], i[1], i[2], none);
    if (o == "mat_tmat_mul") return N::op_mat_tmat_mul(t[0], t[1], t[3], i[0], i[1], i[2], none);
    if (o == "relu") return N::op_relu(t[0], t[3], i[0], none);
    if (o == "relu_leaky") return N::op_relu_leaky(t[0], t[3], i[0], f[0], none);
    if (o == "tanh") return N::op_tanh(t[0], t[3], i[0], none);
    if (o == "sigmoid") return N::op_sigmoid(t[0], t[3], i[0], none);
    if (o == "relu_grad") return N::op_relu_grad(t[0], t[1], t[3], i[0], none);
    if (o == "leaky_relu_grad") return N::op_leaky_relu_grad(t[0], t[1], t[3], f[0], i[0], none);
    if (o == "tanh_grad") return N::op_tanh_grad(t[0], t[1], t[3], i[0], none);
    if (o == "sigmoid_grad") return N::op_sigmoid_grad(t[0], t[1], t[3], i[0], none);
    if (o == "add") return N::op_add(t[0], t[1], t[3], i[0], none);
    if (o == "mse") return N::op_mse(t[0], t[1], t[3], i[0], i[1], none);
    if (o == "mse_grad") return N::op_mse_grad(t[0], t[1], t[3], i[0], none);
    if (o == "sigmoid_cross_entropy") return N::op_sigmoid_cross_entropy(t[0], t[1], t[3], i[0], none);
    if (o == "sigmoid_cross_entropy_grad") return N::op_sigmoid_cross_entropy_grad(t[0], t[1], t[3], i[0], none);
    if (o == "argmax_acc") return N::op_argmax_acc(t[0], t[1], t[3], i[0], i[1], none);
    if (o == "update") return N::op_update(t[3], t[0], t[1], i[0], none);
    if (o == "moment_update") return N::op_moment_update(t[3], t[0], f[0], f[1], i[0], none);
    if (o == "moment_update2") return N::op_moment_update2(t[3], t[0], f[0], f[1], i[0], none);
    // var, t (host counter), m, v
    if (o == "adam_update") return N::op_adam_update(t[3], t[4], t[0], t[1], f[0], f[1], f[2], f[3], i[0], none);
    return nullptr;
}

int seam_node_type(void* node) { return static_cast<rt::Node*>(node)->type; }
void seam_node_free(void* node) { delete static_cast<rt::Node*>(node); }

// The reference's CPU table entry for the node (src/cpu/kernels.cu:218-262).
int seam_run_cpu(void* node)
{
    rt::Node* n = static_cast<rt::Node*>(node);
    try
    {
        cpu::kernels_list[n->type](n);
        return 0;
    }
    catch (const std::exception& e)
    {
        g_error = e.what();
        return 1;
    }
}

// The HIP table entry for the node, through the plain table runner (one synchronisation at the end).
int seam_run_hip(void* node)
{
    try
    {
        hip::run_table({static_cast<rt::Node*>(node)});
        return 0;
    }
    catch (const std::exception& e)
    {
        g_error = e.what();
        return 1;
    }
}

// 1 where the HIP table has an entry for the op code, 0 where it is nullptr.
int seam_hip_has(int type) { return type >= 0 && type < 512 && hip::kernels_list[type] != nullptr; }
int seam_cpu_has(int type) { return type >= 0 && type < 512 && cpu::kernels_list[type] != nullptr; }
}
