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
//
// The planning runner, dcgan-cuda_amd/host/hip_kernels.cc, is compiled into the same library the same
// way -- unchanged, against the reference's node.hh and nodes-list.hh.  The seam_prog_* calls build a
// whole instruction graph in the reference's rt::Graph (src/runtime/graph.cu), order it with the
// reference's rt::Graph::topological_sort as src/ops/graph.cu:194-200 does, and run the resulting
// rt::NodesList through hip::run (fused and paired launches) or, node by node, through the reference's
// CPU table.
#include <cstddef>
#include <cstring>
#include <exception>
#include <string>
#include <vector>

#include "cpu/kernels.hh"
#include "runtime/graph.hh"
#include "runtime/node.hh"
#include "runtime/nodes-list.hh"

#include "hip_runner.hh"
#include "hip_table.hh"

namespace
{
std::string g_error;
}

// An instruction graph owned by the reference's rt::Graph; nodes are addressed by creation order.
struct Prog
{
    rt::Graph graph;
    std::vector<rt::Node*> nodes;
};

rt::Node* make_node(const char* op, float** t, const int* i, const float* f, const std::vector<rt::Node*>& preds);

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
    return make_node(op, t, i, f, {});
}
}  // extern "C"

rt::Node* make_node(const char* op, float** t, const int* i, const float* f, const std::vector<rt::Node*>& none)
{
    const std::string o(op);
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

extern "C" {

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

// ---- whole instruction graphs through the planning runner ----------------------------------------
void* seam_prog_new(void) { return new Prog(); }
void seam_prog_free(void* prog) { delete static_cast<Prog*>(prog); }   // rt::Graph deletes its nodes

// Adds one instruction made by the reference's factory `op` (arguments as for seam_node_new) whose
// predecessors are the instructions pred[0..npred), given by their ids; returns the new id, -1 for
// an unknown factory.
int seam_prog_add(void* prog, const char* op, float** t, const int* i, const float* f, const int* pred, int npred)
{
    Prog* p = static_cast<Prog*>(prog);
    std::vector<rt::Node*> preds;
    for (int q = 0; q < npred; ++q)
        preds.push_back(p->nodes.at((std::size_t)pred[q]));
    rt::Node* n = make_node(op, t, i, f, preds);
    if (!n)
        return -1;
    p->graph.add(n);
    p->nodes.push_back(n);
    return (int)p->nodes.size() - 1;
}

// The order the reference would execute in for the requested instructions (src/ops/graph.cu:196):
// writes up to `cap` ids, returns the length of the list.
int seam_prog_order(void* prog, const int* want, int nwant, int* ids, int cap)
{
    Prog* p = static_cast<Prog*>(prog);
    std::vector<rt::Node*> targets;
    for (int q = 0; q < nwant; ++q)
        targets.push_back(p->nodes.at((std::size_t)want[q]));
    rt::NodesList list(p->graph.topological_sort(targets));
    int n = 0;
    for (rt::Node* node : list.nodes())
    {
        for (std::size_t id = 0; id < p->nodes.size(); ++id)
            if (p->nodes[id] == node && n < cap)
                ids[n] = (int)id;
        ++n;
    }
    return n;
}

// Runs the sorted list node by node through the reference's CPU table (cpu::run_sequential without its
// debug output, src/cpu/runner.cu).
int seam_prog_run_cpu(void* prog, const int* want, int nwant)
{
    Prog* p = static_cast<Prog*>(prog);
    try
    {
        std::vector<rt::Node*> targets;
        for (int q = 0; q < nwant; ++q)
            targets.push_back(p->nodes.at((std::size_t)want[q]));
        rt::NodesList list(p->graph.topological_sort(targets));
        for (rt::Node* n : list.nodes())
            cpu::kernels_list[n->type](n);
        return 0;
    }
    catch (const std::exception& e)
    {
        g_error = e.what();
        return 1;
    }
}

// Runs the sorted list through hip::run.  fuse / pair: the planner's switches.  nkeep < 0: the caller
// names no tensors, as gpu::run's signature has it (every tensor is then kept); otherwise
// keep[0..nkeep) go to hip::set_protected_tensors first, the one call a fused drop-in adds to
// src/ops/graph.cu.  *launches receives the number of steps the plan issued.
int seam_prog_run_hip(void* prog, const int* want, int nwant, int fuse, int pair, float** keep, int nkeep, int* launches)
{
    Prog* p = static_cast<Prog*>(prog);
    try
    {
        std::vector<rt::Node*> targets;
        for (int q = 0; q < nwant; ++q)
            targets.push_back(p->nodes.at((std::size_t)want[q]));
        rt::NodesList list(p->graph.topological_sort(targets));
        hip::set_fusion(fuse != 0);
        hip::set_pairing(pair != 0);
        hip::forget_plans();
        if (nkeep < 0)
            hip::protect_all_tensors();
        else
            hip::set_protected_tensors(std::vector<const dbl_t*>(keep, keep + nkeep));
        hip::run(list);
        if (launches)
            *launches = hip::last_launch_count();
        hip::forget_plans();
        hip::protect_all_tensors();
        return 0;
    }
    catch (const std::exception& e)
    {
        g_error = e.what();
        return 1;
    }
}
}
