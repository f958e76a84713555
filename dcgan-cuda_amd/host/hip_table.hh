// The kernel-table half of the HIP backend: the drop-in for gpu::kernels_list and gpu::run
// (src/gpu/kernels.cu:23-61, src/gpu/runner.cu:10-18).  hip_table.cc needs nothing but rt::Node's
// fields and op codes and the C ABI, so it compiles unchanged against the reference's own
// src/runtime/node.hh: the field names are the same.  The include below uses angle brackets on
// purpose -- the include path, not this file's directory, decides whose rt::Node the table is built
// for (-I <this directory> here, -I <reference>/src/runtime for the reference's).
#pragma once

#include <vector>

#include <node.hh>

using kernel_f = void (*)(rt::Node*);

namespace hip
{

// Indexed by rt::Node::type.  Entries 20 and 31 are nullptr exactly as in the reference
// (conv2d_bias_add lowers to mat_rvect_add, its gradient to mat_sum_cols); the softmax family
// (4, 5, 6, 18) is not on the convolution path and is nullptr as well.
extern kernel_f kernels_list[512];

// Issues the instructions in list order through the table, without a device synchronisation
// between them, and waits once at the end -- gpu::run without its per-node cudaDeviceSynchronize.
void run_table(const std::vector<rt::Node*>& nodes);

// Every launch of the backend is ordered on the default stream.
constexpr void* g_stream = nullptr;

// Throws std::runtime_error(what + dh_last_error()) when a C-ABI call returned non-zero: the
// reference's gpuErrchk convention (src/memory/alloc.cu:6-14).
void check(int rc, const char* what);

// Geometry of a convolution call as the C ABI takes it, decoded from a node the way the reference's
// GPU entries decode it (src/gpu/conv2d.cu; citations at the definitions).
struct ConvGeom
{
    int N, H, W, C, Ho, Wo, O, kh, kw, sh, sw, pt, pl;
};
ConvGeom geom_conv2d(const rt::Node* n);
ConvGeom geom_input_grad(const rt::Node* n);
ConvGeom geom_kernel_grad(const rt::Node* n);
ConvGeom geom_transpose(const rt::Node* n);
ConvGeom geom_transpose_input_grad(const rt::Node* n);
ConvGeom geom_transpose_kernel_grad(const rt::Node* n);

// The operator's name as rt::Node::OP_NAMES spells it ("nop" for the placeholder, "?" outside the table).
const char* op_name(int type);

// Advances the host-side step counter of an adam_update node (node->out2) and returns the
// bias-corrected rate, formed in float exactly as src/gpu/update.cu:81-93 does.
float adam_advance(rt::Node* n);

}  // namespace hip
