// The planning runner of the HIP backend: the drop-in for gpu::run (src/gpu/runner.cu:10-18, called
// from src/ops/graph.cu:194-200 with nothing but the instruction list).  Like hip_table.hh this header
// and hip_kernels.cc behind it need only rt::Node, rt::NodesList and the C ABI, and name both headers
// with angle brackets: the include path decides whether they are built for this repository's mirror
// (-I <this directory>) or, unchanged, for the reference's own src/runtime/node.hh and nodes-list.hh.
#pragma once

#include <cstddef>
#include <vector>

#include <node.hh>
#include <nodes-list.hh>

#include "hip_table.hh"

namespace hip
{

// kernels_list[512] and the plain table runner are declared in hip_table.hh.

// Issues every instruction of the list on the backend's stream, in order, WITHOUT a device
// synchronisation between instructions; returns after one synchronisation at the end.
void run(rt::NodesList& tasks);

// As run(), but leaves the stream running (the caller synchronises before it reads results).
void run_async(rt::NodesList& tasks);

// Pattern-matches the instruction list and replaces operator chains by fused C-ABI calls:
//   conv2d / conv2d_transpose -> mat_rvect_add -> relu|relu_leaky|tanh      (one launch)
//   relu_grad|leaky_relu_grad|tanh_grad -> mat_sum_cols                      (one pass)
//   moment_update + moment_update2 + adam_update of one variable            (one pass)
//   mat_mul_add -> relu|relu_leaky                                          (one launch)
//   sigmoid_cross_entropy + sigmoid_cross_entropy_grad on the same logits [x 2 + the add of the losses]  (one launch)
// Intermediate tensors that other instructions or the caller still read are kept up to date.
// Off by default (DCGAN_HIP_FUSE=1 or set_fusion(true) turns it on).
void set_fusion(bool on);
bool fusion();
// Part of fusion, on by default: two steps of a run that are the same convolution with the same
// filter on independent activations (the discriminator on the real and on the generated batch) are
// issued as one paired launch; filter gradients that only meet in a sum become one contraction.
// Call forget_plans() after changing it.
void set_pairing(bool on);
// Number of steps (single or fused launches; a reduction that follows a split launch not counted) the last run issued.
int last_launch_count();

// Tensors the caller will read after the run: the planner keeps them materialised and is free to leave
// out any other intermediate result (a convolution's output folded into its bias add and activation, a
// bias gradient that only the optimiser reads, ...).  The reference's Graph::run knows them
// (src/ops/graph.cu:201-215 reads compiled_ops_[ops[i]].out_data for every non-null outputs[i]) and
// names them in one call before gpu::run.  Until the first call -- a caller that hands over nothing but
// the instruction list, as src/gpu/runner.cu:10 is declared -- every tensor of the list counts as read
// by the caller and only the fusions that write all their nodes' outputs are made (activation gradient
// + column sums, the three optimiser nodes of a variable, all optimiser steps in one launch, paired
// forward / input-gradient launches).  protect_all_tensors() returns to that state.
void set_protected_tensors(const std::vector<const dbl_t*>& tensors);
void protect_all_tensors();
// Drop the cached plans (call when instructions are deleted or re-created).
void forget_plans();

// When off, rt::execute() in GPU mode returns right after issuing the instructions (the next
// blocking copy or hip::synchronize() waits for them).  On by default.
void set_sync_each_run(bool on);
bool sync_each_run();

// Notes that the device tensor at `dst` is to receive `count` values from host memory before the next
// run reads it.  The run stages and copies the data in front of the first step that touches the tensor
// (after queueing the steps before it), or at its end; src_host must stay valid until that run -- or
// hip::synchronize() -- returns.  Graph::run feeds its inputs this way.
void feed(dbl_t* dst, const dbl_t* src_host, std::size_t count);
// Forgets the inputs noted and not yet copied (a caller that fed inputs and then cannot run).  A run
// that throws forgets them by itself.
void drop_feeds();

void* stream();  // hipStream_t the backend launches on
void synchronize();

}  // namespace hip
