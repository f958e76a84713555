// Backends: one kernel table + one runner per ProgramMode
// (reference: src/gpu/fwd.hh:8 `kernel_f`, src/gpu/kernels.cu:23-61 `gpu::kernels_list[512]`,
// src/gpu/runner.cu:10-18 `gpu::run`, dispatch in src/ops/graph.cu:172-200).
//
// This library ships ONE backend, `hip` (RT_MODE=GPU).  The CPU modes belong to the reference's
// own src/cpu tree; a host program that links it (or a test that links the CPU oracle) can plug
// it in with register_cpu_backend().  Running in a CPU mode without such a registration throws
// -- there is no silent CPU fallback.
#pragma once

#include "hip_table.hh"
#include "mode.hh"
#include "rt_graph.hh"

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

// Tensors the caller will read after the run: the planner keeps them materialised.
void set_protected_tensors(const std::vector<const dbl_t*>& tensors);
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

void* stream();  // hipStream_t the backend launches on
void synchronize();

}  // namespace hip

namespace rt
{
using runner_f = void (*)(NodesList&);
// Plug a CPU backend in for ProgramMode::MONOTHREAD / MULTITHREAD.
void register_cpu_backend(ProgramMode mode, runner_f runner);
// Dispatch on program_mode() (src/ops/graph.cu:172-200).
void execute(NodesList& tasks);
}  // namespace rt
