// Backends: one kernel table + one runner per ProgramMode
// (reference: src/gpu/fwd.hh:8 `kernel_f`, src/gpu/kernels.cu:23-61 `gpu::kernels_list[512]`,
// src/gpu/runner.cu:10-18 `gpu::run`, dispatch in src/ops/graph.cu:172-200).
//
// This library ships ONE backend, `hip` (RT_MODE=GPU).  The CPU modes belong to the reference's
// own src/cpu tree; a host program that links it (or a test that links the CPU oracle) can plug
// it in with register_cpu_backend().  Running in a CPU mode without such a registration throws
// -- there is no silent CPU fallback.
#pragma once

#include "hip_runner.hh"
#include "mode.hh"
#include "rt_graph.hh"


namespace rt
{
using runner_f = void (*)(NodesList&);
// Plug a CPU backend in for ProgramMode::MONOTHREAD / MULTITHREAD.
void register_cpu_backend(ProgramMode mode, runner_f runner);
// Dispatch on program_mode() (src/ops/graph.cu:172-200).
void execute(NodesList& tasks);
}  // namespace rt
