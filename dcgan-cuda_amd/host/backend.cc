// Dispatch of a run on program_mode() (src/ops/graph.cu:172-200): the HIP runner for RT_MODE=GPU, a
// registered CPU runner otherwise.  This library holds no CPU kernels of its own.
#include "backend.hh"

#include <stdexcept>

namespace rt
{
namespace
{
runner_f g_cpu[2] = {nullptr, nullptr};
}

void register_cpu_backend(ProgramMode mode, runner_f runner)
{
    if (mode == ProgramMode::MONOTHREAD) g_cpu[0] = runner;
    if (mode == ProgramMode::MULTITHREAD) g_cpu[1] = runner;
}

void execute(NodesList& tasks)
{
    const ProgramMode mode = program_mode();
    if (mode == ProgramMode::GPU)
    {
        if (hip::sync_each_run())
            hip::run(tasks);
        else
            hip::run_async(tasks);
        return;
    }
    runner_f r = g_cpu[mode == ProgramMode::MONOTHREAD ? 0 : 1];
    if (!r)
        throw std::runtime_error(
            "RT_MODE selects a CPU mode, but this library only holds the HIP backend (RT_MODE=GPU); "
            "the CPU runners are the reference's src/cpu tree -- register one with rt::register_cpu_backend");
    r(tasks);
}
}  // namespace rt
