// Runtime mode switch, selected by the RT_MODE environment variable
// (reference: src/memory/mode.hh:3-11, src/memory/mode.cu:8-36).
//   RT_MODE=GPU  -> ProgramMode::GPU          (this library: the HIP backend)
//   RT_MODE=MCPU -> ProgramMode::MULTITHREAD  (a CPU backend must be registered, see backend.hh)
//   RT_MODE=CPU, unset or anything else -> ProgramMode::MONOTHREAD
// The value is read once and cached, as in the reference.
#pragma once

enum class ProgramMode
{
    MONOTHREAD,
    MULTITHREAD,
    GPU
};

ProgramMode program_mode();

// Test hook: forget the cached mode so that the next program_mode() re-reads RT_MODE.
void program_mode_reset();
