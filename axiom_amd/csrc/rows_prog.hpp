// Compiled fused-row programs, run-time side (rows_prog.hip).
#pragma once

#include <string>

#include "common.hpp"
#include "rows_codegen.hpp"

namespace axhip {

// Matches the program against the compiled kernels: those built into the library first, then (unless AXHIP_JIT=0)
// one compiled through hipRTC when the program is first launched.  Fills `name` (when non-NULL) and launches when
// `launch` is set; *rc receives the launch's error code.  Returns false when the interpreter has to take the
// program (it does not qualify, or run-time compilation is off or failed).
bool rows_prog_dispatch(const AxhipRowsProgram &P, hipStream_t s, bool launch, char *name, size_t name_len, int *rc, bool builtin_only = false);

// Compiles the program's kernel through hipRTC for gfx950 without loading it (needs no device): the check that the
// generator's text is valid for a program shape.
bool rows_prog_compile_only(const AxhipRowsProgram &P, std::string *label, std::string *error);

// how many run-time kernels this process took from the on-disk cache / compiled with hipRTC so far
void rows_prog_jit_counters(int *from_disk, int *compiled);

} // namespace axhip
