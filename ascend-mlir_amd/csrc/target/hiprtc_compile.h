// Compiling the HIP source of a region inside the process, through the runtime-compilation
// library that ships with the HIP runtime (libhiprtc), for hosts that have the runtime but no
// hipcc.  The reference compiles its generated kernel sources with an external compiler
// (lib/Runtime/Compilation/KernelCompiler.cpp drives `bisheng`); this is the same step without
// the external program.
#pragma once

#include <string>
#include <vector>

namespace afir_target {

// The options both compilers are given for a region's source: the emitted kernels use compiler
// builtins only (no device headers), keep every float operation a separate IEEE operation, and
// are built without packed float32 instructions like the rest of the kernels.
const std::vector<std::string> &regionCompileOptions();

// source -> gfx950 code object.  Empty string: done, *image holds the code object.  Otherwise
// the reason (the library is missing, or the compiler's log).
std::string compileWithHiprtc(const std::string &source, std::vector<char> *image);

}  // namespace afir_target
