// The hand-tuned kernel families as region programs.  The library's build
// compiles each into lib/families/<family>.hsaco; a family launcher whose
// specialised kernels do not fit a launch's shapes runs the launch on those
// kernels instead of its own scalar fallbacks.
#pragma once

namespace afir_family {

// y[i] = sum_j (x[i,j] + bias[j])
constexpr const char *kBroadcastAddReducesum =
    "afir-hip-region 1\n"
    "arg in f32 2\narg in f32 1\narg out f32 1\n"
    "segment 2\nsize arg0.0 arg0.1\noutoff 0\n"
    "push arg0 d0 d1\npush arg1 d1\nadd\nreduce sum\nstore\nend\n";

// out[b,j,i] = relu(x[b,i,j]) + c[j]
constexpr const char *kReluBroadcastAddTranspose =
    "afir-hip-region 1\n"
    "arg in f16 3\narg in f16 1\narg out f16 3\n"
    "segment 3\nsize arg0.0 arg0.2 arg0.1\noutoff 0\n"
    "push arg0 d0 d2 d1\nrelu\npush arg1 d1\nadd\nstore\nend\n";

// out[r,:] = table[idx[r],:] * scale + shift
constexpr const char *kGatherScaleShift =
    "afir-hip-region 1\n"
    "arg in f16 2\narg in i32 1\narg in f16 1\narg in f16 1\narg out f16 2\n"
    "segment 2\nsize arg1.0 arg0.1\noutoff 0\n"
    "push arg0 g0:arg1 d1\npush arg2 d1\nmul\npush arg3 d1\nadd\nstore\nend\n";

}  // namespace afir_family
