"""Builds the gfx950 libraries in-tree with hipcc (cross-compiles without a GPU).

    python ascend-mlir_amd/build.py
    python ascend-mlir_amd/build.py --variant OUT.so -DAFIR_MM_KSTAGGER_M=1 [-D...]
        a copy of the kernel library with compile-time choices of the hand-tuned kernels
        changed (what a tile search times against the shipped choice; bin/autotuner calls
        this for parameters named build_<MACRO>)

Outputs (under ascend-mlir_amd/lib/):
    libafir_hip_kernels.so    fused kernels + launcher C ABI
    libAFIRRuntimeCAPI.so     afirt_* C API + host runtime (and bin/: the CLIs)
    families/*.hsaco          the kernel families as compiled region kernels
    libafir_bench_probes.so   measurement aids of bench.py (not part of the product)
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "lib")
OBJ = os.path.join(HERE, "build")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

# -packed-fp32-ops off: the compiler must not form packed f32 instructions.
COMMON = ["-std=c++17", "-O3", "-fPIC", f"--offload-arch={ARCH}",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-Wall", "-Wno-unused-value", "-Wno-unknown-warning-option",
          "-I", os.path.join(ROOT, "include")]
# every f32 add/mul of the elementwise kernels stays a separate IEEE operation
STRICT = ["-ffp-contract=off"]

KERNEL_SOURCES = [
    ("kernels/eltwise.hip", STRICT),
    ("kernels/rowsum.hip", STRICT),
    ("kernels/transpose.hip", STRICT),
    ("kernels/gather.hip", STRICT),
    ("kernels/matmul.hip", []),
    ("kernels/matmul_dma.hip", []),
    ("kernels/matmul_layouts.hip", []),
    ("kernels/region.hip", STRICT),
    ("target/region_program.cpp", []),
    ("target/hip_emitter.cpp", []),
    ("target/hiprtc_compile.cpp", []),
    ("capi/afir_hip_kernels.cpp", []),
]


def _run(cmd):
    p = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in p.stderr.splitlines()
                    if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + err)
    if err.strip():
        sys.stderr.write(err + "\n")


def _compile(src, extra):
    obj = os.path.join(OBJ, src.replace("/", "_") + ".o")
    cmd = [HIPCC, *COMMON, *extra, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    _run(cmd)
    return obj


def build_kernels():
    os.makedirs(LIB, exist_ok=True)
    os.makedirs(OBJ, exist_ok=True)
    with cf.ThreadPoolExecutor(max_workers=min(8, len(KERNEL_SOURCES))) as ex:
        objs = list(ex.map(lambda a: _compile(*a), KERNEL_SOURCES))
    out = os.path.join(LIB, "libafir_hip_kernels.so")
    _run([HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", out, *objs])
    return out


RUNTIME_SOURCES = ["runtime/support.cpp", "runtime/artifact.cpp", "runtime/session.cpp",
                   "runtime/hip_runner.cpp", "capi/afirt_runtime.cpp",
                   "target/region_program.cpp", "target/mlir_translate.cpp", "target/hip_emitter.cpp",
                   "target/hiprtc_compile.cpp"]
HOST = ["-std=c++17", "-O2", "-fPIC", "-Wall", "-Wno-unused-result",
        "-D__HIP_PLATFORM_AMD__", "-I", "/opt/rocm/include", "-I", os.path.join(ROOT, "include")]
CXX = os.environ.get("CXX", "g++")


def _compile_host(src):
    obj = os.path.join(OBJ, "host_" + src.replace("/", "_") + ".o")
    _run([CXX, *HOST, "-c", os.path.join(CSRC, src), "-o", obj])
    return obj


def build_runtime():
    """libAFIRRuntimeCAPI.so (afirt_* C API + host runtime) and the
    runtime-session CLI.  Host code only: compiled with g++ against the HIP
    runtime API; the kernels are reached through dlopen of the kernel library."""
    os.makedirs(LIB, exist_ok=True)
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(os.path.join(HERE, "bin"), exist_ok=True)
    with cf.ThreadPoolExecutor(max_workers=6) as ex:
        objs = list(ex.map(_compile_host, RUNTIME_SOURCES))
    lib = os.path.join(LIB, "libAFIRRuntimeCAPI.so")
    _run([CXX, "-shared", "-fPIC", "-o", lib, *objs, "-L/opt/rocm/lib", "-lamdhip64", "-ldl",
          "-Wl,-rpath,/opt/rocm/lib"])
    main_obj = _compile_host("tools/runtime_session_main.cpp")
    exe = os.path.join(HERE, "bin", "runtime-session")
    _run([CXX, "-o", exe, main_obj, "-L" + LIB, "-lAFIRRuntimeCAPI", "-L/opt/rocm/lib",
          "-lamdhip64", "-ldl", "-Wl,-rpath,$ORIGIN/../lib", "-Wl,-rpath,/opt/rocm/lib"])
    at_obj = _compile_host("tools/autotuner_main.cpp")
    at_exe = os.path.join(HERE, "bin", "autotuner")
    _run([CXX, "-o", at_exe, at_obj, "-L" + LIB, "-lAFIRRuntimeCAPI", "-L/opt/rocm/lib",
          "-lamdhip64", "-ldl", "-Wl,-rpath,$ORIGIN/../lib", "-Wl,-rpath,/opt/rocm/lib"])
    # afir-translate -mlir-to-hip: host-only, no HIP runtime needed
    tr_obj = _compile_host("tools/afir_translate_main.cpp")
    tr_exe = os.path.join(HERE, "bin", "afir-translate")
    _run([CXX, "-o", tr_exe, tr_obj, *[o for o in objs if "target_" in o]])
    return [lib, exe, at_exe, tr_exe]


HIPCC_REGION_FLAGS = ["--genco", "--offload-arch=gfx950", "-O3", "-nogpuinc", "-ffp-contract=off",
                      "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build_families(kernel_lib):
    """The kernel families as compiled region kernels: lib/families/<family>.hsaco, which
    the family launchers fall back on for shapes their specialised kernels do not take."""
    import ctypes
    L = ctypes.CDLL(kernel_lib)
    L.afir_hip_family_program.restype = ctypes.c_char_p
    L.afir_hip_family_program.argtypes = [ctypes.c_char_p]
    L.afir_hip_region_register.argtypes = [ctypes.c_char_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_uint64)]
    L.afir_hip_region_emit_source.argtypes = [ctypes.c_uint64, ctypes.c_char_p, ctypes.c_size_t,
                                              ctypes.POINTER(ctypes.c_size_t)]
    out_dir = os.path.join(LIB, "families")
    os.makedirs(out_dir, exist_ok=True)
    built = []
    for family in ("broadcast_add_reducesum", "relu_broadcast_add_transpose", "gather_scale_shift"):
        text = L.afir_hip_family_program(family.encode())
        handle, n = ctypes.c_uint64(0), ctypes.c_size_t(0)
        os.environ["AFIR_HIP_REGION_GENERIC"] = "1"
        try:
            rc = L.afir_hip_region_register(text, len(text), ctypes.byref(handle))
        finally:
            del os.environ["AFIR_HIP_REGION_GENERIC"]
        if rc or L.afir_hip_region_emit_source(handle, None, 0, ctypes.byref(n)):
            raise RuntimeError(f"cannot emit the source of family {family}")
        buf = ctypes.create_string_buffer(n.value + 1)
        L.afir_hip_region_emit_source(handle, buf, n.value + 1, ctypes.byref(n))
        L.afir_hip_region_unregister(handle)
        src = os.path.join(OBJ, family + ".hip")
        with open(src, "wb") as f:
            f.write(buf.value)
        obj = os.path.join(out_dir, family + ".hsaco")
        _run([HIPCC, *HIPCC_REGION_FLAGS, "-o", obj, src])
        built.append(obj)
    return built


def build_probes():
    """libafir_bench_probes.so: ceiling probes for bench.py (csrc/bench/probes.h), among them
    the direct-to-LDS matmul kernel instantiated with parts of its K loop left out
    (csrc/bench/matmul_feed_probes.h)."""
    os.makedirs(LIB, exist_ok=True)
    os.makedirs(OBJ, exist_ok=True)
    obj = os.path.join(OBJ, "bench_probes.o")
    _run([HIPCC, *COMMON, "-x", "hip", "-c", os.path.join(CSRC, "bench/probes.hip"), "-o", obj])
    out = os.path.join(LIB, "libafir_bench_probes.so")
    _run([HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", out, obj])
    return out


def _source_closure(src):
    """Text of a source file and of every header of this tree it includes, directly or not."""
    import re
    seen, todo, text = set(), [os.path.join(CSRC, src)], []
    while todo:
        path = os.path.normpath(todo.pop())
        if path in seen or not os.path.exists(path):
            continue
        seen.add(path)
        body = open(path).read()
        text.append(body)
        for inc in re.findall(r'^\s*#\s*include\s+"([^"]+)"', body, flags=re.M):
            todo.append(os.path.join(os.path.dirname(path), inc))
            todo.append(os.path.join(ROOT, "include", inc))
    return "\n".join(text)


def build_variant(out, defines):
    """The kernel library with extra -D flags.  A source is recompiled with them when it, or a
    header it includes, uses one of the macros (as a whole identifier); the others keep their
    ordinary objects (compiled here if the build directory does not hold them).  A macro that
    no source uses is an error: the variant would be the shipped library under another name."""
    import re
    names = [re.match(r"-D([A-Za-z_0-9]+)", d).group(1) for d in defines]
    closures = {src: _source_closure(src) for src, _ in KERNEL_SOURCES}
    for n in names:
        if not any(re.search(r"\b" + re.escape(n) + r"\b", t) for t in closures.values()):
            raise SystemExit(f"build.py --variant: no kernel source or header uses {n}")
    tag = "_".join(d[2:].replace("=", "-") for d in defines) or "base"
    vdir = os.path.join(os.path.dirname(os.path.abspath(out)), "obj_" + tag)
    os.makedirs(vdir, exist_ok=True)
    os.makedirs(OBJ, exist_ok=True)

    def one(item):
        src, extra = item
        touched = any(re.search(r"\b" + re.escape(n) + r"\b", closures[src]) for n in names)
        obj = os.path.join(vdir if touched else OBJ, src.replace("/", "_") + ".o")
        if touched or not os.path.exists(obj):
            _run([HIPCC, *COMMON, *extra, *(defines if touched else []), "-x", "hip", "-c",
                  os.path.join(CSRC, src), "-o", obj])
        return obj
    with cf.ThreadPoolExecutor(max_workers=min(8, len(KERNEL_SOURCES))) as ex:
        objs = list(ex.map(one, KERNEL_SOURCES))
    _run([HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", out, *objs])
    # the families' compiled form is looked up beside the library
    fam = os.path.join(LIB, "families")
    link = os.path.join(os.path.dirname(os.path.abspath(out)), "families")
    if os.path.isdir(fam) and not os.path.exists(link):
        os.symlink(fam, link)
    return out


def build_all():
    kernel_lib = build_kernels()
    return [kernel_lib, *build_runtime(), *build_families(kernel_lib), build_probes()]


if __name__ == "__main__":
    if len(sys.argv) > 1 and sys.argv[1] == "--variant":
        if len(sys.argv) < 3 or any(not a.startswith("-D") for a in sys.argv[3:]):
            raise SystemExit("usage: build.py --variant OUT.so [-DNAME=VALUE ...]")
        print("built", build_variant(sys.argv[2], sys.argv[3:]))
    else:
        for path in build_all():
            print("built", os.path.relpath(path, ROOT))
