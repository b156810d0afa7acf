"""Region program -> HIP source -> gfx950 code object, without a GPU: the
emitter accepts every program the translator produces, the source carries the
program and its hash, hipcc accepts it, and the artifact layer stores it
(reference counterpart: the kernel source `afir-translate -mlir-to-cann` prints,
lib/Target/CannKernel/CannTranslation.cpp:2487-2694, compiled by
lib/Runtime/Compilation/KernelCompiler.cpp into the artifact's device binary)."""
import ctypes
import os
import shutil
import subprocess

import pytest

from tests import mlir_cases as MC
from tests import region_cases as RC

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "ascend-mlir_amd", "bin")
TR = os.path.join(BIN, "afir-translate")
RS = os.path.join(BIN, "runtime-session")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
FLAGS = ["--genco", "--offload-arch=gfx950", "-O3", "-nogpuinc", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

PROGRAMS = {n: getattr(RC, n) for n in dir(RC)
            if n.isupper() and isinstance(getattr(RC, n), str) and "segment" in getattr(RC, n)}


def _emit(text):
    return subprocess.run([TR, "-mlir-to-hip", "-", "--emit-hip-source"], input=text, capture_output=True, text=True)


def _fnv1a(data: bytes) -> int:
    h = 0xcbf29ce484222325
    for c in data:
        h = ((h ^ c) * 0x100000001b3) & 0xFFFFFFFFFFFFFFFF
    return h


@pytest.mark.parametrize("name", sorted(PROGRAMS))
def test_every_program_emits_and_compiles(tmp_path, name):
    p = _emit(PROGRAMS[name])
    assert p.returncode == 0, p.stderr
    src = p.stdout
    # the program it was generated from, line by line, and its hash
    canonical = subprocess.run([TR, "-mlir-to-hip", "-"], input=PROGRAMS[name], capture_output=True, text=True).stdout
    body = "".join(l + "\n" for l in canonical.splitlines() if not l.startswith("#"))
    for line in body.splitlines():
        assert "//   " + line in src
    assert "afir_region_program_hash = 0x%016xull" % _fnv1a(body.encode()) in src
    nseg = body.count("\nsegment ")
    for k in range(nseg):
        for variant in ("i32_a", "i32_g", "i64_a", "i64_g"):
            assert f"afir_region_s{k}_{variant}(" in src
    assert "#include" not in src            # builtins only: compiles with -nogpuinc
    (tmp_path / "k.hip").write_text(src)
    q = subprocess.run([HIPCC, *FLAGS, "-o", str(tmp_path / "k.hsaco"), str(tmp_path / "k.hip")],
                       capture_output=True, text=True)
    assert q.returncode == 0, q.stderr[-3000:]
    image = (tmp_path / "k.hsaco").read_bytes()
    assert b"afir_region_s0_i32_a" in image and b"afir_region_program_hash" in image


def test_lane_shapes_follow_the_element_types():
    assert "a lane takes 4 groups of 4 elements per pass" in _emit(RC.C1_ADD_MUL).stdout       # all f32
    assert "a lane takes 4 groups of 8 elements per pass" in _emit(RC.RELU_COL_ADD).stdout     # all f16
    mixed = RC.HEADER + ("arg in f16 2\narg in f32 1\narg out f16 2\nsegment 2\n size arg0.0 arg0.1\n outoff 0\n"
                         " push arg0 d0 d1\n push arg1 d1\n add\n store\nend\n")
    assert "a lane takes 2 groups of 8 elements per pass" in _emit(mixed).stdout


def test_transposed_reads_go_through_lds_tiles():
    src = _emit(RC.C3_RELU_BCAST_TRANSPOSE).stdout      # x[b, i, j] read over the space (b, j, i)
    assert "tiles of 64 (dim 1) x 64 (dim 2) through LDS; a lane takes 1 groups of 8 elements per row" in src
    assert "__attribute__((shared)) static float tile[1][TQ * PITCH];" in src
    assert src.count("__builtin_amdgcn_s_barrier();") == 2          # after the tile is written, before it is reused
    # a program with transposed reads gets no all-segments kernel, others of 2..4 segments do
    assert "afir_region_all_i32_a" not in src
    assert "afir_region_all_i32_a" in _emit(RC.SPLIT_RELU_BRC_ADD_MUL).stdout
    two = RC.HEADER + ("arg in f32 2\narg in f32 2\narg in f32 2\narg out f32 2\nsegment 2\n size arg0.0 arg0.1\n outoff 0\n"
                       " push arg0 d0 d1\n push arg1 d1 d0\n add\n push arg2 d1 d0\n mul\n store\nend\n")
    src = _emit(two).stdout                             # two transposed operands, f32
    assert "tiles of 64 (dim 0) x 64 (dim 1) through LDS; a lane takes 2 groups of 4 elements per row" in src
    assert "static float tile[2][TQ * PITCH];" in src


def test_integer_regions_use_wrapping_integer_arithmetic():
    src = _emit(RC.INT_CHAIN_I32).stdout
    assert "a lane takes 2 groups of 4 elements per row" in src              # i32 everywhere, a transposed read
    assert "static int tile[1][TQ * PITCH];" in src and "ldv_i32<EL, true>" in src
    assert "(int)((unsigned)" in src and "stv_i32<W>(R.out" in src
    body = src[src.index("// ---- segment 0"):]
    assert "fmax_ieee" not in body and "float" not in body
    narrow = _emit(RC.INT_CHAIN_I16).stdout
    assert "(int)(short)" in narrow and "(int)(short)" not in src           # comparisons on 16-bit values
    assert "stv_i16<W>(R.out" in narrow and "ldv_i16<W, " in narrow
    mixed = _emit(RC.INT_MIXED_TO_I16).stdout
    assert "a lane takes 2 groups of 8 elements per pass" in mixed          # 16 bytes of the i16 tensors
    # one streamed byte per byte written: ordinary loads (no non-temporal hint)
    assert "ldv_i16<W, false>(R.in[0].base" in mixed and "ldd_i32(R.in[1].base" in mixed


def test_reductions_also_get_a_workgroup_per_row_kernel():
    src = _emit(RC.C2_BCAST_ADD_ROWSUM).stdout
    assert "rows of exactly 4096 elements: a workgroup per row, the next row in flight" in src
    assert "afir_region_s0_rows_i32(" in src and "afir_region_s0_rows_i64(" in src
    rows = src[src.index("DEV void segment0_rows"):]
    rows = rows[:rows.index("\n}\n")]
    # the bias does not change with the row: loaded once, before the loop, not in the fetch of the next row
    # (the aligned form of each read; the general form next to it is compiled out in this kernel)
    assert rows.count("ldv_f32<W, false>(R.in[1].base, q1 + (A ||") == 1
    assert rows.count("ldv_f32<W, true>(R.in[0].base, q0 + (A ||") == 2
    assert rows.count("__builtin_amdgcn_s_barrier();") == 1
    # ... and the kernels for few long rows and for a handful of very long ones
    for name in ("afir_region_s0_long_i32(", "afir_region_s0_split_i32(", "afir_region_s0_join_i64("):
        assert name in src
    assert "float afir_region_partials[65536];" in src
    plain = _emit(RC.C1_ADD_MUL).stdout                           # parallel segments have none of these
    assert "_rows_" not in plain and "_split_" not in plain and "afir_region_partials" not in plain


def test_short_rows_get_one_group_per_lane_kernels():
    src = _emit(RC.RELU_COL_ADD).stdout
    assert "a lane takes 1 group of 8 elements per pass (for rows of few groups)" in src
    assert "afir_region_s0_slim_i32_a(" in src and "afir_region_s0_slim_i32_v(" in src
    assert "afir_region_s0_slim_i32_g(" not in src and "slim_i64" not in src
    assert "_slim" not in _emit(RC.C3_RELU_BCAST_TRANSPOSE).stdout       # tiled segments have none
    # and the three modes of the ordinary kernels
    for mode in "avg":
        assert f"afir_region_s0_i32_{mode}(" in src and f"afir_region_s0_i64_{mode}(" in src


def test_column_gathers_get_an_lds_staged_kernel():
    src = _emit(RC.RELU_COLGATHER_ADD).stdout
    assert "a workgroup per row, the gathered operand's source row staged in LDS" in src
    assert "a wavefront per row, the gathered operand's source row staged in LDS" in src
    for name in ("afir_region_s0_stage_i32_a(", "afir_region_s0_stage_i32_v(", "afir_region_s0_stage_i64_a(",
                 "afir_region_s0_stagew_i32_a(", "afir_region_s0_stagew_i64_v("):
        assert name in src
    assert "stage_f16(sbase + (bad ? 0 : gi[u][e]))" in src and "afir_region_s0_stage_i32_g(" not in src
    assert "_stage_" not in _emit(RC.C4_GATHER_SCALE_SHIFT).stdout      # rows gathered whole: nothing to stage


def test_identical_reads_are_loaded_once():
    src = _emit(RC.C1_ADD_MUL).stdout           # (a + b) * b reads b twice
    # once in the ordinary form of the segment, once in its one-group-per-lane form
    # (counted on the aligned form of the read; each is followed by its general form)
    assert src.count("ldv_f32<W, true>(R.in[1].base, q1 + (A ||") == 2 and "R.in[2]" not in src


def test_matmul_programs_have_no_source_form():
    prog = subprocess.run([TR, "-mlir-to-hip", "-"], input=MC.MATMUL_BIAS_LEAKY_BF16, capture_output=True, text=True)
    assert prog.returncode == 0
    p = _emit(prog.stdout)
    assert p.returncode == 1 and "hand-written MFMA kernels" in p.stderr
    # MLIR input works as well as a program
    p = subprocess.run([TR, "-mlir-to-hip", "-", "--emit-hip-source"], input=MC.SPLIT_HALVES,
                       capture_output=True, text=True)
    assert p.returncode == 0 and "afir_region_s1_i32_a" in p.stdout


def _compile(tmp_path, env=None, mlir=MC.SPLIT_HALVES):
    src = tmp_path / "k.mlir"
    src.write_text(mlir)
    p = subprocess.run([RS, "--kernel", str(src), "--output", str(tmp_path / "art"), "--name", "k"],
                       capture_output=True, text=True, env=dict(os.environ, **(env or {})))
    assert p.returncode == 0, p.stderr
    return (tmp_path / "art" / "out" / "manifest.txt").read_text().splitlines(), tmp_path / "art"


def test_artifact_holds_source_and_code_object(tmp_path):
    manifest, art = _compile(tmp_path)
    assert "code_object_path=k.hsaco" in manifest
    assert (art / "k.hip").read_text().startswith("// HIP kernels for the fused region 'k'")
    assert b"afir_region_s1_i64_g" in (art / "k.hsaco").read_bytes()
    desc = (art / "k.hipk").read_text()
    assert "code_object=k.hsaco\n" in desc and f"code_object_dir={art}\n" in desc
    assert not (art / "k.hipcc.log").exists()
    # the artifact loads again from its root
    assert subprocess.run([RS, "--artifact-root", str(art)], capture_output=True).returncode == 0


def test_artifact_without_compiler_keeps_the_program(tmp_path):
    manifest, art = _compile(tmp_path, env={"AFIR_HIP_CODEGEN": "0"})
    assert not any(l.startswith("code_object_path=") for l in manifest)
    assert "code_object_note=disabled by AFIR_HIP_CODEGEN=0" in manifest
    assert "program:\nafir-hip-region 1" in (art / "k.hipk").read_text()
    sub = tmp_path / "b"
    sub.mkdir()
    manifest, art = _compile(sub, env={"HIPCC": "/nonexistent/hipcc", "AFIR_HIP_COMPILER": "hipcc"})
    assert any(l.startswith("code_object_note=cannot start /nonexistent/hipcc") for l in manifest)
    assert (art / "k.hip").exists() and not (art / "k.hsaco").exists()


def test_artifact_without_hipcc_is_compiled_inside_the_process(tmp_path):
    """No hipcc on the host (or AFIR_HIP_COMPILER=hiprtc): the HIP runtime's own compiler library
    builds the same source with the same options, and the artifact holds the same kernels."""
    for i, env in enumerate(({"HIPCC": "/nonexistent/hipcc"}, {"AFIR_HIP_COMPILER": "hiprtc"})):
        sub = tmp_path / str(i)
        sub.mkdir()
        manifest, art = _compile(sub, env=env)
        assert "code_object_path=k.hsaco" in manifest, manifest
        image = (art / "k.hsaco").read_bytes()
        assert image[:4] == b"\x7fELF" and b"afir_region_s1_i64_g" in image and b"afir_region_program_hash" in image
        assert subprocess.run([RS, "--artifact-root", str(art)], capture_output=True).returncode == 0


def test_capi_compiles_a_region_inside_the_process(pkg):
    """afir_hip_region_compile: emit + compile + attach without hipcc and without a device."""
    from ascend_mlir_amd import hip_kernels as H
    L = H.load()
    r = H.Region(RC.RELU_COL_ADD)
    assert r.kernel != "fused_region_compiled"
    r.compile(in_process=True)
    assert r.kernel == "fused_region_compiled"
    u64, sz = ctypes.c_uint64, ctypes.c_size_t
    L.afir_hip_region_compile.restype = ctypes.c_uint32
    L.afir_hip_region_compile.argtypes = [u64, ctypes.c_void_p, sz, ctypes.POINTER(sz)]
    n = sz(0)
    assert L.afir_hip_region_compile(u64(r.handle), None, 0, ctypes.byref(n)) == 0 and n.value > 1000
    buf = ctypes.create_string_buffer(n.value)
    assert L.afir_hip_region_compile(u64(r.handle), buf, n.value, None) == 0
    assert buf.raw[:4] == b"\x7fELF" and b"afir_region_s0_i32_a" in buf.raw
    assert L.afir_hip_region_compile(u64(424242), None, 0, None) != 0 and b"no region program" in L.afir_hip_last_error()
    r.close()
    prog = subprocess.run([TR, "-mlir-to-hip", "-"], input=MC.MATMUL_BIAS_LEAKY_BF16, capture_output=True, text=True).stdout
    m = H.Region(prog)
    with pytest.raises(H.AfirHipError, match="no specialised kernel"):
        m.compile(in_process=True)
    m.close()


def test_capi_emit_and_attach_without_gpu(pkg):
    from ascend_mlir_amd import hip_kernels as H
    L = H.load()
    r = H.Region(RC.RELU_COL_ADD)
    src = r.emit_source()
    assert src == _emit(RC.RELU_COL_ADD).stdout.replace("fused region 'region'", "fused region 'region'")
    u64 = ctypes.c_uint64
    L.afir_hip_region_attach_code_object.argtypes = [u64, ctypes.c_char_p, ctypes.c_size_t]
    assert L.afir_hip_region_attach_code_object(u64(r.handle), None, 0) != 0
    assert b"empty image" in L.afir_hip_last_error()
    assert L.afir_hip_region_attach_code_object(u64(999999), b"x" * 16, 16) != 0
    assert b"no region program" in L.afir_hip_last_error()
    # an image is accepted as bytes here; it is checked against the program when first launched
    r.attach_code_object(b"\x7fELF" + b"\0" * 60)
    assert r.kernel == "fused_region_compiled"
    r.close()
    prog = subprocess.run([TR, "-mlir-to-hip", "-"], input=MC.MATMUL_BIAS_LEAKY_BF16, capture_output=True, text=True).stdout
    m = H.Region(prog)
    with pytest.raises(H.AfirHipError, match="no specialised kernel"):
        m.emit_source()
    with pytest.raises(H.AfirHipError, match="take no code object"):
        m.attach_code_object(b"\x7fELF" + b"\0" * 60)
    m.close()


def test_emit_options_change_the_tile_and_the_unroll(tmp_path):
    def emit(text, *flags):
        return subprocess.run([TR, "-mlir-to-hip", "-", "--emit-hip-source", *flags], input=text, capture_output=True, text=True)
    p = emit(RC.C3_RELU_BCAST_TRANSPOSE, "--emit-options", "tile_p=32,tile_q=128")
    assert p.returncode == 0, p.stderr
    assert "tiles of 32 (dim 1) x 128 (dim 2) through LDS; a lane takes 2 groups of 8 elements per row" in p.stdout
    assert "afir_region_emit_options[3] = {32, 128, 0};" in p.stdout
    assert "afir_region_emit_options[3] = {64, 64, 0};" in emit(RC.C3_RELU_BCAST_TRANSPOSE).stdout
    p = emit(RC.C1_ADD_MUL, "--emit-options=unroll=2")
    assert p.returncode == 0 and "a lane takes 2 groups of 4 elements per pass" in p.stdout
    p = emit(RC.C1_ADD_MUL, "--emit-options", "tile_q=100")
    assert p.returncode == 1 and "tile_q must be 64, 128 or 256" in p.stderr
    p = emit(RC.C1_ADD_MUL, "--emit-options", "tiles=3")
    assert p.returncode == 2 and "unknown emit option" in p.stderr
    # through the artifact compiler
    src = tmp_path / "k.region"
    src.write_text(RC.C3_RELU_BCAST_TRANSPOSE)
    q = subprocess.run([RS, "--kernel", str(src), "--output", str(tmp_path / "a"), "--name", "k",
                        "--emit-options", "tile_q=128"], capture_output=True, text=True)
    assert q.returncode == 0, q.stderr
    assert "x 128 (dim 2) through LDS" in (tmp_path / "a" / "k.hip").read_text()
    q = subprocess.run([RS, "--kernel", str(src), "--output", str(tmp_path / "b"), "--name", "k",
                        "--emit-options", "tile_p=48"], capture_output=True, text=True)
    assert q.returncode == 4 and "tile_p must be a multiple of 32" in q.stderr


def test_operations_after_reduce_sum_are_applied_to_the_row_sum_where_it_is_stored():
    src = _emit(RC.MEAN_ROWBIAS).stdout
    assert "float extent_const[8];" in src
    assert src.count("(rt_f16(s) / R.extent_const[0])") >= 4        # every kernel that stores a row sum
    assert "v0[u][e] / " not in src                          # not per element
    chain = _emit(RC.REDUCE_TAIL_CHAIN).stdout
    half, four = "as_f32(0x3f000000u) /* 0.5 */", "as_f32(0x40800000u) /* 4 */"
    assert f"(fmax_ieee(((-(s * {half})) + {four}), 0.f) * (R.extent_const[0] * {half}))" in chain
    plain = _emit(RC.REDUCE_ROWBIAS).stdout
    assert "R.extent_const" not in plain.split("struct SpecArgs", 1)[1].split("};", 1)[1]


def test_extent_constants_outside_the_tail_are_launch_arguments_too():
    """An extent is not known when the kernel is emitted: wherever it stands in the segment it
    is read from the launch arguments, numbered in program order (a literal 0 there once made
    `x / N` a division by zero on the compiled route only)."""
    par = _emit(RC.PARALLEL_DIV_EXTENT)
    assert par.returncode == 0, par.stderr
    assert "= R.extent_const[0];" in par.stdout and "= R.extent_const[1];" in par.stdout
    assert "as_f32(0x00000000u)" not in par.stdout.split("KERNEL void", 1)[0].split("segment0", 1)[1]
    pre = _emit(RC.PRE_REDUCE_DIV_EXTENT).stdout
    assert "= R.extent_const[0];" in pre                    # per element, before the sum
    assert src_count(pre, "(s * R.extent_const[1])") >= 4   # on the sum, numbered after it
    many = RC.PARALLEL_DIV_EXTENT.replace("  const arg0.0\n  mul\n", "  const arg0.0\n  mul\n" * 8)
    p = _emit(many)
    assert p.returncode != 0 and "more than 8 extent constants in a segment" in p.stderr


def src_count(src, needle):
    return src.count(needle)


def test_segments_that_can_separate_reads_from_writes_get_the_phased_kernel():
    """One or two streamed operands, row vectors and per-row values, one element size: the segment
    also has afir_region_s<k>_phased_i32 (eight 16-byte groups per lane, packed results held in
    registers through a timed hold); programs of several such segments also one kernel for all.
    Row sums, transposed reads, gathers along the innermost dim and mixed element sizes do not."""
    c1 = _emit(RC.C1_ADD_MUL).stdout
    assert "PHASED_KERNEL void afir_region_s0_phased_i32(const SpecArgs R)" in c1
    assert "in 2 rounds" in c1 and "u32x4 raw0[U];" in c1 and "u32x4 raw1[U];" in c1 and "rowvec" not in c1
    assert "__builtin_amdgcn_s_sleep(1);" in c1 and "R.hold_ticks" in c1
    c4 = _emit(RC.C4_GATHER_SCALE_SHIFT).stdout
    assert "afir_region_s0_phased_i32" in c4 and "in 1 round" in c4
    assert "rowvec[0 * row_chunks + c]" in c4 and "rowvec[1 * row_chunks + c]" in c4     # scale and shift through LDS
    split = _emit(RC.SPLIT_RELU_BRC_ADD_MUL).stdout
    assert "afir_region_s0_phased_i32" in split and "afir_region_s1_phased_i32" in split
    assert "PHASED_KERNEL void afir_region_all_phased_i32(const SpecAll S)" in split
    for text in (RC.C2_BCAST_ADD_ROWSUM, RC.C3_RELU_BCAST_TRANSPOSE, RC.RELU_COLGATHER_ADD, RC.RELU_COL_ADD):
        assert "_phased_i32" not in _emit(text).stdout
    mixed = RC.C1_ADD_MUL.replace("arg out f32 2", "arg out f16 2")
    assert "_phased_i32" not in _emit(mixed).stdout
