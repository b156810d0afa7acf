#!/usr/bin/env python3
"""Benchmark of the fused-kernel hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|c1|c3|c4|c5|...]
                    [--all/--no-all] [--no-cpu-baseline]

A step is one launch of the workload's fused kernel over one batch of seeded
synthetic input already resident in HBM.  Buffer sets are rotated between
steps: every HBM-bound workload cycles over at least 1 GiB of inputs, so that
none of its reads can be served from the 256 MB last-level cache (see
MIN_CYCLIC_READ_BYTES).  Before the W warmup steps the workload is launched
untimed for --ramp-ms (the device's sustained clocks).  Prints ONE JSON line.

  value            algorithmic GB/s (TFLOP/s for c5) over the K timed steps,
                   wall clock between two device synchronisations
  roofline         algorithmic bytes (flops) per launch / average launch
                   duration from HIP events recorded on the launch stream
                   around the last K - 1 of the same K steps (launches that
                   follow a launch: the host's way from the synchronisation to
                   its first launch is not kernel time), against the published peak
  cpu_baseline     the C restatement of the reference golden ("port"), timed
                   on this host's cores on a bounded sample
  workloads        with --all (default): the same figures for all five
                   configurations, each parity-checked against the oracle, the
                   region-program workloads (g*, i*) and three measured
                   ceilings (ceil_*: probe kernels of libafir_bench_probes.so)
  targets          per configuration: roofline.frac (the event-timed figure),
                   the target it is read against and whether it is met;
                   min_frac_hbm = the lowest of c1..c4
"""
from __future__ import annotations

import argparse
import importlib.util
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "fused-kernel HBM GB/s (% of peak); matmul+epilogue TFLOP/s; 1 GPU"
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published

# HBM bytes per step measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (two runs), scaled by the same counters' reading for a plain 256 MiB copy
# (FETCH_SIZE x 2.0, WRITE_SIZE x 1.0).  Not measured in this run: each figure
# is copied from section (2) of the profiles/ file named beside it, which gives
# the command that produced it.
MEASURED_TRAFFIC = {
    "c1": (201417113, "profiles/add_mul_f32_phased__c1_4096x4096.txt"),
    "c2": (134633066, "profiles/bcast_add_rowsum_f32_wgrow__c2_8192x4096.txt"),
    "c3": (134387302, "profiles/relu_bcast_add_transpose_f16_phased__c3_64x1024x512.txt"),
    "c4": (133898035, "profiles/gather_scale_shift_f16_phased__c4_131072x1024_idx32768.txt"),
    "c5": (1804801024, "profiles/matmul_bias_leakyrelu_dma__c5_8192x8192x8192.txt"),
    "g1": (201432473, "profiles/afir_region_s0_phased_i32__g1_compiled_add_mul_f32_4096x4096.txt"),
    "g2": (134726553, "profiles/afir_region_all_phased_i32__g2_compiled_split_relu_brc_f16_8192x4096.txt"),
    "g3": (134646784, "profiles/afir_region_s0_rows_i32__g3_compiled_bcast_add_rowsum_f32_8192x4096.txt"),
    "g4": (133937868, "profiles/afir_region_s0_phased_i32__g4_compiled_gather_scale_shift_f16_131072x1024_idx32768.txt"),
    "i1": (201611468, "profiles/fused_region_parallel__i1_interpreter_add_mul_f32_4096x4096.txt"),
    "i2": (135332659, "profiles/fused_region_parallel__i2_interpreter_split_relu_brc_f16_8192x4096.txt"),
}

# north_star targets, read on roofline.frac (algorithmic work / event-timed launch duration / published peak)
TARGETS = {"c1": 0.70, "c2": 0.70, "c3": 0.70, "c4": 0.70, "c5": 0.60}
CEILINGS = ["ceil_copy", "ceil_copy_phased", "ceil_read", "ceil_write", "ceil_tilecopy64"]
# m_ta / m_tb: c5's product with A (B) stored transposed, as region programs
# (linalg.matmul_transpose_a / _b of the reference's matmul recogniser)
# m_b16: sixteen independent products of 1024^3 in one launch (linalg.batch_matmul), same epilogue
LAYOUTS = ["m_ta", "m_tb", "m_b16"]
ALL_WORKLOADS = ["c1", "c2", "c3", "c4", "c5", "g1", "g2", "g3", "g4", "i1", "i2"] + LAYOUTS + CEILINGS

# Region programs of the two generic-kernel workloads (grammar:
# ascend-mlir_amd/csrc/target/region_program.h)
REGION_ADD_MUL = """afir-hip-region 1
arg in f32 2
arg in f32 2
arg out f32 2
segment 2
size arg0.0 arg0.1
outoff 0
push arg0 d0 d1
push arg1 d0 d1
add
push arg1 d0 d1
mul
store
end
"""
REGION_BCAST_ADD_ROWSUM = """afir-hip-region 1
arg in f32 2
arg in f32 1
arg out f32 1
segment 2
size arg0.0 arg0.1
outoff 0
push arg0 d0 d1
push arg1 d1
add
reduce sum
store
end
"""
REGION_GATHER_SCALE_SHIFT = """afir-hip-region 1
arg in f16 2
arg in i32 1
arg in f16 1
arg in f16 1
arg out f16 2
segment 2
size arg1.0 arg0.1
outoff 0
push arg0 g0:arg1 d1
push arg2 d1
mul
push arg3 d1
add
store
end
"""
REGION_SPLIT_RELU_BRC_ADD_MUL = """afir-hip-region 1
arg in f16 2
arg in f16 1
arg in f16 1
arg in f16 1
arg in f16 1
arg out f16 2
segment 2
size arg1.0 arg0.1
outoff 0
push arg0 d0 d1
relu
push arg1 d0
add
push arg3 d1
mul
store
end
segment 2
size arg2.0 arg0.1
outoff arg1.0
push arg0 d0 d1 slice arg1.0 0
relu
push arg2 d0
add
push arg4 d1
mul
store
end
"""


def load_package():
    name = "ascend_mlir_amd"
    if name in sys.modules:
        return sys.modules[name]
    pkg_dir = os.path.join(ROOT, "ascend-mlir_amd")
    spec = importlib.util.spec_from_file_location(
        name, os.path.join(pkg_dir, "__init__.py"), submodule_search_locations=[pkg_dir])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


# The last-level cache (256 MB "Infinity Cache", memory side) serves reads of anything that was
# read within the previous 256 MB of reads; writes pass through it.  A plain copy measures
# 6.7 TB/s while the launches cycle over <= 256 MiB of sources and 5.67 TB/s from 512 MiB on
# (the same kernel, the same launch sizes).  Every HBM-bound workload therefore cycles over
# enough copies of its inputs that the bytes it reads come back only after at least this many
# other bytes have been read: what is timed is HBM, not that cache.
MIN_CYCLIC_READ_BYTES = 1 << 30


def sets_for(read_bytes_per_launch):
    return max(2, -(-MIN_CYCLIC_READ_BYTES // int(read_bytes_per_launch)))


class Workload:
    """One configuration: seeded inputs, launch closures over `nsets` buffer
    sets, algorithmic work, parity check and CPU baseline."""

    key = ""
    title = ""
    dtype = ""
    bound = "hbm"

    def work(self):           # bytes (hbm) or flops (mfma) per launch
        raise NotImplementedError


def _dev(torch, a):
    return torch.from_numpy(a).cuda()


def _dev_bf16(torch, bits):
    import numpy as np
    return torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16)


def make_workload(key, torch, H, O, C):
    import numpy as np

    w = Workload()
    w.key = key
    if key == "c1":
        a, b = O.gen_c1()
        w.title = "c1 fused add->mul out=(a+b)*b f32 [4096,4096]"
        w.dtype, w.symbol = "f32", "afir_hip_launch_fused_add_mul"
        w.work = lambda: O.algorithmic_bytes("c1", m=4096, n=4096)
        w.nsets = sets_for(a.nbytes + b.nbytes)
        sets = []
        da, db = _dev(torch, a), _dev(torch, b)
        for i in range(w.nsets):
            ia, ib = (da, db) if i == 0 else (da.clone(), db.clone())
            out = torch.empty_like(ia)
            sets.append((ia, ib, out))
        w.sets = sets
        w.launches = [H.prepare(w.symbol, [s[0].data_ptr(), s[1].data_ptr(), s[2].data_ptr(), 0],
                                H.pack_tiling(4096, 4096)) for s in sets]

        def parity():
            want = O.golden_c1(a, b)
            got = sets[0][2].cpu().numpy()
            return {"bar": "bit-exact", "passed": got.tobytes() == want.tobytes(),
                    "mismatches": int((got != want).sum())}
        w.parity = parity

        def cpu(budget_s):
            t0 = time.perf_counter(); reps = 0
            while True:
                C.add_mul_f32(a, b); reps += 1
                if time.perf_counter() - t0 > budget_s:
                    break
            dt = (time.perf_counter() - t0) / reps
            return w.work() / dt / 1e9, f"full workload, mean of {reps} runs"
        w.cpu = cpu
    elif key == "c2":
        x, bias = O.gen_c2()
        w.title = "c2 broadcast-add-reduce y=rowsum(x+bias) f32 [8192,4096]+[4096]->[8192]"
        w.dtype, w.symbol = "f32", "afir_hip_launch_broadcast_add_reducesum"
        w.work = lambda: O.algorithmic_bytes("c2", m=8192, n=4096)
        w.nsets = sets_for(x.nbytes)
        dx, dbias = _dev(torch, x), _dev(torch, bias)
        sets = []
        for i in range(w.nsets):
            ix = dx if i == 0 else dx.clone()
            sets.append((ix, dbias, torch.empty((8192,), dtype=torch.float32, device="cuda")))
        w.sets = sets
        w.launches = [H.prepare(w.symbol, [s[0].data_ptr(), s[1].data_ptr(), s[2].data_ptr(), 0],
                                H.pack_tiling(8192, 4096)) for s in sets]

        def parity():
            want = O.golden_c2(x, bias).astype(np.float64)
            got = sets[0][2].cpu().numpy().astype(np.float64)
            scale = np.abs(x.astype(np.float64) + bias).sum(axis=1)
            err = np.abs(got - want)
            ok = err <= 1e-5 * np.abs(want) + 1e-7 * scale
            rel = err / np.maximum(np.abs(want), 1e-30)
            return {"bar": "<=1e-5 rel (+1e-7*sum|terms| floor)", "passed": bool(ok.all()),
                    "mismatches": int((~ok).sum()), "max_abs": float(err.max()),
                    "median_rel": float(np.median(rel))}
        w.parity = parity

        def cpu(budget_s):
            t0 = time.perf_counter(); reps = 0
            while True:
                C.bcast_add_rowsum_f32(x, bias); reps += 1
                if time.perf_counter() - t0 > budget_s:
                    break
            dt = (time.perf_counter() - t0) / reps
            return w.work() / dt / 1e9, f"full workload, mean of {reps} runs"
        w.cpu = cpu
    elif key == "c3":
        x, c = O.gen_c3()
        w.title = "c3 relu-broadcast-transpose out=transpose(relu(x)+c) f16 [64,1024,512]->[64,512,1024]"
        w.dtype, w.symbol = "f16", "afir_hip_launch_relu_broadcast_add_transpose"
        w.work = lambda: O.algorithmic_bytes("c3", b=64, m=1024, n=512)
        w.nsets = sets_for(x.nbytes)
        dx, dc = _dev(torch, x), _dev(torch, c)
        sets = []
        for i in range(w.nsets):
            ix = dx if i == 0 else dx.clone()
            sets.append((ix, dc, torch.empty((64, 512, 1024), dtype=torch.float16, device="cuda")))
        w.sets = sets
        w.launches = [H.prepare(w.symbol, [s[0].data_ptr(), s[1].data_ptr(), s[2].data_ptr(), 0],
                                H.pack_tiling(64, 1024, 512)) for s in sets]

        def parity():
            want = O.golden_c3(x, c)
            got = sets[0][2].cpu().numpy()
            return {"bar": "bit-exact (<=1e-2 rel required)",
                    "passed": got.tobytes() == want.tobytes(),
                    "mismatches": int((got.view(np.uint16) != want.view(np.uint16)).sum())}
        w.parity = parity

        def cpu(budget_s):
            t0 = time.perf_counter(); reps = 0
            while True:
                C.relu_bcast_add_transpose_f16(x, c); reps += 1
                if time.perf_counter() - t0 > budget_s:
                    break
            dt = (time.perf_counter() - t0) / reps
            return w.work() / dt / 1e9, f"full workload, mean of {reps} runs"
        w.cpu = cpu
    elif key == "c4":
        table, idx, scale, shift = O.gen_c4()
        w.title = ("c4 gather-elementwise out=table[idx]*scale+shift f16 table [131072,1024], "
                   "int32 idx [32768]")
        w.dtype, w.symbol = "f16", "afir_hip_launch_gather_scale_shift"
        w.work = lambda: O.algorithmic_bytes("c4", nidx=32768, dim=1024)
        # a launch reads 64 MiB of gathered rows: a seeded index vector and a copy of the table of its
        # own per set (16 x 256 MiB), so that no launch finds rows in the 256 MB last-level cache that
        # an earlier one left there (with four tables the launch four steps back still did: the same
        # kernel measured 1-3 % faster, and its best hold shorter)
        w.nsets = sets_for(32768 * 1024 * 2)
        dt_, dsc, dsh = _dev(torch, table), _dev(torch, scale), _dev(torch, shift)
        tables = [dt_] + [dt_.clone() for _ in range(w.nsets - 1)]
        rng = np.random.default_rng(7)
        sets = []
        for i in range(w.nsets):
            ii = idx if i == 0 else rng.integers(0, 131072, 32768, dtype=np.int64).astype(np.int32)
            sets.append((tables[i], _dev(torch, ii), dsc, dsh,
                         torch.empty((32768, 1024), dtype=torch.float16, device="cuda")))
        w.sets = sets
        w.launches = [H.prepare(w.symbol, [s[0].data_ptr(), s[1].data_ptr(), s[2].data_ptr(),
                                           s[3].data_ptr(), s[4].data_ptr(), 0],
                                H.pack_tiling(131072, 1024, 32768)) for s in sets]

        def parity():
            want = O.golden_c4(table, idx, scale, shift)
            got = sets[0][4].cpu().numpy()
            return {"bar": "bit-exact", "passed": got.tobytes() == want.tobytes(),
                    "mismatches": int((got.view(np.uint16) != want.view(np.uint16)).sum())}
        w.parity = parity

        def cpu(budget_s):
            t0 = time.perf_counter(); reps = 0
            while True:
                C.gather_scale_shift_f16(table, idx, scale, shift); reps += 1
                if time.perf_counter() - t0 > budget_s:
                    break
            dt = (time.perf_counter() - t0) / reps
            return w.work() / dt / 1e9, f"full workload, mean of {reps} runs"
        w.cpu = cpu
    elif key == "c5":
        a, b, bias = O.gen_c5()
        w.title = ("c5 matmul-add-leakyrelu out=leakyrelu(A@B+bias,0.01) bf16 8192x8192x8192, "
                   "fp32 accumulate")
        w.dtype, w.symbol, w.bound = "bf16", "afir_hip_launch_matmul_add_leakyrelu", "mfma"
        w.work = lambda: O.algorithmic_flops_c5(8192, 8192, 8192)
        w.nsets = 2
        da, db, dbias = _dev_bf16(torch, a), _dev_bf16(torch, b), _dev_bf16(torch, bias)
        sets = []
        for i in range(w.nsets):
            ia, ib = (da, db) if i == 0 else (da.clone(), db.clone())
            sets.append((ia, ib, dbias,
                         torch.empty((8192, 8192), dtype=torch.bfloat16, device="cuda")))
        w.sets = sets
        w.launches = [H.prepare(w.symbol, [s[0].data_ptr(), s[1].data_ptr(), s[2].data_ptr(),
                                           s[3].data_ptr(), 0],
                                H.pack_tiling(8192, 8192, 8192, H.f32_bits(0.01))) for s in sets]

        def parity():
            rows = np.arange(0, 8192, 61)[:128]          # strided row sample, full K and N
            want = O.golden_c5_rows(a, b, bias, rows, 0.01)
            got = sets[0][3][torch.from_numpy(rows).cuda()].view(torch.int16).cpu().numpy() \
                .view(np.uint16)
            r = O.compare_outputs([(got, "bf16")], [(want, "bf16")], 1e-5, 1e-2)
            nonfinite = O.nonfinite_mismatches(got, want, "bf16")   # the comparator cannot see NaN
            return {"bar": "<=1e-2 rel (atol 1e-5), 128 sampled rows x 8192 cols; no NaN / inf the golden lacks",
                    "passed": bool(r["passed"]) and nonfinite == 0,
                    "mismatches": int(r["mismatches"]) + nonfinite, "nonfinite_mismatches": nonfinite,
                    "max_abs": float(r["max_abs_diff"]),
                    "bit_identical_frac": float((got == want).mean())}
        w.parity = parity

        def cpu(budget_s):
            rows = 64
            t0 = time.perf_counter()
            C.matmul_bias_leakyrelu_bf16(a[:rows], b, bias, 0.01)
            dt = time.perf_counter() - t0
            return (2.0 * rows * 8192 * 8192) / dt / 1e12, \
                f"{rows} of 8192 output rows (full K and N), one run"
        w.cpu = cpu

        def power_evidence():
            """Why the fraction of the published MFMA peak is what it is, in figures
            measured in this run on this workload's operands: the register-only MFMA
            rate (the board power limit sets the clock, and the power an MFMA draws
            depends on its operand values), the same kernel with its feed and its
            LDS reads left out, the vendor GEMM on the same operands, and all of it
            again on constant matrices."""
            from ascend_mlir_amd import bench_probes as P
            flops = w.work()

            def rate(launch, n=10, warm=2):
                for i in range(warm):
                    launch(i)
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for i in range(n):
                    launch(i)
                e1.record()
                torch.cuda.synchronize()
                return flops * n / (e0.elapsed_time(e1) * 1e-3) / 1e12

            def ablated(what):
                calls = [P.prepare("afir_bench_matmul_ablated", s[0].data_ptr(), s[1].data_ptr(), s[2].data_ptr(),
                                   s[3].data_ptr(), 8192, 8192, 8192, what) for s in sets]
                return lambda i: calls[i % len(calls)]()

            ours = lambda i: w.launches[i % len(w.launches)]()
            vendor = lambda i: torch.matmul(sets[i % len(sets)][0], sets[i % len(sets)][1])
            # alternating rounds: each kernel sees the same thermal history
            rounds = {"this_kernel": [], "vendor_gemm": [], "no_feed": [], "no_feed_no_lds_reads": [],
                      "loads_of_one_kib": [], "l2_resident": []}
            for _ in range(3):
                rounds["vendor_gemm"].append(rate(vendor))
                rounds["this_kernel"].append(rate(ours))
                rounds["no_feed"].append(rate(ablated(1)))
                rounds["no_feed_no_lds_reads"].append(rate(ablated(2)))
                rounds["loads_of_one_kib"].append(rate(ablated(3)))
                rounds["l2_resident"].append(rate(ablated(4)))
            med = lambda v: round(sorted(v)[len(v) // 2], 1)
            ev = {"mfma_only_workload_operands_tflops": round(P.mfma_rate(sets[0][0]), 1),
                  "vendor_gemm_tflops": med(rounds["vendor_gemm"]),
                  "vendor_gemm": "torch.matmul (hipBLASLt), no bias / activation, same operands, rounds of 10 "
                                 "launches alternating with this kernel; median of 3",
                  "this_kernel_alternating_tflops": med(rounds["this_kernel"]),
                  "decomposition_tflops": {
                      "mfma_waits_barriers": med(rounds["no_feed_no_lds_reads"]),
                      "plus_lds_operand_reads": med(rounds["no_feed"]),
                      "plus_load_issue_and_lds_writes": med(rounds["loads_of_one_kib"]),
                      "plus_l2_hits_operands_resident_in_l2": med(rounds["l2_resident"]),
                      "plus_l2_misses_the_kernel": med(rounds["this_kernel"])}}
            ones = torch.ones((8192, 8192), dtype=torch.bfloat16, device="cuda")
            ev["mfma_only_constant_operands_tflops"] = round(P.mfma_rate(ones), 1)
            launch = H.prepare(w.symbol, [ones.data_ptr(), ones.data_ptr(), sets[0][2].data_ptr(),
                                          sets[1][3].data_ptr(), 0],
                               H.pack_tiling(8192, 8192, 8192, H.f32_bits(0.01)))
            ev["kernel_constant_operands_tflops"] = round(rate(lambda i: launch(), n=20, warm=3), 1)
            ev["vendor_gemm_constant_operands_tflops"] = round(rate(lambda i: torch.matmul(ones, ones), n=20, warm=3), 1)
            # the board's own power reading against its cap while each kind of operand runs
            # (hwmon of the amdgpu driver; absent where the driver does not expose it)
            cap = _board_power("power1_cap")
            if cap:
                ev["board_power_cap_w"] = cap
                ev["board_power_w_this_kernel_workload_operands"] = _power_while(torch, ours)
                ev["board_power_w_this_kernel_constant_operands"] = _power_while(torch, lambda i: launch())
            return ev
        w.power_evidence = power_evidence
    elif key == "m_b16":
        nb, dim = 16, 1024
        w.title = ("m_b16 batch of 16 matmul-add-leakyrelu bf16 1024x1024x1024 (linalg.batch_matmul + the same epilogue), "
                   "as a region program")
        w.dtype, w.bound, w.no_cpu = "bf16", "mfma", True
        w.work = lambda: nb * O.algorithmic_flops_c5(dim, dim, dim)
        w.nsets = 8
        text = ("afir-hip-region 1\narg in bf16 3\narg in bf16 3\narg in bf16 1\narg out bf16 3\nsegment 3\n"
                " size arg3.0 arg3.1 arg3.2\n outoff 0\n matmul arg0 arg1\n push arg2 d2\n add\n leaky 0.01\n store\nend\n")
        region = H.Region(text)
        parts = [O.gen_c5(dim, dim, dim, seed=O.SEED + z) for z in range(nb)]
        a = np.stack([p[0] for p in parts])
        b = np.stack([p[1] for p in parts])
        bias = parts[0][2]
        da, db, dbias = _dev_bf16(torch, a), _dev_bf16(torch, b), _dev_bf16(torch, bias)
        sets = []
        for i in range(w.nsets):
            ia, ib = (da, db) if i == 0 else (da.clone(), db.clone())
            sets.append((ia, ib, dbias, torch.empty((nb, dim, dim), dtype=torch.bfloat16, device="cuda")))
        w.sets = sets
        w.region = region
        tiling = H.pack_tiling(nb, dim, dim, nb, dim, dim, dim, nb, dim, dim)
        w.launches = [region.prepare([s[0].data_ptr(), s[1].data_ptr(), s[2].data_ptr(), s[3].data_ptr()], tiling) for s in sets]

        def parity():
            rows = np.arange(0, dim, 17)[:32]
            bad = nonfinite = 0
            for z in (0, 7, 15):
                want = O.golden_c5_rows(a[z], b[z], bias, rows, 0.01)
                got = sets[0][3][z][torch.from_numpy(rows).cuda()].view(torch.int16).cpu().numpy().view(np.uint16)
                bad += int(O.compare_outputs([(got, "bf16")], [(want, "bf16")], 1e-5, 1e-2)["mismatches"])
                nonfinite += O.nonfinite_mismatches(got, want, "bf16")
            return {"bar": "<=1e-2 rel (atol 1e-5), 32 sampled rows x 1024 cols of batches 0, 7, 15; no NaN / inf the golden lacks",
                    "passed": bad == 0 and nonfinite == 0, "mismatches": bad + nonfinite,
                    "nonfinite_mismatches": nonfinite, "kernel": H.last_launch()["kernel"]}
        w.parity = parity
    elif key in LAYOUTS:
        # c5's operands, one of them stored transposed; the product is c5's, so its golden is too
        ta = key == "m_ta"
        a, b, bias = O.gen_c5()
        flags = " ta" if ta else " tb"
        w.title = (f"{key} matmul-add-leakyrelu bf16 8192x8192x8192 with {'A stored as [K, M]' if ta else 'B stored as [N, K]'} "
                   f"(linalg.matmul_transpose_{'a' if ta else 'b'}), as a region program")
        w.dtype, w.bound, w.no_cpu = "bf16", "mfma", True
        w.work = lambda: O.algorithmic_flops_c5(8192, 8192, 8192)
        w.nsets = 2
        text = ("afir-hip-region 1\narg in bf16 2\narg in bf16 2\narg in bf16 1\narg out bf16 2\nsegment 2\n"
                f" size arg3.0 arg3.1\n outoff 0\n matmul arg0 arg1{flags}\n push arg2 d1\n add\n leaky 0.01\n store\nend\n")
        region = H.Region(text)
        da, db, dbias = _dev_bf16(torch, a), _dev_bf16(torch, b), _dev_bf16(torch, bias)
        if ta:
            da = da.t().contiguous()
        else:
            db = db.t().contiguous()
        sets = []
        for i in range(w.nsets):
            ia, ib = (da, db) if i == 0 else (da.clone(), db.clone())
            sets.append((ia, ib, dbias, torch.empty((8192, 8192), dtype=torch.bfloat16, device="cuda")))
        w.sets = sets
        w.region = region
        tiling = H.pack_tiling(8192, 8192, 8192, 8192, 8192, 8192, 8192)
        w.launches = [region.prepare([s[0].data_ptr(), s[1].data_ptr(), s[2].data_ptr(), s[3].data_ptr()], tiling) for s in sets]

        def parity():
            rows = np.arange(0, 8192, 61)[:128]
            want = O.golden_c5_rows(a, b, bias, rows, 0.01)
            got = sets[0][3][torch.from_numpy(rows).cuda()].view(torch.int16).cpu().numpy().view(np.uint16)
            r = O.compare_outputs([(got, "bf16")], [(want, "bf16")], 1e-5, 1e-2)
            nonfinite = O.nonfinite_mismatches(got, want, "bf16")
            return {"bar": "<=1e-2 rel (atol 1e-5), 128 sampled rows x 8192 cols; no NaN / inf the golden lacks",
                    "passed": bool(r["passed"]) and nonfinite == 0, "mismatches": int(r["mismatches"]) + nonfinite,
                    "nonfinite_mismatches": nonfinite, "kernel": H.last_launch()["kernel"]}
        w.parity = parity
    elif key in ("g1", "g2", "g3", "g4", "i1", "i2"):
        # Region programs (any fused chain) next to the hand-tuned kernels:
        # g1 / i1 = the c1 chain kept off its fast path, g2 / i2 = the
        # reference's split / relu / broadcast-add / broadcast-mul / concat
        # graph (examples/split-relu-brc-add-mul) at [8192, 4096] f16.
        # g3 / g4 = the c2 row sum and the c4 gather as programs, kept off
        # their fast paths.  g: kernels emitted and compiled for the program;
        # i: the interpreter kernel of the library.
        from oracle import region_oracle as RO
        compiled = key[0] == "g"
        how = "compiled region kernel" if compiled else "region interpreter kernel"
        os.environ["AFIR_HIP_REGION_GENERIC"] = "1"
        if key[1] == "1":
            text = REGION_ADD_MUL
            a, b = O.gen_c1()
            inputs, out_shape, out_dt = [a, b], (4096, 4096), torch.float32
            w.title = f"{key} {how}: (a+b)*b f32 [4096,4096] as a region program"
            w.dtype = "f32"
            work = O.algorithmic_bytes("c1", m=4096, n=4096)
        elif key[1] == "3":
            text = REGION_BCAST_ADD_ROWSUM
            x, bias = O.gen_c2()
            inputs, out_shape, out_dt = [x, bias], (8192,), torch.float32
            w.title = f"{key} {how}: rowsum(x+bias) f32 [8192,4096] as a region program"
            w.dtype = "f32"
            work = O.algorithmic_bytes("c2", m=8192, n=4096)
        elif key[1] == "4":
            text = REGION_GATHER_SCALE_SHIFT
            inputs = list(O.gen_c4())
            out_shape, out_dt = (32768, 1024), torch.float16
            w.title = f"{key} {how}: table[idx]*scale+shift f16 [131072,1024], idx [32768] as a region program"
            w.dtype = "f16"
            work = O.algorithmic_bytes("c4", nidx=32768, dim=1024)
        else:
            text = REGION_SPLIT_RELU_BRC_ADD_MUL
            rng = np.random.default_rng(42)
            m, n = 8192, 4096
            f16 = lambda shape: rng.uniform(-1, 1, shape).astype(np.float32).astype(np.float16)
            inputs = [f16((m, n)), f16((m // 2,)), f16((m // 2,)), f16((n,)), f16((n,))]
            out_shape, out_dt = (m, n), torch.float16
            w.title = (f"{key} {how}: split/relu/bcast-add/bcast-mul/concat f16 [8192,4096] "
                       "(two segments)")
            w.dtype = "f16"
            work = 2 * m * n * 2 + 2 * (m // 2) * 2 + 2 * n * 2
        region = H.Region(text)
        del os.environ["AFIR_HIP_REGION_GENERIC"]
        assert region.kernel == "fused_region"
        if compiled:
            region.compile()     # from lib/region_cache when build() left it there
            assert region.kernel == "fused_region_compiled"
        w.work = lambda: work
        w.nsets = sets_for(32768 * 1024 * 2 if key[1] == "4" else
                           inputs[0].nbytes + (inputs[1].nbytes if key[1] == "1" else 0))
        dev0 = [_dev(torch, x) for x in inputs]
        tables = [dev0[0]] + ([dev0[0].clone() for _ in range(w.nsets - 1)] if key[1] == "4" else [])
        sets = []
        idx_rng = np.random.default_rng(7)
        for i in range(w.nsets):
            if i == 0:
                ins = dev0
            elif key[1] == "4":
                # other rows and a table of its own for every set (as in c4)
                other = idx_rng.integers(0, 131072, 32768, dtype=np.int64).astype(np.int32)
                ins = [tables[i], _dev(torch, other)] + dev0[2:]
            else:
                ins = [dev0[0].clone()] + ([dev0[1].clone()] if key[1] == "1" else dev0[1:])
            sets.append((ins, torch.empty(out_shape, dtype=out_dt, device="cuda")))
        w.sets = sets
        dims = [d for x in inputs for d in x.shape] + list(out_shape)
        w.launches = [region.prepare([t.data_ptr() for t in s[0]] + [s[1].data_ptr()],
                                     H.pack_tiling(*dims)) for s in sets]
        w.region = region

        def parity():
            want = RO.evaluate(text, inputs)
            got = sets[0][1].cpu().numpy()
            if key[1] == "3":      # a sum in another order: the bar of c2
                err = np.abs(got.astype(np.float64) - want.astype(np.float64))
                scale = np.abs(inputs[0].astype(np.float64) + inputs[1]).sum(axis=1)
                ok = err <= 1e-5 * np.abs(want.astype(np.float64)) + 1e-7 * scale
                return {"bar": "<=1e-5 rel (+1e-7*sum|terms| floor) vs the region oracle", "passed": bool(ok.all()),
                        "mismatches": int((~ok).sum()), "max_abs": float(err.max())}
            bits = np.uint16 if key[1] in "24" else np.uint32
            return {"bar": "bit-exact vs the region oracle", "passed": got.tobytes() == want.tobytes(),
                    "mismatches": int((got.view(bits) != want.view(bits)).sum())}
        w.parity = parity

        def cpu(budget_s):
            t0 = time.perf_counter()
            RO.evaluate(text, inputs)
            dt = time.perf_counter() - t0
            return w.work() / dt / 1e9, "full workload, numpy region oracle (1 thread), one run"
        w.cpu = cpu
        w.cpu_cores = 1
    elif key in CEILINGS:
        # Measured ceilings (probe kernels of libafir_bench_probes.so, csrc/bench/probes.h): what
        # this chip sustains on a plain copy, on a copy whose reads and writes are separated in time
        # (what the one-shot kernels of c3 and c4 do), on a read-only and a write-only stream, and on
        # the address pattern of c3's other kernel with the transposition left out.  No oracle:
        # nothing is computed.
        from ascend_mlir_amd import bench_probes as P
        # 128 MiB for the read-only stream: as long a launch as the copies' (a 10 us launch would
        # measure the host's launch rate)
        nbytes = (128 << 20) if key in ("ceil_read", "ceil_write") else (64 << 20)
        w.dtype = "u8"
        w.nsets = sets_for(nbytes)
        w.no_cpu = True
        srcs = [torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device="cuda") for _ in range(w.nsets)]
        if key == "ceil_copy":
            w.title = "ceil_copy: 64 MiB -> 64 MiB, 128-bit non-temporal loads and stores (probe, no arithmetic)"
            dsts = [torch.empty_like(x) for x in srcs]
            w.work = lambda: 2 * nbytes
            w.launches = [P.prepare("afir_bench_copy", a.data_ptr(), b.data_ptr(), nbytes) for a, b in zip(srcs, dsts)]
            w.sets = list(zip(srcs, dsts))
            w.parity = lambda: {"bar": "dst == src", "passed": bool(torch.equal(srcs[0], dsts[0])),
                                "mismatches": int((srcs[0] != dsts[0]).sum().item())}
        elif key == "ceil_copy_phased":
            w.title = ("ceil_copy_phased: 64 MiB -> 64 MiB with every lane resident at once and the stores held "
                       "back until the chip's reads have been served (probe, no arithmetic)")
            dsts = [torch.empty_like(x) for x in srcs]
            w.work = lambda: 2 * nbytes
            w.launches = [P.prepare("afir_bench_copy_phased", a.data_ptr(), b.data_ptr(), nbytes)
                          for a, b in zip(srcs, dsts)]
            w.sets = list(zip(srcs, dsts))
            w.parity = lambda: {"bar": "dst == src", "passed": bool(torch.equal(srcs[0], dsts[0])),
                                "mismatches": int((srcs[0] != dsts[0]).sum().item())}
        elif key == "ceil_write":
            w.title = "ceil_write: 128 MiB write-only stream, 128-bit non-temporal stores (probe)"
            w.work = lambda: nbytes
            w.launches = [P.prepare("afir_bench_fill", a.data_ptr(), nbytes, 7 + i) for i, a in enumerate(srcs)]
            w.sets = [(a,) for a in srcs]

            def parity():
                words = srcs[0].view(torch.int32).view(-1, 4)
                ok = bool((words[:, 0] == 7).all().item()) and bool((words[:, 3] == 21).all().item())
                return {"bar": "every chunk holds the launch's seed", "passed": ok, "mismatches": 0 if ok else 1}
            w.parity = parity
        elif key == "ceil_read":
            w.title = "ceil_read: 128 MiB read-only stream, 128-bit non-temporal loads (probe)"
            sink = torch.zeros(8192, dtype=torch.float32, device="cuda")
            w.work = lambda: nbytes
            w.launches = [P.prepare("afir_bench_read", a.data_ptr(), sink.data_ptr(), nbytes) for a in srcs]
            w.sets = [(a, sink) for a in srcs]
            w.parity = lambda: {"bar": "none: nothing is written", "passed": True, "mismatches": 0}
        else:
            w.title = ("ceil_tilecopy64: c3's address pattern ([64,1024,512] -> [64,512,1024] f16 in 64x64 tiles, "
                       "128-byte runs both ways) without the transposition (probe, registers only)")
            dsts = [torch.empty_like(x) for x in srcs]
            w.work = lambda: 2 * nbytes
            w.launches = [P.prepare("afir_bench_tilecopy64", a.data_ptr(), b.data_ptr(), 64, 1024, 512)
                          for a, b in zip(srcs, dsts)]
            w.sets = list(zip(srcs, dsts))

            def parity():
                # every byte of src lands somewhere in dst: compare the byte histograms
                a = torch.bincount(srcs[0].int(), minlength=256)
                b = torch.bincount(dsts[0].int(), minlength=256)
                return {"bar": "dst is a permutation of src (byte histogram)", "passed": bool(torch.equal(a, b)),
                        "mismatches": int((a != b).sum().item())}
            w.parity = parity
    else:
        raise SystemExit(f"unknown workload {key}")
    return w


def _board_power(name="power1_input"):
    """Watts from the amdgpu driver's hwmon file of the first card that has one, or None."""
    import glob
    for path in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/" + name)):
        try:
            with open(path) as f:
                return round(int(f.read().strip()) / 1e6, 1)
        except (OSError, ValueError):
            continue
    return None


def _power_while(torch, launch, seconds=1.0):
    """Median board power over the second half of `seconds` of back-to-back launches."""
    readings, i = [], 0
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            launch(i)
            i += 1
        torch.cuda.synchronize()
        if time.perf_counter() - t0 > seconds / 2:
            p = _board_power()
            if p is not None:
                readings.append(p)
    return sorted(readings)[len(readings) // 2] if readings else None


def run_workload(w, torch, steps, warmup, ramp_ms=0.0):
    n = len(w.launches)
    # The device takes some 50-100 ms of continuous work to settle at its sustained clocks (the
    # first launches after an idle period run 3-8 % slower): launches of the same workload,
    # untimed, until ramp_ms have passed; then the W warmup steps, then the K timed ones.
    if ramp_ms > 0:
        t_end = time.perf_counter() + ramp_ms * 1e-3
        i = 0
        while time.perf_counter() < t_end:
            for _ in range(16):
                w.launches[i % n]()
                i += 1
            torch.cuda.synchronize()
    for i in range(warmup):
        w.launches[i % n]()
    torch.cuda.synchronize()
    # The wall clock brackets exactly the K timed steps between two synchronisations.  The events
    # bracket the last K - 1 of them: the first event sits behind the first timed launch, so what
    # they time is launches that follow a launch, not the host's way from the synchronisation to
    # its first launch (3-15 us of idle device, which at K = 20 would read as 1-4 % of every step).
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    if steps < 2:
        e0.record()
    for i in range(steps):
        w.launches[i % n]()
        if i == 0 and steps >= 2:
            e0.record()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ev_ms = e0.elapsed_time(e1)
    return wall, ev_ms, (steps - 1 if steps >= 2 else steps)


def summarize(w, wall, ev_ms, steps, ev_steps):
    work = w.work()
    avg_launch_s = ev_ms / 1e3 / ev_steps
    if w.bound == "hbm":
        value, unit = work * steps / wall / 1e9, "GB/s"
        achieved, peak = work / avg_launch_s / 1e9, HBM_PEAK_GBS
    else:
        value, unit = work * steps / wall / 1e12, "TFLOP/s"
        achieved, peak = work / avg_launch_s / 1e12, MFMA_BF16_PEAK_TFLOPS
    traffic, source = MEASURED_TRAFFIC.get(w.key, (None, None))
    roof = {"bound": w.bound, "achieved": round(achieved, 2), "peak": peak, "unit": unit,
            "frac": round(achieved / peak, 4), "traffic": traffic, "traffic_source": source,
            "avg_launch_us": round(avg_launch_s * 1e6, 3),
            "work_per_launch": work}
    return value, unit, roof


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--ramp-ms", type=float, default=100.0,
                    help="untimed launches of the workload for this long before the warmup steps, so that "
                         "the device is at its sustained clocks when the timed region starts (0: none)")
    ap.add_argument("--workload", default="c2", choices=ALL_WORKLOADS)
    ap.add_argument("--all", dest="all", action="store_true", default=True)
    ap.add_argument("--no-all", dest="all", action="store_false")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-power-evidence", action="store_true",
                    help="c5: skip the extra launches on constant operands and the MFMA rate probe "
                         "(keeps a profiler's per-kernel averages to the timed steps)")
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three plain 256 MiB device copies, so that a counter run "
                         "(rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE) holds a kernel of known traffic")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build runs the fused-kernel path on ONE GPU; "
                         "--gpus must be 1 (no collectives or sharding are part of it)")

    import torch
    if not torch.cuda.is_available():
        raise SystemExit("bench.py: no GPU visible; the HIP path has no CPU fallback")
    load_package()
    from ascend_mlir_amd import hip_kernels as H
    H.load()
    from oracle import afir_oracle as O
    from oracle import c_oracle as C

    def steps_for(key):
        if args.steps is not None:
            return args.steps
        return 50 if key in ("c5", "m_ta", "m_tb") else 300

    def warm_for(key):
        if args.warmup is not None:
            return args.warmup
        return 5 if key in ("c5", "m_ta", "m_tb") else 30

    order = [args.workload] + ([k for k in ALL_WORKLOADS if k != args.workload] if args.all else [])
    results = []
    for key in order:
        w = make_workload(key, torch, H, O, C)
        steps, warmup = steps_for(key), warm_for(key)
        wall, ev_ms, ev_steps = run_workload(w, torch, steps, warmup, args.ramp_ms)
        value, unit, roof = summarize(w, wall, ev_ms, steps, ev_steps)
        par = w.parity()
        extra = (w.power_evidence() if hasattr(w, "power_evidence") and not args.no_power_evidence
                 else None)
        entry = {"key": key, "workload": w.title, "value": round(value, 2), "unit": unit, "steps": steps,
                 "warmup": warmup, "ms_per_step": round(wall * 1e3 / steps, 5), "dtype": w.dtype,
                 "buffer_sets": w.nsets, "roofline": roof, "parity": par}
        if extra is not None:
            entry["power_limit_evidence"] = extra
            # the same kernel against what the matrix cores sustain on these operands from registers
            # alone, and against the vendor GEMM (a comparator here, never part of the product path)
            roof["frac_of_mfma_only"] = round(roof["achieved"] / extra["mfma_only_workload_operands_tflops"], 4)
            roof["vs_vendor_gemm"] = round(extra["this_kernel_alternating_tflops"] / extra["vendor_gemm_tflops"], 4)
        if not args.no_cpu_baseline and not getattr(w, "no_cpu", False):
            budget = args.cpu_seconds if key == args.workload else min(3.0, args.cpu_seconds)
            v, sample = w.cpu(budget)
            entry["cpu_baseline"] = {"value": round(v, 4), "unit": unit,
                                     "cores": getattr(w, "cpu_cores", None) or C.threads(),
                                     "kind": "port", "sample": sample,
                                     "host_cpus": os.cpu_count()}
        results.append(entry)
        del w
        torch.cuda.empty_cache()

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    main_e = results[0]
    line = {
        "metric": METRIC, "value": main_e["value"], "unit": main_e["unit"], "n_gpus": 1,
        "steps": main_e["steps"], "warmup": main_e["warmup"],
        "ms_per_step": main_e["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": main_e["dtype"], "data": "synthetic",
        "config": {"workload": main_e["workload"], "seed": 42,
                   "buffer_sets": main_e["buffer_sets"], "ramp_ms": args.ramp_ms},
        "roofline": {k: main_e["roofline"][k] for k in
                     ("bound", "achieved", "peak", "unit", "frac", "traffic")},
        "parity": main_e["parity"],
    }
    line["roofline"]["traffic_source"] = main_e["roofline"]["traffic_source"]
    if "power_limit_evidence" in main_e and not args.all:
        for k in ("frac_of_mfma_only", "vs_vendor_gemm"):
            line["roofline"][k] = main_e["roofline"][k]
        line["power_limit_evidence"] = main_e["power_limit_evidence"]
    if "cpu_baseline" in main_e:
        line["cpu_baseline"] = {k: main_e["cpu_baseline"][k] for k in
                                ("value", "unit", "cores", "kind", "sample")}
    line["device"] = torch.cuda.get_device_name(0)
    if args.all:
        by_key = {e["key"]: e for e in results}
        # The long per-workload array goes first and a compact summary of every configuration
        # last: a log that keeps only the end of this line still holds all five.
        line["workloads"] = results
        # the targets are read on roofline.frac: algorithmic work / average launch duration from HIP
        # events / published peak (value, the wall-clock figure, also holds the host's launch gaps)
        line["targets_read_on"] = "roofline.frac (HIP events on the launch stream), not value (wall clock)"
        line["other_fracs"] = {k: e["roofline"]["frac"] for k, e in by_key.items()
                               if k not in TARGETS and k not in CEILINGS}
        if "c5" in by_key:   # the transposed layouts against the plain one
            for k in ("m_ta", "m_tb"):
                if k in by_key:
                    line["other_fracs"][k + "_vs_c5"] = round(by_key[k]["roofline"]["achieved"] /
                                                              by_key["c5"]["roofline"]["achieved"], 4)
        ceil = {k: by_key[k]["roofline"]["achieved"] for k in CEILINGS
                if k in by_key}
        if ceil:
            line["measured_ceilings_gbs"] = ceil
        if "c5" in by_key:
            r5, ev = by_key["c5"]["roofline"], by_key["c5"].get("power_limit_evidence") or {}
            line["c5_summary"] = {"frac": r5["frac"], "tflops": r5["achieved"], "avg_launch_us": r5["avg_launch_us"],
                                  "frac_of_mfma_only": r5.get("frac_of_mfma_only"),
                                  "vs_vendor_gemm": r5.get("vs_vendor_gemm"),
                                  "vendor_gemm_tflops": ev.get("vendor_gemm_tflops"),
                                  "this_kernel_alternating_tflops": ev.get("this_kernel_alternating_tflops"),
                                  "board_power_w": ev.get("board_power_w_this_kernel_workload_operands"),
                                  "board_power_cap_w": ev.get("board_power_cap_w")}
        line["targets"] = {k: {"frac": by_key[k]["roofline"]["frac"], "target": t,
                               "met": by_key[k]["roofline"]["frac"] >= t,
                               "parity": by_key[k]["parity"]["passed"],
                               "us": by_key[k]["roofline"]["avg_launch_us"]}
                           for k, t in TARGETS.items() if k in by_key}
        line["min_frac_hbm"] = min(v["frac"] for k, v in line["targets"].items() if k != "c5")
    print(json.dumps(line))


if __name__ == "__main__":
    main()
