#!/usr/bin/env python3
"""Times the gather family (out = table[idx] * scale + shift, f16) over row lengths and row
counts, with the kernels that separate reads from writes switched on and off
(AFIR_HIP_PHASED, read at every launch), and prints one table line per shape: which kernel each
setting launched, its grid, the average launch time and the algorithmic GB/s (gathered rows +
output + indices + the two vectors).

Every shape is checked once, bit for bit, against the same expression in torch
(float32 arithmetic, one rounding to f16).  The timed launches rotate over eight index vectors
into a table of at least 1 GiB (131072 rows or more), so that a launch finds few of its rows in
the 256 MB last-level cache.

    gather_shapes.py [--steps N]

Needs a GPU."""
import argparse
import importlib.util
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
SHAPES = [(256, 131072), (1024, 32768), (1024, 65536), (4096, 4096), (4096, 8192), (4096, 16384), (4096, 32768),
          (8192, 2048), (8192, 4096), (8192, 5120), (8192, 8192), (8192, 32768)]
MIN_TABLE_ROWS, MIN_TABLE_BYTES = 131072, 1 << 30


def load_package():
    pkg_dir = os.path.dirname(HERE)
    spec = importlib.util.spec_from_file_location("ascend_mlir_amd", os.path.join(pkg_dir, "__init__.py"),
                                                  submodule_search_locations=[pkg_dir])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["ascend_mlir_amd"] = mod
    spec.loader.exec_module(mod)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--steps", type=int, default=200)
    args = ap.parse_args()
    import torch
    load_package()
    from ascend_mlir_amd import hip_kernels as H
    H.load()
    g = torch.Generator(device="cuda").manual_seed(42)
    print("# dim  rows  MiB_gathered | phased: kernel grid us GB/s | unphased: kernel grid us GB/s | ratio", flush=True)
    for dim, nidx in SHAPES:
        TABLE_ROWS = max(MIN_TABLE_ROWS, MIN_TABLE_BYTES // (dim * 2))
        table = (torch.randn(TABLE_ROWS, dim, device="cuda", generator=g) * 0.02).to(torch.float16)
        scale = (torch.rand(dim, device="cuda", generator=g) + 0.5).to(torch.float16)
        shift = (torch.rand(dim, device="cuda", generator=g) * 0.2 - 0.1).to(torch.float16)
        idxs = [torch.randint(0, TABLE_ROWS, (nidx,), device="cuda", generator=g, dtype=torch.int32) for _ in range(8)]
        outs = [torch.empty(nidx, dim, device="cuda", dtype=torch.float16) for _ in range(2)]
        work = 2 * nidx * dim * 2 + nidx * 4 + 2 * dim * 2
        want = (table[idxs[0].long()].float() * scale.float() + shift.float()).to(torch.float16)
        cells = []
        for phased in ("1", "0"):
            os.environ["AFIR_HIP_PHASED"] = phased
            tiling = H.pack_tiling(TABLE_ROWS, dim, nidx)
            ws = torch.zeros(4, dtype=torch.int32, device="cuda")
            calls = [H.prepare("afir_hip_launch_gather_scale_shift",
                               [table.data_ptr(), idxs[i].data_ptr(), scale.data_ptr(), shift.data_ptr(),
                                outs[i % 2].data_ptr(), ws.data_ptr()], tiling) for i in range(8)]
            calls[0]()
            torch.cuda.synchronize()
            note = H.last_launch()
            if not torch.equal(outs[0], want):
                raise SystemExit(f"mismatch at dim {dim} rows {nidx} phased {phased}")
            t_end = time.perf_counter() + 0.05
            while time.perf_counter() < t_end:
                for i in range(8):
                    calls[i]()
                torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(args.steps):
                calls[i % 8]()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / args.steps
            cells.append((note["kernel"], note["workgroups"], us, work / us / 1e3))
        os.environ.pop("AFIR_HIP_PHASED", None)
        (k1, g1, u1, b1), (k0, g0, u0, b0) = cells
        print(f"{dim:5d} {nidx:6d} {nidx * dim * 2 / 2**20:7.0f} | {k1} {g1} {u1:.2f} {b1:.0f} | {k0} {g0} {u0:.2f} {b0:.0f} | {u0 / u1:.3f}",
              flush=True)
        del table, idxs, outs, want


if __name__ == "__main__":
    main()
