#!/usr/bin/env python3
"""Tile search for one of the hand-tuned kernel families at its benchmark shape,
the way the reference's examples drive its autotuner (examples/*/tiling_space.json
+ tools/autotuner): seeded inputs and the expected output (numpy, float32
arithmetic and one rounding to the storage type, as the reference's gen_data.py
scripts compute their goldens) are written as .npy files, then bin/autotuner
builds the kernel library once per combination of the build_<MACRO> parameters
in the family's tiling_space.json, launches and validates every candidate and
scores it by kernel time.

    autotune_family.py eltwise|rowsum|transpose-family|gather|matmul [--out DIR] [--repeats N] [--space FILE]

Needs a GPU and hipcc.  Prints the autotuner's candidate table; best_config.json
is left in DIR."""
import argparse
import os
import subprocess
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
# copies of the tensors the timed launches rotate over: at least 1 GiB of inputs read between two
# launches on the same copy, so that the 256 MB last-level cache serves none of the reads
BUFFER_SETS = {"eltwise": 8, "rowsum": 8, "transpose-family": 16, "gather": 16, "matmul": 2}


def bf16_bits(x):
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_to_f32(b):
    return (b.astype(np.uint32) << 16).view(np.float32)


def save_bf16(path, bits):
    np.save(path, np.ascontiguousarray(bits).view("V2"))     # bf16 travels as 2-byte void, like the reference's NpyIO


def generate(family, out):
    rng = np.random.default_rng(42)
    p = lambda name: os.path.join(out, name + ".npy")
    if family == "eltwise":
        a = rng.uniform(-1, 1, (4096, 4096)).astype(np.float32)
        b = rng.uniform(-1, 1, (4096, 4096)).astype(np.float32)
        np.save(p("a"), a); np.save(p("b"), b); np.save(p("expected"), (a + b) * b)
        return ["a", "b"], "0", "0"
    if family == "rowsum":
        x = rng.standard_normal((8192, 4096), dtype=np.float32)
        bias = rng.uniform(-1, 1, (4096,)).astype(np.float32)
        np.save(p("x"), x); np.save(p("bias"), bias)
        np.save(p("expected"), (x + bias[None, :]).sum(axis=1, dtype=np.float32))
        return ["x", "bias"], "2e-3", "1e-5"       # a float32 sum in another order
    if family == "transpose-family":
        x = rng.standard_normal((64, 1024, 512), dtype=np.float32).astype(np.float16)
        c = rng.uniform(-0.5, 0.5, (512,)).astype(np.float32).astype(np.float16)
        e = (np.maximum(x.astype(np.float32), 0) + c.astype(np.float32)[None, None, :]).astype(np.float16)
        np.save(p("x"), x); np.save(p("c"), c); np.save(p("expected"), np.ascontiguousarray(e.transpose(0, 2, 1)))
        return ["x", "c"], "0", "0"
    if family == "gather":
        table = (rng.standard_normal((131072, 1024), dtype=np.float32) * np.float32(0.02)).astype(np.float16)
        idx = rng.integers(0, 131072, 32768, dtype=np.int64).astype(np.int32)
        scale = rng.uniform(0.5, 1.5, (1024,)).astype(np.float32).astype(np.float16)
        shift = rng.uniform(-0.1, 0.1, (1024,)).astype(np.float32).astype(np.float16)
        e = (table[idx].astype(np.float32) * scale.astype(np.float32) + shift.astype(np.float32)).astype(np.float16)
        for n, v in (("table", table), ("idx", idx), ("scale", scale), ("shift", shift), ("expected", e)):
            np.save(p(n), v)
        return ["table", "idx", "scale", "shift"], "0", "0"
    if family == "matmul":
        k = 8192
        a = bf16_bits(rng.standard_normal((8192, k), dtype=np.float32) / np.float32(np.sqrt(k)))
        b = bf16_bits(rng.standard_normal((k, 8192), dtype=np.float32) / np.float32(np.sqrt(k)))
        bias = bf16_bits(rng.uniform(-0.1, 0.1, (8192,)).astype(np.float32))
        v = bf16_to_f32(a) @ bf16_to_f32(b) + bf16_to_f32(bias)[None, :]
        e = bf16_bits(np.maximum(v, v * np.float32(0.01)))
        for n, bits in (("a", a), ("b", b), ("bias", bias), ("expected", e)):
            save_bf16(p(n), bits)
        return ["a", "b", "bias"], "1e-5", "1e-2"
    raise SystemExit(f"unknown family {family}")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("family", choices=["eltwise", "rowsum", "transpose-family", "gather", "matmul"])
    ap.add_argument("--out", default=None)
    ap.add_argument("--repeats", default="200")
    ap.add_argument("--space", default="tiling_space.json",
                    help="file in the family's directory (tiling_space_unphased.json: the eltwise / gather / "
                         "transpose kernels that do not separate reads from writes)")
    args = ap.parse_args()
    out = args.out or f"/tmp/autotune-{args.family}"
    os.makedirs(out, exist_ok=True)
    inputs, atol, rtol = generate(args.family, out)
    here = os.path.join(HERE, "autotune-" + args.family)
    cmd = [os.path.join(HERE, "..", "bin", "autotuner"), "--space", os.path.join(here, args.space),
           "--kernel", os.path.join(here, "kernel.region"),
           "--inputs", ",".join(os.path.join(out, n + ".npy") for n in inputs),
           "--expected", os.path.join(out, "expected.npy"), "--atol", atol, "--rtol", rtol,
           "--repeats", args.repeats, "--buffer-sets", str(BUFFER_SETS[args.family]), "--ramp-ms", "100",
           "--build-dir", os.path.join(out, "artifacts"),
           "--shape", "S=1", "--output", os.path.join(out, "best_config.json")]
    print("+", " ".join(cmd), flush=True)
    sys.exit(subprocess.run(cmd).returncode)


if __name__ == "__main__":
    main()
