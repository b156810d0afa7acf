#!/usr/bin/env python3
"""Writes tests/golden/reference_examples.npz: inputs and expected outputs of
the reference's example graphs, produced by the reference's OWN golden scripts
(examples/*/gen_data.py, gen_inputs.py, seed 42) at reduced, deliberately
ragged sizes so that the fixture stays a few tens of KB.

Run in the authoring container, where the reference tree is mounted:

    python tests/golden/make_fixtures.py [/root/reference]

Each script is executed as a child process with an output directory of its
own; nothing of the reference is copied, only the arrays it writes are kept.
The tests load the .npz with numpy.load(allow_pickle=False).
"""
import os
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

# example dir, script, size arguments, name of the output-dir flag
RUNS = [
    ("broadcast-add-reduce", "gen_data.py", ["--m", "40", "--n", "75"], "--out-dir"),
    ("relu-broadcast-transpose", "gen_inputs.py", ["--m", "70", "--n", "33"], "--out-dir"),
    ("gather-elementwise-fusion", "gen_data.py", ["--m", "16", "--n", "96", "--k", "50"], "--out-dir"),
    ("matmul-add-leakyrelu", "gen_data.py", ["--M", "128", "--K", "64", "--N", "128"], "--out-dir"),
    ("add-broadcast-concat", "gen_inputs.py", ["--M", "24", "--N", "40"], "--outdir"),
    ("split-relu-brc-add-mul", "gen_data.py", ["--M", "32", "--N", "40"], "--outdir"),
    ("real-npu-microcases", "gen_data.py", [], "--out-dir"),
]


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    arrays = {}
    for example, script, size_args, out_flag in RUNS:
        with tempfile.TemporaryDirectory() as tmp:
            subprocess.run([sys.executable, os.path.join(ref, "examples", example, script), *size_args,
                            out_flag, tmp], check=True, stdout=subprocess.DEVNULL)
            for root, _, files in os.walk(tmp):
                for f in sorted(files):
                    if not f.endswith(".npy"):
                        continue
                    rel = os.path.relpath(os.path.join(root, f), tmp)[:-4].replace(os.sep, "/")
                    if example == "real-npu-microcases" and not rel.startswith(("relu_only", "broadcast_add")):
                        continue     # the copy / const cases exercise Ascend data movement only
                    if example == "matmul-add-leakyrelu" and rel in ("input0", "input1", "input2", "output0"):
                        continue     # the same arrays under the names the mix runner wants
                    arrays[f"{example}/{rel}"] = np.load(os.path.join(root, f), allow_pickle=False)
    out = os.path.join(HERE, "reference_examples.npz")
    np.savez_compressed(out, **arrays)
    for k, v in arrays.items():
        print(f"{k:60s} {v.dtype} {v.shape}")
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
