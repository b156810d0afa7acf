#!/bin/bash
# Tile search for a fused region with a transposed operand, the way the
# reference's examples drive its autotuner (examples/*/tiling_space.json +
# tools/autotuner): out[b, j, i] = f16(relu(x[b, i, j]) + c[j]) on
# x f16 [64, 1024, 512].  Searched: the LDS tile of the emitted kernel
# (emit_tile_p x emit_tile_q) and the grid size (block_dim_values); every
# candidate is compiled, launched and validated bit-exactly, the score is its
# kernel time in ns.
#   usage: run.sh [output dir]      (needs a GPU and hipcc)
set -e
HERE="$(cd "$(dirname "$0")" && pwd)"
OUT="${1:-/tmp/autotune-transpose}"
mkdir -p "$OUT"
python3 - "$OUT" <<'PY'
import sys
import numpy as np
out = sys.argv[1]
rng = np.random.default_rng(42)
x = rng.standard_normal((64, 1024, 512), dtype=np.float32).astype(np.float16)
c = rng.uniform(-0.5, 0.5, (512,)).astype(np.float32).astype(np.float16)
e = (np.maximum(x.astype(np.float32), 0) + c.astype(np.float32)[None, None, :]).astype(np.float16)
np.save(out + "/x.npy", x)
np.save(out + "/c.npy", c)
np.save(out + "/expected.npy", np.ascontiguousarray(e.transpose(0, 2, 1)))
PY
"$HERE/../../bin/autotuner" --space "$HERE/tiling_space.json" --kernel "$HERE/kernel.region" \
  --inputs "$OUT/x.npy,$OUT/c.npy" --expected "$OUT/expected.npy" --shape B=64 --atol 0 --rtol 0 \
  --repeats 200 --buffer-sets 16 --ramp-ms 100 --build-dir "$OUT/artifacts" --output "$OUT/best_config.json"
