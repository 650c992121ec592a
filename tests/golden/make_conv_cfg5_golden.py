"""Writes tests/golden/conv_cfg5_rows.npz: the fifth benchmark configuration's convolution
(8 clouds x 16384 points at 128^3, 200 -> 200 channels, 5^3 offsets) as the CPU oracle
computes it -- the restatement of the reference's per-offset gather -> GEMM -> scatter-add
(src/conv/indice_conv.h:296-338) takes minutes at this size, so it runs here, once, and the
GPU test compares against what it wrote: 2048 sampled output rows and the column sums of
the whole output.

Inputs are seeded numpy draws (the same on every machine); the test regenerates them.

Run from the repository root:  python tests/golden/make_conv_cfg5_golden.py
"""
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
for p in (os.path.join(ROOT, "ss-conv_amd"), os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)

import oracle as O  # noqa: E402
import synth  # noqa: E402

SAMPLE_ROWS = 2048


def cfg5_inputs():
    """Voxels, features and filters of the layer: clouds of seed 1, numbers of seed 9."""
    cfg = synth.CONFIGS["cfg5"]
    pts, _, ids = synth.config_clouds("cfg5", seed=1)
    idx = synth.voxel_indices(pts, ids, cfg["grid"])
    c = sum(cfg["mult_in"] * (2 * l + 1) for l in range(cfg["lmax"] + 1))
    K = cfg["kernel"] ** 3
    rng = np.random.default_rng(9)
    f = rng.standard_normal((idx.shape[0], c), dtype=np.float32)
    w = (rng.standard_normal((K, c, c), dtype=np.float32) / np.float32((K * c) ** 0.5))
    return cfg, idx, f, w


def main():
    cfg, idx, f, w = cfg5_inputs()
    grid = cfg["grid"]
    t0 = time.time()
    o_idx, pairs, num = O.canonicalize(*O.rulebook(idx, cfg["batch"], [grid] * 3, cfg["kernel"],
                                                   cfg["stride"], cfg["padding"]))
    n_out = o_idx.shape[0]
    print("rulebook: %d -> %d rows, %d pairs, %.1f s" % (idx.shape[0], n_out, int(num.sum()),
                                                        time.time() - t0), flush=True)
    t0 = time.time()
    out = O.conv_fwd(f, w, pairs, num, n_out, matmul=np.matmul)
    print("conv_fwd: %.1f s" % (time.time() - t0), flush=True)
    rows = np.sort(np.random.default_rng(10).choice(n_out, size=SAMPLE_ROWS, replace=False))
    np.savez(os.path.join(ROOT, "tests", "golden", "conv_cfg5_rows.npz"),
             n_in=np.int64(idx.shape[0]), n_out=np.int64(n_out), pairs=np.int64(num.sum()),
             rows=rows.astype(np.int32), out_rows=out[rows].astype(np.float32),
             out_row_keys=o_idx[rows].astype(np.int32),
             col_sums=out.astype(np.float64).sum(0),
             sq_sum=np.float64((out.astype(np.float64) ** 2).sum()))


if __name__ == "__main__":
    main()
