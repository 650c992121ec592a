"""Writes tests/golden/rulebook_cases.npz and rulebook_transposed_cases.npz from the
REFERENCE's own CPU rulebook (src/conv/geometry.h:140-189, 190-237, 241-288), compiled where
it lies by oracle/Makefile into oracle/_ref/libssc_ref.so.  Run once in a container that has
/root/reference; the .npz files (inputs and expected outputs only) are committed.

    python tests/golden/make_rulebook_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(HERE)), "oracle"))
import oracle as O  # noqa: E402

CASES = [
    # name, batch, grid, n_voxels, kernel, stride, padding, dilation, subm, seed
    ("k3s1p1", 2, 8, 60, 3, 1, 1, 1, False, 1),
    ("k3s2p1", 2, 9, 80, 3, 2, 1, 1, False, 2),
    ("k2s2p0", 3, 8, 70, 2, 2, 0, 1, False, 3),
    ("k5s1p2", 1, 10, 90, 5, 1, 2, 1, False, 4),
    ("k3s2p0", 2, 7, 50, 3, 2, 0, 1, False, 5),
    ("k3s3p1", 2, 8, 50, 3, 3, 1, 1, False, 6),
    ("k3s1p2d2", 2, 12, 120, 3, 1, 2, 2, False, 7),
    ("subm_k3", 2, 8, 100, 3, 1, 1, 1, True, 8),
    ("subm_k5", 2, 10, 150, 5, 1, 2, 1, True, 9),
    ("unsorted_rows", 2, 8, 60, 3, 1, 1, 1, False, 10),
]


TRANSPOSED_CASES = [
    # name, batch, grid, n_voxels, kernel, stride, padding, dilation, output_padding, seed
    ("t_k3s2p1", 2, 5, 40, 3, 2, 1, 1, 0, 21),
    ("t_k3s2p1o1", 2, 5, 40, 3, 2, 1, 1, 1, 22),
    ("t_k2s2p0", 3, 4, 30, 2, 2, 0, 1, 0, 23),
    ("t_k3s1p1", 2, 8, 60, 3, 1, 1, 1, 0, 24),
    ("t_k3s1p0d2", 2, 7, 50, 3, 1, 0, 2, 0, 25),
    ("t_k4s3p1", 1, 4, 20, 4, 3, 1, 1, 0, 26),
    ("t_k5s1p2", 1, 6, 40, 5, 1, 2, 1, 0, 27),
]


def voxels(rng, batch, grid, n, shuffle):
    cells = rng.choice(batch * grid ** 3, size=n, replace=False)
    if not shuffle:
        cells.sort()
    b, r = cells // grid ** 3, cells % grid ** 3
    return np.stack([b, r // grid ** 2, (r // grid) % grid, r % grid], 1).astype(np.int32)


def main():
    assert O.ref_lib() is not None, "build oracle/_ref first: make -C oracle ref"
    out = {}
    for name, batch, grid, n, k, s, p, d, subm, seed in CASES:
        rng = np.random.default_rng(seed)
        idx = voxels(rng, batch, grid, n, shuffle=(name == "unsorted_rows"))
        o_idx, pairs, num, o_shape = O.ref_rulebook(idx, batch, [grid] * 3, k, s, p, d, subm)
        out[name + "/params"] = np.array([batch, grid, k, s, p, d, int(subm)], dtype=np.int32)
        out[name + "/indices"] = idx
        out[name + "/out_indices"] = o_idx
        out[name + "/pairs"] = pairs
        out[name + "/num"] = num
    # The known answer recorded when the reference code was first compiled:
    idx = np.array([[0, 0, 0, 0], [0, 1, 2, 3], [0, 3, 3, 3]], dtype=np.int32)
    o_idx, pairs, num, _ = O.ref_rulebook(idx, 1, [4, 4, 4], 3, 1, 1)
    assert o_idx.shape[0] == 30
    out["known/params"] = np.array([1, 4, 3, 1, 1, 1, 0], dtype=np.int32)
    out["known/indices"] = idx
    out["known/out_indices"] = o_idx
    out["known/pairs"] = pairs
    out["known/num"] = num
    np.savez_compressed(os.path.join(HERE, "rulebook_cases.npz"), **out)
    print("wrote", len(out) // 5, "cases")
    out = {}
    for name, batch, grid, n, k, s, p, d, op, seed in TRANSPOSED_CASES:
        rng = np.random.default_rng(seed)
        idx = voxels(rng, batch, grid, n, shuffle=False)
        o_idx, pairs, num, o_shape = O.ref_rulebook(idx, batch, [grid] * 3, k, s, p, d,
                                                    transpose=True, out_padding=op)
        out[name + "/params"] = np.array([batch, grid, k, s, p, d, op] + list(o_shape),
                                         dtype=np.int32)
        out[name + "/indices"] = idx
        out[name + "/out_indices"] = o_idx
        out[name + "/pairs"] = pairs
        out[name + "/num"] = num
    np.savez_compressed(os.path.join(HERE, "rulebook_transposed_cases.npz"), **out)
    print("wrote", len(out) // 5, "transposed cases")


if __name__ == "__main__":
    main()
