"""Pins the rulebook oracle (oracle/ssc_oracle.c) without a GPU:
golden vectors produced by the reference's own compiled CPU code, the compiled
reference itself when it is present, a brute-force statement of the definition,
and structural invariants."""
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "rulebook_cases.npz")


def _cases():
    z = np.load(GOLDEN)
    names = sorted({k.split("/")[0] for k in z.files})
    return z, names


def random_voxels(rng, batch, grid, n):
    cells = np.sort(rng.choice(batch * grid ** 3, size=n, replace=False))
    b, r = cells // grid ** 3, cells % grid ** 3
    return np.stack([b, r // grid ** 2, (r // grid) % grid, r % grid], 1).astype(np.int32)


def brute_force_pairs(idx, grid_out, k, s, p, d):
    """The definition: input voxel i and tap (kx,ky,kz) give output o = (i + p - k*d)/s
    when that is integral and inside the output grid."""
    out = {}
    for row, (b, x, y, z) in enumerate(idx):
        for kx in range(k):
            for ky in range(k):
                for kz in range(k):
                    o = []
                    for c, kk in ((x, kx), (y, ky), (z, kz)):
                        t = c + p - kk * d
                        if t < 0 or t % s or t // s >= grid_out:
                            o = None
                            break
                        o.append(t // s)
                    if o is not None:
                        out.setdefault((kx * k + ky) * k + kz, []).append((row, (b, *o)))
    return out


@pytest.mark.parametrize("name", _cases()[1])
def test_oracle_matches_reference_golden(name, oracle):
    z, _ = _cases()
    batch, grid, k, s, p, d, subm = [int(v) for v in z[name + "/params"]]
    o_idx, pairs, num, _ = oracle.rulebook(z[name + "/indices"], batch, [grid] * 3, k, s, p, d,
                                           bool(subm))
    assert np.array_equal(num, z[name + "/num"])
    assert np.array_equal(o_idx, z[name + "/out_indices"])
    assert np.array_equal(pairs, z[name + "/pairs"])


GOLDEN_T = os.path.join(os.path.dirname(__file__), "golden", "rulebook_transposed_cases.npz")


def _transposed_cases():
    z = np.load(GOLDEN_T)
    return z, sorted({k.split("/")[0] for k in z.files})


@pytest.mark.parametrize("name", _transposed_cases()[1])
def test_oracle_matches_reference_golden_transposed(name, oracle):
    """Transposed rulebooks written by the reference's getIndicePairsDeConv
    (src/conv/geometry.h:190-237; tests/golden/make_rulebook_golden.py)."""
    z, _ = _transposed_cases()
    batch, grid, k, s, p, d, op = [int(v) for v in z[name + "/params"][:7]]
    o_idx, pairs, num, shape = oracle.rulebook(z[name + "/indices"], batch, [grid] * 3, k, s, p, d,
                                               transpose=True, out_padding=op)
    assert shape == [int(v) for v in z[name + "/params"][7:]]
    assert np.array_equal(num, z[name + "/num"])
    assert np.array_equal(o_idx, z[name + "/out_indices"])
    assert np.array_equal(pairs, z[name + "/pairs"])


@pytest.mark.parametrize("grid,k,s,p,d,op", [(5, 3, 2, 1, 1, 0), (5, 3, 2, 1, 1, 1),
                                             (4, 2, 2, 0, 1, 0), (6, 3, 1, 0, 2, 0),
                                             (4, 4, 3, 1, 1, 2)])
def test_transposed_oracle_matches_definition_and_compiled_reference(grid, k, s, p, d, op, oracle):
    """The definition: input voxel i and tap k give output i*s - p + k*d where that lies inside
    (i-1)*s - 2p + k + output_padding cells per axis; pairs in ascending input row.  And the
    adjoint property: every pair (i -> o, k) is a pair (o -> i, k) of the regular rulebook of
    the same window over the reached cells."""
    rng = np.random.default_rng(grid * 10 + k)
    idx = random_voxels(rng, 2, grid, 30)
    o_idx, pairs, num, shape = oracle.rulebook(idx, 2, [grid] * 3, k, s, p, d, transpose=True,
                                               out_padding=op)
    extent = (grid - 1) * s - 2 * p + k + op
    assert shape == [extent] * 3
    want = {}
    for row, (b, x, y, z) in enumerate(idx):
        for kx in range(k):
            for ky in range(k):
                for kz in range(k):
                    o = [c * s - p + kk * d for c, kk in ((x, kx), (y, ky), (z, kz))]
                    if all(0 <= v < extent for v in o):
                        want.setdefault((kx * k + ky) * k + kz, []).append((row, (b, *o)))
    assert int(num.sum()) == sum(len(v) for v in want.values())
    for kk in range(k ** 3):
        got = [(int(i), tuple(int(v) for v in o_idx[o])) for i, o in
               zip(pairs[kk, 0, :num[kk]], pairs[kk, 1, :num[kk]])]
        assert got == want.get(kk, [])
    assert len({tuple(r) for r in o_idx.tolist()}) == o_idx.shape[0]
    if oracle.ref_lib() is not None:
        ref = oracle.ref_rulebook(idx, 2, [grid] * 3, k, s, p, d, transpose=True, out_padding=op)
        for x, y in zip((o_idx, pairs, num), ref[:3]):
            assert np.array_equal(x, y)
    if (extent + 2 * p - d * (k - 1) - 1) // s + 1 >= grid:  # the regular window lands on the grid
        c_idx, c_pairs, c_num = oracle.canonicalize(o_idx, pairs, num, shape)
        r_idx, r_pairs, r_num, r_shape = oracle.rulebook(c_idx, 2, shape, k, s, p, d)
        back = {}
        for kk in range(k ** 3):
            for i, o in zip(r_pairs[kk, 0, :r_num[kk]], r_pairs[kk, 1, :r_num[kk]]):
                back.setdefault(kk, set()).add((tuple(r_idx[o]), tuple(c_idx[i])))
        for kk in range(k ** 3):
            for i, o in zip(c_pairs[kk, 0, :c_num[kk]], c_pairs[kk, 1, :c_num[kk]]):
                assert (tuple(idx[i]), tuple(c_idx[o])) in back.get(kk, set())


def test_known_answer(oracle):
    """indices (0,0,0),(1,2,3),(3,3,3) on a 4^3 grid, k3 s1 p1: 30 outputs, 34 pairs."""
    idx = np.array([[0, 0, 0, 0], [0, 1, 2, 3], [0, 3, 3, 3]], dtype=np.int32)
    o_idx, pairs, num, shape = oracle.rulebook(idx, 1, [4, 4, 4], 3, 1, 1)
    assert shape == [4, 4, 4] and o_idx.shape[0] == 30
    assert num.tolist() == [1, 2, 1, 1, 2, 1, 0, 1, 1, 1, 2, 1, 1, 3, 2, 0, 2, 2, 0, 1, 1, 0, 2,
                            2, 0, 2, 2]
    assert o_idx[:8, 1:].tolist() == [[1, 1, 1], [1, 1, 0], [1, 0, 1], [1, 0, 0], [0, 1, 1],
                                      [0, 1, 0], [0, 0, 1], [0, 0, 0]]
    assert pairs[13, 0, :3].tolist() == [0, 1, 2] and pairs[13, 1, :3].tolist() == [7, 16, 26]


@pytest.mark.parametrize("grid,k,s,p,d,subm", [(8, 3, 1, 1, 1, 0), (9, 3, 2, 1, 1, 0),
                                               (8, 2, 2, 0, 1, 0), (10, 5, 1, 2, 1, 0),
                                               (7, 3, 2, 0, 1, 0), (12, 3, 1, 2, 2, 0),
                                               (8, 3, 1, 1, 1, 1), (6, 4, 2, 1, 1, 0)])
def test_oracle_matches_compiled_reference(grid, k, s, p, d, subm, oracle):
    if oracle.ref_lib() is None:
        pytest.skip("oracle/_ref/libssc_ref.so not built (reference sources absent)")
    rng = np.random.default_rng(grid * 100 + k)
    idx = random_voxels(rng, 2, grid, 80)
    a = oracle.rulebook(idx, 2, [grid] * 3, k, s, p, d, bool(subm))
    b = oracle.ref_rulebook(idx, 2, [grid] * 3, k, s, p, d, bool(subm))
    for x, y in zip(a[:3], b[:3]):
        assert np.array_equal(x, y)


@pytest.mark.parametrize("grid,k,s,p,d", [(6, 3, 1, 1, 1), (7, 3, 2, 1, 1), (6, 2, 2, 0, 1),
                                          (8, 3, 1, 2, 2), (5, 3, 3, 0, 1), (6, 5, 1, 2, 1)])
def test_oracle_matches_brute_force_definition(grid, k, s, p, d, oracle):
    rng = np.random.default_rng(7)
    idx = random_voxels(rng, 2, grid, 40)
    o_idx, pairs, num, shape = oracle.rulebook(idx, 2, [grid] * 3, k, s, p, d)
    want = brute_force_pairs(idx, shape[0], k, s, p, d)
    assert int(num.sum()) == sum(len(v) for v in want.values())
    outs = set()
    for kk in range(k ** 3):
        got = [(int(i), tuple(int(v) for v in o_idx[o])) for i, o in
               zip(pairs[kk, 0, :num[kk]], pairs[kk, 1, :num[kk]])]
        assert got == want.get(kk, [])  # CPU order: ascending input row
        outs.update(o for _, o in got)
    assert outs == {tuple(int(v) for v in r) for r in o_idx}  # exactly the reached cells
    assert len(outs) == o_idx.shape[0]


def test_invariants_stride1(oracle):
    rng = np.random.default_rng(3)
    grid, k = 10, 3
    idx = random_voxels(rng, 2, grid, 120)
    o_idx, pairs, num, _ = oracle.rulebook(idx, 2, [grid] * 3, k, 1, 1)
    # an interior voxel owns all K taps; a boundary voxel loses the clipped ones
    per_voxel = np.zeros(idx.shape[0], dtype=int)
    for kk in range(27):
        rows_in, rows_out = pairs[kk, 0, :num[kk]], pairs[kk, 1, :num[kk]]
        assert len(set(rows_in.tolist())) == num[kk] == len(set(rows_out.tolist()))
        assert np.all(pairs[kk, :, num[kk]:] == -1)
        np.add.at(per_voxel, rows_in, 1)
    expect = np.prod([np.minimum(idx[:, a] + 1, grid - 1) - np.maximum(idx[:, a] - 1, 0) + 1
                      for a in (1, 2, 3)], axis=0)
    assert np.array_equal(per_voxel, expect)
    # outputs = clipped dilation of the inputs
    dil = set()
    for b, x, y, z in idx:
        for dx in (-1, 0, 1):
            for dy in (-1, 0, 1):
                for dz in (-1, 0, 1):
                    c = (x + dx, y + dy, z + dz)
                    if all(0 <= v < grid for v in c):
                        dil.add((b, *c))
    assert dil == {tuple(r) for r in o_idx.tolist()}
    # canonical order: ascending flat key, pairs ascending in input row
    c_idx, c_pairs, c_num = oracle.canonicalize(o_idx, pairs, num, [grid] * 3)
    keys = oracle.flat_key(c_idx, [grid] * 3)
    assert np.all(np.diff(keys) > 0)
    for kk in range(27):
        assert np.all(np.diff(c_pairs[kk, 0, :c_num[kk]]) > 0)
        # inputs sorted by key => outputs of one offset ascending as well
        assert np.all(np.diff(c_pairs[kk, 1, :c_num[kk]]) > 0)


def test_invariants_subm(oracle):
    rng = np.random.default_rng(4)
    idx = random_voxels(rng, 2, 8, 150)
    o_idx, pairs, num, _ = oracle.rulebook(idx, 2, [8] * 3, 3, 1, 0, 1, subm=True)
    assert np.array_equal(o_idx, idx)
    assert np.array_equal(num, num[::-1])  # i sees j through k <=> j sees i through K-1-k
    assert num[13] == idx.shape[0]
    assert np.array_equal(pairs[13, 0, :num[13]], pairs[13, 1, :num[13]])


def test_empty_input(oracle):
    o_idx, pairs, num, _ = oracle.rulebook(np.zeros((0, 4), np.int32), 1, [8] * 3, 3, 1, 1)
    assert o_idx.shape == (0, 4) and pairs.shape == (27, 2, 0) and num.sum() == 0


def test_stride_with_dilation_is_refused(oracle):
    """The reference asserts stride == 1 or dilation == 1 per axis (ss_conv/sp_ops/conv.py:50-51):
    its candidate enumeration (geometry.h:18-80) yields offsets outside the kernel otherwise."""
    idx = np.array([[0, 2, 2, 2]], dtype=np.int32)
    with pytest.raises(ValueError):
        oracle.rulebook(idx, 1, [8] * 3, [1, 1, 3], [3, 1, 1], [2, 0, 1], [2, 1, 1])
    # on different axes both are fine
    o_idx, _, num, _ = oracle.rulebook(idx, 1, [8] * 3, [1, 1, 3], [1, 2, 1], [0, 0, 1], [1, 1, 2])
    assert o_idx.shape[0] == int(num.sum()) == 2  # z + 1 - 2 kz in {3, 1, -1}: two inside


def test_anisotropic_geometries_against_brute_force(oracle):
    """Kernel size, stride, padding and dilation differing per axis on a non-cubic grid: the
    pairs must be exactly those (input, offset) whose output position is integral and inside
    the output grid: out * s = in + p - k * d."""
    rng = np.random.default_rng(12)
    for _ in range(40):
        shape = [int(rng.integers(3, 10)) for _ in range(3)]
        ks = [int(rng.integers(1, 4)) for _ in range(3)]
        st = [int(rng.integers(1, 4)) for _ in range(3)]
        dl = [int(rng.integers(1, 3)) if s == 1 else 1 for s in st]
        pd = [int(rng.integers(0, 3)) for _ in range(3)]
        out_shape = [(n + 2 * p - d * (k - 1) - 1) // s + 1
                     for n, p, d, k, s in zip(shape, pd, dl, ks, st)]
        if min(out_shape) < 1:
            continue
        cells = 2 * shape[0] * shape[1] * shape[2]
        n = int(rng.integers(1, min(cells, 60) + 1))
        flat = np.sort(rng.choice(cells, size=n, replace=False))
        vol = shape[0] * shape[1] * shape[2]
        b, r = flat // vol, flat % vol
        idx = np.stack([b, r // (shape[1] * shape[2]), (r // shape[2]) % shape[1],
                        r % shape[2]], 1).astype(np.int32)
        o_idx, pairs, num, o_shape = oracle.rulebook(idx, 2, shape, ks, st, pd, dl)
        assert list(o_shape) == out_shape
        want = set()
        for i, (bb, x, y, z) in enumerate(idx):
            for kx in range(ks[0]):
                for ky in range(ks[1]):
                    for kz in range(ks[2]):
                        num_ = [x + pd[0] - kx * dl[0], y + pd[1] - ky * dl[1], z + pd[2] - kz * dl[2]]
                        if any(v % s for v, s in zip(num_, st)):
                            continue
                        o = [v // s for v, s in zip(num_, st)]
                        if all(0 <= v < m for v, m in zip(o, out_shape)):
                            want.add((i, (kx * ks[1] + ky) * ks[2] + kz, bb, *o))
        got = set()
        for k in range(len(num)):
            for j in range(int(num[k])):
                i, o = int(pairs[k, 0, j]), int(pairs[k, 1, j])
                got.add((i, k, *[int(v) for v in o_idx[o]]))
        assert got == want, (shape, ks, st, pd, dl)
