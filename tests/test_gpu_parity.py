"""GPU parity: every native entry point against the CPU oracle on seeded inputs.

Bars: rulebooks, voxel indices and every other integer result bit-exact;
fp32 results within rel-L2 1e-5 (conv, which re-associates sums on MFMA) or
bit-exact where the kernel keeps the oracle's operation order (pools, voxel
means, interpolation)."""
import numpy as np
import pytest
import torch

import synth

pytestmark = pytest.mark.gpu

REL_L2 = 1e-5


def rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    den = np.linalg.norm(b)
    return np.linalg.norm(a - b) / (den if den > 0 else 1.0)


def random_voxels(rng, batch, grid, n):
    cells = rng.choice(batch * grid ** 3, size=n, replace=False)
    cells.sort()
    b, r = cells // grid ** 3, cells % grid ** 3
    return np.stack([b, r // grid ** 2, (r // grid) % grid, r % grid], 1).astype(np.int32)


def gpu_rulebook(idx, batch, grid, k, s, p, d=1, subm=False, device="cuda"):
    from ss_conv.sp_ops.ops import get_indice_pairs
    t = torch.from_numpy(idx).to(device)
    out, pairs, num = get_indice_pairs(t, batch, [grid] * 3, k, s, p, d, 0, subm)
    torch.cuda.synchronize()
    return out.cpu().numpy(), pairs.cpu().numpy(), num.cpu().numpy()


RULEBOOK_CASES = [
    # batch, grid, n, k, stride, pad, dil, subm
    (2, 8, 60, 3, 1, 1, 1, False),
    (2, 9, 80, 3, 2, 1, 1, False),
    (3, 8, 70, 2, 2, 0, 1, False),
    (1, 10, 90, 5, 1, 2, 1, False),
    (2, 8, 100, 3, 1, 1, 1, True),
    (2, 7, 50, 3, 2, 0, 1, False),
    (2, 8, 50, 3, 3, 1, 1, False),
    (2, 12, 200, 3, 1, 2, 2, False),
    (4, 16, 1500, 3, 1, 1, 1, False),
    (2, 8, 1, 3, 1, 1, 1, False),
    (1, 4, 64, 3, 1, 1, 1, False),   # full grid
    (2, 16, 300, 5, 1, 2, 1, True),
]


@pytest.mark.parametrize("case", RULEBOOK_CASES)
def test_rulebook_matches_oracle(case, oracle, device):
    batch, grid, n, k, s, p, d, subm = case
    rng = np.random.default_rng(hash(case) % 2 ** 31)
    idx = random_voxels(rng, batch, grid, n)
    print("case", case, flush=True)
    o_idx, o_pairs, o_num, o_shape = oracle.rulebook(idx, batch, [grid] * 3, k, s, p, d, subm)
    if not subm:
        o_idx, o_pairs, o_num = oracle.canonicalize(o_idx, o_pairs, o_num, o_shape)
    g_idx, g_pairs, g_num = gpu_rulebook(idx, batch, grid, k, s, p, d, subm)
    assert np.array_equal(g_num, o_num)
    assert np.array_equal(g_idx, o_idx)
    assert np.array_equal(g_pairs, o_pairs)


TRANSPOSED_CASES = [
    # batch, grid, n, k, stride, pad, dil, output_padding
    (2, 5, 40, 3, 2, 1, 1, 0),
    (2, 5, 40, 3, 2, 1, 1, 1),
    (3, 4, 30, 2, 2, 0, 1, 0),
    (2, 8, 60, 3, 1, 1, 1, 0),
    (2, 7, 50, 3, 1, 0, 2, 0),
    (1, 4, 20, 4, 3, 1, 1, 0),
    (2, 16, 1200, 3, 2, 1, 1, 1),
    (1, 6, 216, 3, 2, 0, 1, 0),   # full grid
]


@pytest.mark.parametrize("case", TRANSPOSED_CASES)
def test_transposed_rulebook_matches_oracle(case, oracle, device):
    """transpose=True (src/conv/geometry.h:82-138, 190-237): bit-exact against the oracle in
    canonical order, and against the golden rulebooks of the reference's own code where the
    case is one of them."""
    from ss_conv.sp_ops.ops import get_indice_pairs
    batch, grid, n, k, s, p, d, op = case
    rng = np.random.default_rng(hash(case) % 2 ** 31)
    idx = random_voxels(rng, batch, grid, n)
    print("case", case, flush=True)
    o_idx, o_pairs, o_num, o_shape = oracle.rulebook(idx, batch, [grid] * 3, k, s, p, d,
                                                     transpose=True, out_padding=op)
    o_idx, o_pairs, o_num = oracle.canonicalize(o_idx, o_pairs, o_num, o_shape)
    g_idx, g_pairs, g_num = get_indice_pairs(torch.from_numpy(idx).to(device), batch, [grid] * 3,
                                             k, s, p, d, op, False, True)
    assert np.array_equal(g_num.cpu().numpy(), o_num)
    assert np.array_equal(g_idx.cpu().numpy(), o_idx)
    assert np.array_equal(g_pairs.cpu().numpy(), o_pairs)


def test_transposed_rulebook_matches_reference_golden(oracle, device):
    import os
    from ss_conv.sp_ops.ops import get_indice_pairs
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "rulebook_transposed_cases.npz"))
    for name in sorted({k.split("/")[0] for k in z.files}):
        batch, grid, k, s, p, d, op = [int(v) for v in z[name + "/params"][:7]]
        shape = [int(v) for v in z[name + "/params"][7:]]
        want = oracle.canonicalize(z[name + "/out_indices"], z[name + "/pairs"], z[name + "/num"],
                                   shape)
        got = get_indice_pairs(torch.from_numpy(z[name + "/indices"]).to(device), batch,
                               [grid] * 3, k, s, p, d, op, False, True)
        for g, w in zip(got, want):
            assert np.array_equal(g.cpu().numpy(), w), name


def test_transposed_convolution_layer(oracle, device):
    """SparseConvolution(transposed=True), forward and both gradients, against the oracle's
    convolution over the oracle's transposed rulebook, and against torch's dense
    conv_transpose3d of the same layer (an independent statement: the reference's
    transposed convolution reaches out = in*s - p + k, torch's the same cells)."""
    from ss_conv.sp_ops.conv import SparseConvolution
    from ss_conv.sp_ops.tensor import SparseTensor
    rng = np.random.default_rng(77)
    batch, grid, n, cin, cout, k, s, p, op = 2, 6, 70, 5, 7, 3, 2, 1, 1
    idx = random_voxels(rng, batch, grid, n)
    x = rng.normal(size=(n, cin)).astype(np.float32)
    layer = SparseConvolution(3, cin, cout, k, stride=s, padding=p, output_padding=op, bias=False,
                              transposed=True).to(device)
    w = layer.weight.detach().cpu().numpy().reshape(k ** 3, cin, cout)
    feats = torch.from_numpy(x).to(device).requires_grad_(True)
    out = layer(SparseTensor(feats, torch.from_numpy(idx).to(device), [grid] * 3, batch))
    o_idx, o_pairs, o_num, o_shape = oracle.rulebook(idx, batch, [grid] * 3, k, s, p, 1,
                                                     transpose=True, out_padding=op)
    o_idx, o_pairs, o_num = oracle.canonicalize(o_idx, o_pairs, o_num, o_shape)
    assert list(out.spatial_shape) == o_shape == [(grid - 1) * s - 2 * p + k + op] * 3
    assert np.array_equal(out.indices.cpu().numpy(), o_idx)
    ref = oracle.conv_fwd(x, w, o_pairs, o_num, o_idx.shape[0])
    assert rel_l2(out.features.detach().cpu().numpy(), ref) < REL_L2
    # dense statement: torch's transposed convolution wants [Cin, Cout, kx, ky, kz]
    dense_in = torch.zeros((batch, cin, grid, grid, grid), dtype=torch.float64)
    dense_in[idx[:, 0], :, idx[:, 1], idx[:, 2], idx[:, 3]] = torch.from_numpy(x).double()
    wd = torch.from_numpy(w).double().reshape(k, k, k, cin, cout).permute(3, 4, 0, 1, 2)
    dense = torch.nn.functional.conv_transpose3d(dense_in, wd, stride=s, padding=p,
                                                 output_padding=op)
    got = dense[o_idx[:, 0], :, o_idx[:, 1], o_idx[:, 2], o_idx[:, 3]].numpy()
    assert rel_l2(out.features.detach().cpu().numpy(), got) < REL_L2
    mask = torch.ones(dense.shape[0], dense.shape[2], dense.shape[3], dense.shape[4], dtype=torch.bool)
    mask[o_idx[:, 0], o_idx[:, 1], o_idx[:, 2], o_idx[:, 3]] = False
    assert float(dense.permute(0, 2, 3, 4, 1)[mask].abs().max()) == 0.0  # nothing outside the active rows
    # gradients through the same pairs
    g_out = rng.normal(size=ref.shape).astype(np.float32)
    out.features.backward(torch.from_numpy(g_out).to(device))
    d_in, d_w = oracle.conv_bwd(x, w, g_out, o_pairs, o_num)
    assert rel_l2(feats.grad.cpu().numpy(), d_in) < REL_L2
    assert rel_l2(layer.weight.grad.cpu().numpy().reshape(k ** 3, cin, cout), d_w) < REL_L2


@pytest.mark.parametrize("case", [RULEBOOK_CASES[1], RULEBOOK_CASES[4], RULEBOOK_CASES[8]])
@pytest.mark.parametrize("shuffle", [False, True])
def test_rulebook_count_then_emit_entry_points(case, shuffle, device):
    """The library offers the rulebook in two ways: ssc_rulebook_count(_ordered) followed
    by ssc_rulebook_emit (the host waits for the number of outputs before anything else is
    queued), and ssc_rulebook_begin / ssc_rulebook_finish / ssc_rulebook_rows (the pair
    lists are queued before the wait; the one the Python side calls).  Both give the same
    tensors and the same order flag."""
    import ctypes
    from ss_conv import _ext
    batch, grid, n, k, s, p, d, subm = case
    rng = np.random.default_rng(11)
    idx = random_voxels(rng, batch, grid, n)
    if shuffle:
        idx = idx[rng.permutation(idx.shape[0])]
    print("case", case, shuffle, flush=True)
    t = torch.from_numpy(idx).to(device)
    out_shape = [grid] * 3 if subm else [(grid + 2 * p - d * (k - 1) - 1) // s + 1] * 3
    want = _ext.get_indice_pairs_3d(t, batch, out_shape, [grid] * 3, [k] * 3, [s] * 3, [p] * 3,
                                    [d] * 3, [0] * 3, int(subm), 0)
    g = _ext._geometry(batch, out_shape, [k] * 3, [s] * 3, [p] * 3, [d] * 3, subm, 0)
    lib = _ext._lib
    nbytes = lib.ssc_rulebook_workspace_bytes(ctypes.byref(g), n)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
    n_out, in_order = ctypes.c_int32(0), ctypes.c_int32(-1)
    assert lib.ssc_rulebook_count_ordered(t.data_ptr(), n, ctypes.byref(g), ws.data_ptr(), nbytes,
                                          ctypes.byref(n_out), ctypes.byref(in_order), None) == 0
    assert n_out.value == want[0].shape[0]
    assert bool(in_order.value) == _ext.rulebook_meta(want[1]).canonical[0] == (not shuffle)
    K = k ** 3
    out = torch.full((max(n_out.value, 1), 4), -7, dtype=torch.int32, device=device)
    pairs = torch.full((K, 2, n), -7, dtype=torch.int32, device=device)
    num = torch.full((K,), -7, dtype=torch.int32, device=device)
    assert lib.ssc_rulebook_emit(t.data_ptr(), n, ctypes.byref(g), ws.data_ptr(), nbytes,
                                 None if subm else out.data_ptr(), pairs.data_ptr(),
                                 num.data_ptr(), None) == 0
    torch.cuda.synchronize()
    if not subm:
        assert torch.equal(out[:n_out.value], want[0])
    assert torch.equal(pairs, want[1]) and torch.equal(num, want[2])


def test_rulebook_clean_table_contract(oracle, device):
    """ssc_rulebook_begin with a table the caller keeps between calls: it must be all zero
    again when the call's kernels are done, whatever geometries share it, and the rulebook
    must be the one the call without it builds (and the oracle's)."""
    import ctypes
    from ss_conv import _ext
    lib = _ext._lib
    rng = np.random.default_rng(21)
    table = None
    for batch, grid, n, k, p in ((2, 32, 3000, 3, 1), (1, 64, 9000, 5, 2), (3, 32, 500, 3, 1),
                                 (2, 32, 4000, 3, 0)):
        idx = random_voxels(rng, batch, grid, n)
        t = torch.from_numpy(idx).to(device)
        os_ = grid + 2 * p - (k - 1)
        g = _ext._geometry(batch, [os_] * 3, [k] * 3, [1] * 3, [p] * 3, [1] * 3, 0, 0)
        gref = ctypes.byref(g)
        need = lib.ssc_rulebook_clean_table_bytes(gref, n)
        if os_ % 32 == 0:
            assert need > 0
        if table is None or table.numel() < need:
            table = torch.zeros(max(need, 1), dtype=torch.uint8, device=device)
        K = k ** 3
        results = []
        for with_table in (True, False, True):
            nbytes = lib.ssc_rulebook_workspace_bytes(gref, n)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
            pairs = torch.full((K, 2, n), -7, dtype=torch.int32, device=device)
            num = torch.full((K,), -7, dtype=torch.int32, device=device)
            n_out, in_order = ctypes.c_int32(0), ctypes.c_int32(-1)
            assert lib.ssc_rulebook_begin(t.data_ptr(), n, gref, ws.data_ptr(), nbytes,
                                          pairs.data_ptr(), num.data_ptr(), None, 0,
                                          table.data_ptr() if with_table and need else None,
                                          table.numel() if with_table and need else 0, None) == 0
            assert lib.ssc_rulebook_finish(gref, n, ctypes.byref(n_out), ctypes.byref(in_order)) == 0
            out = torch.empty((max(n_out.value, 1), 4), dtype=torch.int32, device=device)
            assert lib.ssc_rulebook_rows(gref, n, ws.data_ptr(), nbytes, out.data_ptr(), None) == 0
            torch.cuda.synchronize()
            assert int(table.count_nonzero().item()) == 0, (batch, grid, n, k, p)
            assert in_order.value == 1
            results.append((out[:n_out.value].cpu().numpy(), pairs.cpu().numpy(), num.cpu().numpy()))
        want = oracle.canonicalize(*oracle.rulebook(idx, batch, [grid] * 3, k, 1, p))
        for got in results:
            for a, b in zip(got, want):
                assert np.array_equal(a, b)


def test_rulebook_few_voxels_in_a_large_grid(oracle, device):
    """300 voxels in 40 x 128^3 cells: the table has 2.6 M words, the input five chunks.
    (The blocks that decode the table into output rows ride on the grid of the kernel that
    writes the pairs, which is sized by the input: here they must stride over the table.)"""
    rng = np.random.default_rng(3)
    cells = np.unique(rng.integers(0, 40 * 128 ** 3, size=300))
    b, r = cells // 128 ** 3, cells % 128 ** 3
    idx = np.stack([b, r // 128 ** 2, (r // 128) % 128, r % 128], 1).astype(np.int32)
    o = oracle.canonicalize(*oracle.rulebook(idx, 40, [128] * 3, 3, 1, 1))
    g = gpu_rulebook(idx, 40, 128, 3, 1, 1)
    for a, b in zip(g, o):
        assert np.array_equal(a, b)


def test_rulebook_unsorted_input_rows(oracle, device):
    """Input rows in arbitrary order: outputs still ascending by key, pairs ascending in input row."""
    rng = np.random.default_rng(5)
    idx = random_voxels(rng, 2, 10, 150)
    idx = idx[rng.permutation(idx.shape[0])]
    o = oracle.canonicalize(*oracle.rulebook(idx, 2, [10] * 3, 3, 1, 1))
    g = gpu_rulebook(idx, 2, 10, 3, 1, 1)
    for a, b in zip(g, o):
        assert np.array_equal(a, b)


def test_rulebook_empty_and_errors(device):
    from ss_conv import _ext
    empty = torch.zeros((0, 4), dtype=torch.int32, device=device)
    out, pairs, num = _ext.get_indice_pairs_3d(empty, 1, [8] * 3, [8] * 3, [3] * 3, [1] * 3, [1] * 3,
                                               [1] * 3, [0] * 3, 0, 0)
    assert out.shape == (0, 4) and pairs.shape == (27, 2, 0) and int(num.sum()) == 0
    one = torch.zeros((1, 4), dtype=torch.int32, device=device)
    with pytest.raises(RuntimeError):  # kernel volume 343 > 256 (reference: indice_conv.h:44)
        _ext.get_indice_pairs_3d(one, 1, [8] * 3, [8] * 3, [7] * 3, [1] * 3, [3] * 3, [1] * 3,
                                 [0] * 3, 0, 0)
    with pytest.raises(RuntimeError):  # wrong list length (reference: indice_conv.h:33-39)
        _ext.get_indice_pairs_3d(one, 1, [8] * 3, [8] * 3, [3] * 2, [1] * 3, [1] * 3, [1] * 3,
                                 [0] * 3, 0, 0)


def test_rulebook_without_any_output(oracle, device):
    """A stride can step over every candidate of a voxel: no active output at all.  The
    rulebook is empty, and convolution, pooling and their gradients on it return empty or
    zero tensors (the reference allocates zero-row tensors, indice_conv.h:49-56,278)."""
    from ss_conv import _ext
    idx = np.array([[0, 1, 0, 0], [1, 4, 2, 1]], dtype=np.int32)
    geo = dict(batch=2, shape=[13, 4, 4], ks=[2, 2, 2], st=[3, 3, 2], pd=[1, 2, 1])
    o_idx, o_pairs, o_num, _ = oracle.rulebook(idx, geo["batch"], geo["shape"], geo["ks"],
                                               geo["st"], geo["pd"])
    assert o_idx.shape[0] == 0 and int(o_num.sum()) == 0
    t = torch.from_numpy(idx).to(device)
    from ss_conv.sp_ops.ops import get_indice_pairs
    out, pairs, num = get_indice_pairs(t, geo["batch"], geo["shape"], geo["ks"], geo["st"],
                                       geo["pd"], 1, 0, False)
    assert out.shape == (0, 4) and int(num.sum()) == 0 and bool((pairs == -1).all())
    f = torch.randn((2, 8), device=device)
    w = torch.randn((2, 2, 2, 8, 12), device=device)
    y = _ext.indice_conv_fp32(f, w, pairs, num, 0, 0, 0)
    assert y.shape == (0, 12)
    d_in, d_w = _ext.indice_conv_backward_fp32(f, w, y, pairs, num, 0, 0)
    assert d_in.shape == f.shape and not d_in.any() and d_w.shape == w.shape and not d_w.any()
    assert _ext.indice_maxpool_fp32(f, pairs, num, 0).shape == (0, 8)
    rf = _ext.indiceSummaryRF(pairs, num, 0)
    assert rf.shape == (0,)
    assert _ext.indice_avgpool_fp32(f, pairs, num, 0, rf).shape == (0, 8)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_anisotropic_geometries_match_oracle(seed, oracle, device):
    """Kernel size, stride, padding and dilation differing per axis, non-cubic grids, inputs
    in key order or shuffled, regular and submanifold: rulebook bit-exact, convolution
    (forward, both gradients) and both pools against the oracle, 40 seeded cases a seed."""
    from ss_conv import _ext
    from ss_conv.sp_ops.ops import get_indice_pairs
    rng = np.random.default_rng(seed)
    done = 0
    while done < 40:
        batch = int(rng.integers(1, 4))
        shape = [int(rng.integers(3, 14)) for _ in range(3)]
        ks = [int(rng.integers(1, 4)) for _ in range(3)]
        st = [int(rng.integers(1, 4)) for _ in range(3)]
        dl = [int(rng.integers(1, 3)) if t == 1 else 1 for t in st]
        pd = [int(rng.integers(0, 3)) for _ in range(3)]
        subm = bool(rng.integers(0, 4) == 0)
        if subm:
            ks, st = [k | 1 for k in ks], [1, 1, 1]
        out_shape = [(n + 2 * p - d * (k - 1) - 1) // t + 1
                     for n, p, d, k, t in zip(shape, pd, dl, ks, st)]
        if min(out_shape) < 1:
            continue
        done += 1
        cells = batch * shape[0] * shape[1] * shape[2]
        n = int(rng.integers(1, min(cells, 400) + 1))
        flat = np.sort(rng.choice(cells, size=n, replace=False))
        vol = shape[0] * shape[1] * shape[2]
        b, r = flat // vol, flat % vol
        idx = np.stack([b, r // (shape[1] * shape[2]), (r // shape[2]) % shape[1],
                        r % shape[2]], 1).astype(np.int32)
        if rng.integers(0, 3) == 0:
            idx = idx[rng.permutation(n)]
        case = (batch, shape, ks, st, pd, dl, subm, n)
        print("case", case, flush=True)
        raw = oracle.rulebook(idx, batch, shape, ks, st, pd, dl, subm)
        # submanifold outputs keep the input numbering; regular ones are numbered by key
        o_idx, o_pairs, o_num = raw[:3] if subm else oracle.canonicalize(*raw)
        g = get_indice_pairs(torch.from_numpy(idx).to(device), batch, shape, ks, st, pd, dl, 0, subm)
        for got, want in zip(g, (o_idx, o_pairs, o_num)):
            assert np.array_equal(got.cpu().numpy(), want), case
        K = ks[0] * ks[1] * ks[2]
        n_out = o_idx.shape[0]
        cin, cout = int(rng.choice([3, 8, 16, 37, 64, 72])), int(rng.choice([5, 16, 24, 64, 80]))
        f = rng.normal(size=(n, cin)).astype(np.float32)
        w = (rng.normal(size=(K, cin, cout)) / np.sqrt(K * cin)).astype(np.float32)
        go = rng.normal(size=(n_out, cout)).astype(np.float32)
        ft, wt, got_ = [torch.from_numpy(a).to(device) for a in (f, w, go)]
        wt = wt.reshape(*ks, cin, cout)
        y = _ext.indice_conv_fp32(ft, wt, g[1], g[2], n_out, 0, int(subm))
        d_in, d_w = _ext.indice_conv_backward_fp32(ft, wt, got_, g[1], g[2], 0, int(subm))
        assert rel_l2(y.cpu().numpy(), oracle.conv_fwd(f, w, o_pairs, o_num, n_out,
                                                       matmul=np.matmul)) < REL_L2, case
        r_in, r_w = oracle.conv_bwd(f, w, go, o_pairs, o_num)
        assert rel_l2(d_in.cpu().numpy(), r_in) < REL_L2, case
        assert rel_l2(d_w.cpu().numpy().reshape(K, cin, cout), r_w) < REL_L2, case
        c = int(rng.choice([4, 7, 32]))
        pf = rng.normal(size=(n, c)).astype(np.float32)
        pt = torch.from_numpy(pf).to(device)
        mx = _ext.indice_maxpool_fp32(pt, g[1], g[2], n_out)
        assert np.array_equal(mx.cpu().numpy(), oracle.maxpool_fwd(pf, o_pairs, o_num, n_out)), case
        rf = _ext.indiceSummaryRF(g[1], g[2], n_out)
        o_rf = oracle.summary_rf(o_pairs, o_num, n_out)
        assert np.array_equal(rf.cpu().numpy(), o_rf), case
        av = _ext.indice_avgpool_fp32(pt, g[1], g[2], n_out, rf)
        assert np.array_equal(av.cpu().numpy(),
                              oracle.avgpool_fwd(pf, o_pairs, o_num, n_out, o_rf)), case


def test_rulebook_config1_sizes(oracle, device):
    c = synth.CONFIGS["cfg1"]
    pts, _, ids = synth.config_clouds("cfg1")
    idx = synth.voxel_indices(pts, ids, c["grid"])
    o = oracle.canonicalize(*oracle.rulebook(idx, c["batch"], [c["grid"]] * 3, 3, 1, 1))
    g = gpu_rulebook(idx, c["batch"], c["grid"], 3, 1, 1)
    for a, b in zip(g, o):
        assert np.array_equal(a, b)


CONV_CASES = [
    # n_vox, grid, k, s, p, cin, cout
    (300, 10, 3, 1, 1, 32, 32),
    (300, 10, 3, 1, 1, 64, 128),
    (200, 10, 3, 2, 1, 128, 256),
    (200, 8, 3, 1, 1, 3, 152),
    (150, 8, 5, 1, 2, 200, 200),
    (100, 8, 3, 1, 1, 5, 7),
    (100, 8, 2, 2, 0, 16, 20),
    (900, 12, 3, 1, 1, 64, 64),
    # many tiles per workgroup range, several tiles per range boundary, 2 column blocks
    (6000, 24, 3, 1, 1, 64, 80),
    # two channel chunks on the buffer-load gather path, 3 column blocks
    (1500, 16, 3, 1, 1, 128, 136),
    # a single chunk with three 16-channel quarters in use, both gather paths
    (700, 12, 3, 1, 1, 40, 64),
    (700, 12, 3, 1, 1, 37, 24),
]


def _conv_case(oracle, device, n, grid, k, s, p, cin, cout, seed, permuted=False, shuffle=False):
    from ss_conv import _ext
    rng = np.random.default_rng(seed)
    idx = random_voxels(rng, 2, grid, n)
    if shuffle:
        idx = idx[rng.permutation(n)]
    feats = rng.normal(size=(n, cin)).astype(np.float32)
    K = k ** 3
    w = (rng.normal(size=(K, cin, cout)) / np.sqrt(K * cin)).astype(np.float32)
    o_idx, o_pairs, o_num = oracle.canonicalize(*oracle.rulebook(idx, 2, [grid] * 3, k, s, p))
    # fp64 accumulation of the same sums as the reference's gather-GEMM-scatter
    ref = np.zeros((o_idx.shape[0], cout), dtype=np.float64)
    for kk in range(K):
        m = int(o_num[kk])
        if m:
            np.add.at(ref, o_pairs[kk, 1, :m],
                      feats[o_pairs[kk, 0, :m]].astype(np.float64) @ w[kk].astype(np.float64))
    # and the fp32 restatement must agree with it
    ref32 = oracle.conv_fwd(feats, w, o_pairs, o_num, o_idx.shape[0], matmul=np.matmul)
    assert rel_l2(ref32, ref) < REL_L2

    g_idx, g_pairs, g_num = [torch.from_numpy(x).to(device) for x in
                             gpu_rulebook(idx, 2, grid, k, s, p)]
    wt = torch.from_numpy(w).to(device)
    if permuted:  # the reference's layout: [Cout, Cin, k, k, k] permuted to [k, k, k, Cin, Cout]
        wt = wt.permute(2, 1, 0).contiguous().reshape(cout, cin, k, k, k).permute(2, 3, 4, 1, 0)
        assert not wt.is_contiguous()
    else:
        wt = wt.reshape(k, k, k, cin, cout)
    out = _ext.indice_conv_fp32(torch.from_numpy(feats).to(device), wt, g_pairs, g_num,
                                g_idx.shape[0], 0, 0)
    torch.cuda.synchronize()
    err = rel_l2(out.cpu().numpy(), ref)
    assert err < REL_L2, err
    return out, ref


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_matches_oracle(case, oracle, device):
    print("case", case, flush=True)
    n, grid, k, s, p, cin, cout = case
    _conv_case(oracle, device, n, grid, k, s, p, cin, cout, seed=11)


def test_conv_reference_filter_layout(oracle, device):
    _conv_case(oracle, device, 300, 10, 3, 1, 1, 32, 48, seed=12, permuted=True)


def test_conv_unsorted_pairs(oracle, device):
    """Input rows in arbitrary order make the per-offset output rows unsorted: the re-ordering path."""
    _conv_case(oracle, device, 300, 10, 3, 1, 1, 32, 32, seed=13, shuffle=True)


def test_conv_is_reproducible(oracle, device):
    a, _ = _conv_case(oracle, device, 900, 12, 3, 1, 1, 64, 64, seed=14)
    b, _ = _conv_case(oracle, device, 900, 12, 3, 1, 1, 64, 64, seed=14)
    assert torch.equal(a, b)


@pytest.mark.parametrize("shape", [(64, 72), (128, 136), (40, 8), (37, 3)])
def test_conv_lone_last_column_group(shape, oracle, device):
    """Cout = 64 b + (1..16) with b <= 2: the full blocks of 64 columns take a launch each and
    the last group of 16 the kernel's one-column-group form (four consumer waves sharing the
    row blocks of the one group).  Against the oracle, bit-reproducible, and equal up to
    the order of the float sums to the launch that gives the group a column block of its own
    (ssc_conv_tuning flag 2)."""
    from ss_conv import _ext
    cin, cout = shape
    print("shape", shape, flush=True)
    a, ref = _conv_case(oracle, device, 2500, 16, 3, 1, 1, cin, cout, seed=31)
    b, _ = _conv_case(oracle, device, 2500, 16, 3, 1, 1, cin, cout, seed=31)
    assert torch.equal(a, b)
    try:
        assert _ext._lib.ssc_conv_tuning(1 | 2) == 0
        c, _ = _conv_case(oracle, device, 2500, 16, 3, 1, 1, cin, cout, seed=31)
    finally:
        _ext._lib.ssc_conv_tuning(1)
    assert rel_l2(a.cpu().numpy(), c.cpu().numpy()) < 1e-6
    # the sizes the plan functions report follow the flag back
    assert _ext._lib.ssc_conv_plan_bytes(1000, 27, cin, cout, 1000) > 0


def test_plans_are_kept_apart_by_tuning_setting(device):
    """ssc_conv_tuning changes what a plan looks like (here: a launch of its own for the lone
    last column group, or a column block of its own): the binding keys the plans it keeps
    with a rulebook by the setting they were built under, so a call under another setting
    over the same pairs tensor builds its own plan instead of walking the old one."""
    from ss_conv import _ext
    from ss_conv.sp_ops.ops import get_indice_pairs
    rng = np.random.default_rng(8)
    idx = torch.from_numpy(random_voxels(rng, 2, 16, 2500)).to(device)
    o_idx, pairs, num = get_indice_pairs(idx, 2, [16] * 3, 3, 1, 1)
    f = torch.randn(idx.shape[0], 64, device=device)
    w = torch.randn(3, 3, 3, 64, 72, device=device) / 40.0
    n_out = o_idx.shape[0]
    a = _ext.indice_conv_fp32(f, w, pairs, num, n_out, 0, 0)
    meta = _ext.rulebook_meta(pairs)
    assert len(meta.plans) == 1
    try:
        assert _ext._lib.ssc_conv_tuning(1 | 2) == 0
        b = _ext.indice_conv_fp32(f, w, pairs, num, n_out, 0, 0)
        assert len(meta.plans) == 2
    finally:
        _ext._lib.ssc_conv_tuning(1)
    c = _ext.indice_conv_fp32(f, w, pairs, num, n_out, 0, 0)
    assert len(meta.plans) == 2 and torch.equal(a, c)
    assert rel_l2(b.cpu().numpy(), a.cpu().numpy()) < 1e-6


@pytest.mark.parametrize("shape", [(200, 72), (256, 200), (197, 70), (260, 136)])
def test_conv_five_group_form(shape, oracle, device):
    """More than 192 input channels (four chunks or more) and Cout = 64 b + (1..16), b >= 1:
    one launch per block of 64 columns, the last of which takes the lone last group of 16
    along as a fifth one (every wave multiplies one of its row blocks for it).  Against the
    oracle, bit-reproducible, and equal up to the order of the float sums to the launch that
    gives the group a column block of its own (ssc_conv_tuning flag 8)."""
    from ss_conv import _ext
    cin, cout = shape
    print("shape", shape, flush=True)
    a, ref = _conv_case(oracle, device, 2500, 16, 3, 1, 1, cin, cout, seed=37)
    b, _ = _conv_case(oracle, device, 2500, 16, 3, 1, 1, cin, cout, seed=37)
    assert torch.equal(a, b)
    try:
        assert _ext._lib.ssc_conv_tuning(1 | 8) == 0
        c, _ = _conv_case(oracle, device, 2500, 16, 3, 1, 1, cin, cout, seed=37)
    finally:
        _ext._lib.ssc_conv_tuning(1)
    assert rel_l2(a.cpu().numpy(), c.cpu().numpy()) < 1e-6
    assert _ext._lib.ssc_conv_plan_bytes(1000, 27, cin, cout, 1000) > 0


@pytest.mark.parametrize("case", [(2500, 16, 3, 1, 1, 64, 128), (900, 12, 3, 2, 1, 128, 256),
                                  (400, 10, 5, 1, 2, 200, 200), (5, 8, 3, 1, 1, 5, 7),
                                  (2500, 16, 3, 1, 1, 64, 72), (1, 4, 3, 1, 1, 16, 16)])
def test_conv_schedule_filled_range_by_range(case, oracle, device):
    """Plans with one range to a workgroup have their schedule filled by the launch that counts
    the ranges' row blocks, every range at the groups it takes from a shared cursor; with
    ssc_conv_tuning flag 512 a launch of its own fills it with the ranges in order.  The
    convolution's result does not depend on where a range's groups lie: bit-equal, run after
    run."""
    from ss_conv import _ext
    print("case", case, flush=True)
    n, grid, k, s, p, cin, cout = case
    a, _ = _conv_case(oracle, device, n, grid, k, s, p, cin, cout, seed=43)
    a2, _ = _conv_case(oracle, device, n, grid, k, s, p, cin, cout, seed=43)
    try:
        assert _ext._lib.ssc_conv_tuning(1 | 512) == 0
        b, _ = _conv_case(oracle, device, n, grid, k, s, p, cin, cout, seed=43)
    finally:
        _ext._lib.ssc_conv_tuning(1)
    assert torch.equal(a, a2)
    assert torch.equal(a, b)


@pytest.mark.parametrize("case", [(2500, 16, 3, 1, 1, 64, 128), (900, 12, 3, 2, 1, 128, 256),
                                  (400, 10, 5, 1, 2, 200, 200), (5, 8, 3, 1, 1, 5, 7),
                                  (2500, 16, 3, 1, 1, 64, 72), (3000, 16, 3, 1, 1, 3, 152)])
@pytest.mark.parametrize("flags", [32, 128, 32 | 128])
def test_conv_second_work_split(case, flags, oracle, device):
    """The work split made twice (plans of long kernels; forced here by ssc_conv_tuning flag
    32) and two ranges of output rows to a workgroup, paired by the row-block groups they
    came to (plans of middle size; forced by flag 128): either moves the boundaries between
    the workgroups' ranges of output rows, nothing else.  Against the oracle, and equal to the plan of one split up to the
    order of the float sums: an output row's products are added offset by offset within a
    row-block group and chunk by chunk over the groups, and which offsets share a group
    moves with the tiles.  With one channel chunk and no lone last group that order is
    fixed: bit-equal."""
    from ss_conv import _ext
    print("case", case, "flags", flags, flush=True)
    n, grid, k, s, p, cin, cout = case
    a, _ = _conv_case(oracle, device, n, grid, k, s, p, cin, cout, seed=41)
    try:
        assert _ext._lib.ssc_conv_tuning(1 | flags) == 0
        b, _ = _conv_case(oracle, device, n, grid, k, s, p, cin, cout, seed=41)
        c, _ = _conv_case(oracle, device, n, grid, k, s, p, cin, cout, seed=41)
    finally:
        _ext._lib.ssc_conv_tuning(1)
    assert torch.equal(b, c)
    if cin <= 64 and cout % 64 == 0:
        assert torch.equal(a, b)
    else:
        assert rel_l2(a.cpu().numpy(), b.cpu().numpy()) < 1e-6


def test_conv_random_layers(device):
    """Forty seeded random layers -- channel counts on both sides of every block and chunk
    boundary (1 ... 260 in, 1 ... 200 out), kernels 1-3, strides 1-2, regular, submanifold and
    transposed rulebooks -- forward and both gradients against a float64 statement of the
    same sums (one GEMM and one index_add per offset, src/conv/indice_conv.h:296-338,
    385-421) evaluated with torch on the GPU."""
    from ss_conv import _ext
    from ss_conv.sp_ops.ops import get_indice_pairs
    rng = np.random.default_rng(2024)
    for it in range(40):
        batch, grid, n = int(rng.integers(1, 4)), int(rng.integers(5, 18)), int(rng.integers(1, 3000))
        k, s = int(rng.choice([1, 2, 3])), int(rng.choice([1, 2]))
        p = int(rng.integers(0, k))
        tr = bool(rng.integers(0, 4) == 0)
        subm = (not tr) and k == 3 and bool(rng.integers(0, 5) == 0)
        cin = int(rng.choice([1, 3, 5, 8, 16, 37, 40, 64, 72, 100, 128, 152, 200, 197, 260]))
        cout = int(rng.choice([1, 3, 7, 8, 16, 17, 24, 64, 65, 72, 80, 96, 129, 136, 144, 152, 200]))
        print("layer", it, (batch, grid, n, k, s, p, tr, subm, cin, cout), flush=True)
        idx = torch.from_numpy(random_voxels(rng, batch, grid, min(n, batch * grid ** 3))).to(device)
        o_idx, pairs, num = get_indice_pairs(idx, batch, [grid] * 3, k, s, p, 1, 0, subm, tr)
        n_in, n_out, K = idx.shape[0], o_idx.shape[0], k ** 3
        gen = torch.Generator(device).manual_seed(it)
        f = torch.randn((n_in, cin), device=device, generator=gen)
        w = torch.randn((K, cin, cout), device=device, generator=gen) / (K * cin) ** 0.5
        go = torch.randn((n_out, cout), device=device, generator=gen)
        w5 = w.reshape(k, k, k, cin, cout)
        out = _ext.indice_conv_fp32(f, w5, pairs, num, n_out, 0, int(subm))
        d_in, d_w = _ext.indice_conv_backward_fp32(f, w5, go, pairs, num, 0, int(subm))
        ref = torch.zeros((n_out, cout), dtype=torch.float64, device=device)
        ref_in = torch.zeros((n_in, cin), dtype=torch.float64, device=device)
        ref_w = torch.zeros((K, cin, cout), dtype=torch.float64, device=device)
        for kk, m in enumerate(num.cpu().tolist()):
            if m:
                i_rows, o_rows = pairs[kk, 0, :m].long(), pairs[kk, 1, :m].long()
                fi, gk, wk = f[i_rows].double(), go[o_rows].double(), w[kk].double()
                ref.index_add_(0, o_rows, fi @ wk)
                ref_in.index_add_(0, i_rows, gk @ wk.t())
                ref_w[kk] = fi.t() @ gk
        for got, want in ((out, ref), (d_in, ref_in), (d_w.reshape(K, cin, cout), ref_w)):
            if want.numel():
                err = float((got.double() - want).norm() / want.norm().clamp_min(1e-30))
                assert err < REL_L2, (it, err)


def test_conv_inverse(oracle, device):
    """inverse=1 swaps the pair planes: features live on the outputs of the forward rulebook."""
    from ss_conv import _ext
    rng = np.random.default_rng(21)
    idx = random_voxels(rng, 2, 10, 200)
    o_idx, o_pairs, o_num = oracle.canonicalize(*oracle.rulebook(idx, 2, [10] * 3, 3, 2, 1))
    n_out = o_idx.shape[0]
    feats = rng.normal(size=(n_out, 16)).astype(np.float32)
    w = rng.normal(size=(27, 16, 24)).astype(np.float32)
    ref = oracle.conv_fwd(feats, w, o_pairs, o_num, idx.shape[0], inverse=True, matmul=np.matmul)
    out = _ext.indice_conv_fp32(torch.from_numpy(feats).to(device),
                                torch.from_numpy(w).to(device).reshape(3, 3, 3, 16, 24),
                                torch.from_numpy(o_pairs).to(device),
                                torch.from_numpy(o_num).to(device), idx.shape[0], 1, 0)
    assert rel_l2(out.cpu().numpy(), ref) < REL_L2


@pytest.mark.parametrize("k,s,p,c", [(2, 2, 0, 64), (3, 2, 1, 32), (3, 1, 1, 5), (2, 2, 0, 256)])
def test_pools_match_oracle(k, s, p, c, oracle, device):
    from ss_conv import _ext
    rng = np.random.default_rng(31)
    idx = random_voxels(rng, 2, 12, 400)
    feats = rng.normal(size=(400, c)).astype(np.float32)
    o_idx, o_pairs, o_num = oracle.canonicalize(*oracle.rulebook(idx, 2, [12] * 3, k, s, p))
    n_out = o_idx.shape[0]
    ft = torch.from_numpy(feats).to(device)
    pt = torch.from_numpy(o_pairs).to(device)
    nt = torch.from_numpy(o_num).to(device)
    mx = _ext.indice_maxpool_fp32(ft, pt, nt, n_out).cpu().numpy()
    assert np.array_equal(mx, oracle.maxpool_fwd(feats, o_pairs, o_num, n_out))
    rf = _ext.indiceSummaryRF(pt, nt, n_out)
    assert np.array_equal(rf.cpu().numpy(), oracle.summary_rf(o_pairs, o_num, n_out))
    full = torch.full((n_out,), k ** 3, dtype=torch.int32, device=device)
    av = _ext.indice_avgpool_fp32(ft, pt, nt, n_out, full).cpu().numpy()
    assert np.array_equal(av, oracle.avgpool_fwd(feats, o_pairs, o_num, n_out))
    av2 = _ext.indice_avgpool_fp32(ft, pt, nt, n_out, rf).cpu().numpy()
    assert np.array_equal(av2, oracle.avgpool_fwd(feats, o_pairs, o_num, n_out,
                                                  rf.cpu().numpy()))


@pytest.mark.parametrize("c", [1, 32, 200, 512])
def test_segment_pools(c, oracle, device):
    from ss_conv.pool import GlobalAvgPool, GlobalMaxPool
    rng = np.random.default_rng(41)
    lens = [5, 1, 300, 17, 64]
    offsets = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    feats = rng.normal(size=(offsets[-1], c)).astype(np.float32)
    feats[10:40, 0] = 2.5  # ties: the first row of the maximum wins
    ft, ot = torch.from_numpy(feats).to(device), torch.from_numpy(offsets).to(device)
    avg = GlobalAvgPool()(ft, ot).cpu().numpy()
    assert rel_l2(avg, oracle.segment_avg(feats, offsets)) < 1e-6
    mx = GlobalMaxPool()(ft, ot).cpu().numpy()
    o_max, o_idx = oracle.segment_max(feats, offsets)
    assert np.array_equal(mx, o_max)
    from ss_conv import _ext
    out = torch.zeros((len(lens), c), device=device)
    arg = torch.zeros((len(lens), c), dtype=torch.int32, device=device)
    _ext.global_maxpool_fp(ft, ot, out, arg, len(lens), c)
    assert np.array_equal(arg.cpu().numpy(), o_idx)


def test_segment_pool_empty_segment(oracle, device):
    from ss_conv import _ext
    feats = np.arange(12, dtype=np.float32).reshape(4, 3)
    offsets = np.array([0, 2, 2, 4], dtype=np.int32)
    ft, ot = torch.from_numpy(feats).to(device), torch.from_numpy(offsets).to(device)
    out = torch.zeros((3, 3), device=device)
    arg = torch.zeros((3, 3), dtype=torch.int32, device=device)
    _ext.global_avgpool_fp(ft, ot, out, arg, 3, 3)
    o = oracle.segment_avg(feats, offsets)
    assert np.array_equal(np.isnan(out.cpu().numpy()), np.isnan(o))
    _ext.global_maxpool_fp(ft, ot, out, arg, 3, 3)
    om, oi = oracle.segment_max(feats, offsets)
    assert np.array_equal(out.cpu().numpy(), om) and np.array_equal(arg.cpu().numpy(), oi)


@pytest.mark.parametrize("mode", [1, 2, 3, 4])
def test_point2voxel_matches_oracle(mode, oracle, device):
    from ss_conv.sp_ops.voxelize import Point2Voxel
    pts, feats, ids = synth.make_clouds(3, 700, seed=3, channels=6)
    pts = pts * 1.2  # some points fall outside and are filtered
    grid = 16
    ref = oracle.point2voxel(pts, feats, ids, [grid] * 3, [2.0 / grid] * 3, mode)
    p2v = Point2Voxel([grid] * 3, [2.0 / grid] * 3, mode)
    vp, st, vi, flag = p2v(torch.from_numpy(pts).to(device), torch.from_numpy(feats).to(device),
                           torch.from_numpy(ids).to(device))
    assert np.array_equal(vp.cpu().numpy(), ref["valid_points"])
    assert np.array_equal(vi.cpu().numpy(), ref["valid_ids"])
    assert np.array_equal(flag.cpu().numpy(), ref["flag"])
    assert np.array_equal(st.indices.cpu().numpy(), ref["indices"])
    assert st.batch_size == max(ref["batch_size"], int(ref["valid_ids"].max()) + 1)
    assert np.array_equal(st.features.cpu().numpy(), ref["features"])


@pytest.mark.parametrize("n,dims", [(1, [1, 3, 3, 3]), (500, [2, 4, 5, 6]), (20000, [3, 17, 9, 33]),
                                    (4000, [2, 64, 64, 64])])
def test_unique_rows_both_entry_point_pairs(n, dims, device):
    """Sorted distinct voxel rows, inverse, counts and the largest count
    (torch.unique(dim=0, return_inverse=True, return_counts=True) in
    ss_conv/sp_ops/voxelize.py:88), through ssc_unique_count + ssc_unique_emit and through
    ssc_unique_build + ssc_unique_rows."""
    from ss_conv import _ext
    gen = torch.Generator().manual_seed(n)
    rows = torch.stack([torch.randint(0, d, (n,), generator=gen) for d in dims], 1).int().to(device)
    print("n", n, "dims", dims, flush=True)
    want_u, want_inv, want_cnt = torch.unique(rows.long(), dim=0, return_inverse=True,
                                              return_counts=True)
    u1, inv1, cnt1 = _ext.unique_rows(rows, dims, return_counts=True)
    u2, inv2, cnt2, largest = _ext.unique_rows_max(rows, dims)
    for u, inv, cnt in ((u1, inv1, cnt1), (u2, inv2, cnt2)):
        assert torch.equal(u.long(), want_u)
        assert torch.equal(inv.long(), want_inv)
        assert torch.equal(cnt.long(), want_cnt)
    assert largest == int(want_cnt.max())


def test_point2voxel_empty_batch_element(oracle, device):
    """A batch element whose points all fall outside gets one zero point (voxelize.py:68-78)."""
    from ss_conv.sp_ops.voxelize import Point2Voxel
    pts, feats, ids = synth.make_clouds(3, 100, seed=4, channels=2)
    pts[ids == 1] = 50.0
    ref = oracle.point2voxel(pts, feats, ids, [8] * 3, [0.25] * 3, 4)
    vp, st, vi, flag = Point2Voxel([8] * 3, [0.25] * 3)(
        torch.from_numpy(pts).to(device), torch.from_numpy(feats).to(device),
        torch.from_numpy(ids).to(device))
    assert flag.cpu().tolist() == [1.0, 0.0, 1.0] == ref["flag"].tolist()
    assert np.array_equal(st.indices.cpu().numpy(), ref["indices"])
    assert np.array_equal(st.features.cpu().numpy(), ref["features"])
    # everything outside (voxelize.py:52-56)
    pts[:] = 50.0
    ref = oracle.point2voxel(pts, feats, ids, [8] * 3, [0.25] * 3, 4)
    vp, st, vi, flag = Point2Voxel([8] * 3, [0.25] * 3)(
        torch.from_numpy(pts).to(device), torch.from_numpy(feats).to(device),
        torch.from_numpy(ids).to(device))
    assert flag.cpu().tolist() == [0.0, 0.0, 0.0]
    assert np.array_equal(st.indices.cpu().numpy(), ref["indices"])


def test_point2voxel_gapped_ids_feed_a_convolution(oracle, device):
    """Clouds whose batch ids have gaps (1, 4, 6): the SparseTensor's batch size is 1 + the
    largest id, so the layer that follows finds every row inside its grid, and its result is
    that of the same clouds numbered 0, 1, 2."""
    from ss_conv.sp_ops.conv import SparseConvolution
    from ss_conv.sp_ops.voxelize import Point2Voxel
    pts, feats, ids = synth.make_clouds(3, 300, seed=5, channels=4)
    gapped = np.array([1, 4, 6], dtype=np.int64)[ids]
    grid = 8
    torch.manual_seed(0)
    conv = SparseConvolution(3, 4, 6, 3, stride=1, padding=1, bias=False).to(device)
    outs = []
    for use in (ids, gapped):
        p2v = Point2Voxel([grid] * 3, [2.0 / grid] * 3)
        _, st, _, _ = p2v(*[torch.from_numpy(a).to(device) for a in (pts, feats, use)])
        assert st.batch_size == int(use.max()) + 1
        with torch.no_grad():
            outs.append(conv(st))
    a, b = outs
    remap = torch.tensor([1, 4, 6], dtype=torch.int32, device=device)
    assert torch.equal(remap[a.indices[:, 0].long()], b.indices[:, 0])
    assert torch.equal(a.indices[:, 1:], b.indices[:, 1:])
    assert torch.equal(a.features, b.features)
    for mod in (1, 2):  # both paths of the module (one call; filter, unique, lists)
        p2v = Point2Voxel([grid] * 3, [2.0 / grid] * 3)
        if mod == 2:
            p2v._n_ids_hint = None
        _, st, _, _ = p2v(*[torch.from_numpy(x).to(device) for x in (pts, feats, gapped)])
        assert st.batch_size == 7


def test_point2voxel_unsorted_ids_and_outliers(oracle, device):
    """Points in arbitrary order (batch ids not sorted: the torch path) and in batch
    order (the native filter) give the oracle's result; some points lie outside the grid."""
    from ss_conv.sp_ops.voxelize import Point2Voxel
    pts, feats, ids = synth.make_clouds(4, 300, seed=9, channels=6)
    pts = pts * 1.2  # pushes part of every cloud outside [-1, 1]^3
    grid = 8
    rng = np.random.default_rng(3)
    for perm in (np.arange(len(ids)), rng.permutation(len(ids))):
        p, f, i = pts[perm], feats[perm], ids[perm]
        ref = oracle.point2voxel(p, f, i, [grid] * 3, [2.0 / grid] * 3, 4)
        vp, st, vi, flag = Point2Voxel([grid] * 3, [2.0 / grid] * 3)(
            torch.from_numpy(p).to(device), torch.from_numpy(f).to(device),
            torch.from_numpy(i).to(device))
        assert np.array_equal(st.indices.cpu().numpy(), ref["indices"])
        assert np.array_equal(vp.cpu().numpy(), ref["valid_points"])
        assert np.array_equal(vi.cpu().numpy(), ref["valid_ids"])
        assert np.array_equal(st.features.cpu().numpy(), ref["features"])
        assert flag.cpu().tolist() == ref["flag"].tolist()


@pytest.mark.parametrize("seed", [1, 2])
def test_point_voxel_random_configurations(seed, oracle, device):
    """Point2Voxel and Voxel2Point on 40 seeded configurations a seed: 1-5 clouds (some empty,
    some entirely outside, ids with gaps, points in batch order or shuffled), non-cubic voxel
    limits, anisotropic voxel extents, all four reduction modes, points exactly on cell faces
    and duplicated points.  Voxel lists, features, 3-NN indices and distances bit-exact."""
    from ss_conv.sp_ops.functional import three_nn
    from ss_conv.sp_ops.voxelize import Point2Voxel, Voxel2Point
    rng = np.random.default_rng(seed)
    for case in range(40):
        B = int(rng.integers(1, 6))
        limit = [int(rng.integers(2, 20)) for _ in range(3)]
        unit = [float(rng.choice([0.05, 0.1, 0.125, 0.3, 0.07])) for _ in range(3)]
        mode = int(rng.integers(1, 5))
        C = int(rng.choice([1, 3, 6, 16, 33]))
        counts = [int(rng.integers(0, 300)) for _ in range(B)]
        if sum(counts) == 0:
            counts[0] = 5
        ids = np.concatenate([np.full(c, b, dtype=np.int64) for b, c in enumerate(counts)])
        if rng.integers(0, 3) == 0:
            ids = ids * 2 + 1
        n = len(ids)
        half = 0.5 * np.array(limit) * np.array(unit)
        scale = float(rng.choice([0.5, 1.0, 1.3]))
        pts = (rng.uniform(-1, 1, size=(n, 3)) * half * scale).astype(np.float32)
        on_face = rng.integers(0, 10, size=n) == 0
        u32 = np.array(unit, np.float32)
        pts[on_face] = (np.round(pts[on_face] / u32) * u32).astype(np.float32)
        if n > 4:
            pts[rng.integers(0, n, size=n // 8)] = pts[rng.integers(0, n, size=n // 8)]
        if rng.integers(0, 4) == 0 and B > 1:
            pts[ids == ids[0]] = 1e3
        feats = rng.normal(size=(n, C)).astype(np.float32)
        if rng.integers(0, 4) == 0:
            perm = rng.permutation(n)
            pts, feats, ids = pts[perm], feats[perm], ids[perm]
        print("case", case, B, limit, unit, mode, C, n, flush=True)
        ref = oracle.point2voxel(pts, feats, ids, limit, unit, mode)
        vp, st, vi, flag = Point2Voxel(limit, unit, mode)(
            torch.from_numpy(pts).to(device), torch.from_numpy(feats).to(device),
            torch.from_numpy(ids).to(device))
        assert np.array_equal(vp.cpu().numpy(), ref["valid_points"]), case
        assert np.array_equal(vi.cpu().numpy(), ref["valid_ids"]), case
        assert np.array_equal(flag.cpu().numpy(), ref["flag"]), case
        assert np.array_equal(st.indices.cpu().numpy(), ref["indices"]), case
        assert st.batch_size == max(ref["batch_size"], int(ref["valid_ids"].max()) + 1), case
        assert np.array_equal(st.features.cpu().numpy(), ref["features"]), case
        v2p = Voxel2Point(unit_voxel_extent=unit)
        out = v2p(st, vp, vi)
        want, _, _ = oracle.voxel2point(st.indices.cpu().numpy(), st.features.cpu().numpy(), limit,
                                        vp.cpu().numpy(), vi.cpu().numpy(), unit_voxel_extent=unit)
        assert rel_l2(out.cpu().numpy(), want) < REL_L2, case
        centres = v2p._get_vertice_feats(st)[0]
        target = torch.cat([vi.float().unsqueeze(1), vp], 1).contiguous()
        dist, idx = three_nn(target, centres)
        odist, oidx = oracle.three_nn(target.cpu().numpy(), centres.cpu().numpy())
        assert np.array_equal(idx.cpu().numpy(), oidx), case
        assert np.array_equal(dist.cpu().numpy(), odist), case


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_three_nn_grid_equals_plain_scan(seed, device):
    """The grid search among voxel centres returns the plain scan's distances and indices,
    ties included: dense and nearly empty grids, anisotropic cells, voxel rows in arbitrary
    order, queries inside, on cell faces, outside the grid and in batch elements without
    voxels (the last kinds make the call fall back to the plain scan)."""
    from ss_conv import _ext
    rng = np.random.default_rng(seed)
    for case in range(25):
        batch = int(rng.integers(1, 5))
        dims = [int(rng.integers(1, 20)) for _ in range(3)]
        unit = np.array([float(rng.choice([0.05, 0.1, 0.3, 1.0])) for _ in range(3)], np.float32)
        origin = (np.float32(-0.5) * (unit * np.array(dims, np.float32))).astype(np.float32)
        cells = batch * dims[0] * dims[1] * dims[2]
        fill = float(rng.choice([0.002, 0.05, 0.5, 1.0]))
        m = max(1, min(cells, int(cells * fill)))
        flat = rng.choice(cells, size=m, replace=False)
        if rng.integers(0, 2):
            flat.sort()
        vol = dims[0] * dims[1] * dims[2]
        b, r = flat // vol, flat % vol
        vox = np.stack([b, r // (dims[1] * dims[2]), (r // dims[2]) % dims[1], r % dims[2]],
                       1).astype(np.int32)
        centres = np.concatenate([vox[:, :1].astype(np.float32),
                                  vox[:, 1:].astype(np.float32) * unit + origin
                                  + np.float32(0.5) * unit], 1).astype(np.float32)
        n = int(rng.integers(1, 600))
        extent = unit * np.array(dims, np.float32)
        pts = (rng.uniform(-0.5, 0.5, size=(n, 3)) * extent * float(rng.choice([1.0, 1.0, 2.5])))
        pts = pts.astype(np.float32)
        on_face = rng.integers(0, 6, size=n) == 0
        pts[on_face] = (np.round(pts[on_face] / unit) * unit).astype(np.float32)
        exact = rng.integers(0, 6, size=n) == 0   # exactly on a centre: ties between neighbours
        pts[exact] = centres[rng.integers(0, m, size=int(exact.sum())), 1:]
        qb = rng.integers(0, batch + 1, size=n).astype(np.float32)  # batch + 1: no such element
        unknown = np.concatenate([qb[:, None], pts], 1).astype(np.float32)
        print("case", case, batch, dims, unit.tolist(), m, n, flush=True)
        u_t, k_t, v_t = [torch.from_numpy(a).to(device) for a in (unknown, centres, vox)]
        d_grid, i_grid = _ext.three_nn_grid(u_t, k_t, v_t, batch, dims, origin, unit)
        d_ref = torch.empty((n, 3), dtype=torch.float32, device=device)
        i_ref = torch.empty((n, 3), dtype=torch.int32, device=device)
        _ext.three_nn(n, m, u_t, k_t, d_ref, i_ref)
        assert torch.equal(d_grid, d_ref), case
        assert torch.equal(i_grid, i_ref), case


def test_voxel2point_matches_oracle(oracle, device):
    from ss_conv.sp_ops.voxelize import Point2Voxel, Voxel2Point
    pts, feats, ids = synth.make_clouds(3, 500, seed=6, channels=10)
    grid = 16
    dp, df, di = [torch.from_numpy(x).to(device) for x in (pts, feats, ids)]
    vp, st, vi, _ = Point2Voxel([grid] * 3, [2.0 / grid] * 3)(dp, df, di)
    out = Voxel2Point(unit_voxel_extent=[2.0 / grid] * 3)(st, vp, vi)
    ref, ridx, rw = oracle.voxel2point(st.indices.cpu().numpy(), st.features.cpu().numpy(),
                                       [grid] * 3, vp.cpu().numpy(), vi.cpu().numpy(),
                                       unit_voxel_extent=[2.0 / grid] * 3)
    assert rel_l2(out.cpu().numpy(), ref) < 1e-6
    # index parity of the search itself, including ties
    from ss_conv.sp_ops.functional import three_nn
    centres = Voxel2Point(unit_voxel_extent=[2.0 / grid] * 3)._get_vertice_feats(st)[0]
    target = torch.cat([vi.float().unsqueeze(1), vp], 1).contiguous()
    dist, idx = three_nn(target, centres)
    odist, oidx = oracle.three_nn(target.cpu().numpy(), centres.cpu().numpy())
    assert np.array_equal(idx.cpu().numpy(), oidx)
    assert np.array_equal(dist.cpu().numpy(), odist)
    c2, f2, b2 = Voxel2Point(voxel_extent=[2.0] * 3)(st)
    assert c2.shape == (st.indices.shape[0], 3) and f2 is st.features


def test_three_nn_unsorted_and_many_tiles(oracle, device):
    """Known rows in arbitrary order (batch elements interleaved) and more than one
    tile of 256 rows per batch element: the tile skipping must not change a result."""
    from ss_conv.sp_ops.functional import three_nn
    rng = np.random.default_rng(21)
    m, n, nb = 3000, 700, 5
    known = np.concatenate([rng.integers(0, nb, size=(m, 1)).astype(np.float32),
                            rng.integers(0, 12, size=(m, 3)).astype(np.float32) * 0.25], 1)
    unknown = np.concatenate([rng.integers(0, nb + 1, size=(n, 1)).astype(np.float32),
                              rng.uniform(0, 3, size=(n, 3)).astype(np.float32)], 1)
    for kn in (known, known[np.argsort(known[:, 0], kind="stable")]):
        dist, idx = three_nn(torch.from_numpy(unknown).to(device).contiguous(),
                             torch.from_numpy(np.ascontiguousarray(kn)).to(device))
        odist, oidx = oracle.three_nn(unknown, np.ascontiguousarray(kn))
        assert np.array_equal(idx.cpu().numpy(), oidx)
        assert np.array_equal(dist.cpu().numpy(), odist)


def test_kernel_combine_matches_einsum(oracle, device):
    from ss_conv.utils.kernel import SE3Kernel
    torch.manual_seed(0)
    for rs_in, rs_out, size in [([(2, 0), (2, 1), (2, 2), (2, 3)], [(2, 0), (2, 1), (2, 2), (2, 3)], 3),
                                ([(3, 0)], [(2, 0), (1, 1), (1, 2)], 3),
                                ([(1, 0), (2, 2)], [(2, 1), (1, 4)], 5)]:
        ker = SE3Kernel(rs_in, rs_out, size).to(device)
        got = ker().detach().cpu().numpy()
        bases = [[getattr(ker, "kernel_%d_%d" % (i, j)) for j in range(len(ker.Rs_in))]
                 for i in range(len(ker.Rs_out))]
        bases = [[None if b is None else b.cpu().numpy() for b in row] for row in bases]
        ref = oracle.combine(ker.weight.detach().cpu().numpy(), bases, ker.multiplicities_out,
                             ker.dims_out, ker.multiplicities_in, ker.dims_in, size)
        assert got.shape == ref.shape
        assert rel_l2(got, ref) < 1e-6
        # synthesis and packing in one launch: the same dense kernel, and the packed filters
        # that ssc_conv_pack_filters_f32 makes of it, bit for bit
        from ss_conv import _ext
        both = ker(pack=True).detach()
        assert np.array_equal(both.cpu().numpy(), got)
        fused = ker.packed
        w = both.permute(2, 3, 4, 1, 0)
        packed = _ext.prepack_filters(w, ker.n_in, ker.n_out)
        assert fused is not None and fused.numel() == packed.numel()
        assert torch.equal(fused, packed)


def test_convolution_layer_end_to_end(oracle, device):
    """Point2Voxel -> Convolution against the oracle pipeline and against dense conv3d."""
    import torch.nn.functional as F
    from ss_conv.convolution import Convolution
    from ss_conv.sp_ops.voxelize import Point2Voxel
    torch.manual_seed(1)
    rs = [(2, 0), (2, 1), (2, 2), (2, 3)]
    pts, feats, ids = synth.make_clouds(2, 300, seed=8, channels=32)
    grid = 12
    conv = Convolution(rs, rs, 3, stride=1, padding=1).to(device).eval()
    _, st, _, _ = Point2Voxel([grid] * 3, [2.0 / grid] * 3)(
        *[torch.from_numpy(x).to(device) for x in (pts, feats, ids)])
    with torch.no_grad():
        out = conv(st)
    dense_kernel = conv.kernel().detach()  # [Cout, Cin, k, k, k]
    want = F.conv3d(st.dense().cpu().double(), dense_kernel.cpu().double(), stride=1, padding=1)
    got = out.dense().cpu().double()
    assert rel_l2(got.numpy(), want.numpy()) < REL_L2
    w = dense_kernel.permute(2, 3, 4, 1, 0).reshape(27, 32, 32).cpu().numpy()
    o_idx, o_pairs, o_num = oracle.canonicalize(*oracle.rulebook(
        st.indices.cpu().numpy(), 2, [grid] * 3, 3, 1, 1))
    assert np.array_equal(out.indices.cpu().numpy(), o_idx)
    ref = oracle.conv_fwd(st.features.cpu().numpy(), w, o_pairs, o_num, o_idx.shape[0],
                          matmul=np.matmul)
    assert rel_l2(out.features.cpu().numpy(), ref) < REL_L2


BWD_CASES = [
    # n_vox, grid, k, s, p, cin, cout
    (300, 10, 3, 1, 1, 32, 32),
    (900, 12, 3, 1, 1, 64, 128),
    (200, 10, 3, 2, 1, 128, 72),
    (200, 8, 3, 1, 1, 3, 152),
    (150, 8, 5, 1, 2, 40, 24),
    (100, 8, 2, 2, 0, 5, 7),
]


@pytest.mark.parametrize("case", BWD_CASES)
def test_conv_backward_matches_oracle(case, oracle, device):
    """Input and filter gradients through the C ABI against the restated backward."""
    from ss_conv import _ext
    print("case", case, flush=True)
    n, grid, k, s, p, cin, cout = case
    rng = np.random.default_rng(41)
    idx = random_voxels(rng, 2, grid, n)
    feats = rng.normal(size=(n, cin)).astype(np.float32)
    K = k ** 3
    w = (rng.normal(size=(K, cin, cout)) / np.sqrt(K * cin)).astype(np.float32)
    o_idx, o_pairs, o_num = oracle.canonicalize(*oracle.rulebook(idx, 2, [grid] * 3, k, s, p))
    g_out = rng.normal(size=(o_idx.shape[0], cout)).astype(np.float32)
    ref_in, ref_w = oracle.conv_bwd(feats, w, g_out, o_pairs, o_num)
    g_idx, g_pairs, g_num = [torch.from_numpy(x).to(device) for x in
                             gpu_rulebook(idx, 2, grid, k, s, p)]
    wt = torch.from_numpy(w).to(device).reshape(k, k, k, cin, cout)
    d_in, d_w = _ext.indice_conv_backward_fp32(
        torch.from_numpy(feats).to(device), wt, torch.from_numpy(g_out).to(device), g_pairs,
        g_num, 0, 0)
    assert d_w.shape == wt.shape
    assert rel_l2(d_in.cpu().numpy(), ref_in) < REL_L2
    assert rel_l2(d_w.cpu().numpy().reshape(K, cin, cout), ref_w) < REL_L2
    # twice the same bits
    d_in2, d_w2 = _ext.indice_conv_backward_fp32(
        torch.from_numpy(feats).to(device), wt, torch.from_numpy(g_out).to(device), g_pairs,
        g_num, 0, 0)
    assert torch.equal(d_w, d_w2) and torch.equal(d_in, d_in2)
    # the inverse convolution's backward: roles of the two row planes exchanged
    wi = torch.from_numpy(np.ascontiguousarray(np.transpose(w, (0, 2, 1)))).to(device) \
        .reshape(k, k, k, cout, cin)
    e_in, e_w = _ext.indice_conv_backward_fp32(
        torch.from_numpy(g_out).to(device), wi, torch.from_numpy(feats).to(device), g_pairs,
        g_num, 1, 0)
    oref_in, oref_w = oracle.conv_bwd(g_out, np.transpose(w, (0, 2, 1)).copy(), feats, o_pairs,
                                      o_num, inverse=True)
    assert rel_l2(e_in.cpu().numpy(), oref_in) < REL_L2
    assert rel_l2(e_w.cpu().numpy().reshape(K, cout, cin), oref_w) < REL_L2


@pytest.mark.parametrize("geom", [dict(stride=1, padding=1), dict(stride=2, padding=1),
                                  dict(stride=1, padding=1, subm=True),
                                  dict(stride=1, padding=1, subm=True, indice_key="k")])
def test_training_layer_filters_ride_on_the_rulebook(geom, device):
    """A training-mode Convolution leaves the synthesis and packing of its filters to the first
    launch of the rulebook it queues (to a launch of its own when the rulebook is already
    there: the second call under an indice_key).  Same filters, same plan as the
    evaluation-mode layer, which synthesises them by itself: bit-equal rows, and the dense
    kernel the autograd graph holds equals the module's."""
    from ss_conv.convolution import Convolution
    from ss_conv.sp_ops.tensor import SparseTensor
    torch.manual_seed(4)
    rs_in, rs_out = [(3, 0), (2, 1), (1, 2)], [(4, 0), (3, 1), (1, 2)]
    rng = np.random.default_rng(6)
    grid, n = 11, 400
    idx = torch.from_numpy(random_voxels(rng, 2, grid, n)).to(device)
    conv = Convolution(rs_in, rs_out, 3, **geom).to(device)
    feats = torch.from_numpy(rng.normal(size=(n, conv.in_channels)).astype(np.float32)).to(device)
    make = lambda: SparseTensor(feats, idx, [grid] * 3, 2)  # noqa: E731
    with torch.no_grad():
        conv.eval()
        want = conv(make())
        conv.train()
        x = make()
        got = conv(x)
        again = conv(x) if geom.get("indice_key") else None  # the rulebook is cached now
    assert torch.equal(got.indices, want.indices)
    assert torch.equal(got.features, want.features)
    if again is not None:
        assert torch.equal(again.features, want.features)


def test_index_work_on_a_second_stream(device):
    """Rulebooks and plans are queued on a second stream of the device, the convolutions and
    pools on the caller's: a stack of layers over changing inputs, calls following each other
    without a wait, gives bit for bit what it gives with everything on one stream.  Inputs are
    made by torch kernels on the caller's stream right before each pass (the second stream
    has to wait for them), the rulebooks under an indice_key are reused by later layers, and
    tensors are dropped while kernels that read them may still be queued (the allocator must
    not hand their memory out early)."""
    from ss_conv import _ext
    from ss_conv.convolution import Convolution
    from ss_conv.pool import MaxPool
    from ss_conv.sp_ops.tensor import SparseTensor
    torch.manual_seed(12)
    rs0, rs1, rs2 = [(4, 0), (2, 1)], [(6, 0), (3, 1), (1, 2)], [(8, 0), (4, 1)]
    layers = [Convolution(rs0, rs1, 3, stride=1, padding=1).to(device),
              Convolution(rs1, rs1, 3, stride=1, padding=1, subm=True, indice_key="a").to(device),
              Convolution(rs1, rs2, 3, stride=2, padding=1).to(device),
              Convolution(rs2, rs2, 3, stride=1, padding=1, subm=True, indice_key="b").to(device),
              Convolution(rs2, rs2, 3, stride=1, padding=1, subm=True, indice_key="b").to(device)]
    pool = MaxPool(2, 2)
    for m in layers:
        m.train()
    grid, n = 20, 3000
    rng = np.random.default_rng(21)
    clouds = [torch.from_numpy(random_voxels(rng, 2, grid, n)).to(device) for _ in range(4)]

    def run_all():
        outs = []
        for it in range(8):
            idx = clouds[it % 4].clone()  # a new tensor, written on the caller's stream
            feats = torch.randn(n, layers[0].in_channels, device=device,
                                generator=torch.Generator(device).manual_seed(it))
            x = SparseTensor(feats * 1.5, idx, [grid] * 3, 2)
            for m in layers:
                x = m(x)
            y = pool(x)
            outs.append((x.features, x.indices, y.features, y.indices))
            del x, y, idx, feats
        torch.cuda.synchronize()
        return outs

    keep = _ext._INDEX_STREAM_MIN_WORK, _ext._INDEX_STREAM_MIN_FLOPS
    was = _ext.index_stream(True)
    try:
        # (these layers are far below the size it is meant for)
        _ext._INDEX_STREAM_MIN_WORK = _ext._INDEX_STREAM_MIN_FLOPS = 0
        with torch.no_grad():
            two = run_all()
            again = run_all()
            _ext.index_stream(False)
            one = run_all()
    finally:
        _ext._INDEX_STREAM_MIN_WORK, _ext._INDEX_STREAM_MIN_FLOPS = keep
        _ext.index_stream(was)
    for a, b, c in zip(two, again, one):
        for ta, tb, tc in zip(a, b, c):
            assert torch.equal(ta, tc)
            assert torch.equal(tb, tc)


def test_index_work_on_a_second_stream_training_step(device):
    """A training step -- forward, loss, backward through three layers, the first two sharing
    a rulebook under an indice_key -- with rulebooks and plans on the second stream: the
    gradients of the features and of every layer's weights equal those of the same step on
    one stream, bit for bit, over several steps that follow each other without a wait."""
    from ss_conv import _ext
    from ss_conv.convolution import Convolution
    from ss_conv.sp_ops.tensor import SparseTensor
    torch.manual_seed(13)
    rs0, rs1 = [(4, 0), (2, 1)], [(6, 0), (3, 1), (1, 2)]
    layers = [Convolution(rs0, rs1, 3, stride=1, padding=1, subm=True, indice_key="s").to(device),
              Convolution(rs1, rs1, 3, stride=1, padding=1, subm=True, indice_key="s").to(device),
              Convolution(rs1, rs0, 3, stride=2, padding=1).to(device)]
    for m in layers:
        m.train()
    grid, n = 18, 2500
    rng = np.random.default_rng(22)
    clouds = [torch.from_numpy(random_voxels(rng, 2, grid, n)).to(device) for _ in range(3)]

    def run_all():
        outs = []
        for it in range(5):
            idx = clouds[it % 3].clone()
            feats = torch.randn(n, layers[0].in_channels, device=device,
                                generator=torch.Generator(device).manual_seed(100 + it))
            feats.requires_grad_(True)
            for m in layers:
                m.zero_grad(set_to_none=True)
            x = SparseTensor(feats, idx, [grid] * 3, 2)
            for m in layers:
                x = m(x)
            (x.features * x.features).sum().backward()
            outs.append([feats.grad.clone()] + [m.kernel.weight.grad.clone() for m in layers])
        torch.cuda.synchronize()
        return outs

    keep = _ext._INDEX_STREAM_MIN_WORK, _ext._INDEX_STREAM_MIN_FLOPS
    was = _ext.index_stream(True)
    try:
        _ext._INDEX_STREAM_MIN_WORK = _ext._INDEX_STREAM_MIN_FLOPS = 0
        two = run_all()
        _ext.index_stream(False)
        one = run_all()
    finally:
        _ext._INDEX_STREAM_MIN_WORK, _ext._INDEX_STREAM_MIN_FLOPS = keep
        _ext.index_stream(was)
    for a, b in zip(two, one):
        for ta, tb in zip(a, b):
            assert torch.equal(ta, tb)


def test_layer_gradients(oracle, device):
    """loss.backward() through Convolution: gradient of the input features against the
    restated backward, gradient of kernel.weight against torch autograd through an
    einsum statement of the kernel synthesis (ss_conv/utils/kernel.py:267-299)."""
    from ss_conv.convolution import Convolution
    from ss_conv.sp_ops.tensor import SparseTensor
    torch.manual_seed(2)
    rs_in, rs_out = [(2, 0), (1, 1), (1, 2)], [(3, 0), (2, 1)]
    rng = np.random.default_rng(5)
    grid, n = 9, 250
    idx = random_voxels(rng, 2, grid, n)
    conv = Convolution(rs_in, rs_out, 3, stride=1, padding=1).to(device).train()
    cin, cout = conv.in_channels, conv.out_channels
    feats = torch.from_numpy(rng.normal(size=(n, cin)).astype(np.float32)).to(device)
    feats.requires_grad_(True)
    x = SparseTensor(feats, torch.from_numpy(idx).to(device), [grid] * 3, 2)
    out = conv(x)
    g_out = torch.from_numpy(rng.normal(size=tuple(out.features.shape)).astype(np.float32))
    (out.features * g_out.to(device)).sum().backward()

    ker = conv.kernel
    w_dense = ker().detach().permute(2, 3, 4, 1, 0).reshape(27, cin, cout).cpu().numpy()
    o_idx, o_pairs, o_num = oracle.canonicalize(*oracle.rulebook(idx, 2, [grid] * 3, 3, 1, 1))
    assert np.array_equal(out.indices.cpu().numpy(), o_idx)
    ref_in, ref_w = oracle.conv_bwd(feats.detach().cpu().numpy(), w_dense, g_out.numpy(), o_pairs,
                                    o_num)
    assert rel_l2(feats.grad.cpu().numpy(), ref_in) < REL_L2
    # kernel.weight: chain ref_w [K, Cin, Cout] through the synthesis, in float64 on the CPU
    wt = ker.weight.detach().cpu().double().requires_grad_(True)
    rows, off = [], 0
    for i, (mi, di) in enumerate(zip(ker.multiplicities_out, ker.dims_out)):
        cols = []
        for j, (mj, dj) in enumerate(zip(ker.multiplicities_in, ker.dims_in)):
            kij = getattr(ker, "kernel_%d_%d" % (i, j))
            if kij is None:
                cols.append(torch.zeros(mi * di, mj * dj, 3, 3, 3, dtype=torch.float64))
                continue
            nb = kij.size(0)
            wb = wt[off:off + mi * mj * nb].view(mi, mj, nb)
            off += mi * mj * nb
            blk = torch.einsum("uvn,nabxyz->uavbxyz", wb, kij.detach().cpu().double())
            cols.append(blk.reshape(mi * di, mj * dj, 3, 3, 3))
        rows.append(torch.cat(cols, 1))
    dense = torch.cat(rows, 0)  # [Cout, Cin, 3, 3, 3]
    assert rel_l2(dense.detach().permute(2, 3, 4, 1, 0).reshape(27, cin, cout).numpy(),
                  w_dense) < 1e-6
    (dense.permute(2, 3, 4, 1, 0).reshape(27, cin, cout) *
     torch.from_numpy(ref_w).double()).sum().backward()
    assert rel_l2(ker.weight.grad.cpu().numpy(), wt.grad.numpy()) < REL_L2


@pytest.mark.parametrize("k,s,p,c", [(2, 2, 0, 64), (3, 2, 1, 32), (3, 1, 1, 5)])
def test_pool_backward_matches_oracle(k, s, p, c, oracle, device):
    """Max / avg pooling gradients through autograd (bit-exact: same order of additions)."""
    from ss_conv.sp_ops.functional import indice_avgpool, indice_maxpool
    rng = np.random.default_rng(23)
    n, grid = 400, 10
    idx = random_voxels(rng, 2, grid, n)
    feats = rng.normal(size=(n, c)).astype(np.float32)
    o_idx, o_pairs, o_num = oracle.canonicalize(*oracle.rulebook(idx, 2, [grid] * 3, k, s, p))
    g_idx, g_pairs, g_num = [torch.from_numpy(x).to(device) for x in
                             gpu_rulebook(idx, 2, grid, k, s, p)]
    g_out = rng.normal(size=(o_idx.shape[0], c)).astype(np.float32)
    for op, name in ((indice_maxpool, "max"), (indice_avgpool, "avg")):
        x = torch.from_numpy(feats).to(device).requires_grad_(True)
        y = op(x, g_pairs, g_num, g_idx.shape[0])
        (y * torch.from_numpy(g_out).to(device)).sum().backward()
        if name == "max":
            pooled = oracle.maxpool_fwd(feats, o_pairs, o_num, o_idx.shape[0])
            ref = oracle.maxpool_bwd(feats, pooled, g_out, o_pairs, o_num)
        else:
            ref = oracle.avgpool_bwd(g_out, o_pairs, o_num, n,
                                     np.full(o_idx.shape[0], k ** 3, dtype=np.int32))
        assert np.array_equal(x.grad.cpu().numpy(), ref), name


def test_segment_voxel_interp_backward(oracle, device):
    from ss_conv.sp_ops.functional import (global_avgpool, global_maxpool, voxelization,
                                           three_interpolate)
    rng = np.random.default_rng(29)
    n, c = 500, 70
    feats = rng.normal(size=(n, c)).astype(np.float32)
    offsets = np.array([0, 120, 120, 333, 500], dtype=np.int32)
    g = rng.normal(size=(4, c)).astype(np.float32)
    offs = torch.from_numpy(offsets).to(device)
    x = torch.from_numpy(feats).to(device).requires_grad_(True)
    (global_avgpool(x, offs) * torch.from_numpy(g).to(device))[[0, 2, 3]].sum().backward()
    ref = oracle.segment_avg_bwd(g, offsets, n)
    assert np.array_equal(x.grad.cpu().numpy(), ref)
    x = torch.from_numpy(feats).to(device).requires_grad_(True)
    (global_maxpool(x, offs) * torch.from_numpy(g).to(device))[[0, 2, 3]].sum().backward()
    _, arg = oracle.segment_max(feats, offsets)
    g_used = g.copy()
    g_used[1] = 0  # the empty segment's output (-inf) is left out of the loss
    assert np.array_equal(x.grad.cpu().numpy(), oracle.segment_max_bwd(g_used, arg, n))
    # voxel mean
    inverse = rng.integers(0, 60, size=n).astype(np.int32)
    inverse[:60] = np.arange(60)
    counts = np.bincount(inverse, minlength=60)
    maps = oracle.voxel_map(inverse, 60, int(counts.max()), 4)
    gv = rng.normal(size=(60, c)).astype(np.float32)
    x = torch.from_numpy(feats).to(device).requires_grad_(True)
    y = voxelization(x, torch.from_numpy(maps).to(device), 4)
    (y * torch.from_numpy(gv).to(device)).sum().backward()
    assert np.array_equal(x.grad.cpu().numpy(), oracle.voxel_reduce_bwd(gv, maps, 4, n))
    # interpolation (atomic accumulation: tolerance, not bit equality)
    m, q = 90, 400
    vf = rng.normal(size=(m, c)).astype(np.float32)
    idx3 = rng.integers(0, m, size=(q, 3)).astype(np.int32)
    w3 = rng.uniform(size=(q, 3)).astype(np.float32)
    gq = rng.normal(size=(q, c)).astype(np.float32)
    x = torch.from_numpy(vf).to(device).requires_grad_(True)
    y = three_interpolate(x, torch.from_numpy(idx3).to(device), torch.from_numpy(w3).to(device))
    (y * torch.from_numpy(gq).to(device)).sum().backward()
    assert rel_l2(x.grad.cpu().numpy(), oracle.three_interp_bwd(gq, idx3, w3, m)) < REL_L2


def test_point2voxel_passes_gradients_to_the_point_features(device):
    """Voxel means are differentiable in the point features (the reference keeps them in the
    autograd graph through its boolean-mask indexing, voxelize.py:60-83, and voxelize_bp):
    a point inside the grid receives gv[its voxel] / (points in the voxel), a dropped one 0."""
    from ss_conv.sp_ops.voxelize import Point2Voxel
    pts, feats, ids = synth.make_clouds(3, 400, seed=8, channels=5)
    pts = pts * 1.2  # part of every cloud falls outside
    grid = 8
    unit = np.float32(2.0 / grid)
    x = torch.from_numpy(feats).to(device).requires_grad_(True)
    vp, st, vi, _ = Point2Voxel([grid] * 3, [2.0 / grid] * 3)(
        torch.from_numpy(pts).to(device), x, torch.from_numpy(ids).to(device))
    gv = torch.randn_like(st.features)
    st.features.backward(gv)
    half = np.float32(0.5) * (np.float32(grid) * unit)
    inside = (np.abs(pts) > half).sum(1) == 0
    assert inside.sum() == vp.shape[0] and 0 < inside.sum() < len(ids)
    cells = ((pts[inside] + half) / unit).astype(np.int32)
    keys = ((ids[inside] * (grid + 1) + cells[:, 0]) * (grid + 1) + cells[:, 1]) * (grid + 1) + cells[:, 2]
    vox = st.indices.cpu().numpy().astype(np.int64)
    vkeys = ((vox[:, 0] * (grid + 1) + vox[:, 1]) * (grid + 1) + vox[:, 2]) * (grid + 1) + vox[:, 3]
    inv = np.searchsorted(vkeys, keys)
    assert np.array_equal(vkeys[inv], keys)
    counts = np.bincount(inv, minlength=len(vkeys)).astype(np.float32)
    want = np.zeros_like(feats)
    want[inside] = gv.cpu().numpy()[inv] / counts[inv][:, None]
    assert x.grad is not None
    assert rel_l2(x.grad.cpu().numpy(), want) < 1e-6


def test_downsampling_block(oracle, device):
    """Strided convolution followed by MaxPool and AvgPool (k=2, s=2)."""
    import torch.nn.functional as F
    from ss_conv.convolution import Convolution
    from ss_conv.pool import MaxPool, AvgPool
    from ss_conv.sp_ops.voxelize import Point2Voxel
    torch.manual_seed(2)
    pts, feats, ids = synth.make_clouds(2, 400, seed=9, channels=4)
    grid = 16
    conv = Convolution([(4, 0)], [(2, 0), (2, 1)], 3, stride=2, padding=1).to(device).eval()
    _, st, _, _ = Point2Voxel([grid] * 3, [2.0 / grid] * 3)(
        *[torch.from_numpy(x).to(device) for x in (pts, feats, ids)])
    with torch.no_grad():
        y = conv(st)
        mx = MaxPool(2, 2)(y)
        av = AvgPool(2, 2)(y)
    assert list(y.spatial_shape) == [8, 8, 8] and list(mx.spatial_shape) == [4, 4, 4]
    dy = y.dense().cpu()
    assert rel_l2(mx.dense().cpu().numpy(), F.max_pool3d(F.relu(dy), 2, 2).numpy()) < 1e-6
    assert rel_l2(av.dense().cpu().numpy(), F.avg_pool3d(dy, 2, 2).numpy()) < 1e-6


def test_submanifold_reuse_and_inverse(oracle, device):
    """subm=True keeps the active set (dense conv3d sampled at the input sites), layers
    sharing an indice_key reuse one rulebook, and an inverse convolution maps a strided
    layer's output back onto the sites of its input (sp_ops/conv.py:124-136)."""
    import torch.nn.functional as F
    from ss_conv.convolution import Convolution
    from ss_conv.sp_ops.tensor import SparseTensor
    torch.manual_seed(4)
    rng = np.random.default_rng(8)
    grid, n = 10, 300
    idx = random_voxels(rng, 2, grid, n)
    rs = [(4, 0), (2, 1)]
    feats = torch.from_numpy(rng.normal(size=(n, 10)).astype(np.float32)).to(device)
    x = SparseTensor(feats, torch.from_numpy(idx).to(device), [grid] * 3, 2)
    a = Convolution(rs, rs, 3, padding=1, subm=True, indice_key="s1").to(device).eval()
    b = Convolution(rs, rs, 3, padding=1, subm=True, indice_key="s1").to(device).eval()
    with torch.no_grad():
        y = a(x)
        assert list(x.indice_dict.keys()) == ["s1"]
        pairs_first = x.indice_dict["s1"][2]
        z = b(y)
        assert z.indice_dict["s1"][2] is pairs_first  # the rulebook was not rebuilt
    assert torch.equal(y.indices, x.indices) and torch.equal(z.indices, x.indices)
    want = F.conv3d(x.dense().cpu().double(), a.kernel().detach().cpu().double(), padding=1)
    t = torch.from_numpy(idx).long()
    assert rel_l2(y.features.cpu().numpy(), want[t[:, 0], :, t[:, 1], t[:, 2], t[:, 3]].numpy()) \
        < REL_L2
    # strided layer and its inverse
    down = Convolution(rs, rs, 3, stride=2, padding=1, indice_key="d1").to(device).eval()
    up = Convolution(rs, rs, 3, indice_key="d1", inverse=True).to(device).eval()
    with torch.no_grad():
        d = down(z)
        u = up(d)
    assert torch.equal(u.indices, x.indices) and list(u.spatial_shape) == [grid] * 3
    # the inverse convolution is the transpose of the strided one over the same pairs
    o_idx, o_pairs, o_num = oracle.canonicalize(*oracle.rulebook(idx, 2, [grid] * 3, 3, 2, 1))
    w_up = up.kernel().detach().permute(2, 3, 4, 1, 0).reshape(27, 10, 10).cpu().numpy()
    ref = oracle.conv_fwd(d.features.cpu().numpy(), w_up, o_pairs, o_num, n, inverse=True,
                          matmul=np.matmul)
    assert rel_l2(u.features.cpu().numpy(), ref) < REL_L2


def test_training_step_end_to_end(device):
    """Point2Voxel -> Convolution -> BatchNorm -> ReLU -> strided Convolution -> MaxPool ->
    GlobalAvgPool + Voxel2Point, loss.backward(), one SGD step: every parameter receives
    a finite gradient and the loss of the same batch goes down."""
    from ss_conv.batchnorm import BatchNorm
    from ss_conv.convolution import Convolution
    from ss_conv.pool import MaxPool, GlobalAvgPool
    from ss_conv.sp_ops.voxelize import Point2Voxel, Voxel2Point
    torch.manual_seed(3)
    rs_in = [(4, 0)]
    rs_conv = [(12, 0)]  # scalar fields only, so that a plain ReLU is equivariant
    pts, feats, ids = synth.make_clouds(2, 400, seed=12, channels=4)
    grid = 12
    conv = Convolution(rs_in, rs_conv, 3, stride=1, padding=1).to(device)
    bn = BatchNorm(rs_conv).to(device)
    conv2 = Convolution(rs_conv, [(8, 0)], 3, stride=2, padding=1).to(device)
    params = list(conv.parameters()) + list(bn.parameters()) + list(conv2.parameters())
    opt = torch.optim.SGD(params, lr=1e-2)
    dp, df, di = [torch.from_numpy(x).to(device) for x in (pts, feats, ids)]
    target = torch.randn(2, 8, device=device)

    def loss_fn():
        vp, st, vi, _ = Point2Voxel([grid] * 3, [2.0 / grid] * 3)(dp, df.clone().requires_grad_(True), di)
        y = bn(conv(st))
        y.features = torch.relu(y.features)
        y = MaxPool(2, 2)(conv2(y))
        pooled = GlobalAvgPool()(y)
        back = Voxel2Point(unit_voxel_extent=[2.0 / 3] * 3)(y, vp, vi)
        return ((pooled - target) ** 2).mean() + 1e-3 * (back ** 2).mean()

    conv.train(); conv2.train(); bn.train()
    l0 = loss_fn()
    opt.zero_grad()
    l0.backward()
    for p in params:
        assert p.grad is not None and torch.isfinite(p.grad).all()
    assert float(conv.kernel.weight.grad.abs().sum()) > 0
    opt.step()
    l1 = loss_fn()
    assert l1.item() < l0.item()


def test_cpu_tensor_is_rejected(device):
    from ss_conv import _ext
    with pytest.raises(RuntimeError):
        _ext.get_indice_pairs_3d(torch.zeros((1, 4), dtype=torch.int32), 1, [8] * 3, [8] * 3,
                                 [3] * 3, [1] * 3, [1] * 3, [1] * 3, [0] * 3, 0, 0)


# ---- SE(3) batch norm + gated non-linearity ---------------------------------------------------
BNACT_CASES = [
    # Rs of the activation, rows, layers ("bn", "act", "fused"), training
    ([(4, 0), (4, 1), (4, 2)], 1000, "fused", True),
    ([(4, 0), (4, 1), (4, 2)], 1000, "fused", False),
    ([(4, 0), (4, 1), (4, 2)], 777, "bn", True),
    ([(4, 0), (4, 1), (4, 2)], 777, "bn", False),
    ([(4, 0), (4, 1), (4, 2)], 777, "act", True),
    ([(3, 0), (2, 1), (2, 2)], 333, "fused", True),            # 23 columns: the scalar-width kernels
    ([(3, 0), (2, 1), (2, 2)], 333, "act", True),
    ([(8, 0), (8, 1), (8, 2), (8, 3), (8, 4)], 5000, "fused", True),   # 232 columns
    ([(32, 0), (32, 1), (32, 2), (32, 3)], 3000, "fused", True),       # 608 columns: several passes
    ([(2, 0), (1, 1)], 3, "fused", True),
    ([(16, 0)], 100, "fused", True),                                   # scalars only, no gates
]


def _bnact_modules(Rs, acts, device, rng):
    from ss_conv.activation import Activation
    from ss_conv.batchnorm import BatchNorm
    n_gates = sum(m for m, _ in Rs[1:])
    Rs_bn = list(Rs) + ([(n_gates, 0)] if n_gates else [])
    bn = BatchNorm(Rs_bn).to(device)
    act = Activation(Rs, acts).to(device)
    with torch.no_grad():
        for p in list(bn.parameters()) + list(act.parameters()):
            p.copy_(torch.from_numpy(rng.normal(size=tuple(p.shape)).astype(np.float32)))
        bn.weight.add_(1.0)
        bn.running_mean.copy_(torch.from_numpy(rng.normal(size=tuple(bn.running_mean.shape)).astype(np.float32)))
        bn.running_var.copy_(torch.from_numpy(rng.uniform(0.5, 2, size=tuple(bn.running_var.shape)).astype(np.float32)))
    return bn, act, Rs_bn


@pytest.mark.parametrize("case", BNACT_CASES)
def test_batchnorm_activation_match_oracle(case, oracle, device):
    from ss_conv.fused import BatchNormActivation
    from ss_conv.sp_ops.tensor import SparseTensor
    Rs, n, which, training = case
    print("case", case, flush=True)
    rng = np.random.default_rng(len(Rs) * 1000 + n)
    bn, act, Rs_bn = _bnact_modules(Rs, (torch.relu, torch.sigmoid), device, rng)
    c_in = sum(m * (2 * l + 1) for m, l in Rs_bn)
    x_np = (rng.normal(size=(n, c_in)) * 2 + 0.3).astype(np.float32)
    x = torch.from_numpy(x_np).to(device).requires_grad_(True)
    module = {"bn": bn, "act": act, "fused": BatchNormActivation(bn, act)}[which]
    module.train(training)
    running = (bn.running_mean.cpu().numpy().copy(), bn.running_var.cpu().numpy().copy())
    st = SparseTensor(x, torch.zeros(n, 4, dtype=torch.int32, device=device), [4, 4, 4], 1)
    # the layers must run on the library's kernels here, not on their torch code
    from ss_conv import _ext
    calls = {"fwd": 0, "bwd": 0}
    real_fwd, real_bwd = _ext.bnact_forward, _ext.bnact_backward

    def counted_fwd(*a, **k):
        calls["fwd"] += 1
        return real_fwd(*a, **k)

    def counted_bwd(*a, **k):
        calls["bwd"] += 1
        return real_bwd(*a, **k)

    _ext.bnact_forward, _ext.bnact_backward = counted_fwd, counted_bwd
    try:
        y = module(st).features
        dy_np = rng.normal(size=tuple(y.shape)).astype(np.float32)
        y.backward(torch.from_numpy(dy_np).to(device))
        torch.cuda.synchronize()
    finally:
        _ext.bnact_forward, _ext.bnact_backward = real_fwd, real_bwd
    assert calls == {"fwd": 1, "bwd": 1}, calls

    sb = act.scalar_act.bias if act.scalar_act is not None else None
    gb = act.gate_act.bias if act.gate_act is not None else None
    as_np = lambda t: None if t is None else t.detach().cpu().numpy()  # noqa: E731
    params = dict(weight=as_np(bn.weight), bias=as_np(bn.bias), scalar_bias=as_np(sb),
                  gate_bias=as_np(gb))
    use_bn, use_act = which in ("bn", "fused"), which in ("act", "fused")
    kw = dict(training=training, act_scalar="relu", act_gate="sigmoid" if gb is not None else None,
              running=running)
    args = (Rs_bn if use_bn else None, Rs if use_act else None, params)
    want = oracle.bn_gate_fwd(x_np, *args, **kw)
    assert rel_l2(y.detach().cpu().numpy(), want) < REL_L2
    grads = oracle.bn_gate_bwd(x_np, dy_np, *args, **kw)
    assert rel_l2(x.grad.cpu().numpy(), grads["x"]) < REL_L2
    got = dict(weight=bn.weight.grad, bias=bn.bias.grad, scalar_bias=None if sb is None else sb.grad,
               gate_bias=None if gb is None else gb.grad)
    for k, g in grads.items():
        if k == "x":
            continue
        assert got[k] is not None, k
        assert rel_l2(got[k].cpu().numpy(), g) < 1e-4, k   # sums over all rows in fp32
    if use_bn and training:
        _, rm, rv = oracle.batchnorm_fwd(x_np, Rs_bn, params["weight"], params["bias"], *running)
        assert rel_l2(bn.running_mean.cpu().numpy(), rm) < REL_L2
        assert rel_l2(bn.running_var.cpu().numpy(), rv) < REL_L2


def test_batchnorm_activation_other_cases(oracle, device):
    """tanh activations, layers without bias or affine parameters, an activation the kernels
    do not cover (torch code on the GPU), and reproducibility."""
    from ss_conv.activation import Activation
    from ss_conv.batchnorm import BatchNorm
    from ss_conv.fused import BatchNormActivation
    from ss_conv.sp_ops.tensor import SparseTensor
    rng = np.random.default_rng(77)
    Rs = [(4, 0), (3, 1), (2, 2)]
    Rs_bn = Rs + [(5, 0)]
    n, c_in = 600, 4 + 9 + 10 + 5
    x_np = rng.normal(size=(n, c_in)).astype(np.float32)
    idx = torch.zeros(n, 4, dtype=torch.int32, device=device)

    def run(bn, act):
        m = BatchNormActivation(bn, act).to(device).train()
        st = SparseTensor(torch.from_numpy(x_np).to(device), idx, [4, 4, 4], 1)
        return m(st).features.detach().cpu().numpy()

    y = run(BatchNorm(Rs_bn, affine=False), Activation(Rs, (torch.tanh, torch.tanh), bias=False))
    want = oracle.bn_gate_fwd(x_np, Rs_bn, Rs, {}, act_scalar="tanh", act_gate="tanh")
    assert rel_l2(y, want) < REL_L2
    y = run(BatchNorm(Rs_bn), Activation(Rs, (None, torch.sigmoid)))
    want = oracle.bn_gate_fwd(x_np, Rs_bn, Rs, {}, act_scalar=None, act_gate="sigmoid")
    assert rel_l2(y, want) < REL_L2
    y1 = run(BatchNorm(Rs_bn), Activation(Rs, (torch.relu, torch.sigmoid)))
    y2 = run(BatchNorm(Rs_bn), Activation(Rs, (torch.relu, torch.sigmoid)))
    assert np.array_equal(y1, y2)
    # softplus is not one of the kernels' activations: the layers fall back to torch ops
    soft = torch.nn.functional.softplus
    act = Activation(Rs, (soft, torch.sigmoid))
    assert not act._kernel_ok
    y = run(BatchNorm(Rs_bn), act)
    z, _, _ = oracle.batchnorm_fwd(x_np, Rs_bn)
    z[:, :4] = np.log1p(np.exp(z[:, :4]))
    want = oracle.gate_fwd(z, Rs, act_scalar=None, act_gate="sigmoid")
    assert rel_l2(y, want) < REL_L2


def test_conv_order_promise_follows_the_input_order(oracle, device):
    """The rulebook reports whether its input rows came in key order; only then may the
    convolution skip its own order check.  Both ways must give the oracle's result."""
    from ss_conv import _ext
    from ss_conv.sp_ops.ops import get_indice_pairs
    rng = np.random.default_rng(21)
    n, grid, cin, cout, k = 400, 10, 32, 48, 3
    idx_sorted = random_voxels(rng, 2, grid, n)
    feats = rng.normal(size=(n, cin)).astype(np.float32)
    w = (rng.normal(size=(k ** 3, cin, cout)) / np.sqrt(27 * cin)).astype(np.float32)
    perm = rng.permutation(n)
    for idx, f, want_flag in ((idx_sorted, feats, True), (idx_sorted[perm], feats[perm], False)):
        t = torch.from_numpy(idx).to(device)
        o_idx, pairs, num = get_indice_pairs(t, 2, [grid] * 3, k, 1, 1, 1, 0, False)
        assert _ext.rulebook_meta(pairs).canonical == (want_flag, True)
        out = _ext.indice_conv_fp32(torch.from_numpy(f).to(device),
                                    torch.from_numpy(w).to(device).reshape(k, k, k, cin, cout),
                                    pairs, num, o_idx.shape[0], 0, 0)
        r_idx, r_pairs, r_num = oracle.canonicalize(*oracle.rulebook(idx, 2, [grid] * 3, k, 1, 1))
        # the oracle numbers pairs by input row as given, outputs by key: same convention
        ref = oracle.conv_fwd(f, w, r_pairs, r_num, r_idx.shape[0], matmul=np.matmul)
        assert np.array_equal(o_idx.cpu().numpy(), r_idx)
        assert rel_l2(out.cpu().numpy(), ref) < REL_L2
        # the input gradient accumulates into input rows: always in order
        go = rng.normal(size=(r_idx.shape[0], cout)).astype(np.float32)
        gi, _ = _ext.indice_conv_backward_fp32(
            torch.from_numpy(f).to(device),
            torch.from_numpy(w).to(device).reshape(k, k, k, cin, cout),
            torch.from_numpy(go).to(device), pairs, num, 0, 0)
        want, _ = oracle.conv_bwd(f, w, go, r_pairs, r_num)
        assert rel_l2(gi.cpu().numpy(), want) < REL_L2


def test_conv_call_replays_in_a_hip_graph(device):
    """The convolution call enqueues kernels only (no host read, no memset), so a captured
    graph of it can be replayed: every replay, with eager work and synchronisations in
    between, gives the bits of the eager call on the same buffers."""
    from ss_conv import _ext
    rng = np.random.default_rng(31)
    grid, n, cin, cout = 16, 2500, 64, 96
    idx = random_voxels(rng, 2, grid, n)
    g_idx, g_pairs, g_num = [torch.from_numpy(x).to(device) for x in
                             gpu_rulebook(idx, 2, grid, 3, 1, 1)]
    n_out = g_idx.shape[0]
    f = torch.randn((n, cin), device=device)
    w = torch.randn((3, 3, 3, cin, cout), device=device) / (27 * cin) ** 0.5
    eager = _ext.indice_conv_fp32(f, w, g_pairs, g_num, n_out, 0, 0)  # also the warm-up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            captured = _ext.indice_conv_fp32(f, w, g_pairs, g_num, n_out, 0, 0)
    torch.cuda.current_stream().wait_stream(side)
    for trial in range(4):
        if trial:  # new values in the captured input buffers, eager result for them
            f.copy_(torch.randn((n, cin), device=device))
            w.copy_(torch.randn((3, 3, 3, cin, cout), device=device) / (27 * cin) ** 0.5)
            eager = _ext.indice_conv_fp32(f, w, g_pairs, g_num, n_out, 0, 0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured, eager), trial


@pytest.mark.parametrize("rs", [[(8, 0), (8, 1), (8, 2), (8, 3)], [(3, 0), (2, 2)], [(5, 1)]])
def test_dropout_kernel_matches_expanded_masks(rs, device):
    """Dropout on the GPU: masks drawn as the reference draws them (ss_conv/dropout.py:32-45),
    multiplied in by ssc_field_scale_f32 -- same bits as the expanded product, forward and
    backward."""
    from ss_conv.dropout import Dropout
    from ss_conv.sp_ops.tensor import SparseTensor
    n = 3000
    c = sum(m * (2 * l + 1) for m, l in rs)
    drop = Dropout(rs, p=0.4).to(device).train()
    x = torch.randn(n, c, device=device, requires_grad=True)
    idx = torch.zeros((n, 4), dtype=torch.int32, device=device)
    state = torch.cuda.get_rng_state(device)
    y = drop(SparseTensor(x, idx, [4, 4, 4], 1)).features
    torch.cuda.set_rng_state(state, device)
    noises = []
    for m, l in rs:
        noise = x.new_empty(n, m).bernoulli_(0.6).div_(0.6)
        noises.append(noise.unsqueeze(2).expand(-1, -1, 2 * l + 1).contiguous().view(n, -1))
    noise = torch.cat(noises, dim=1)
    assert torch.equal(y, x.detach() * noise)
    g = torch.randn_like(y)
    y.backward(g)
    assert torch.equal(x.grad, g * noise)
    drop.eval()
    t = SparseTensor(x.detach(), idx, [4, 4, 4], 1)
    assert drop(t).features is t.features


def test_backbone_forward_matches_oracle(oracle, device):
    """The fourth benchmark configuration at reduced size: Point2Voxel -> four stages of
    [Convolution k3 -> BatchNorm -> gated Activation] with irreps (8,8,8,8) -> (16,...) ->
    (32,...) -> (32,...), stride 2 at stages 2 and 3 -> GlobalAvgPool and Voxel2Point, in
    training mode (batch statistics), against the oracle's composition of the same steps."""
    from ss_conv.activation import Activation
    from ss_conv.batchnorm import BatchNorm
    from ss_conv.convolution import Convolution
    from ss_conv.fused import BatchNormActivation
    from ss_conv.pool import GlobalAvgPool
    from ss_conv.sp_ops.voxelize import Point2Voxel, Voxel2Point
    torch.manual_seed(3)
    batch, grid = 3, 24
    pts, feats, ids = synth.make_clouds(batch, 700, seed=10, channels=3)
    rs_in = [(3, 0)]
    stages = [(synth.irreps(8, 3), 1), (synth.irreps(16, 3), 2), (synth.irreps(32, 3), 2),
              (synth.irreps(32, 3), 1)]
    p2v = Point2Voxel([grid] * 3, [2.0 / grid] * 3)
    vp, st, vi, _ = p2v(*[torch.from_numpy(x).to(device) for x in (pts, feats, ids)])
    # oracle side starts from the same voxels
    o_idx = st.indices.cpu().numpy()
    o_feat = st.features.cpu().numpy().astype(np.float64)
    shape = [grid] * 3
    x = st
    for si, (rs, stride) in enumerate(stages):
        n_gates = sum(m for m, _ in rs[1:])
        rs_gated = rs + [(n_gates, 0)]
        conv = Convolution(rs_in, rs_gated, 3, stride=stride, padding=1).to(device).train()
        block = BatchNormActivation(BatchNorm(rs_gated), Activation(rs, (torch.relu, torch.sigmoid)))
        block = block.to(device).train()
        with torch.no_grad():
            for p in block.parameters():
                p.add_(torch.randn_like(p) * 0.3)
            x = block(conv(x))
        # oracle: rulebook, convolution with the layer's synthesised kernel, batch norm, gate
        cin = sum(m * (2 * l + 1) for m, l in rs_in)
        cout = sum(m * (2 * l + 1) for m, l in rs_gated)
        w = conv.kernel().detach().permute(2, 3, 4, 1, 0).reshape(27, cin, cout).cpu().numpy()
        r_idx, r_pairs, r_num, r_shape = oracle.rulebook(o_idx, batch, shape, 3, stride, 1)
        r_idx, r_pairs, r_num = oracle.canonicalize(r_idx, r_pairs, r_num, r_shape)
        y = oracle.conv_fwd(o_feat.astype(np.float32), w, r_pairs, r_num, r_idx.shape[0],
                            matmul=np.matmul)
        as_np = lambda t: t.detach().cpu().numpy()  # noqa: E731
        params = dict(weight=as_np(block.bn.weight), bias=as_np(block.bn.bias),
                      scalar_bias=as_np(block.act.scalar_act.bias),
                      gate_bias=as_np(block.act.gate_act.bias))
        o_feat = oracle.bn_gate_fwd(y, rs_gated, rs, params, training=True)
        o_idx, shape, rs_in = r_idx, list(r_shape), rs
        assert np.array_equal(x.indices.cpu().numpy(), o_idx), si
        err = rel_l2(x.features.cpu().numpy(), o_feat)
        print("stage", si, "rows", o_idx.shape[0], "rel-l2", err, flush=True)
        assert err < REL_L2, (si, err)
    # heads: per-cloud mean of the voxel features, and the features read back at the points
    offs = x.get_offsets().int().contiguous()
    pooled = GlobalAvgPool()(x.features.contiguous(), offs).cpu().numpy()
    want = oracle.segment_avg(o_feat.astype(np.float32), offs.cpu().numpy())
    assert rel_l2(pooled, want) < REL_L2
    v2p = Voxel2Point(unit_voxel_extent=[2.0 / s for s in shape])
    at_points = v2p(x, vp, vi).cpu().numpy()
    want = oracle.voxel2point(o_idx, o_feat.astype(np.float32), shape, vp.cpu().numpy(),
                              vi.cpu().numpy(), unit_voxel_extent=[2.0 / s for s in shape])[0]
    assert rel_l2(at_points, want) < REL_L2


def test_rows_outside_the_grid_are_reported(device):
    """A batch index beyond batch_size (regular rulebook), a coordinate equal to the shape
    (submanifold rulebook) and a row outside dims (unique rows) would address memory outside
    the bit table: the rows are skipped on the device and the call raises ValueError."""
    from ss_conv import _ext
    from ss_conv.sp_ops.ops import get_indice_pairs
    rng = np.random.default_rng(5)
    idx = random_voxels(rng, 2, 8, 100)
    bad_batch = idx.copy()
    bad_batch[17, 0] = 2
    with pytest.raises(ValueError, match="outside the grid"):
        get_indice_pairs(torch.from_numpy(bad_batch).to(device), 2, [8] * 3, 3, 1, 1, 1, 0, False)
    negative = idx.copy()
    negative[3, 0] = -1
    with pytest.raises(ValueError, match="outside the grid"):
        get_indice_pairs(torch.from_numpy(negative).to(device), 2, [8] * 3, 3, 2, 1, 1, 0, False)
    on_the_face = idx.copy()
    on_the_face[40, 2] = 8
    with pytest.raises(ValueError, match="outside the grid"):
        get_indice_pairs(torch.from_numpy(on_the_face).to(device), 2, [8] * 3, 3, 1, 1, 1, 0, True)
    # the same row is fine for a regular convolution: its taps are clipped to the grid
    t = torch.from_numpy(on_the_face).to(device)
    o_idx, pairs, num = get_indice_pairs(t, 2, [8] * 3, 3, 1, 1, 1, 0, False)
    assert int(o_idx[:, 1:].max()) <= 7 and int(o_idx[:, 1:].min()) >= 0
    with pytest.raises(ValueError, match="outside the grid"):
        _ext.unique_rows(t, [2, 8, 8, 8])
    with pytest.raises(ValueError, match="outside the grid"):
        _ext.unique_rows_max(t, [2, 8, 8, 8])
    u, inv, cnt, largest = _ext.unique_rows_max(t, [2, 9, 9, 9])
    assert u.shape[0] == 100 and largest == 1
    # the good rulebook still works after the failed calls
    o2, p2, n2 = get_indice_pairs(torch.from_numpy(idx).to(device), 2, [8] * 3, 3, 1, 1, 1, 0, False)
    assert int(n2.sum()) > 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("subm", [False, True])
def test_cached_plan_gives_identical_results(subm, oracle, device):
    """Convolutions over one rulebook share the row-block schedule: the second call of a
    (direction, channel counts) combination reuses the plan built by the first and must
    return the same bits, as must the one-call entry point; forward, input gradient and a
    layer with other channel counts each keep their own plan; an in-place edit of the pairs
    drops the promise."""
    from ss_conv import _ext
    from ss_conv.sp_ops.ops import get_indice_pairs
    rng = np.random.default_rng(31)
    n, grid, cin, cout, k = 3000, 20, 64, 96, 3
    idx = random_voxels(rng, 2, grid, n)
    t = torch.from_numpy(idx).to(device)
    o_idx, pairs, num = get_indice_pairs(t, 2, [grid] * 3, k, 1, 1, 1, 0, subm)
    n_out = o_idx.shape[0]
    meta = _ext.rulebook_meta(pairs)
    assert meta is not None and meta.canonical == (True, True) and len(meta.plans) == 0
    f = torch.randn((n, cin), device=device)
    w = torch.randn((k, k, k, cin, cout), device=device) / (27 * cin) ** 0.5
    go = torch.randn((n_out, cout), device=device)
    out1 = _ext.indice_conv_fp32(f, w, pairs, num, n_out, 0, int(subm))
    assert len(meta.plans) == 1
    out2 = _ext.indice_conv_fp32(f, w, pairs, num, n_out, 0, int(subm))
    assert len(meta.plans) == 1 and torch.equal(out1, out2)
    # a clone carries no promise: order check, schedule and kernel in one call
    out3 = _ext.indice_conv_fp32(f, w, pairs.clone(), num, n_out, 0, int(subm))
    assert torch.equal(out1, out3)
    r_idx, r_pairs, r_num, r_shape = oracle.rulebook(idx, 2, [grid] * 3, k, 1, 1, 1, subm)
    if not subm:
        r_idx, r_pairs, r_num = oracle.canonicalize(r_idx, r_pairs, r_num, r_shape)
    ref = oracle.conv_fwd(f.cpu().numpy(), w.reshape(27, cin, cout).cpu().numpy(), r_pairs, r_num,
                          n_out, matmul=np.matmul)
    assert rel_l2(out1.cpu().numpy(), ref) < REL_L2
    # new filter values, same plan (the filters are packed again)
    w2 = w * 0.5
    assert rel_l2(_ext.indice_conv_fp32(f, w2, pairs, num, n_out, 0, int(subm)).cpu().numpy(),
                  0.5 * ref) < REL_L2
    # filters changed in place: the packed copy kept on the tensor must not be reused
    w2.mul_(4.0)
    assert rel_l2(_ext.indice_conv_fp32(f, w2, pairs, num, n_out, 0, int(subm)).cpu().numpy(),
                  2.0 * ref) < REL_L2
    gi1, gw1 = _ext.indice_conv_backward_fp32(f, w, go, pairs, num, 0, int(subm))
    assert len(meta.plans) == 2
    gi2, gw2 = _ext.indice_conv_backward_fp32(f, w, go, pairs, num, 0, int(subm))
    assert len(meta.plans) == 2 and torch.equal(gi1, gi2) and torch.equal(gw1, gw2)
    gi3, gw3 = _ext.indice_conv_backward_fp32(f, w, go, pairs.clone(), num, 0, int(subm))
    assert torch.equal(gi1, gi3) and torch.equal(gw1, gw3)
    ri, rw = oracle.conv_bwd(f.cpu().numpy(), w.reshape(27, cin, cout).cpu().numpy(),
                             go.cpu().numpy(), r_pairs, r_num)
    assert rel_l2(gi1.cpu().numpy(), ri) < REL_L2
    # other channel counts over the same rulebook: a plan of their own
    fh = torch.randn((n, 24), device=device)
    wh = torch.randn((k, k, k, 24, 40), device=device)
    oh = _ext.indice_conv_fp32(fh, wh, pairs, num, n_out, 0, int(subm))
    assert len(meta.plans) == 3
    assert torch.equal(oh, _ext.indice_conv_fp32(fh, wh, pairs.clone(), num, n_out, 0, int(subm)))
    # half precision over the same rulebook
    o16 = _ext.indice_conv_half(f.half(), w.half(), pairs, num, n_out, 0, int(subm))
    assert len(meta.plans) == 4
    assert torch.equal(o16, _ext.indice_conv_half(f.half(), w.half(), pairs.clone(), num, n_out, 0,
                                                  int(subm)))
    # an in-place edit of the pairs: the promise and the plans no longer count
    pairs[:, :, 0] += 0
    assert _ext.rulebook_meta(pairs) is None
    assert torch.equal(out1, _ext.indice_conv_fp32(f, w, pairs, num, n_out, 0, int(subm)))


def test_layer_reuses_plan_under_an_indice_key(device):
    """Two submanifold layers under one indice_key, and a second forward of the same layer in
    evaluation mode: the rulebook, the plan and the packed filters are built once."""
    from ss_conv import _ext
    from ss_conv.sp_ops.conv import SparseConvolution
    from ss_conv.sp_ops.tensor import SparseTensor
    rng = np.random.default_rng(8)
    idx = random_voxels(rng, 2, 16, 1500)
    t = torch.from_numpy(idx).to(device)
    torch.manual_seed(0)
    a = SparseConvolution(3, 32, 32, 3, subm=True, bias=False, indice_key="s").to(device).eval()
    b = SparseConvolution(3, 32, 32, 3, subm=True, bias=False, indice_key="s").to(device).eval()
    x = torch.randn((idx.shape[0], 32), device=device)
    with torch.no_grad():
        st = SparseTensor(x, t, [16] * 3, 2)
        y = b(a(st))
        pairs = st.indice_dict["s"][2]
        meta = _ext.rulebook_meta(pairs)
        assert meta is not None and len(meta.plans) == 1
        packed_a = a.weight._ssc_packed[1]
        st2 = SparseTensor(x, t, [16] * 3, 2)
        st2.indice_dict = st.indice_dict
        y2 = b(a(st2))
        assert len(meta.plans) == 1 and a.weight._ssc_packed[1] is packed_a
        assert torch.equal(y.features, y2.features)
        # the layers one by one through the one-call entry point
        z = _ext.indice_conv_fp32(x, a.weight, pairs.clone(), st.indice_dict["s"][3],
                                  idx.shape[0], 0, 1)
        z = _ext.indice_conv_fp32(z, b.weight, pairs.clone(), st.indice_dict["s"][3],
                                  idx.shape[0], 0, 1)
        assert torch.equal(z, y.features)


def test_cloned_pairs_keep_their_plan(device):
    """The plans of a rulebook belong to the SparseTensor (plan_dict, keyed like indice_dict),
    not to one tensor object: pairs that come back as a clone under the same key are bound
    to the same plans after one comparison, pairs with other contents are not, and the plans
    kept per rulebook are evicted least recently used first."""
    from ss_conv import _ext
    from ss_conv.sp_ops.conv import SparseConvolution
    from ss_conv.sp_ops.tensor import SparseTensor
    rng = np.random.default_rng(3)
    idx = random_voxels(rng, 2, 12, 700)
    t = torch.from_numpy(idx).to(device)
    torch.manual_seed(5)
    layer = SparseConvolution(3, 16, 24, 3, stride=1, padding=1, subm=True, bias=False,
                              indice_key="s").to(device)
    x = torch.randn((idx.shape[0], 16), device=device)
    with torch.no_grad():
        st = SparseTensor(x, t, [12] * 3, 2)
        y = layer(st)
        meta = st.plan_dict["s"]
        assert y.plan_dict is st.plan_dict and len(meta.plans) == 1
        plan = next(iter(meta.plans.values()))
        # the same rulebook as other tensor objects
        outids, ind, pairs, num, shape = st.indice_dict["s"]
        st2 = SparseTensor(x, t, [12] * 3, 2)
        st2.indice_dict = {"s": (outids, ind, pairs.clone(), num.clone(), shape)}
        st2.plan_dict = st.plan_dict
        calls = []
        keep = _ext._lib.ssc_conv_plan_build
        _ext._lib.ssc_conv_plan_build = lambda *a: calls.append(1) or keep(*a)
        try:
            y2 = layer(st2)
        finally:
            _ext._lib.ssc_conv_plan_build = keep
        assert not calls and torch.equal(y2.features, y.features)
        assert next(iter(st.plan_dict["s"].plans.values())) is plan
        # other pairs under the key: no binding, the call builds its own schedule
        other = pairs.clone()
        other[0, :, :2] = pairs[0, :, :2].flip(1)  # the same pairs in another order
        st3 = SparseTensor(x, t, [12] * 3, 2)
        st3.indice_dict = {"s": (outids, ind, other, num, shape)}
        st3.plan_dict = st.plan_dict
        y3 = layer(st3)
        assert _ext.rulebook_meta(other) is None
        assert rel_l2(y3.features.cpu().numpy(), y.features.cpu().numpy()) < 1e-6
        # least recently used first
        for c in range(_ext.RulebookMeta.MAX_PLANS + 2):
            meta.put_plan(("k", c), object())
            assert meta.get_plan(("k", 0)) is not None  # kept alive by use
        assert len(meta.plans) == _ext.RulebookMeta.MAX_PLANS
        assert meta.get_plan(("k", 1)) is None and meta.get_plan(("k", 0)) is not None


def test_packed_filters_follow_explicit_invalidation(device):
    """The packed copy of a layer's filters is reused while the weight's version counter
    stands still; an edit through .data does not move it, forget_packed does."""
    from ss_conv import _ext
    from ss_conv.sp_ops.conv import SparseConvolution
    from ss_conv.sp_ops.tensor import SparseTensor
    rng = np.random.default_rng(4)
    idx = random_voxels(rng, 1, 10, 300)
    t = torch.from_numpy(idx).to(device)
    torch.manual_seed(6)
    layer = SparseConvolution(3, 8, 8, 3, stride=1, padding=1, bias=False).to(device).eval()
    x = torch.randn((idx.shape[0], 8), device=device)
    with torch.no_grad():
        y0 = layer(SparseTensor(x, t, [10] * 3, 1)).features
        layer.weight.mul_(2.0)  # moves the version counter: repacked
        y1 = layer(SparseTensor(x, t, [10] * 3, 1)).features
        assert torch.allclose(y1, 2.0 * y0, rtol=1e-6, atol=1e-6)
        layer.weight.data.mul_(0.5)  # does not: the stale copy is used until told
        _ext.forget_packed(layer.weight)
        y2 = layer(SparseTensor(x, t, [10] * 3, 1)).features
        assert torch.allclose(y2, y0, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("subm,stride", [(False, 1), (False, 2), (True, 1)])
def test_fused_rulebook_conv_equals_the_two_calls(subm, stride, device):
    """A layer without a cached rulebook runs rulebook and convolution as one native
    sequence (one autograd node); a layer that finds the rulebook under its indice_key runs
    the convolution alone.  Same rulebook, same output bits, same gradients."""
    from ss_conv.sp_ops.conv import SparseConvolution
    from ss_conv.sp_ops.ops import get_indice_pairs
    from ss_conv.sp_ops.functional import indice_conv, indice_subm_conv
    from ss_conv.sp_ops.tensor import SparseTensor
    rng = np.random.default_rng(77)
    idx = random_voxels(rng, 3, 14, 900)
    t = torch.from_numpy(idx).to(device)
    torch.manual_seed(1)
    layer = SparseConvolution(3, 24, 40, 3, stride=stride, padding=1, subm=subm, bias=True,
                              indice_key="k").to(device)
    x1 = torch.randn((idx.shape[0], 24), device=device, requires_grad=True)
    st = SparseTensor(x1, t, [14] * 3, 3)
    y1 = layer(st)                      # fused: builds the rulebook
    outids, _, pairs, num, _ = st.indice_dict["k"]
    g_idx, g_pairs, g_num = get_indice_pairs(t, 3, [14] * 3, 3, stride, 1, 1, 0, subm)
    assert torch.equal(outids, g_idx) and torch.equal(pairs, g_pairs) and torch.equal(num, g_num)
    go = torch.randn_like(y1.features)
    y1.features.backward(go)
    gx1, gw1, gb1 = x1.grad.clone(), layer.weight.grad.clone(), layer.bias.grad.clone()
    layer.zero_grad()
    x2 = x1.detach().clone().requires_grad_(True)
    st2 = SparseTensor(x2, t, [14] * 3, 3)
    st2.indice_dict = st.indice_dict    # cached rulebook: convolution alone
    y2 = layer(st2)
    assert torch.equal(y1.indices, y2.indices) and torch.equal(y1.features, y2.features)
    y2.features.backward(go)
    assert torch.equal(gx1, x2.grad) and torch.equal(gw1, layer.weight.grad)
    assert torch.equal(gb1, layer.bias.grad)
    fn = indice_subm_conv if subm else indice_conv
    y3 = fn(x1.detach(), layer.weight.detach(), g_pairs.clone(), g_num, g_idx.shape[0])
    assert torch.equal(y3 + layer.bias.detach(), y1.features.detach())


@pytest.mark.parametrize("batch,grid,n_vox", [(4, 64, 45000), (2, 32, 45000)])
def test_strided_layer_with_its_plan_cut_by_the_rulebook(batch, grid, n_vox, device):
    """A strided layer's rulebook counts the pairs of every table word while it marks the
    outputs and places the range boundaries of the convolution's plan itself.  Whether the
    outputs outnumber the inputs (a sparse cloud, first case) or not (a dense one, second
    case) decides what the plan looks like -- two ranges to a workgroup or one, at these
    sizes -- and is known only when the rulebook's totals arrive: the rulebook places the
    cut of either plan.  Same rulebook as get_indice_pairs, same output as the convolution
    over those pairs, whose plan comes from its own passes over the pairs (the same sums in
    another order)."""
    from ss_conv.sp_ops.conv import SparseConvolution
    from ss_conv.sp_ops.ops import get_indice_pairs
    from ss_conv.sp_ops.functional import indice_conv
    from ss_conv.sp_ops.tensor import SparseTensor
    rng = np.random.default_rng(31)
    idx = random_voxels(rng, batch, grid, n_vox)
    t = torch.from_numpy(idx).to(device)
    torch.manual_seed(3)
    layer = SparseConvolution(3, 16, 256, 3, stride=2, padding=1, bias=False,
                              indice_key="s").to(device)
    x = torch.randn((idx.shape[0], 16), device=device)
    with torch.no_grad():
        st = SparseTensor(x, t, [grid] * 3, batch)
        y = layer(st)
        outids, _, pairs, num, _ = st.indice_dict["s"]
        g_idx, g_pairs, g_num = get_indice_pairs(t, batch, [grid] * 3, 3, 2, 1, 1, 0, False)
        assert torch.equal(outids, g_idx) and torch.equal(pairs, g_pairs)
        assert torch.equal(num, g_num)
        n_out = g_idx.shape[0]
        assert (n_out > n_vox) == (grid == 64), (n_out, n_vox)
        y2 = indice_conv(x, layer.weight, g_pairs, g_num, n_out)
        assert torch.allclose(y.features, y2, rtol=1e-5, atol=1e-5)
        # against the oracle on a sample of rows: float64 sums over the pairs
        gp = g_pairs.cpu().numpy()
        gn = g_num.cpu().numpy()
        w = layer.weight.detach().cpu().numpy().reshape(27, 16, 256).astype(np.float64)
        xf = x.cpu().numpy().astype(np.float64)
        rows = rng.choice(n_out, size=64, replace=False)
        want = np.zeros((64, 256))
        pos = {int(r): j for j, r in enumerate(rows)}
        for k in range(27):
            o = gp[k, 1, :gn[k]]
            hit = np.nonzero(np.isin(o, rows))[0]
            for h in hit:
                want[pos[int(o[h])]] += xf[gp[k, 0, h]] @ w[k]
        got = y.features[torch.from_numpy(rows).to(device)].cpu().numpy()
        assert np.abs(got - want).max() <= 1e-4 * max(np.abs(want).max(), 1.0)


@pytest.mark.parametrize("seed", [0, 1])
def test_fused_layer_random_geometries(seed, oracle, device):
    """The layer's own sequence -- rulebook, the plan's range boundaries placed by the
    rulebook, convolution -- on geometries of every kind: kernel size, stride, padding and
    dilation differing per axis, grids that are no cubes and whose rows are no whole table
    words, a few thousand voxels, so that a plan has many ranges; sparse and dense clouds
    (outputs more or fewer than inputs).  Rulebook bit-exact against the oracle's, features
    against the oracle's convolution over those pairs."""
    from ss_conv.sp_ops.conv import SparseConvolution
    from ss_conv.sp_ops.tensor import SparseTensor
    rng = np.random.default_rng(1000 + seed)
    done = 0
    while done < 14:
        batch = int(rng.integers(1, 4))
        shape = [int(rng.integers(8, 40)) for _ in range(3)]
        if rng.integers(0, 2):
            shape[2] = int(rng.choice([32, 64]))  # whole table words: the dilation path at stride 1
        ks = [int(rng.integers(1, 4)) for _ in range(3)]
        st = [int(rng.integers(1, 4)) for _ in range(3)]
        if rng.integers(0, 3) == 0:
            st = [1, 1, 1]
        dl = [int(rng.integers(1, 3)) if t == 1 else 1 for t in st]
        pd = [int(rng.integers(0, 3)) for _ in range(3)]
        out_shape = [(n + 2 * p - d * (k - 1) - 1) // t + 1
                     for n, p, d, k, t in zip(shape, pd, dl, ks, st)]
        if min(out_shape) < 1 or ks == [1, 1, 1]:
            continue
        done += 1
        cells = batch * shape[0] * shape[1] * shape[2]
        n = int(rng.integers(1500, 9000))
        n = min(n, int(cells * float(rng.choice([0.05, 0.3, 0.9]))) + 1)
        flat = np.sort(rng.choice(cells, size=n, replace=False))
        vol = shape[0] * shape[1] * shape[2]
        b, r = flat // vol, flat % vol
        idx = np.stack([b, r // (shape[1] * shape[2]), (r // shape[2]) % shape[1],
                        r % shape[2]], 1).astype(np.int32)
        cin, cout = int(rng.choice([4, 12, 16, 24])), int(rng.choice([16, 40, 64, 72, 256]))
        case = (batch, shape, ks, st, pd, dl, n, cin, cout)
        print("case", case, flush=True)
        o_idx, o_pairs, o_num = oracle.canonicalize(*oracle.rulebook(idx, batch, shape, ks, st, pd,
                                                                     dl, False))
        torch.manual_seed(seed * 100 + done)
        layer = SparseConvolution(3, cin, cout, ks, stride=st, padding=pd, dilation=dl,
                                  bias=False, indice_key="r").to(device)
        f = rng.normal(size=(n, cin)).astype(np.float32)
        with torch.no_grad():
            x = SparseTensor(torch.from_numpy(f).to(device), torch.from_numpy(idx).to(device),
                             shape, batch)
            y = layer(x)
        outids, _, pairs, num, _ = x.indice_dict["r"]
        assert np.array_equal(outids.cpu().numpy(), o_idx), case
        assert np.array_equal(pairs.cpu().numpy(), o_pairs), case
        assert np.array_equal(num.cpu().numpy(), o_num), case
        assert list(y.spatial_shape) == out_shape, case
        K = ks[0] * ks[1] * ks[2]
        w = layer.weight.detach().cpu().numpy().reshape(K, cin, cout)
        want = oracle.conv_fwd(f, w, o_pairs, o_num, o_idx.shape[0], matmul=np.matmul)
        assert rel_l2(y.features.cpu().numpy(), want) < REL_L2, case


def test_fused_layer_on_a_dense_grid(device):
    """A grid the outputs nearly fill: the layer sizes its plan for the bound on the number
    of outputs (every cell: 4 x 64^3) before that number arrives, and the real number (about
    0.9 M) falls where the work split uses a finer grid than it would for the bound.  The
    buffers sized for the bound must do."""
    from ss_conv.sp_ops.conv import SparseConvolution
    from ss_conv.sp_ops.ops import get_indice_pairs
    from ss_conv.sp_ops.functional import indice_conv
    from ss_conv.sp_ops.tensor import SparseTensor
    rng = np.random.default_rng(5)
    idx = random_voxels(rng, 4, 64, 75000)
    t = torch.from_numpy(idx).to(device)
    torch.manual_seed(2)
    layer = SparseConvolution(3, 64, 64, 3, stride=1, padding=1, bias=False).to(device)
    x = torch.randn((idx.shape[0], 64), device=device)
    with torch.no_grad():
        y = layer(SparseTensor(x, t, [64] * 3, 4))
        n_out = y.indices.shape[0]
        assert 0.67 * 4 * 64 ** 3 < n_out < 4 * 64 ** 3, n_out
        g_idx, g_pairs, g_num = get_indice_pairs(t, 4, [64] * 3, 3, 1, 1, 1, 0, False)
        assert torch.equal(y.indices, g_idx)
        y2 = indice_conv(x, layer.weight, g_pairs, g_num, n_out)
        # (the layer's plan has its range boundaries from the rulebook, the call's from its
        # own passes over the pairs: the same sums in another order)
        assert rel_l2(y.features.cpu().numpy(), y2.cpu().numpy()) < 1e-6
        # against float64 sums over the pairs
        w = layer.weight.double().reshape(27, 64, 64)
        ref = torch.zeros((n_out, 64), dtype=torch.float64, device=device)
        for k in range(27):
            m = int(g_num[k])
            ref.index_add_(0, g_pairs[k, 1, :m].long(), x[g_pairs[k, 0, :m].long()].double() @ w[k])
        assert rel_l2(y.features.double().cpu().numpy(), ref.cpu().numpy()) < 1e-5


def _p2v_same(a, b):
    """Two Point2Voxel results, field by field, bit for bit."""
    (vp1, st1, vi1, f1), (vp2, st2, vi2, f2) = a, b
    assert torch.equal(vp1, vp2) and torch.equal(vi1, vi2) and torch.equal(f1, f2)
    assert torch.equal(st1.indices, st2.indices) and st1.batch_size == st2.batch_size
    assert torch.equal(st1.features, st2.features)
    assert list(st1.spatial_shape) == list(st2.spatial_shape)


@pytest.mark.parametrize("mode", [1, 2, 3, 4])
def test_point2voxel_one_call_path(mode, oracle, device):
    """Point2Voxel runs the whole forward as one native call with one wait of the host when
    the batch ids fit the tables it sized beforehand (ids below 64 on a first call, below 1 +
    the largest id of the last call afterwards).  Its result equals the oracle's and that of
    the step-by-step path, bit for bit: filtered points, ids, flags, voxel rows, voxel
    features."""
    from ss_conv.sp_ops.voxelize import Point2Voxel
    pts, feats, ids = synth.make_clouds(3, 700, seed=3, channels=6)
    pts = pts * 1.2  # some points fall outside and are filtered
    pts[ids == 1] = 50.0  # a cloud left without points: one zero point
    grid = 16
    ref = oracle.point2voxel(pts, feats, ids, [grid] * 3, [2.0 / grid] * 3, mode)
    p2v = Point2Voxel([grid] * 3, [2.0 / grid] * 3, mode)
    args = [torch.from_numpy(a).to(device) for a in (pts, feats, ids)]
    p2v._n_ids_hint = None  # (no tables sized beforehand: the step-by-step path)
    first = p2v(*args)
    assert p2v.last_path == "native filter"
    second = p2v(*args)
    assert p2v.last_path == "one call"
    _p2v_same(first, second)
    fresh = Point2Voxel([grid] * 3, [2.0 / grid] * 3, mode)
    _p2v_same(fresh(*args), second)  # a module's first call
    assert fresh.last_path == "one call"
    vp, st, vi, flag = second
    assert np.array_equal(vp.cpu().numpy(), ref["valid_points"])
    assert np.array_equal(vi.cpu().numpy(), ref["valid_ids"])
    assert np.array_equal(flag.cpu().numpy(), ref["flag"])
    assert np.array_equal(st.indices.cpu().numpy(), ref["indices"])
    assert st.batch_size == max(ref["batch_size"], int(ref["valid_ids"].max()) + 1)
    assert np.array_equal(st.features.cpu().numpy(), ref["features"])
    # ids beyond what the module has seen: the call notices and another path is taken
    more = ids + 5
    third = p2v(args[0], args[1], torch.from_numpy(more).to(device))
    assert p2v.last_path == "native filter"
    ref3 = oracle.point2voxel(pts, feats, more, [grid] * 3, [2.0 / grid] * 3, mode)
    assert np.array_equal(third[1].indices.cpu().numpy(), ref3["indices"])
    assert np.array_equal(third[1].features.cpu().numpy(), ref3["features"])
    # unsorted ids: not for the native paths at all
    perm = np.random.default_rng(0).permutation(len(ids))
    fourth = p2v(*[torch.from_numpy(a[perm]).to(device) for a in (pts, feats, ids)])
    assert p2v.last_path == "torch filter"
    ref4 = oracle.point2voxel(pts[perm], feats[perm], ids[perm], [grid] * 3, [2.0 / grid] * 3, mode)
    assert np.array_equal(fourth[1].features.cpu().numpy(), ref4["features"])


@pytest.mark.parametrize("mode", [1, 2, 3, 4])
def test_point2voxel_one_call_crowded_voxels_and_wide_rows(mode, oracle, device):
    """Voxels with hundreds of points, spread over thousands of row numbers (the ordered
    reduction walks several windows of its row bit map), and feature rows wider than one
    pass of the wave over the channels."""
    from ss_conv.sp_ops.voxelize import Point2Voxel
    rng = np.random.default_rng(12)
    n_per, B, C, grid = 6000, 2, 300, 4
    pts = rng.uniform(-0.999, 0.999, size=(B * n_per, 3)).astype(np.float32)
    feats = rng.normal(size=(B * n_per, C)).astype(np.float32)
    ids = np.repeat(np.arange(B, dtype=np.int64), n_per)
    ref = oracle.point2voxel(pts, feats, ids, [grid] * 3, [2.0 / grid] * 3, mode)
    p2v = Point2Voxel([grid] * 3, [2.0 / grid] * 3, mode)
    args = [torch.from_numpy(a).to(device) for a in (pts, feats, ids)]
    p2v._n_ids_hint = None  # (the step-by-step path first)
    first = p2v(*args)
    assert p2v.last_path == "native filter"
    second = p2v(*args)
    assert p2v.last_path == "one call"
    _p2v_same(first, second)
    assert second[1].indices.shape[0] == B * grid ** 3
    assert np.array_equal(second[1].features.cpu().numpy(), ref["features"])


def test_point2voxel_one_call_random_configurations(oracle, device):
    """The one-call path on seeded configurations: 1-5 clouds (some empty, some entirely
    outside, ids with gaps), non-cubic limits, anisotropic extents, all modes, points on
    cell faces, duplicated points."""
    from ss_conv.sp_ops.voxelize import Point2Voxel
    rng = np.random.default_rng(5)
    taken = 0
    for case in range(40):
        B = int(rng.integers(1, 6))
        limit = [int(rng.integers(2, 20)) for _ in range(3)]
        unit = [float(rng.choice([0.05, 0.1, 0.125, 0.3, 0.07])) for _ in range(3)]
        mode = int(rng.integers(1, 5))
        C = int(rng.choice([1, 3, 6, 16, 33]))
        counts = [int(rng.integers(0, 300)) for _ in range(B)]
        if sum(counts) == 0:
            counts[0] = 5
        ids = np.concatenate([np.full(c, b, dtype=np.int64) for b, c in enumerate(counts)])
        if rng.integers(0, 3) == 0:
            ids = ids * 2 + 1
        n = len(ids)
        half = 0.5 * np.array(limit) * np.array(unit)
        pts = (rng.uniform(-1.15, 1.15, size=(n, 3)) * half).astype(np.float32)
        on_face = rng.integers(0, n, size=max(1, n // 10))
        pts[on_face, rng.integers(0, 3)] = (np.round(pts[on_face, 0] / unit[0]) * unit[0]).astype(np.float32)
        dup = rng.integers(0, n, size=max(1, n // 8))
        pts[dup] = pts[rng.integers(0, n, size=len(dup))]
        if B > 1 and rng.integers(0, 3) == 0:
            pts[ids == ids[0]] = 1e3  # first cloud entirely outside
        feats = rng.normal(size=(n, C)).astype(np.float32)
        print("case", case, "B", B, "limit", limit, "mode", mode, "C", C, "n", n, flush=True)
        ref = oracle.point2voxel(pts, feats, ids, limit, unit, mode)
        p2v = Point2Voxel(limit, unit, mode)
        args = [torch.from_numpy(a).to(device) for a in (pts, feats, ids)]
        p2v(*args)
        vp, st, vi, flag = p2v(*args)
        if p2v.last_path == "one call":
            taken += 1
        assert np.array_equal(vp.cpu().numpy(), ref["valid_points"]), case
        assert np.array_equal(vi.cpu().numpy(), ref["valid_ids"]), case
        assert np.array_equal(flag.cpu().numpy(), ref["flag"]), case
        assert np.array_equal(st.indices.cpu().numpy(), ref["indices"]), case
        assert np.array_equal(st.features.cpu().numpy(), ref["features"]), case
    assert taken >= 30


@pytest.mark.parametrize("mode", [2, 3, 4])
def test_point2voxel_one_call_gradients(mode, oracle, device):
    """The gradient of the point features through the one-call path equals the one through
    the per-voxel point lists (voxelize_bp) of the other path."""
    from ss_conv.sp_ops.voxelize import Point2Voxel
    pts, feats, ids = synth.make_clouds(3, 400, seed=8, channels=5)
    pts = pts * 1.2
    grid = 6
    p2v = Point2Voxel([grid] * 3, [2.0 / grid] * 3, mode)
    tp, ti = torch.from_numpy(pts).to(device), torch.from_numpy(ids).to(device)
    grads = []
    gv = None
    p2v._n_ids_hint = None  # (the first call by the other path)
    for _ in range(2):
        x = torch.from_numpy(feats).to(device).requires_grad_(True)
        vp, st, vi, _ = p2v(tp, x, ti)
        if gv is None:
            gv = torch.randn_like(st.features)
        st.features.backward(gv)
        grads.append(x.grad.clone())
    assert p2v.last_path == "one call"
    assert torch.equal(grads[0], grads[1])


EPILOGUE_CASES = [
    # Rs of the activation, Cin, kernel, stride, pad, subm, indice_key
    ([(10, 0), (6, 1), (4, 2), (2, 3)], 16, 3, 1, 1, False, None),    # 62 + 12 gates -> 80 columns
    ([(10, 0), (6, 1), (4, 2), (2, 3)], 16, 3, 1, 1, True, "s0"),     # subm, cached rulebook
    ([(32, 0), (32, 1), (32, 2)], 40, 3, 2, 1, False, None),          # 288 outputs, several blocks
    ([(3, 0), (2, 1), (2, 2)], 5, 2, 2, 0, False, None),              # 19 outputs: scalar stores
    ([(16, 0)], 8, 3, 1, 1, False, None),                             # scalars only, no gates
    # 6.9 MB of packed filters in four column blocks: one column block per XCD
    ([(40, 0), (24, 1), (16, 2)], 256, 3, 1, 1, False, None),
    # plans of the five-group form (200 and 256 input channels, 80 computed columns in 5
    # groups): the epilogue of the fifth group
    ([(10, 0), (6, 1), (4, 2), (2, 3)], 200, 3, 1, 1, False, None),
    ([(20, 0), (8, 1), (4, 2)], 256, 3, 2, 1, False, None),
]


@pytest.mark.parametrize("case", EPILOGUE_CASES)
def test_conv_epilogue_block_matches_oracle(case, oracle, device):
    """fused.ConvBatchNormActivation in evaluation mode (ssc_conv_run_epilogue_f32: batch
    norm constants and gate applied while the convolution stores its rows) against
    oracle.bn_gate_fwd(oracle.conv_fwd(.)), and against the three layers run one after the
    other on the GPU; in training mode the block is the three layers."""
    from ss_conv import _ext
    from ss_conv.fused import ConvBatchNormActivation
    from ss_conv.sp_ops.conv import SparseConvolution
    from ss_conv.sp_ops.tensor import SparseTensor
    Rs, cin, k, s, p, subm, key = case
    print("case", case, flush=True)
    rng = np.random.default_rng(cin * 100 + k)
    bn, act, Rs_bn = _bnact_modules(Rs, (torch.relu, torch.sigmoid), device, rng)
    c_conv = sum(m * (2 * l + 1) for m, l in Rs_bn)
    c_act = sum(m * (2 * l + 1) for m, l in Rs)
    conv = SparseConvolution(3, cin, c_conv, k, s, p, bias=False, subm=subm, indice_key=key).to(device)
    block = ConvBatchNormActivation(conv, bn, act).eval()
    batch, grid, n = 2, 10, 500
    idx = random_voxels(rng, batch, grid, n)
    x_np = rng.normal(size=(n, cin)).astype(np.float32)
    w_np = conv.weight.detach().cpu().numpy().reshape(-1, cin, c_conv)

    def tensor():
        return SparseTensor(torch.from_numpy(x_np).to(device), torch.from_numpy(idx).to(device),
                            [grid] * 3, batch)

    calls = {"epi": 0}
    real = _ext._lib.ssc_conv_run_epilogue_f32

    def counted(*a):
        calls["epi"] += 1
        return real(*a)

    _ext._lib.ssc_conv_run_epilogue_f32 = counted
    try:
        with torch.no_grad():
            st = tensor()
            y1 = block(st)
            if key is not None:   # second layer of the same key: the cached rulebook
                st2 = tensor()
                st2.indice_dict = y1.indice_dict
                y2 = block(st2)
                assert torch.equal(y1.features, y2.features)
            torch.cuda.synchronize()
    finally:
        _ext._lib.ssc_conv_run_epilogue_f32 = real
    assert calls["epi"] == (2 if key is not None else 1), calls
    assert y1.features.shape[1] == c_act

    r = oracle.rulebook(idx, batch, [grid] * 3, k, s, p, 1, subm)
    o_idx, o_pairs, o_num = r[:3] if subm else oracle.canonicalize(*r)
    z = oracle.conv_fwd(x_np, w_np, o_pairs, o_num, o_idx.shape[0])
    sb, gb = act.biases()
    as_np = lambda t: None if t is None else t.detach().cpu().numpy()  # noqa: E731
    params = dict(weight=as_np(bn.weight), bias=as_np(bn.bias), scalar_bias=as_np(sb),
                  gate_bias=as_np(gb))
    running = (bn.running_mean.cpu().numpy().copy(), bn.running_var.cpu().numpy().copy())
    want = oracle.bn_gate_fwd(z, Rs_bn, Rs, params, training=False, act_scalar="relu",
                              act_gate="sigmoid" if gb is not None else None, running=running)
    assert np.array_equal(y1.indices.cpu().numpy(), o_idx)
    assert rel_l2(y1.features.cpu().numpy(), want) < REL_L2
    # the three layers one after the other
    with torch.no_grad():
        sep = act(bn(conv(tensor())))
    assert rel_l2(y1.features.cpu().numpy(), sep.features.cpu().numpy()) < 1e-6
    # a change of the running statistics is seen by the next call
    with torch.no_grad():
        bn.running_var.mul_(1.5)
        y3 = block(tensor())
        sep = act(bn(conv(tensor())))
    assert rel_l2(y3.features.cpu().numpy(), sep.features.cpu().numpy()) < 1e-6
    # training mode: batch statistics, autograd -- the separate layers
    block.train()
    xt = torch.from_numpy(x_np).to(device).requires_grad_(True)
    yt = block(SparseTensor(xt, torch.from_numpy(idx).to(device), [grid] * 3, batch))
    yt.features.sum().backward()
    assert xt.grad is not None and yt.features.shape[1] == c_act


@pytest.mark.parametrize("fields", [([(6, 0), (5, 1), (3, 2)], 12), ([(20, 0), (8, 1), (4, 2)], 200)])
def test_conv_epilogue_block_other_layers(fields, oracle, device):
    """The evaluation-mode block with tanh activations (the kernel's general form), with a
    batch norm or an activation only, on half-precision rows, and the cases that stay with
    the separate layers (a convolution with bias, an empty input): always the result of the
    three layers run one after the other.  (The second set of fields: 200 input channels and
    80 computed columns, a plan of the five-group form.)"""
    from ss_conv import _ext
    from ss_conv.activation import Activation
    from ss_conv.batchnorm import BatchNorm
    from ss_conv.fused import ConvBatchNormActivation
    from ss_conv.sp_ops.conv import SparseConvolution
    from ss_conv.sp_ops.tensor import SparseTensor
    rng = np.random.default_rng(5)
    Rs, cin = fields
    batch, grid, n = 2, 9, 400
    idx = torch.from_numpy(random_voxels(rng, batch, grid, n)).to(device)
    x = torch.from_numpy(rng.normal(size=(n, cin)).astype(np.float32)).to(device)

    def tensor(feats=x, rows=idx):
        return SparseTensor(feats, rows, [grid] * 3, batch)

    calls = {"epi": 0}
    real = _ext._lib.ssc_conv_run_epilogue_f32
    real_half = _ext._lib.ssc_conv_run_epilogue_f16

    def counted(*a):
        calls["epi"] += 1
        return real(*a)

    def counted_half(*a):
        calls["epi"] += 1
        return real_half(*a)

    def check(block, expect_kernel, make=tensor, tol=1e-6):
        before = calls["epi"]
        with torch.no_grad():
            got = block(make()).features
            y = block.conv(make())
            if block.bn is not None:
                y = block.bn(y)
            if block.activation is not None:
                y = block.activation(y)
        assert calls["epi"] - before == (1 if expect_kernel else 0)
        assert got.shape == y.features.shape
        if got.numel():
            assert rel_l2(got.float().cpu().numpy(), y.features.float().cpu().numpy()) < tol

    _ext._lib.ssc_conv_run_epilogue_f32 = counted
    _ext._lib.ssc_conv_run_epilogue_f16 = counted_half
    try:
        bn, act, Rs_bn = _bnact_modules(Rs, (torch.tanh, torch.tanh), device, rng)
        c_conv = bn.num_channels
        conv = SparseConvolution(3, cin, c_conv, 3, 1, 1, bias=False).to(device)
        check(ConvBatchNormActivation(conv, bn, act).eval(), True)
        # oracle for the tanh block
        block = ConvBatchNormActivation(conv, bn, act).eval()
        with torch.no_grad():
            out = block(tensor())
        r = oracle.rulebook(idx.cpu().numpy(), batch, [grid] * 3, 3, 1, 1)
        o_idx, o_pairs, o_num = oracle.canonicalize(*r)
        z = oracle.conv_fwd(x.cpu().numpy(), conv.weight.detach().cpu().numpy().reshape(27, cin, c_conv),
                            o_pairs, o_num, o_idx.shape[0])
        sb, gb = act.biases()
        as_np = lambda t: None if t is None else t.detach().cpu().numpy()  # noqa: E731
        want = oracle.bn_gate_fwd(z, Rs_bn, Rs, dict(weight=as_np(bn.weight), bias=as_np(bn.bias),
                                                     scalar_bias=as_np(sb), gate_bias=as_np(gb)),
                                  training=False, act_scalar="tanh", act_gate="tanh",
                                  running=(as_np(bn.running_mean), as_np(bn.running_var)))
        assert rel_l2(out.features.cpu().numpy(), want) < REL_L2
        # batch norm only, activation only (no biases), relu scalars without gate activation
        check(ConvBatchNormActivation(conv, bn, None).eval(), True)
        check(ConvBatchNormActivation(conv, None, Activation(Rs, (torch.relu, torch.sigmoid),
                                                             bias=False).to(device)).eval(), True)
        conv2 = SparseConvolution(3, cin, sum(m * (2 * l + 1) for m, l in Rs), 3, 1, 1,
                                  bias=False).to(device)
        check(ConvBatchNormActivation(conv2, BatchNorm(Rs).to(device),
                                      Activation(Rs, (torch.relu, None)).to(device)).eval(), True)
        # half-precision rows and filters (ssc_conv_run_epilogue_f16; the tables stay float32)
        check(ConvBatchNormActivation(conv.half(), None, Activation(Rs, (torch.relu, torch.sigmoid),
                                                                    bias=False).to(device)).eval(),
              True, make=lambda: tensor(x.half()), tol=2e-3)
        # (with the batch norm, whose own forward does not take half rows: against the
        # float32 block)
        before = calls["epi"]
        with torch.no_grad():
            got = ConvBatchNormActivation(conv, bn, act).eval()(tensor(x.half())).features
        conv.float()
        with torch.no_grad():
            want = ConvBatchNormActivation(conv, bn, act).eval()(tensor()).features
        assert calls["epi"] - before == 2 and got.dtype == torch.float16
        assert rel_l2(got.float().cpu().numpy(), want.cpu().numpy()) < 4e-3
        # not for the kernel: bias, no rows, nothing to apply
        biased = SparseConvolution(3, cin, c_conv, 3, 1, 1, bias=True).to(device)
        check(ConvBatchNormActivation(biased, bn, act).eval(), False)
        check(ConvBatchNormActivation(conv, bn, act).eval(), False,
              make=lambda: tensor(x[:0], idx[:0]))
        check(ConvBatchNormActivation(conv, None, None).eval(), False)
    finally:
        _ext._lib.ssc_conv_run_epilogue_f32 = real
        _ext._lib.ssc_conv_run_epilogue_f16 = real_half


def test_voxel2point_one_call_equals_the_separate_steps(oracle, device):
    """ssc_v2p_interpolate_f32 (centres, search, weights and interpolation in one call, what
    Voxel2Point.forward runs) against the module's step-by-step form and the oracle: output,
    and the gradient with respect to the voxel features; clouds with a far-away point (the
    list of unsettled queries), an empty batch element and points on the grid's upper face."""
    from ss_conv.sp_ops.voxelize import Point2Voxel, Voxel2Point
    for seed, grid, npts in ((6, 16, 500), (9, 8, 300), (12, 32, 2000)):
        pts, feats, ids = synth.make_clouds(3, npts, seed=seed, channels=12)
        pts = pts.copy()
        pts[0] = [0.99, 0.99, 0.99]      # a corner of the grid
        pts[1] = [1.0, -1.0, 1.0]        # on the upper face: voxel index == shape
        ids = ids.copy()
        ids[ids == 1] = 2                # batch element 1 has no points
        dp, df, di = [torch.from_numpy(x).to(device) for x in (pts, feats, ids)]
        vp, st, vi, _ = Point2Voxel([grid] * 3, [2.0 / grid] * 3)(dp, df, di)
        for kw in (dict(unit_voxel_extent=[2.0 / grid] * 3), dict(voxel_extent=[2.0] * 3)):
            v2p = Voxel2Point(**kw)
            st.features = st.features.detach().requires_grad_(True)
            out = v2p(st, vp, vi)
            g = torch.randn_like(out)
            out.backward(g)
            grad_one = st.features.grad.clone()
            keep = Voxel2Point.__dict__["_one_call_ok"]
            Voxel2Point._one_call_ok = staticmethod(lambda *a: False)
            try:
                st.features = st.features.detach().requires_grad_(True)
                ref = v2p(st, vp, vi)
                ref.backward(g)
            finally:
                Voxel2Point._one_call_ok = keep
            assert rel_l2(out.detach().cpu().numpy(), ref.detach().cpu().numpy()) < 1e-6
            assert rel_l2(grad_one.cpu().numpy(), st.features.grad.cpu().numpy()) < 1e-6
            want, _, _ = oracle.voxel2point(st.indices.cpu().numpy(),
                                            st.features.detach().cpu().numpy(), [grid] * 3,
                                            vp.cpu().numpy(), vi.cpu().numpy(), **kw)
            assert rel_l2(out.detach().cpu().numpy(), want) < 1e-6
