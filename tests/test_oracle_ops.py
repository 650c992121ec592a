"""Pins the remaining oracle functions against library routines and closed forms:
dense conv3d / max_pool3d / avg_pool3d, numpy reductions, brute force."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F


def random_voxels(rng, batch, grid, n):
    cells = np.sort(rng.choice(batch * grid ** 3, size=n, replace=False))
    b, r = cells // grid ** 3, cells % grid ** 3
    return np.stack([b, r // grid ** 2, (r // grid) % grid, r % grid], 1).astype(np.int32)


def dense(idx, feats, batch, grid):
    d = torch.zeros(batch, feats.shape[1], grid, grid, grid, dtype=torch.float64)
    t = torch.from_numpy(idx).long()
    d[t[:, 0], :, t[:, 1], t[:, 2], t[:, 3]] = torch.from_numpy(feats).double()
    return d


def at_rows(dense_out, idx):
    t = torch.from_numpy(idx).long()
    return dense_out[t[:, 0], :, t[:, 1], t[:, 2], t[:, 3]].numpy()


@pytest.mark.parametrize("k,s,p,d", [(3, 1, 1, 1), (3, 2, 1, 1), (2, 2, 0, 1), (5, 1, 2, 1),
                                     (3, 1, 2, 2), (3, 3, 0, 1)])
def test_conv_equals_dense_conv3d(k, s, p, d, oracle):
    """Sparse conv over the rulebook == F.conv3d (cross-correlation, kernel index
    (kx*k+ky)*k+kz) sampled at the active outputs; every other output cell is 0."""
    rng = np.random.default_rng(1)
    grid, cin, cout = 9, 5, 7
    idx = random_voxels(rng, 2, grid, 70)
    feats = rng.normal(size=(70, cin)).astype(np.float32)
    w = rng.normal(size=(k ** 3, cin, cout)).astype(np.float32)
    o_idx, pairs, num, shape = oracle.rulebook(idx, 2, [grid] * 3, k, s, p, d)
    for mm in (None, np.matmul):
        out = oracle.conv_fwd(feats, w, pairs, num, o_idx.shape[0], matmul=mm)
        kernel = torch.from_numpy(w).double().reshape(k, k, k, cin, cout).permute(4, 3, 0, 1, 2)
        want = F.conv3d(dense(idx, feats, 2, grid), kernel, stride=s, padding=p, dilation=d)
        assert list(want.shape[2:]) == shape
        assert np.allclose(out, at_rows(want, o_idx), rtol=1e-4, atol=1e-5)
        mask = torch.ones_like(want[:, 0], dtype=torch.bool)
        t = torch.from_numpy(o_idx).long()
        mask[t[:, 0], t[:, 1], t[:, 2], t[:, 3]] = False
        assert float(want.abs().sum(1)[mask].max()) == 0.0


@pytest.mark.parametrize("k,s,p", [(3, 1, 1), (3, 2, 1), (2, 2, 0)])
def test_conv_backward_equals_dense_autograd(k, s, p, oracle):
    """The restated backward equals torch's autograd through F.conv3d on the densified
    input: gradient with respect to the active inputs and to the kernel, for an output
    gradient that is zero at inactive outputs."""
    rng = np.random.default_rng(31)
    batch, grid, n, cin, cout = 2, 7, 60, 3, 4
    idx = random_voxels(rng, batch, grid, n)
    feats = rng.normal(size=(n, cin)).astype(np.float32)
    K = k ** 3
    w = rng.normal(size=(K, cin, cout)).astype(np.float32)
    o_idx, pairs, num, o_shape = oracle.rulebook(idx, batch, [grid] * 3, k, s, p)
    g_out = rng.normal(size=(o_idx.shape[0], cout)).astype(np.float32)
    d_in, d_w = oracle.conv_bwd(feats, w, g_out, pairs, num)

    x = dense(idx, feats, batch, grid).requires_grad_(True)
    kernel = torch.from_numpy(w).double().reshape(k, k, k, cin, cout).permute(4, 3, 0, 1, 2) \
        .contiguous().requires_grad_(True)
    out = F.conv3d(x, kernel, stride=s, padding=p)
    assert list(out.shape[2:]) == [int(v) for v in o_shape]
    go = torch.zeros_like(out)
    t = torch.from_numpy(o_idx).long()
    go[t[:, 0], :, t[:, 1], t[:, 2], t[:, 3]] = torch.from_numpy(g_out).double()
    out.backward(go)
    ref_in = at_rows(x.grad, idx)
    ref_w = kernel.grad.permute(2, 3, 4, 1, 0).reshape(K, cin, cout).numpy()
    assert np.allclose(d_in, ref_in, atol=1e-4)
    assert np.allclose(d_w, ref_w, atol=1e-4)
    # the input gradient of an inverse convolution flows the other way through the pairs
    d_in_inv, d_w_inv = oracle.conv_bwd(g_out, np.transpose(w, (0, 2, 1)).copy(), feats, pairs,
                                        num, inverse=True)
    assert d_in_inv.shape == g_out.shape and d_w_inv.shape == (K, cout, cin)
    assert np.allclose(d_w_inv, np.transpose(d_w, (0, 2, 1)), atol=1e-4)


def test_conv_inverse_is_transpose(oracle):
    """<conv(x), y> == <x, conv_inverse(y)> with the transposed per-offset matrices."""
    rng = np.random.default_rng(2)
    idx = random_voxels(rng, 1, 8, 50)
    o_idx, pairs, num, _ = oracle.rulebook(idx, 1, [8] * 3, 3, 2, 1)
    x = rng.normal(size=(50, 4)).astype(np.float32)
    y = rng.normal(size=(o_idx.shape[0], 6)).astype(np.float32)
    w = rng.normal(size=(27, 4, 6)).astype(np.float32)
    fwd = oracle.conv_fwd(x, w, pairs, num, o_idx.shape[0], matmul=np.matmul)
    inv = oracle.conv_fwd(y, np.ascontiguousarray(w.transpose(0, 2, 1)), pairs, num, 50,
                          inverse=True, matmul=np.matmul)
    assert np.isclose((fwd * y).sum(), (x * inv).sum(), rtol=1e-4)


def test_gather_scatter_match_compiled_reference(oracle):
    if oracle.ref_lib() is None:
        pytest.skip("oracle/_ref/libssc_ref.so not built")
    rng = np.random.default_rng(3)
    idx = random_voxels(rng, 2, 8, 60)
    o_idx, pairs, num, _ = oracle.rulebook(idx, 2, [8] * 3, 3, 1, 1)
    x = rng.normal(size=(60, 8)).astype(np.float32)
    w = rng.normal(size=(27, 8, 12)).astype(np.float32)
    a = oracle.conv_fwd(x, w, pairs, num, o_idx.shape[0], matmul=np.matmul)
    b = oracle.ref_gather_scatter_conv(x, w, pairs, num, o_idx.shape[0])
    assert np.array_equal(a, b)


@pytest.mark.parametrize("k,s,p", [(2, 2, 0), (3, 2, 1), (3, 1, 1)])
def test_pools_equal_dense_pools(k, s, p, oracle):
    rng = np.random.default_rng(4)
    grid, c = 8, 6
    idx = random_voxels(rng, 2, grid, 90)
    feats = rng.normal(size=(90, c)).astype(np.float32)
    o_idx, pairs, num, _ = oracle.rulebook(idx, 2, [grid] * 3, k, s, p)
    d = dense(idx, feats, 2, grid)
    mx = oracle.maxpool_fwd(feats, pairs, num, o_idx.shape[0])
    want = F.max_pool3d(F.relu(d), k, s, p)  # output starts at zero: max(0, .)
    assert np.allclose(mx, at_rows(want, o_idx))
    av = oracle.avgpool_fwd(feats, pairs, num, o_idx.shape[0])
    want = F.avg_pool3d(d, k, s, p, count_include_pad=True)
    assert np.allclose(av, at_rows(want, o_idx), atol=1e-6)
    rf = oracle.summary_rf(pairs, num, o_idx.shape[0])
    ones = dense(idx, np.ones((90, 1), np.float32), 2, grid)
    cnt = F.avg_pool3d(ones, k, s, p, count_include_pad=True) * k ** 3
    assert np.array_equal(rf, np.rint(at_rows(cnt, o_idx)[:, 0]).astype(np.int32))
    if oracle.ref_lib() is not None:
        assert np.array_equal(mx, oracle.ref_maxpool_fwd(feats, pairs, num, o_idx.shape[0]))


@pytest.mark.parametrize("k,s,p", [(2, 2, 0), (3, 2, 1), (3, 1, 1)])
def test_pool_backward_equals_dense_autograd(k, s, p, oracle):
    """Backward of avg pooling equals autograd through F.avg_pool3d; backward of max pooling
    equals autograd through F.max_pool3d(relu(.)) on data without ties (every positive
    window maximum unique)."""
    rng = np.random.default_rng(13)
    batch, grid, n, c = 2, 8, 150, 3
    idx = random_voxels(rng, batch, grid, n)
    feats = rng.normal(size=(n, c)).astype(np.float32)
    o_idx, pairs, num, shape = oracle.rulebook(idx, batch, [grid] * 3, k, s, p)
    g_out = rng.normal(size=(o_idx.shape[0], c)).astype(np.float32)
    t = torch.from_numpy(o_idx).long()

    x = dense(idx, feats, batch, grid).requires_grad_(True)
    y = F.avg_pool3d(x, k, s, p, count_include_pad=True)
    go = torch.zeros_like(y)
    go[t[:, 0], :, t[:, 1], t[:, 2], t[:, 3]] = torch.from_numpy(g_out).double()
    y.backward(go)
    rf = np.full(o_idx.shape[0], k ** 3, dtype=np.int32)
    got = oracle.avgpool_bwd(g_out, pairs, num, n, rf)
    assert np.allclose(got, at_rows(x.grad, idx), atol=1e-6)

    x = dense(idx, feats, batch, grid).requires_grad_(True)
    y = F.max_pool3d(torch.relu(x), k, s, p)
    y.backward(go)
    pooled = oracle.maxpool_fwd(feats, pairs, num, o_idx.shape[0])
    got = oracle.maxpool_bwd(feats, pooled, g_out, pairs, num)
    # inputs <= 0 never equal a positive maximum; where the window maximum is 0 (all
    # inputs negative) neither side passes a gradient to a real input
    assert np.allclose(got, at_rows(x.grad, idx), atol=1e-6)


def test_segment_and_voxel_backward(oracle):
    """Segment pools, voxel mean and interpolation backward against torch autograd."""
    rng = np.random.default_rng(17)
    n, c = 40, 3
    feats = rng.normal(size=(n, c)).astype(np.float32)
    offsets = np.array([0, 7, 7, 25, 40], dtype=np.int32)
    g = rng.normal(size=(4, c)).astype(np.float32)
    x = torch.from_numpy(feats).double().requires_grad_(True)
    segs = [x[a:b] for a, b in zip(offsets[:-1], offsets[1:])]
    mean = torch.stack([s.mean(0) if len(s) else torch.zeros(c, dtype=torch.float64) for s in segs])
    (mean * torch.from_numpy(g).double()).sum().backward()
    assert np.allclose(oracle.segment_avg_bwd(g, offsets, n), x.grad.numpy(), atol=1e-6)
    x.grad = None
    mx = torch.stack([s.max(0)[0] if len(s) else torch.zeros(c, dtype=torch.float64) for s in segs])
    (mx * torch.from_numpy(g).double()).sum().backward()
    _, arg = oracle.segment_max(feats, offsets)
    assert np.allclose(oracle.segment_max_bwd(g, arg, n), x.grad.numpy(), atol=1e-6)
    # voxel mean: 3 voxels over 7 points
    inverse = np.array([0, 2, 0, 1, 2, 2, 0], dtype=np.int32)
    maps = oracle.voxel_map(inverse, 3, 3, 4)
    pf = rng.normal(size=(7, c)).astype(np.float32)
    gv = rng.normal(size=(3, c)).astype(np.float32)
    x = torch.from_numpy(pf).double().requires_grad_(True)
    vm = torch.stack([x[torch.from_numpy(np.nonzero(inverse == v)[0])].mean(0) for v in range(3)])
    (vm * torch.from_numpy(gv).double()).sum().backward()
    assert np.allclose(oracle.voxel_reduce_bwd(gv, maps, 4, 7), x.grad.numpy(), atol=1e-6)
    # interpolation
    m, q = 9, 20
    vf = rng.normal(size=(m, c)).astype(np.float32)
    idx3 = rng.integers(0, m, size=(q, 3)).astype(np.int32)
    w3 = rng.uniform(size=(q, 3)).astype(np.float32)
    gq = rng.normal(size=(q, c)).astype(np.float32)
    x = torch.from_numpy(vf).double().requires_grad_(True)
    out = sum(x[torch.from_numpy(idx3[:, j]).long()] * torch.from_numpy(w3[:, j:j + 1]).double()
              for j in range(3))
    (out * torch.from_numpy(gq).double()).sum().backward()
    assert np.allclose(oracle.three_interp_bwd(gq, idx3, w3, m), x.grad.numpy(), atol=1e-5)


def test_segment_pools(oracle):
    rng = np.random.default_rng(5)
    lens = [4, 1, 33, 7]
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    x = rng.normal(size=(off[-1], 9)).astype(np.float32)
    x[6:20, 3] = 4.0
    avg = oracle.segment_avg(x, off)
    mx, arg = oracle.segment_max(x, off)
    for s in range(len(lens)):
        seg = x[off[s]:off[s + 1]]
        assert np.allclose(avg[s], seg.mean(0), rtol=1e-5, atol=1e-6)
        assert np.array_equal(mx[s], seg.max(0))
        assert np.array_equal(arg[s], seg.argmax(0) + off[s])  # first occurrence
    e_avg = oracle.segment_avg(x, np.array([0, 0, 3], np.int32))
    assert np.isnan(e_avg[0]).all()
    e_max, e_arg = oracle.segment_max(x, np.array([0, 0, 3], np.int32))
    assert np.isneginf(e_max[0]).all() and (e_arg[0] == -1).all()


@pytest.mark.parametrize("mode", [1, 2, 3, 4])
def test_point2voxel_semantics(mode, oracle):
    rng = np.random.default_rng(6)
    n, grid = 400, 8
    pts = rng.uniform(-1.2, 1.2, size=(n, 3)).astype(np.float32)
    feats = rng.normal(size=(n, 3)).astype(np.float32)
    ids = np.sort(rng.integers(0, 3, size=n)).astype(np.int64)
    r = oracle.point2voxel(pts, feats, ids, [grid] * 3, [2.0 / grid] * 3, mode)
    inside = (np.abs(pts) <= 1.0).all(1)
    assert np.array_equal(r["valid_points"], pts[inside])
    assert r["counts"].sum() == inside.sum() == r["inverse"].size
    vox = r["indices"]
    assert vox[:, 1:].min() >= 0 and vox[:, 1:].max() < grid
    keys = oracle.flat_key(vox, [grid] * 3)
    assert np.all(np.diff(keys) > 0)  # sorted, unique
    exact = np.floor((pts[inside].astype(np.float64) + 1.0) / (2.0 / grid)).astype(np.int32)
    assert np.array_equal(vox[r["inverse"], 1:], exact)
    vf = feats[inside]
    for v in range(0, vox.shape[0], 7):
        members = np.nonzero(r["inverse"] == v)[0]
        want = {1: vf[members[0]], 2: vf[members[-1]], 3: vf[members].sum(0),
                4: vf[members].mean(0)}[mode]
        assert np.allclose(r["features"][v], want, rtol=1e-5, atol=1e-6)
        if mode >= 3:
            assert r["maps"][v, 0] == members.size
            assert np.array_equal(r["maps"][v, 1:1 + members.size], members)


def test_three_nn_and_interpolation(oracle):
    rng = np.random.default_rng(7)
    known = np.concatenate([rng.integers(0, 2, size=(60, 1)), rng.integers(0, 5, size=(60, 3))],
                           1).astype(np.float32)  # integer grid: plenty of distance ties
    known[:3, 0] = 5  # a batch with exactly three members
    query = np.concatenate([rng.integers(0, 2, size=(40, 1)), rng.uniform(0, 4, size=(40, 3))],
                           1).astype(np.float32)
    query[0] = known[7]
    query[1, 0] = 5
    query[2, 0] = 9  # no member at all
    dist, idx = oracle.three_nn(query, known)
    for q in range(40):
        same = np.nonzero(known[:, 0] == query[q, 0])[0]
        d2 = ((known[same, 1:] - query[q, 1:]).astype(np.float32) ** 2)
        d2 = (d2[:, 0] + d2[:, 1]) + d2[:, 2]
        order = same[np.argsort(d2, kind="stable")]  # ties keep the lower index
        m = min(3, order.size)
        assert np.array_equal(idx[q, :m], order[:m])
        assert np.allclose(dist[q, :m] ** 2, np.sort(d2)[:m], rtol=1e-6)
        assert np.all(np.isinf(dist[q, m:])) and np.all(idx[q, m:] == 0)
    feats = rng.normal(size=(60, 5)).astype(np.float32)
    w = rng.uniform(size=(40, 3)).astype(np.float32)
    out = oracle.three_interp(feats, idx, w)
    want = (feats[idx] * w[:, :, None]).sum(1)
    assert np.allclose(out, want, rtol=1e-5, atol=1e-6)


def test_combine_equals_einsum(oracle):
    rng = np.random.default_rng(8)
    m_out, d_out, m_in, d_in, size = [2, 1], [1, 3], [3, 2], [1, 5], 3
    bases = [[rng.normal(size=(nb, do, di, size, size, size)).astype(np.float32)
              if nb else None for di, nb in zip(d_in, row)]
             for do, row in zip(d_out, [[2, 1], [0, 3]])]
    n_w = sum(mo * mi * (b.shape[0] if b is not None else 0)
              for mo, row in zip(m_out, bases) for mi, b in zip(m_in, row))
    w = rng.normal(size=n_w).astype(np.float32)
    got = oracle.combine(w, bases, m_out, d_out, m_in, d_in, size)
    assert got.shape == (2 * 1 + 1 * 3, 3 * 1 + 2 * 5, 3, 3, 3)
    off = 0
    r0 = 0
    for i, mo in enumerate(m_out):
        c0 = 0
        for j, mi in enumerate(m_in):
            b = bases[i][j]
            blk = got[r0:r0 + mo * d_out[i], c0:c0 + mi * d_in[j]]
            if b is None:
                assert not blk.any()
            else:
                nb = b.shape[0]
                wt = torch.from_numpy(w[off:off + mo * mi * nb]).reshape(mo, mi, nb)
                off += mo * mi * nb
                want = torch.einsum("uvb,bijxyz->uivjxyz", wt, torch.from_numpy(b))
                assert np.allclose(blk, want.reshape(blk.shape).numpy(), atol=1e-5)
            c0 += mi * d_in[j]
        r0 += mo * d_out[i]


def _h(x):
    """x rounded to binary16 by struct's codec (round to nearest even), as a float."""
    import struct
    return struct.unpack("<e", struct.pack("<e", float(x)))[0]


def test_half_pools_known_answers(oracle):
    """The half-precision pools round after every operation (at::Half's operators,
    src/pool/indice_avgpool_cuda_functor.cu:46): known answers rounded by hand with struct's
    binary16 codec, one window of three inputs; where every step is exact in half the result
    equals the float routine's; the maximum equals the float routine on the widened rows."""
    # one output row, three offsets with one pair each
    pairs = np.zeros((3, 2, 1), dtype=np.int32)
    pairs[:, 0, 0] = [0, 1, 2]
    num = np.ones(3, dtype=np.int32)
    vals = [0.7, 2.3, 5.1]
    feats = np.array(vals, dtype=np.float16).reshape(3, 1)
    rf = np.array([3], dtype=np.int32)
    acc = 0.0
    for v in vals:  # products of float(half) operands: exact in double, one rounding to float
        q = _h(np.float32(np.float32(_h(v)) / np.float32(3.0)))
        acc = _h(np.float32(np.float32(acc) + np.float32(q)))
    got = oracle.avgpool_fwd_half(feats, pairs, num, 1, rf)
    assert got.dtype == np.float16 and float(got[0, 0]) == acc
    # rounding at every step shows: the float routine, rounded once at the end, differs
    once = _h(oracle.avgpool_fwd(feats.astype(np.float32), pairs, num, 1, rf)[0, 0])
    assert once != acc
    # backward: din[i] = half(dout / half(rf)) for each of the three inputs
    g = np.array([[0.3]], dtype=np.float16)
    din = oracle.avgpool_bwd_half(g, pairs, num, 3, rf)
    assert all(float(din[i, 0]) == _h(np.float32(np.float32(_h(0.3)) / np.float32(3.0))) for i in range(3))

    # exact cases: small integers and a power-of-two window
    rng = np.random.default_rng(5)
    idx = random_voxels(rng, 2, 8, 120)
    o_idx, pairs, num, _ = oracle.rulebook(idx, 2, [8] * 3, 2, 2, 0)
    n_out = o_idx.shape[0]
    ints = rng.integers(-8, 9, size=(120, 5)).astype(np.float32)
    av = oracle.avgpool_fwd_half(ints, pairs, num, n_out)       # rf = 8: every quotient exact
    assert np.array_equal(av.astype(np.float32), oracle.avgpool_fwd(ints, pairs, num, n_out))
    x = rng.normal(size=(120, 5)).astype(np.float16)
    mx = oracle.maxpool_fwd_half(x, pairs, num, n_out)
    assert np.array_equal(mx.astype(np.float32),
                          oracle.maxpool_fwd(x.astype(np.float32), pairs, num, n_out))
    # max backward: integer gradients add exactly, so half and float routines agree
    gi = rng.integers(-4, 5, size=(n_out, 5)).astype(np.float32)
    a = oracle.maxpool_bwd_half(x, mx, gi, pairs, num)
    b = oracle.maxpool_bwd(x.astype(np.float32), mx.astype(np.float32), gi, pairs, num)
    assert np.array_equal(a.astype(np.float32), b)
    # a window with overlap (3, stride 1): sums of halves that do round -- against a scalar
    # loop with struct's codec
    o_idx, pairs, num, _ = oracle.rulebook(idx, 2, [8] * 3, 3, 1, 1)
    n_out = o_idx.shape[0]
    rf = oracle.summary_rf(pairs, num, n_out)
    x1 = rng.normal(size=(120, 1)).astype(np.float16)
    got = oracle.avgpool_fwd_half(x1, pairs, num, n_out, rf)
    want = np.zeros(n_out)
    for k in range(pairs.shape[0]):
        for j in range(int(num[k])):
            i, o = int(pairs[k, 0, j]), int(pairs[k, 1, j])
            q = _h(np.float32(np.float32(x1[i, 0]) / np.float32(_h(float(rf[o])))))
            want[o] = _h(np.float32(np.float32(want[o]) + np.float32(q)))
    assert np.array_equal(got[:, 0].astype(np.float64), want)
