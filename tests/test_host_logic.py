"""Host-side logic that needs no GPU: shape arithmetic, the sparse tensor type,
the C ABI surface, the steerable basis and the torch-op layers."""
import ctypes
import math
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---- C ABI ----------------------------------------------------------------------------
def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "ssc.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ssc_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from ss_conv import _ext
    lib = ctypes.CDLL(_ext.LIB_PATH)
    names = _declared_symbols()
    assert len(names) >= 24
    for n in names:
        assert hasattr(lib, n), "libssc.so does not export %s" % n
    assert set(names) == set(_ext.EXPORTED_SYMBOLS), \
        set(names).symmetric_difference(_ext.EXPORTED_SYMBOLS)
    assert lib.ssc_version() >= 100


def test_host_argument_checks_need_no_gpu():
    """Checks that run before any kernel launch (reference: indice_conv.h:33-44)."""
    from ss_conv import _ext
    lib = _ext._lib
    g = _ext._geometry(1, [8] * 3, [7] * 3, [1] * 3, [3] * 3, [1] * 3, 0, 0)
    assert lib.ssc_rulebook_workspace_bytes(ctypes.byref(g), 10) == 0  # 7^3 = 343 > 256
    n_out = ctypes.c_int32(-5)
    rc = lib.ssc_rulebook_count(None, 10, ctypes.byref(g), None, 0, ctypes.byref(n_out), None)
    assert rc == _ext.SSC_ERUNTIME and b"kernel volume" in lib.ssc_last_error()
    g = _ext._geometry(1, [8] * 3, [3] * 3, [2] * 3, [1] * 3, [2] * 3, 0, 0)
    rc = lib.ssc_rulebook_count(None, 10, ctypes.byref(g), None, 0, ctypes.byref(n_out), None)
    assert rc == _ext.SSC_EINVAL
    g = _ext._geometry(1, [8] * 3, [3] * 3, [1] * 3, [1] * 3, [1] * 3, 0, 1)
    assert lib.ssc_rulebook_workspace_bytes(ctypes.byref(g), 10) > 0  # transposed: a geometry
    g = _ext._geometry(64, [512] * 3, [3] * 3, [1] * 3, [1] * 3, [1] * 3, 0, 0)
    assert lib.ssc_rulebook_count(None, 10, ctypes.byref(g), None, 0, ctypes.byref(n_out),
                                  None) == _ext.SSC_ERUNTIME  # 64 * 512^3 >= 2^31
    # empty input: no work, no pointers touched
    g = _ext._geometry(1, [8] * 3, [3] * 3, [1] * 3, [1] * 3, [1] * 3, 0, 0)
    assert lib.ssc_rulebook_count(None, 0, ctypes.byref(g), None, 0, ctypes.byref(n_out), None) == 0
    assert n_out.value == 0
    assert lib.ssc_conv_workspace_bytes(1000, 27, 64, 128, 500) > 0
    assert lib.ssc_conv_fwd_f32(None, 0, 0, None, 0, 0, 0, 4, None, 0, None, 27, 0, 0, None, 0,
                                None, 0, None) == _ext.SSC_EINVAL
    assert lib.ssc_voxel_map(None, None, None, 5, 5, 1, 9, None) == _ext.SSC_EINVAL  # bad mode


def test_cpu_tensors_are_rejected():
    from ss_conv import _ext
    with pytest.raises(RuntimeError, match="GPU only"):
        _ext.get_indice_pairs_3d(torch.zeros((1, 4), dtype=torch.int32), 1, [8] * 3, [8] * 3,
                                 [3] * 3, [1] * 3, [1] * 3, [1] * 3, [0] * 3, 0, 0)
    with pytest.raises(RuntimeError):
        _ext.get_indice_pairs_3d(torch.zeros((1, 3), dtype=torch.int32), 1, [8] * 3, [8] * 3,
                                 [3] * 3, [1] * 3, [1] * 3, [1] * 3, [0] * 3, 0, 0)
    with pytest.raises(RuntimeError, match="GPU only"):
        _ext.indice_conv_fp32(torch.zeros(2, 4), torch.zeros(3, 3, 3, 4, 4),
                              torch.zeros((27, 2, 2), dtype=torch.int32),
                              torch.zeros(27, dtype=torch.int32), 2, 0, 0)


def test_plan_buffers_sized_for_a_bound_serve_every_smaller_row_count():
    """A layer sizes plan and scratch for an upper bound of the number of output rows before
    that number is known; the plan is then built for the real number.  The sizes must not
    shrink when n_out grows, across the thresholds where the work split changes its grid
    (fewer than 2048 rows to a range) and its number of ranges."""
    from ss_conv import _ext
    lib = _ext._lib
    for K, c_in, c_out, stride in ((27, 64, 64, 200000), (27, 64, 128, 57304), (125, 200, 200, 106731),
                                   (8, 256, 256, 85349), (27, 3, 152, 30000), (27, 512, 608, 4000)):
        sizes = []
        ns = sorted(set([1, 15, 16, 17, 63, 64, 65, 1000, 2047 * 128, 2048 * 128, 2048 * 256 - 1,
                         2048 * 256, 2048 * 256 + 1, 2048 * 512 - 1, 2048 * 512, 2048 * 512 + 1,
                         600000, 750000, 900000, 1048576, 3000000] +
                        [int(1.17 ** e) for e in range(10, 100)]))
        for n in ns:
            sizes.append((lib.ssc_conv_plan_bytes(n, K, c_in, c_out, stride),
                          lib.ssc_conv_plan_scratch_bytes(n, K, c_in, c_out, stride),
                          lib.ssc_conv_workspace_bytes(n, K, c_in, c_out, stride)))
        for a, b, n in zip(sizes, sizes[1:], ns[1:]):
            assert b[0] >= a[0] and b[1] >= a[1] and b[2] >= a[2], (K, c_in, c_out, n, a, b)
    # the case of the report: bound 1048576 rows, 900000 real ones
    assert lib.ssc_conv_plan_scratch_bytes(1048576, 27, 64, 64, 200000) >= \
        lib.ssc_conv_plan_scratch_bytes(900000, 27, 64, 64, 200000)


def test_tile_cut_of_a_range():
    """Every tile of a range has rows, the heights add up to the range, tiles but the last
    keep room for spilled row blocks behind them and the last one fits the window -- also
    for ranges of hundreds of tiles (tens of millions of output rows)."""
    from ss_conv import _ext
    lib = _ext._lib
    nt, h, win = ctypes.c_int32(), ctypes.c_int32(), ctypes.c_int32()
    for c_in, c_out in ((64, 128), (200, 200), (64, 72), (3, 16)):
        rows_list = list(range(0, 1400)) + [304 * k + d for k in (5, 50, 300, 440, 441, 600, 2000, 7000)
                                            for d in (-161, -1, 0, 1, 23, 24, 25, 135, 137, 303)]
        for rows in rows_list:
            assert lib.ssc_conv_tile_cut(rows, c_in, c_out, ctypes.byref(nt), ctypes.byref(h),
                                         ctypes.byref(win)) == 0
            if rows == 0:
                assert nt.value == 0
                continue
            n, hh, w = nt.value, h.value, win.value
            assert n >= 1 and hh >= 1
            last = rows - (n - 1) * hh
            assert 0 < last <= w, (rows, n, hh, w)
            if n > 1:
                # a tile and the 160 (192) rows of spill behind it fit the window, give or
                # take the slack of 24 rows
                assert hh + 136 <= w, (rows, n, hh, w)
    assert lib.ssc_conv_tile_cut(-1, 64, 64, ctypes.byref(nt), ctypes.byref(h),
                                 ctypes.byref(win)) == _ext.SSC_EINVAL


# ---- shape arithmetic and the tensor type ---------------------------------------------------
@pytest.mark.parametrize("size,k,s,p,d", [(64, 3, 1, 1, 1), (64, 3, 2, 1, 1), (32, 2, 2, 0, 1),
                                          (17, 5, 1, 2, 1), (20, 3, 1, 2, 2), (9, 3, 3, 0, 1)])
def test_conv_output_size_matches_torch(size, k, s, p, d):
    from ss_conv.sp_ops.ops import get_conv_output_size
    out = get_conv_output_size([size] * 3, [k] * 3, [s] * 3, [p] * 3, [d] * 3)
    ref = torch.nn.functional.conv3d(torch.zeros(1, 1, size, size, size),
                                     torch.zeros(1, 1, k, k, k), stride=s, padding=p, dilation=d)
    assert out == list(ref.shape[2:])
    assert get_conv_output_size([size], [-1], [1], [0], [1]) == [1]


def test_sparse_tensor_container():
    from ss_conv.sp_ops.tensor import SparseTensor
    idx = torch.tensor([[0, 0, 1, 2], [0, 3, 3, 3], [1, 2, 0, 1]], dtype=torch.int32)
    feats = torch.arange(6, dtype=torch.float32).reshape(3, 2)
    st = SparseTensor(feats, idx, [4, 4, 4], 2)
    d = st.dense()
    assert d.shape == (2, 2, 4, 4, 4) and d.sum() == feats.sum()
    assert torch.equal(d[1, :, 2, 0, 1], feats[2])
    assert st.dense(channels_first=False).shape == (2, 4, 4, 4, 2)
    assert st.get_offsets().tolist() == [0, 2, 3]
    assert st.spatial_size == 64 and abs(st.sparity - 3 / 128) < 1e-12
    assert st.find_indice_pair(None) is None and st.find_indice_pair("a") is None
    st.indice_dict["a"] = 1
    assert st.find_indice_pair("a") == 1


def test_conv1x1_is_a_matrix_product():
    """1x1x1 kernels bypass the rulebook (reference: sp_ops/conv.py:116-122)."""
    from ss_conv.sp_ops.conv import SparseConvolution
    from ss_conv.sp_ops.tensor import SparseTensor
    torch.manual_seed(0)
    conv = SparseConvolution(3, 4, 6, kernel_size=1, bias=True)
    idx = torch.tensor([[0, 0, 1, 2], [0, 3, 3, 3]], dtype=torch.int32)
    x = torch.randn(2, 4)
    st = SparseTensor(x.clone(), idx, [4, 4, 4], 1)
    out = conv(st)
    assert out is st
    want = x @ conv.weight.reshape(4, 6) + conv.bias
    assert torch.allclose(out.features, want)


# ---- steerable basis -----------------------------------------------------------------------
def test_real_harmonics_and_wigner_conventions():
    from ss_conv.utils import SO3
    dt = torch.float64
    A = SO3.xyz_vector_basis_to_spherical_basis().to(dt)
    _, to3, to5 = [t.to(dt) for t in SO3.tensor3x3_repr_basis_to_spherical_basis()]
    old = torch.get_default_dtype()
    torch.set_default_dtype(dt)
    try:
        for a, b, c in [(0.3, 1.2, 2.2), (5.0, 0.2, 1.0), (2.0, 2.9, 4.0)]:
            R = SO3.rot(a, b, c)
            # anchors stated by the reference (utils/SO3.py:282-292, 304-335)
            assert torch.allclose(SO3.irr_repr(1, a, b, c) @ A, A @ R, atol=1e-12)
            assert torch.allclose(SO3.irr_repr(1, a, b, c) @ to3, to3 @ SO3.tensor3x3_repr(a, b, c),
                                  atol=1e-12)
            assert torch.allclose(SO3.irr_repr(2, a, b, c) @ to5, to5 @ SO3.tensor3x3_repr(a, b, c),
                                  atol=1e-12)
            assert torch.allclose(SO3.irr_repr(0, a, b, c), torch.ones(1, 1))
        for l in range(7):
            # representation property and orthogonality (utils/SO3.py:340-357)
            D1, D2 = SO3.wigner_D_np(l, .3, .5, .7), SO3.wigner_D_np(l, 1.3, 2.5, .1)
            a, b, c = SO3.compose(.3, .5, .7, 1.3, 2.5, .1)
            assert np.abs(D1 @ D2 - SO3.wigner_D_np(l, a.item(), b.item(), c.item())).max() < 1e-10
            assert np.abs(D1 @ D1.T - np.eye(2 * l + 1)).max() < 1e-10
            # Y(R x) = D(R) Y(x) on fresh points (utils/SO3.py:360-383)
            x = np.random.default_rng(l).normal(size=(9, 3))
            R = SO3._rot_np(.3, .5, .7)
            assert np.abs(SO3.real_sh_np(l, x @ R.T) - D1 @ SO3.real_sh_np(l, x)).max() < 1e-10
    finally:
        torch.set_default_dtype(old)
    # orthonormality on the sphere (quadrature on a fine Fibonacci set) and known low orders
    n = 20000
    k = np.arange(n) + 0.5
    z = 1 - 2 * k / n
    phi = k * math.pi * (3 - math.sqrt(5))
    X = np.stack([np.sqrt(1 - z * z) * np.cos(phi), np.sqrt(1 - z * z) * np.sin(phi), z], -1)
    Y = np.concatenate([SO3.real_sh_np(l, X) for l in range(4)], 0)
    assert np.abs(Y @ Y.T * (4 * math.pi / n) - np.eye(16)).max() < 2e-3
    c1 = math.sqrt(3 / (4 * math.pi))
    assert np.allclose(SO3.real_sh_np(1, X), c1 * X[:, [1, 2, 0]].T)
    assert np.allclose(SO3.real_sh_np(0, np.zeros(3)), 1 / math.sqrt(4 * math.pi))
    assert np.allclose(SO3.real_sh_np(3, np.zeros(3)), 0.0)


@pytest.mark.parametrize("J,li,lo", [(0, 0, 0), (1, 1, 0), (1, 1, 1), (2, 1, 1), (3, 2, 1),
                                     (0, 2, 2), (4, 2, 2), (5, 3, 2)])
def test_intertwiner_q_j(J, li, lo):
    from ss_conv.utils import SO3
    Q = SO3.basis_transformation_Q_J(J, li, lo).numpy()
    assert Q.shape == ((2 * lo + 1) * (2 * li + 1), 2 * J + 1)
    assert abs(np.linalg.norm(Q) - 1) < 1e-12
    for a, b, c in [(0.1, 0.2, 0.3), (3.0, 1.5, 4.2)]:
        Rt = np.kron(SO3.wigner_D_np(lo, a, b, c), SO3.wigner_D_np(li, a, b, c))
        assert np.abs(Rt @ Q - Q @ SO3.wigner_D_np(J, a, b, c)).max() < 1e-9


def test_kernel_basis_counts_norms_and_equivariance():
    """Numbers of basis elements, the per-element scale, the weight count
    (reference: utils/kernel.py:133-139,161-167,245-249) and equivariance of the
    sampled basis under the +pi/2 turn about y (asserted inside the constructor)."""
    from ss_conv.utils.kernel import SE3Kernel
    rs = [(2, l) for l in range(4)]
    ker = SE3Kernel(rs, rs, 3)
    table = [[2, 1, 1, 1], [1, 4, 3, 2], [1, 3, 5, 3], [1, 2, 3, 5]]
    n_w = 0
    for i in range(4):
        for j in range(4):
            b = getattr(ker, "kernel_%d_%d" % (i, j))
            assert b.shape == (table[i][j], 2 * i + 1, 2 * j + 1, 3, 3, 3)
            want = math.sqrt((2 * i + 1) / (table[i][j] * 8))
            assert torch.allclose(b.flatten(1).norm(dim=1), torch.full((table[i][j],), want),
                                  rtol=1e-5)
            n_w += 2 * 2 * table[i][j]
    assert ker.weight.numel() == n_w == 152
    assert ker.n_in == ker.n_out == 32
    assert sorted(ker.state_dict().keys()) == sorted(
        ["weight"] + ["kernel_%d_%d" % (i, j) for i in range(4) for j in range(4)])
    k5 = SE3Kernel([(1, 0), (1, 2)], [(1, 1)], 5)
    assert [getattr(k5, "kernel_0_%d" % j).shape[0] for j in range(2)] == [2, 6]


def test_kernel_basis_rotation_equivariance_of_dense_kernel():
    """A dense kernel built from the basis commutes with the 90-degree rotations of
    the grid: K(R x) = D_out(R) K(x) D_in(R)^T for R = quarter turns about z and y."""
    from ss_conv.utils.kernel import SE3Kernel
    from ss_conv.utils import SO3
    torch.manual_seed(3)
    rs_in, rs_out = [(1, 0), (1, 1), (1, 2)], [(1, 1), (1, 2)]
    ker = SE3Kernel(rs_in, rs_out, 5)
    bases = [[getattr(ker, "kernel_%d_%d" % (i, j)).double() for j in range(3)] for i in range(2)]

    def block_diag(rs, a, b, c):
        mats = [torch.tensor(SO3.wigner_D_np(l, a, b, c)) for m, l in rs for _ in range(m)]
        return torch.block_diag(*mats)

    w = ker.weight.detach().double()
    rows, off = [], 0
    for i in range(2):
        cols = []
        for j in range(3):
            nb = bases[i][j].shape[0]
            cols.append(torch.einsum("b,bijxyz->ijxyz", w[off:off + nb], bases[i][j]))
            off += nb
        rows.append(torch.cat(cols, 1))
    K = torch.cat(rows, 0)  # [Cout, Cin, x, y, z]
    # u = +pi/2 about y: (u^-1 x) sampling is transpose(x,z) then flip z (utils/kernel.py:52)
    moved = K.transpose(2, 4).flip(4)
    back = torch.einsum("ij,jkxyz,kl->ilxyz", block_diag(rs_out, 0, math.pi / 2, 0), moved,
                        block_diag(rs_in, 0, -math.pi / 2, 0))
    assert torch.allclose(back, K, atol=1e-6)  # the buffers are stored in float32
    # u = +pi/2 about z: (x,y) -> (-y,x), so K(u^-1 x)[ix,iy] = K[iy,-ix]
    moved = K.transpose(2, 3).flip(2)
    back = torch.einsum("ij,jkxyz,kl->ilxyz", block_diag(rs_out, math.pi / 2, 0, 0), moved,
                        block_diag(rs_in, -math.pi / 2, 0, 0))
    assert torch.allclose(back, K, atol=1e-6)


# ---- torch-op layers -----------------------------------------------------------------------
class _Holder:
    def __init__(self, f):
        self.features = f


def _batchnorm_loops(x, Rs, mean, var, weight, bias, eps, training):
    """Loop-per-field statement of the reference layer (batchnorm.py:49-136)."""
    outs, new_mean, new_var = [], [], []
    ix = im = iv = 0
    for m, l in Rs:
        d = 2 * l + 1
        f = x[:, ix:ix + m * d].reshape(-1, m, d)
        ix += m * d
        if d == 1:
            mu = f.mean(0).reshape(-1) if training else mean[im:im + m]
            new_mean.append(mu)
            f = f - mu.reshape(1, m, 1)
        nrm = (f ** 2).sum(2).mean(0) if training else var[iv:iv + m]
        new_var.append(nrm)
        scale = (nrm + eps).pow(-0.5) * weight[iv:iv + m]
        f = f * scale.reshape(1, m, 1)
        if d == 1:
            f = f + bias[im:im + m].reshape(1, m, 1)
            im += m
        iv += m
        outs.append(f.reshape(-1, m * d))
    return torch.cat(outs, 1), torch.cat(new_mean), torch.cat(new_var)


@pytest.mark.parametrize("training", [True, False])
def test_batchnorm_matches_per_field_loops(training):
    from ss_conv.batchnorm import BatchNorm
    torch.manual_seed(0)
    Rs = [(3, 0), (2, 1), (2, 2), (1, 0)]
    bn = BatchNorm(Rs)
    with torch.no_grad():
        bn.weight.uniform_(0.5, 1.5)
        bn.bias.uniform_(-1, 1)
        bn.running_mean.uniform_(-1, 1)
        bn.running_var.uniform_(0.5, 2)
    bn.train(training)
    x = torch.randn(50, 3 + 6 + 10 + 1) * 2 + 0.3
    rm, rv = bn.running_mean.clone(), bn.running_var.clone()
    want, mu, nv = _batchnorm_loops(x, Rs, rm, rv, bn.weight.detach(), bn.bias.detach(), bn.eps,
                                    training)
    h = _Holder(x.clone())
    out = bn(h)
    assert out is h
    assert torch.allclose(h.features, want, atol=1e-5)
    if training:
        assert torch.allclose(bn.running_mean, 0.9 * rm + 0.1 * mu, atol=1e-6)
        assert torch.allclose(bn.running_var, 0.9 * rv + 0.1 * nv, atol=1e-6)
    assert sorted(bn.state_dict().keys()) == ["bias", "running_mean", "running_var", "weight"]
    with pytest.raises(AssertionError):
        bn(_Holder(torch.randn(5, 7)))


def test_gated_activation():
    from ss_conv.activation import Activation
    torch.manual_seed(1)
    Rs = [(3, 0), (2, 1), (1, 2)]
    act = Activation(Rs, (torch.relu, torch.sigmoid))
    with torch.no_grad():
        act.scalar_act.bias.uniform_(-1, 1)
        act.gate_act.bias.uniform_(-1, 1)
    x = torch.randn(20, 3 + 6 + 5 + 3)  # fields then one gate per non-scalar field
    h = _Holder(x.clone())
    assert act(h) is h
    y = h.features
    assert y.shape == (20, 14)
    assert torch.allclose(y[:, :3], torch.relu(x[:, :3] + act.scalar_act.bias))
    gate = torch.sigmoid(x[:, 14:] + act.gate_act.bias)
    assert torch.allclose(y[:, 3:6], x[:, 3:6] * gate[:, 0:1])
    assert torch.allclose(y[:, 6:9], x[:, 6:9] * gate[:, 1:2])
    assert torch.allclose(y[:, 9:14], x[:, 9:14] * gate[:, 2:3])
    assert sorted(act.state_dict().keys()) == ["gate_act.bias", "scalar_act.bias"]
    ident = Activation(Rs, (None, None))
    h = _Holder(x.clone())
    ident(h)
    assert torch.equal(h.features, x)


def test_dropout():
    from ss_conv.dropout import Dropout
    torch.manual_seed(2)
    Rs = [(2, 0), (3, 1)]
    x = torch.ones(200, 2 + 9)
    drop = Dropout(Rs, p=0.5)
    drop.eval()
    h = _Holder(x)
    assert drop(h).features is x
    drop.train()
    y = drop(_Holder(x.clone())).features
    assert set(y.unique().tolist()) <= {0.0, 2.0}
    v = y[:, 2:].reshape(200, 3, 3)
    assert torch.equal(v[:, :, 0], v[:, :, 1]) and torch.equal(v[:, :, 0], v[:, :, 2])
    assert 0.3 < (y == 0).float().mean() < 0.7


def test_dropout_draws_the_masks_like_the_reference():
    """Same seed, same masks: one new_empty(n, m).bernoulli_(1 - p).div_(1 - p) per entry of
    Rs, in order, expanded over the 2l+1 components (ss_conv/dropout.py:32-45)."""
    from ss_conv.dropout import Dropout
    Rs = [(3, 0), (0, 1), (2, 1), (1, 2)]
    x = torch.randn(50, 3 + 6 + 5)
    drop = Dropout(Rs, p=0.3).train()
    torch.manual_seed(7)
    y = drop(_Holder(x.clone())).features
    torch.manual_seed(7)
    noises = []
    for m, l in Rs:
        if m == 0:
            continue
        noise = x.new_empty(50, m).bernoulli_(0.7).div_(0.7)
        noises.append(noise.unsqueeze(2).expand(-1, -1, 2 * l + 1).contiguous().view(50, -1))
    assert torch.equal(y, x * torch.cat(noises, dim=1))
    for p, value in ((0.0, x), (1.0, torch.zeros_like(x))):
        assert torch.equal(Dropout(Rs, p=p).train()(_Holder(x.clone())).features, value)


def test_synthetic_generator_is_seeded():
    import synth
    a = synth.make_clouds(2, 100, seed=5, rotate=True, channels=3)
    b = synth.make_clouds(2, 100, seed=5, rotate=True, channels=3)
    for x, y in zip(a, b):
        assert np.array_equal(x, y)
    assert np.abs(a[0]).max() < 1.0 and a[1].shape == (200, 3) and a[2].tolist()[99:101] == [0, 1]
    idx = synth.voxel_indices(a[0], a[2], 16)
    assert idx.min() >= 0 and idx[:, 1:].max() < 16


def test_layers_outside_the_native_layouts():
    """A gated activation whose first entry is not a scalar field keeps the torch code (the
    gate tables would ask for gates the reference never counts); a transposed convolution
    is a layer like any other (its output size follows ops.py:26-36 of the reference)."""
    from ss_conv import bnact
    from ss_conv.activation import Activation
    from ss_conv.sp_ops.conv import SparseConvolution
    assert bnact.canonical([(4, 0), (2, 1), (2, 2)])
    assert bnact.canonical([(0, 0), (2, 1)])
    assert not bnact.canonical([(4, 1), (2, 2)])
    assert not bnact.canonical([(4, 0), (2, 0)])
    act = Activation([(4, 1), (2, 2)], (torch.relu, torch.sigmoid))
    assert not act._kernel_ok
    layer = SparseConvolution(3, 4, 4, 3, stride=2, padding=1, output_padding=1, transposed=True)
    assert layer.transposed and layer.output_padding == [1, 1, 1]
    from ss_conv.sp_ops.ops import get_deconv_output_size
    assert get_deconv_output_size([5, 6, 7], [3] * 3, [2] * 3, [1] * 3, [1] * 3, [1] * 3) == \
        [10, 12, 14]


def test_epilogue_layout_keeps_gates_with_their_columns():
    """bnact.epilogue_layout: every output column appears once, in order inside its block;
    a gated column's gate sits in the same block of 64; data runs start at multiples of 4;
    gates that no column reads are not computed; sizes are multiples of 4."""
    from ss_conv import bnact
    cases = [[(10, 0), (6, 1), (4, 2), (2, 3)], [(32, 0), (32, 1), (32, 2), (32, 3)],
             [(3, 0), (2, 1), (2, 2)], [(16, 0)], [(0, 0), (20, 3)], [(4, 0), (3, 0), (5, 1)]]
    for Rs in cases:
        tables, c_out, n_gates = bnact.gate_layout(Rs, True, True)
        lay = bnact.epilogue_layout(c_out, tables["out_mode"].tolist(), tables["gate_col"].tolist())
        src, mode, gate, dest = (lay[k].tolist() for k in ("src", "mode", "gate", "dest"))
        n = len(src)
        assert n % 4 == 0 and len(mode) == len(gate) == len(dest) == n
        stored = [(dest[c], c) for c in range(n) if mode[c] != 3]
        assert sorted(d for d, _ in stored) == list(range(c_out))
        for d, c in stored:
            assert src[c] == d and mode[c] == int(tables["out_mode"][d])
            if c % 4 == 0:
                assert d % 4 == 0
            if mode[c] == 2:
                g = gate[c]
                first, count = lay["gate_run"].tolist()[2 * (c // 64):2 * (c // 64) + 2]
                assert g // 64 == c // 64 and mode[g] == 3 and count <= 16
                assert first <= g < first + count and (first + count - 1) // 64 == c // 64
                assert src[g] == int(tables["gate_col"][d])
        used = {int(tables["gate_col"][d]) for d in range(c_out) if int(tables["out_mode"][d]) == 2}
        computed = {src[c] for c in range(n) if mode[c] == 3 and src[c] >= 0}
        assert computed == used
    # no activation: identity order, padded to a multiple of 4
    lay = bnact.epilogue_layout(10)
    assert lay["src"].tolist() == list(range(10)) + [-1, -1]
    assert lay["mode"].tolist() == [0] * 10 + [3, 3]
    assert lay["gate_run"].tolist() == [12, 0]
