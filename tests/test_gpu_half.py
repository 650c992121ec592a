"""GPU parity of the half-precision convolution entry points (ssc_conv_fwd_f16,
ssc_conv_bwd_filter_f16; reference: indice_conv_half / indice_conv_backward_half,
src/ss_conv_ops.cu:74-83).

The library multiplies half values exactly, accumulates in fp32 (forward and input
gradient on v_mfma_f32_16x16x32_f16, filter gradient on fp32 MFMA over widened rows) and
rounds every result element to half once.  Two bars:
  * against the oracle: the sums of the half-valued inputs taken in float64 are exact to
    well below half precision, so every result element must lie within half a unit in the
    last place of half of them (plus the fp32 accumulation error, which the fp32 tests
    bound at rel-L2 1e-5);
  * against the fp32 entry points on the widened inputs, at any size: the filter gradient
    runs the same operations in the same order, so rounding the fp32 result must give the
    same bits; forward and input gradient add the same exact products in another order, so
    they may differ from the rounded fp32 result by one unit in the last place at most.
"""
import numpy as np
import pytest
import torch

import synth
from test_gpu_parity import gpu_rulebook, random_voxels, rel_l2

pytestmark = pytest.mark.gpu

HALF_EPS = 2.0 ** -11     # half a unit in the last place, relative (normal numbers)
HALF_TINY = 2.0 ** -25    # the same, absolute, for subnormal results
ACC_SLACK = 1e-5          # fp32 accumulation error, relative to the rms of the result


def within_half_rounding(got, exact):
    got = np.asarray(got, dtype=np.float64)
    exact = np.asarray(exact, dtype=np.float64)
    rms = np.sqrt(np.mean(exact ** 2)) if exact.size else 0.0
    bound = HALF_EPS * np.abs(exact) + HALF_TINY + ACC_SLACK * rms
    bad = np.abs(got - exact) > bound
    return not bad.any(), int(bad.sum())


def within_one_ulp(got_half, want_fp32):
    """got_half (torch half) against the fp32 result it should be a rounding of."""
    got = got_half.detach().double()
    want = want_fp32.detach().double()
    rms = float(want.pow(2).mean().sqrt()) if want.numel() else 0.0
    bound = 2.0 ** -10 * want.abs() + 2.0 ** -24 + ACC_SLACK * rms
    return bool(((got - want).abs() <= bound).all())


def conv_sums(feats, w, pairs, num, n_out):
    """float64 sums of the reference's gather-GEMM-scatter (src/conv/indice_conv.h:296-338)."""
    ref = np.zeros((n_out, w.shape[2]), dtype=np.float64)
    for k in range(w.shape[0]):
        m = int(num[k])
        if m:
            np.add.at(ref, pairs[k, 1, :m],
                      feats[pairs[k, 0, :m]].astype(np.float64) @ w[k].astype(np.float64))
    return ref


HALF_CASES = [
    # n_vox, grid, k, s, p, cin, cout
    (300, 10, 3, 1, 1, 32, 32),      # rows of 64 bytes, one chunk
    (900, 12, 3, 1, 1, 64, 128),     # whole chunks: the plain buffer-load gather
    (1500, 16, 3, 1, 1, 128, 136),   # two chunks, three column blocks
    (200, 10, 3, 2, 1, 40, 72),      # a partial chunk on the buffer-load gather
    (100, 8, 3, 1, 1, 5, 7),         # odd widths: scalar loads and stores
    (150, 8, 5, 1, 2, 37, 24),
    (6000, 24, 3, 1, 1, 64, 80),     # many tiles per workgroup
]


def _half_inputs(case, seed, shuffle=False):
    n, grid, k, s, p, cin, cout = case
    rng = np.random.default_rng(seed)
    idx = random_voxels(rng, 2, grid, n)
    if shuffle:
        idx = idx[rng.permutation(n)]
    K = k ** 3
    feats = rng.normal(size=(n, cin)).astype(np.float16)
    w = (rng.normal(size=(K, cin, cout)) / np.sqrt(K * cin)).astype(np.float16)
    return idx, feats, w


@pytest.mark.parametrize("case", HALF_CASES)
def test_conv_half_matches_oracle(case, oracle, device):
    from ss_conv import _ext
    print("case", case, flush=True)
    n, grid, k, s, p, cin, cout = case
    idx, feats, w = _half_inputs(case, 51)
    o_idx, o_pairs, o_num = oracle.canonicalize(*oracle.rulebook(idx, 2, [grid] * 3, k, s, p))
    ref = conv_sums(feats, w, o_pairs, o_num, o_idx.shape[0])
    # the restated fp32 convolution on the same (widened) values agrees with those sums
    ref32 = oracle.conv_fwd(feats.astype(np.float32), w.astype(np.float32), o_pairs, o_num,
                            o_idx.shape[0], matmul=np.matmul)
    assert rel_l2(ref32, ref) < 1e-5

    g_idx, g_pairs, g_num = [torch.from_numpy(x).to(device) for x in
                             gpu_rulebook(idx, 2, grid, k, s, p)]
    f_h = torch.from_numpy(feats).to(device)
    w_h = torch.from_numpy(w).to(device).reshape(k, k, k, cin, cout)
    out = _ext.indice_conv_half(f_h, w_h, g_pairs, g_num, g_idx.shape[0], 0, 0)
    assert out.dtype == torch.float16 and tuple(out.shape) == (o_idx.shape[0], cout)
    ok, n_bad = within_half_rounding(out.cpu().numpy(), ref)
    assert ok, n_bad
    out32 = _ext.indice_conv_fp32(f_h.float(), w_h.float(), g_pairs, g_num, g_idx.shape[0], 0, 0)
    assert within_one_ulp(out, out32)


def test_conv_half_inverse_unsorted_and_strided_filters(oracle, device):
    """The pair planes swapped, rows in arbitrary order (the re-ordering path) and the
    reference's permuted filter view [Cout, Cin, k, k, k] -> [k, k, k, Cin, Cout]."""
    from ss_conv import _ext
    case = (300, 10, 3, 2, 1, 24, 16)
    n, grid, k, s, p, cin, cout = case
    idx, _, w = _half_inputs(case, 52, shuffle=True)
    rng = np.random.default_rng(53)
    # the rulebook itself is covered by the rulebook tests; here it only supplies pairs
    g_idx, g_pairs, g_num = [torch.from_numpy(x).to(device) for x in
                             gpu_rulebook(idx, 2, grid, k, s, p)]
    n_out = g_idx.shape[0]
    # features on the outputs of the rulebook, results on its inputs
    feats = rng.normal(size=(n_out, cin)).astype(np.float16)
    pairs = g_pairs.cpu().numpy()
    num = g_num.cpu().numpy()
    ref = np.zeros((n, cout), dtype=np.float64)
    for kk in range(k ** 3):
        m = int(num[kk])
        np.add.at(ref, pairs[kk, 0, :m],
                  feats[pairs[kk, 1, :m]].astype(np.float64) @ w[kk].astype(np.float64))
    wt = torch.from_numpy(w).to(device)
    wt = wt.permute(2, 1, 0).contiguous().reshape(cout, cin, k, k, k).permute(2, 3, 4, 1, 0)
    assert not wt.is_contiguous()
    out = _ext.indice_conv_half(torch.from_numpy(feats).to(device), wt, g_pairs, g_num, n, 1, 0)
    ok, n_bad = within_half_rounding(out.cpu().numpy(), ref)
    assert ok, n_bad


BWD_HALF_CASES = [
    (300, 10, 3, 1, 1, 32, 32),
    (900, 12, 3, 1, 1, 64, 128),
    (200, 10, 3, 2, 1, 128, 72),
    (100, 8, 2, 2, 0, 5, 7),
    (150, 8, 5, 1, 2, 40, 24),
]


@pytest.mark.parametrize("case", BWD_HALF_CASES)
def test_conv_backward_half_matches_oracle(case, oracle, device):
    from ss_conv import _ext
    print("case", case, flush=True)
    n, grid, k, s, p, cin, cout = case
    K = k ** 3
    idx, feats, w = _half_inputs(case, 54)
    rng = np.random.default_rng(55)
    o_idx, o_pairs, o_num = oracle.canonicalize(*oracle.rulebook(idx, 2, [grid] * 3, k, s, p))
    g_out = rng.normal(size=(o_idx.shape[0], cout)).astype(np.float16)
    # float64 statements of the two gradients (src/conv/indice_conv.h:385-421)
    ref_in = np.zeros((n, cin), dtype=np.float64)
    ref_w = np.zeros((K, cin, cout), dtype=np.float64)
    for kk in range(K):
        m = int(o_num[kk])
        if m:
            fi = feats[o_pairs[kk, 0, :m]].astype(np.float64)
            go = g_out[o_pairs[kk, 1, :m]].astype(np.float64)
            ref_w[kk] = fi.T @ go
            np.add.at(ref_in, o_pairs[kk, 0, :m], go @ w[kk].astype(np.float64).T)
    # the restated backward agrees with them
    chk_in, chk_w = oracle.conv_bwd(feats.astype(np.float32), w.astype(np.float32),
                                    g_out.astype(np.float32), o_pairs, o_num)
    assert rel_l2(chk_in, ref_in) < 1e-5 and rel_l2(chk_w, ref_w) < 1e-5

    g_idx, g_pairs, g_num = [torch.from_numpy(x).to(device) for x in
                             gpu_rulebook(idx, 2, grid, k, s, p)]
    f_h = torch.from_numpy(feats).to(device)
    w_h = torch.from_numpy(w).to(device).reshape(k, k, k, cin, cout)
    go_h = torch.from_numpy(g_out).to(device)
    d_in, d_w = _ext.indice_conv_backward_half(f_h, w_h, go_h, g_pairs, g_num, 0, 0)
    assert d_in.dtype == torch.float16 and d_w.dtype == torch.float16
    assert d_w.shape == w_h.shape and tuple(d_in.shape) == (n, cin)
    ok, n_bad = within_half_rounding(d_in.cpu().numpy(), ref_in)
    assert ok, ("input gradient", n_bad)
    ok, n_bad = within_half_rounding(d_w.cpu().numpy().reshape(K, cin, cout), ref_w)
    assert ok, ("filter gradient", n_bad)
    e_in, e_w = _ext.indice_conv_backward_fp32(f_h.float(), w_h.float(), go_h.float(), g_pairs,
                                               g_num, 0, 0)
    assert within_one_ulp(d_in, e_in) and torch.equal(d_w, e_w.half())


def test_conv_half_benchmark_size_equals_rounded_fp32(device):
    """The second benchmark configuration (32 clouds, 64^3, 64 -> 128 channels): the half
    entry points give the rounded results of the fp32 entry points (the filter gradient bit
    for bit, the others to one unit in the last place)."""
    from ss_conv import _ext
    from ss_conv.sp_ops.ops import get_indice_pairs
    cfg = synth.CONFIGS["cfg2"]
    pts, _, ids = synth.config_clouds("cfg2", seed=3)
    grid, k = cfg["grid"], cfg["kernel"]
    t = torch.from_numpy(synth.voxel_indices(pts, ids, grid)).to(device)
    out_idx, pairs, num = get_indice_pairs(t, cfg["batch"], [grid] * 3, k, cfg["stride"],
                                           cfg["padding"], 1, 0, False)
    cin = sum(cfg["mult_in"] * (2 * l + 1) for l in range(cfg["lmax"] + 1))
    cout = sum(cfg["mult_out"] * (2 * l + 1) for l in range(cfg["lmax"] + 1))
    assert (cin, cout) == (64, 128)
    gen = torch.Generator(device).manual_seed(5)
    f_h = torch.randn((t.shape[0], cin), device=device, generator=gen).half()
    w_h = (torch.randn((k, k, k, cin, cout), device=device, generator=gen)
           / (27 * cin) ** 0.5).half()
    n_out = out_idx.shape[0]
    out = _ext.indice_conv_half(f_h, w_h, pairs, num, n_out, 0, 0)
    out32 = _ext.indice_conv_fp32(f_h.float(), w_h.float(), pairs, num, n_out, 0, 0)
    assert within_one_ulp(out, out32)
    go_h = torch.randn((n_out, cout), device=device, generator=gen).half()
    d_in, d_w = _ext.indice_conv_backward_half(f_h, w_h, go_h, pairs, num, 0, 0)
    e_in, e_w = _ext.indice_conv_backward_fp32(f_h.float(), w_h.float(), go_h.float(), pairs, num,
                                               0, 0)
    assert within_one_ulp(d_in, e_in) and torch.equal(d_w, e_w.half())


def test_conv_half_empty_and_dtype_errors(device):
    from ss_conv import _ext
    pairs = torch.full((27, 2, 0), -1, dtype=torch.int32, device=device)
    num = torch.zeros(27, dtype=torch.int32, device=device)
    f = torch.zeros((0, 8), dtype=torch.float16, device=device)
    w = torch.zeros((3, 3, 3, 8, 12), dtype=torch.float16, device=device)
    out = _ext.indice_conv_half(f, w, pairs, num, 5, 0, 0)
    assert out.dtype == torch.float16 and tuple(out.shape) == (5, 12) and not out.any()
    with pytest.raises(RuntimeError):
        _ext.indice_conv_half(f.float(), w, pairs, num, 5, 0, 0)
    with pytest.raises(RuntimeError):
        _ext.indice_conv_fp32(f, w, pairs, num, 5, 0, 0)


def test_convolution_layer_on_half_features(device):
    """Convolution on a half-precision SparseTensor: the kernel is synthesised in fp32 and
    rounded to the features' type; forward and gradients equal the fp32 layer's on the
    widened values to one unit in the last place of half."""
    from ss_conv.convolution import Convolution
    from ss_conv.sp_ops.tensor import SparseTensor
    torch.manual_seed(4)
    rng = np.random.default_rng(6)
    grid = 12
    idx = torch.from_numpy(random_voxels(rng, 2, grid, 500)).to(device)
    rs_in, rs_out = synth.irreps(8, 3), synth.irreps(16, 3)
    conv = Convolution(rs_in, rs_out, 3, stride=1, padding=1).to(device).train()
    cin = sum(m * (2 * l + 1) for m, l in rs_in)
    x_h = torch.randn((500, cin), device=device).half().requires_grad_(True)
    y = conv(SparseTensor(x_h, idx, [grid] * 3, 2)).features
    assert y.dtype == torch.float16
    w_h = conv.kernel().permute(2, 3, 4, 1, 0).half()
    x32 = x_h.detach().float().requires_grad_(True)
    from ss_conv.sp_ops import functional as Fsp
    from ss_conv.sp_ops.ops import get_indice_pairs
    out_idx, pairs, num = get_indice_pairs(idx, 2, [grid] * 3, 3, 1, 1, 1, 0, False)
    y32 = Fsp.indice_conv(x32, w_h.float(), pairs, num, out_idx.shape[0])
    assert within_one_ulp(y, y32)
    g = torch.randn_like(y32).half()
    y.backward(g)
    y32.backward(g.float())
    assert within_one_ulp(x_h.grad, x32.grad)
    assert conv.kernel.weight.grad is not None and torch.isfinite(conv.kernel.weight.grad).all()


@pytest.mark.parametrize("k,s,p,c", [(2, 2, 0, 64), (3, 2, 1, 32), (3, 1, 1, 5), (3, 1, 1, 12)])
def test_half_pools_match_oracle(k, s, p, c, oracle, device):
    """ssc_pool_{max,avg}_f16 and their gradients (indice_maxpool_half, indice_avgpool_half,
    indice_*pool_backward_half; src/ss_conv_ops_api.cpp:29-35) against the oracle's half
    routines, bit for bit: every operation rounds to half, in the order of the offsets.
    Forward through the raw entry points, backward through autograd as a layer runs it."""
    from ss_conv import _ext
    from ss_conv.sp_ops.functional import indice_avgpool, indice_maxpool
    rng = np.random.default_rng(41)
    n, grid = 400, 10
    idx = random_voxels(rng, 2, grid, n)
    feats = rng.normal(size=(n, c)).astype(np.float16)
    o_idx, o_pairs, o_num = oracle.canonicalize(*oracle.rulebook(idx, 2, [grid] * 3, k, s, p))
    n_out = o_idx.shape[0]
    g_idx, g_pairs, g_num = [torch.from_numpy(x).to(device) for x in
                             gpu_rulebook(idx, 2, grid, k, s, p)]
    ft = torch.from_numpy(feats).to(device)
    mx = _ext.indice_maxpool_half(ft, g_pairs, g_num, n_out)
    assert mx.dtype == torch.half
    want_mx = oracle.maxpool_fwd_half(feats, o_pairs, o_num, n_out)
    assert np.array_equal(mx.cpu().numpy(), want_mx)
    rf = _ext.indiceSummaryRF(g_pairs, g_num, n_out)
    for r in (torch.full((n_out,), k ** 3, dtype=torch.int32, device=device), rf):
        av = _ext.indice_avgpool_half(ft, g_pairs, g_num, n_out, r)
        want = oracle.avgpool_fwd_half(feats, o_pairs, o_num, n_out, r.cpu().numpy())
        assert np.array_equal(av.cpu().numpy(), want)
    g_out = rng.normal(size=(n_out, c)).astype(np.float16)
    gt = torch.from_numpy(g_out).to(device)
    x = ft.clone().requires_grad_(True)
    indice_maxpool(x, g_pairs, g_num, n_out).backward(gt)
    assert np.array_equal(x.grad.cpu().numpy(),
                          oracle.maxpool_bwd_half(feats, want_mx, g_out, o_pairs, o_num))
    x = ft.clone().requires_grad_(True)
    indice_avgpool(x, g_pairs, g_num, n_out).backward(gt)
    want = oracle.avgpool_bwd_half(g_out, o_pairs, o_num, n,
                                   np.full(n_out, k ** 3, dtype=np.int32))
    assert np.array_equal(x.grad.cpu().numpy(), want)
    with pytest.raises(RuntimeError):
        _ext.indice_maxpool_half(ft.float(), g_pairs, g_num, n_out)
