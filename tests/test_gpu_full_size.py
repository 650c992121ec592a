"""GPU parity at the full sizes of the benchmark configurations (2 clouds x 1024 points at
32^3; 32 clouds x 2048 points at 64^3 with stride 1 and 2; the backbone on 32 clouds x 1024
points at 64^3; 8 clouds x 16384 points at 128^3 with a 5^3 kernel).

Rulebooks: bit-exact against the oracle, which runs these sizes in seconds.
Convolution, forward and both gradients: against the oracle's gather-GEMM-scatter where
that finishes in seconds, and at every size against a float64 statement of the same sums
(src/conv/indice_conv.h:296-338, 385-421) evaluated with torch on the GPU -- a different
formulation (one GEMM and one index_add per offset) of the same numbers -- plus two
properties that do not depend on the size: linearity in the features, and the column sums
of the output, which must equal sum_k (sum of the gathered rows of offset k) . W[k]."""
import numpy as np
import pytest
import torch

import synth
from test_gpu_parity import REL_L2, rel_l2

pytestmark = pytest.mark.gpu

FULL = ["cfg1", "cfg2", "cfg3", "cfg5"]


def _channels(cfg, key):
    return sum(cfg[key] * (2 * l + 1) for l in range(cfg["lmax"] + 1))


def _voxels(name):
    cfg = synth.CONFIGS[name]
    pts, _, ids = synth.config_clouds(name, seed=1)
    return cfg, synth.voxel_indices(pts, ids, cfg["grid"])


def _gpu_rulebook(cfg, idx, device):
    from ss_conv.sp_ops.ops import get_indice_pairs
    t = torch.from_numpy(idx).to(device)
    return get_indice_pairs(t, cfg["batch"], [cfg["grid"]] * 3, cfg["kernel"], cfg["stride"],
                            cfg["padding"], 1, 0, False)


def _rel(a, b):
    return float((a.double() - b).norm() / b.norm().clamp_min(1e-300))


@pytest.mark.parametrize("name", FULL)
def test_rulebook_full_size_matches_oracle(name, oracle, device):
    print("config", name, flush=True)
    cfg, idx = _voxels(name)
    want = oracle.canonicalize(*oracle.rulebook(idx, cfg["batch"], [cfg["grid"]] * 3,
                                                cfg["kernel"], cfg["stride"], cfg["padding"]))
    got = _gpu_rulebook(cfg, idx, device)
    for g, w in zip(got, want):
        assert np.array_equal(g.cpu().numpy(), w)


@pytest.mark.parametrize("name", FULL)
def test_conv_full_size(name, oracle, device):
    cfg = synth.CONFIGS[name]
    _conv_full_size(name, _channels(cfg, "mult_in"), _channels(cfg, "mult_out"), oracle, device,
                    with_oracle=name != "cfg5")  # cfg5's CPU restatement takes minutes


@pytest.mark.parametrize("channels", [(64, 72), (128, 136), (152, 8)])
def test_conv_full_size_lone_last_group(channels, oracle, device):
    """Channel counts whose last group of 16 output columns runs the kernel's
    one-column-group form (both gradients included: the input gradient of 64 -> 72 is a
    72 -> 64 convolution), on the clouds of the second configuration."""
    _conv_full_size("cfg2", channels[0], channels[1], oracle, device, with_oracle=True)


def _conv_full_size(name, cin, cout, oracle, device, with_oracle):
    from ss_conv import _ext
    print("config", name, cin, cout, flush=True)
    cfg, idx = _voxels(name)
    k = cfg["kernel"]
    K = k ** 3
    out_idx, pairs, num = _gpu_rulebook(cfg, idx, device)
    n_in, n_out = idx.shape[0], out_idx.shape[0]
    nums = num.cpu().numpy()
    gen = torch.Generator(device).manual_seed(9)
    f = torch.randn((n_in, cin), device=device, generator=gen)
    w = torch.randn((K, cin, cout), device=device, generator=gen) / (K * cin) ** 0.5
    w5 = w.reshape(k, k, k, cin, cout)
    go = torch.randn((n_out, cout), device=device, generator=gen)

    out = _ext.indice_conv_fp32(f, w5, pairs, num, n_out, 0, 0)
    d_in, d_w = _ext.indice_conv_backward_fp32(f, w5, go, pairs, num, 0, 0)

    # float64 statement of the three results, offset by offset
    ref = torch.zeros((n_out, cout), dtype=torch.float64, device=device)
    ref_in = torch.zeros((n_in, cin), dtype=torch.float64, device=device)
    ref_w = torch.zeros((K, cin, cout), dtype=torch.float64, device=device)
    col_sums = torch.zeros(cout, dtype=torch.float64, device=device)
    for kk in range(K):
        m = int(nums[kk])
        if m == 0:
            continue
        i_rows, o_rows = pairs[kk, 0, :m].long(), pairs[kk, 1, :m].long()
        fi, gk, wk = f[i_rows].double(), go[o_rows].double(), w[kk].double()
        ref.index_add_(0, o_rows, fi @ wk)
        ref_in.index_add_(0, i_rows, gk @ wk.t())
        ref_w[kk] = fi.t() @ gk
        col_sums += fi.sum(0) @ wk
    assert _rel(out, ref) < REL_L2
    assert _rel(d_in, ref_in) < REL_L2
    assert _rel(d_w.reshape(K, cin, cout), ref_w) < REL_L2
    # column sums: every pair counted once, none dropped
    assert _rel(out.double().sum(0), col_sums) < REL_L2
    # linearity in the features
    f2 = torch.randn((n_in, cin), device=device, generator=gen)
    out2 = _ext.indice_conv_fp32(f2, w5, pairs, num, n_out, 0, 0)
    mix = _ext.indice_conv_fp32(2.0 * f + f2, w5, pairs, num, n_out, 0, 0)
    assert _rel(mix, 2.0 * out.double() + out2.double()) < REL_L2
    # rows no pair lands on are zero (every active output has at least one pair here, so
    # this holds trivially unless the rulebook and the convolution disagree on n_out)
    assert out.shape == (n_out, cout) and bool(torch.isfinite(out).all())
    if with_oracle:  # the CPU restatement of these sizes takes seconds
        o_ref = oracle.conv_fwd(f.cpu().numpy(), w.cpu().numpy(), pairs.cpu().numpy(), nums,
                                n_out, matmul=np.matmul)
        assert rel_l2(out.cpu().numpy(), o_ref) < REL_L2


def test_conv_cfg5_against_the_oracle_fixture(device):
    """The fifth configuration's convolution (200 -> 200 channels, 125 offsets: the five-group
    form, three launches) against the CPU oracle at full size.  The oracle needs minutes
    for this layer, so tests/golden/make_conv_cfg5_golden.py ran it once and kept 2048
    sampled output rows, their voxel keys, the column sums and the sum of squares of the
    whole output; the inputs are seeded numpy draws, regenerated here."""
    import os
    import sys
    from ss_conv import _ext
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    sys.path.insert(0, here)
    try:
        from make_conv_cfg5_golden import cfg5_inputs
    finally:
        sys.path.remove(here)
    gold = np.load(os.path.join(here, "conv_cfg5_rows.npz"))
    cfg, idx, f, w = cfg5_inputs()
    k = cfg["kernel"]
    c = f.shape[1]
    out_idx, pairs, num = _gpu_rulebook(cfg, idx, device)
    n_out = out_idx.shape[0]
    assert idx.shape[0] == int(gold["n_in"]) and n_out == int(gold["n_out"])
    assert int(num.sum().item()) == int(gold["pairs"])
    rows = torch.from_numpy(gold["rows"]).long().to(device)
    assert np.array_equal(out_idx[rows].cpu().numpy(), gold["out_row_keys"])
    tf = torch.from_numpy(f).to(device)
    tw = torch.from_numpy(w).to(device).reshape(k, k, k, c, c)
    out = _ext.indice_conv_fp32(tf, tw, pairs, num, n_out, 0, 0)
    got = out[rows].cpu().numpy()
    assert rel_l2(got, gold["out_rows"]) < REL_L2
    # every element of the sampled rows, not only their norm
    scale = float(np.sqrt((gold["out_rows"].astype(np.float64) ** 2).mean()))
    assert float(np.abs(got - gold["out_rows"]).max()) < 1e-4 * scale
    assert rel_l2(out.double().sum(0).cpu().numpy(), gold["col_sums"]) < REL_L2
    sq = float((out.double() ** 2).sum().item())
    assert abs(sq - float(gold["sq_sum"])) < 1e-5 * float(gold["sq_sum"])


def test_downsampling_block_full_size(oracle, device):
    """The third configuration as stated: the stride-2 layer (128 -> 256 channels) on 32
    clouds x 2048 points at 64^3, then MaxPool and AvgPool with kernel 2, stride 2 over its
    85 k x 256 output -- rulebooks and pooled rows bit-exact against the oracle (the pools
    keep the reference's operation order), the convolution against the oracle's
    gather-GEMM-scatter."""
    from ss_conv.pool import AvgPool, MaxPool
    from ss_conv.sp_ops.conv import SparseConvolution
    from ss_conv.sp_ops.tensor import SparseTensor
    cfg, idx = _voxels("cfg3")
    grid, batch = cfg["grid"], cfg["batch"]
    cin, cout = _channels(cfg, "mult_in"), _channels(cfg, "mult_out")
    rng = np.random.default_rng(12)
    f = rng.standard_normal((idx.shape[0], cin), dtype=np.float32)
    torch.manual_seed(3)
    conv = SparseConvolution(3, cin, cout, 3, stride=2, padding=1, bias=False).to(device)
    t = torch.from_numpy(idx).to(device)
    with torch.no_grad():
        y = conv(SparseTensor(torch.from_numpy(f).to(device), t, [grid] * 3, batch))
        mx = MaxPool(2, 2)(y)
        av = AvgPool(2, 2)(y)
    o_idx, o_pairs, o_num = oracle.canonicalize(*oracle.rulebook(idx, batch, [grid] * 3, 3, 2, 1))
    assert np.array_equal(y.indices.cpu().numpy(), o_idx)
    assert y.features.shape == (o_idx.shape[0], cout) and cout == 256
    w = conv.weight.detach().reshape(27, cin, cout).cpu().numpy()
    ref = oracle.conv_fwd(f, w, o_pairs, o_num, o_idx.shape[0], matmul=np.matmul)
    y_np = y.features.cpu().numpy()
    assert rel_l2(y_np, ref) < REL_L2
    half = [int(v) for v in y.spatial_shape]
    assert half == [grid // 2] * 3
    p_idx, p_pairs, p_num = oracle.canonicalize(*oracle.rulebook(o_idx, batch, half, 2, 2, 0))
    assert np.array_equal(mx.indices.cpu().numpy(), p_idx)
    assert np.array_equal(av.indices.cpu().numpy(), p_idx)
    # the pools on the GPU's own convolution output: bit for bit
    assert np.array_equal(mx.features.cpu().numpy(),
                          oracle.maxpool_fwd(y_np, p_pairs, p_num, p_idx.shape[0]))
    assert np.array_equal(av.features.cpu().numpy(),
                          oracle.avgpool_fwd(y_np, p_pairs, p_num, p_idx.shape[0]))


def test_layer_chain_full_size(device):
    """cfg3's stride-2 layer followed by average pooling and the global pools at full size:
    sizes and invariants (pooling a non-negative tensor's maximum dominates its average;
    the segment mean of a constant column is the constant)."""
    from ss_conv.pool import AvgPool, MaxPool, GlobalAvgPool
    from ss_conv.sp_ops.tensor import SparseTensor
    cfg, idx = _voxels("cfg3")
    t = torch.from_numpy(idx).to(device)
    x = torch.rand((idx.shape[0], 64), device=device)
    x[:, 0] = 3.0
    st = SparseTensor(x, t, [cfg["grid"]] * 3, cfg["batch"])
    mx = MaxPool(3, 2, 1)(SparseTensor(x, t, [cfg["grid"]] * 3, cfg["batch"]))
    av = AvgPool(3, 2, 1)(st)
    assert torch.equal(mx.indices, av.indices)
    assert bool((mx.features >= av.features - 1e-6).all())
    assert bool((mx.features[:, 0] == 3.0).all())
    offs = av.get_offsets().int().contiguous()
    pooled = GlobalAvgPool()(mx.features.contiguous(), offs)
    assert pooled.shape == (cfg["batch"], 64)
    assert torch.allclose(pooled[:, 0], torch.full((cfg["batch"],), 3.0, device=device))


def test_backbone_full_size(oracle, device):
    """The fourth configuration at its real size: Point2Voxel (32 clouds x 1024 points, 64^3)
    -> four stages of [Convolution k3 -> BatchNorm -> gated Activation], irreps (8,8,8,8) ->
    (16,...) -> (32,...) -> (32,...), stride 2 at stages 2 and 3 -> GlobalAvgPool and
    Voxel2Point.  Every stage is checked by itself on the tensors the GPU path hands it:
    the rulebook bit-exact against the oracle, the convolution against a float64 statement
    of the same sums (one GEMM and one index_add per offset) plus the column-sum property,
    batch norm + gate, the segment mean and the interpolation against the oracle, and the
    grid search for the three nearest voxel centres against the plain scan, bit for bit, on
    the last stage's 16^3 grid."""
    from ss_conv import _ext
    from ss_conv.activation import Activation
    from ss_conv.batchnorm import BatchNorm
    from ss_conv.convolution import Convolution
    from ss_conv.fused import BatchNormActivation
    from ss_conv.pool import GlobalAvgPool
    from ss_conv.sp_ops.voxelize import Point2Voxel, Voxel2Point
    torch.manual_seed(4)
    batch, grid = 32, 64
    pts, feats, ids = synth.make_clouds(batch, 1024, seed=1, channels=3)
    p2v = Point2Voxel([grid] * 3, [2.0 / grid] * 3)
    vp, x, vi, _ = p2v(*[torch.from_numpy(a).to(device) for a in (pts, feats, ids)])
    ref = oracle.point2voxel(pts, feats, ids, [grid] * 3, [2.0 / grid] * 3)
    assert np.array_equal(x.indices.cpu().numpy(), ref["indices"])
    assert np.array_equal(x.features.cpu().numpy(), ref["features"])
    shape = [grid] * 3
    rs_in = [(3, 0)]
    as_np = lambda t: t.detach().cpu().numpy()  # noqa: E731
    for si, (mult, stride) in enumerate(((8, 1), (16, 2), (32, 2), (32, 1))):
        rs = synth.irreps(mult, 3)
        n_gates = sum(m for m, _ in rs[1:])
        rs_gated = rs + [(n_gates, 0)]
        cin = sum(m * (2 * l + 1) for m, l in rs_in)
        cout = sum(m * (2 * l + 1) for m, l in rs_gated)
        conv = Convolution(rs_in, rs_gated, 3, stride=stride, padding=1).to(device).train()
        block = BatchNormActivation(BatchNorm(rs_gated), Activation(rs, (torch.relu, torch.sigmoid)))
        block = block.to(device).train()
        print("stage", si + 1, "rows in", x.features.shape[0], cin, "->", cout, flush=True)
        in_idx, f = x.indices, x.features
        with torch.no_grad():
            for p in block.parameters():
                p.add_(torch.randn_like(p) * 0.3)
            y = conv(x)
            w = conv.kernel().detach().permute(2, 3, 4, 1, 0).reshape(27, cin, cout)
        out_idx, _, pairs, num, _ = y.indice_dict[None]
        want = oracle.canonicalize(*oracle.rulebook(as_np(in_idx), batch, shape, 3, stride, 1))
        for g, r in zip((out_idx, pairs, num), want):
            assert np.array_equal(as_np(g), r), si
        n_out = out_idx.shape[0]
        nums = as_np(num)
        ref64 = torch.zeros((n_out, cout), dtype=torch.float64, device=device)
        col_sums = torch.zeros(cout, dtype=torch.float64, device=device)
        for kk in range(27):
            m = int(nums[kk])
            if m == 0:
                continue
            fi = f[pairs[kk, 0, :m].long()].double()
            ref64.index_add_(0, pairs[kk, 1, :m].long(), fi @ w[kk].double())
            col_sums += fi.sum(0) @ w[kk].double()
        assert _rel(y.features, ref64) < REL_L2, si
        assert _rel(y.features.double().sum(0), col_sums) < REL_L2, si
        del ref64
        y_np = as_np(y.features)
        with torch.no_grad():
            x = block(y)
        params = dict(weight=as_np(block.bn.weight), bias=as_np(block.bn.bias),
                      scalar_bias=as_np(block.act.scalar_act.bias),
                      gate_bias=as_np(block.act.gate_act.bias))
        o_feat = oracle.bn_gate_fwd(y_np, rs_gated, rs, params, training=True)
        err = rel_l2(as_np(x.features), o_feat)
        print("  rows out", n_out, "pairs", int(nums.sum()), "bn+gate rel-l2", err, flush=True)
        assert err < REL_L2, (si, err)
        # the same block in evaluation mode as one kernel (batch norm constants and gate
        # applied while the convolution stores its rows) against the three layers one after
        # the other and against the oracle on the float64 sums
        from ss_conv.fused import ConvBatchNormActivation
        from ss_conv.sp_ops.tensor import SparseTensor
        one = ConvBatchNormActivation(conv, block.bn, block.act).eval()
        with torch.no_grad():
            got = one(SparseTensor(f, in_idx, shape, batch))
            sep = block(conv(SparseTensor(f, in_idx, shape, batch)))
        assert torch.equal(got.indices, sep.indices)
        assert _rel(got.features, sep.features.double()) < 1e-6, si
        running = (as_np(block.bn.running_mean), as_np(block.bn.running_var))
        o_eval = oracle.bn_gate_fwd(y_np, rs_gated, rs, params, training=False, running=running)
        assert rel_l2(as_np(got.features), o_eval) < REL_L2, si
        conv.train()
        block.train()
        shape = [int(v) for v in y.spatial_shape]
        rs_in = rs
    assert shape == [16, 16, 16]
    # heads
    offs = x.get_offsets().int().contiguous()
    pooled = GlobalAvgPool()(x.features.contiguous(), offs)
    want = oracle.segment_avg(as_np(x.features), as_np(offs))
    assert rel_l2(as_np(pooled), want) < REL_L2
    unit = [2.0 / s for s in shape]
    v2p = Voxel2Point(unit_voxel_extent=unit)
    at_points = v2p(x, vp, vi)
    want = oracle.voxel2point(as_np(x.indices), as_np(x.features), shape, as_np(vp), as_np(vi),
                              unit_voxel_extent=unit)[0]
    assert rel_l2(as_np(at_points), want) < REL_L2
    # the grid search against the plain scan on this stage's voxels
    centres, _ = v2p._get_vertice_feats(x)
    queries = torch.cat([vi.float().unsqueeze(1), vp], dim=1).contiguous()
    u, origin = v2p._grid(x)
    d_grid, i_grid = _ext.three_nn_grid(queries, centres, x.indices.contiguous(), batch,
                                        [s + 1 for s in shape], origin, u)
    d_scan = torch.empty_like(d_grid)
    i_scan = torch.empty_like(i_grid)
    _ext.three_nn(queries.shape[0], centres.shape[0], queries, centres, d_scan, i_scan)
    assert torch.equal(i_grid, i_scan) and torch.equal(d_grid, d_scan)
