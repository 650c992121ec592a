"""CPU oracle for the sparse steerable convolution hot path.

TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, __graft_entry__.smoke()
and bench.py's cpu_baseline leg may import this module; the product package
never does.

Every function restates the reference algorithm in NumPy on top of the scalar
C routines of ssc_oracle.c and cites the reference file:line it follows
(paths relative to the reference's SS_Conv_lib/).  When oracle/_ref/libssc_ref.so
is present (the reference's own CPU sources, compiled by oracle/Makefile) the
``ref_*`` functions call it; tests use them to pin the restatement.

Pinning status (what each function is checked against, see tests/test_oracle_*.py):
  rulebook_conv / rulebook_subm   reference CPU build (_ref), committed golden
                                  vectors, brute-force definition, invariants
  conv_fwd                        torch.nn.functional.conv3d closed form; _ref gather/scatter
  maxpool_fwd                     F.max_pool3d(relu(dense)); _ref functor
  avgpool_fwd                     F.avg_pool3d(count_include_pad=True)
  *pool_*_half                    maximum: the float routine on the widened rows (exact);
                                  average: hand-rounded known answers (binary16 codec of
                                  struct), exact cases equal to the float routine
  segment_avg / segment_max       numpy reductions
  point2voxel                     np.unique(axis=0) semantics, per-voxel means, invariants
  three_nn / three_interp         brute force with argsort on tiny inputs
  combine                         torch.einsum on the same buffers (library routine)
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_ORACLE_SO = os.path.join(_HERE, "_build", "libssc_oracle.so")
_REF_SO = os.path.join(_HERE, "_ref", "libssc_ref.so")

_ip = ctypes.POINTER(ctypes.c_int)
_fp = ctypes.POINTER(ctypes.c_float)


def build(force=False):
    """Compile the checker libraries with oracle/Makefile (gcc only)."""
    import subprocess
    args = ["make", "-C", _HERE, "-j3"]
    if force:
        args.insert(1, "-B")
    subprocess.run(args, check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)


def _load(path):
    return ctypes.CDLL(path) if os.path.exists(path) else None


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_ORACLE_SO):
            build()
        _lib = ctypes.CDLL(_ORACLE_SO)
    return _lib


def ref_lib():
    """The compiled reference CPU code, or None when it was never built."""
    global _ref
    if _ref is None and os.path.exists(_REF_SO):
        try:
            import torch  # noqa: F401  (libc10 must be resolvable)
        except Exception:
            pass
        _ref = ctypes.CDLL(_REF_SO)
    return _ref


def _i(a):
    return a.ctypes.data_as(_ip)


def _f(a):
    return a.ctypes.data_as(_fp)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _triple(v):
    if isinstance(v, (list, tuple, np.ndarray)):
        assert len(v) == 3
        return [int(x) for x in v]
    return [int(v)] * 3


# ---------------------------------------------------------------------------
# geometry
# ---------------------------------------------------------------------------
def conv_output_size(in_shape, ksize, stride, padding, dilation):
    """ss_conv/sp_ops/ops.py:13-23."""
    out = []
    for i in range(len(in_shape)):
        size = (in_shape[i] + 2 * padding[i] - dilation[i] * (ksize[i] - 1) - 1) // stride[i] + 1
        out.append(1 if ksize[i] == -1 else size)
    return out


def deconv_output_size(in_shape, ksize, stride, padding, dilation, output_padding):
    """ss_conv/sp_ops/ops.py:26-36 (the dilation does not enter the reference's formula)."""
    return [(in_shape[i] - 1) * stride[i] - 2 * padding[i] + ksize[i] + output_padding[i]
            for i in range(len(in_shape))]


def flat_key(idx, shape):
    """((b*X+x)*Y+y)*Z+z, utils/tensorview.h:457-468 plus the batch term of
    src/conv/indice_cuda_functor.cu:60-61."""
    idx = np.asarray(idx, dtype=np.int64)
    return ((idx[:, 0] * shape[0] + idx[:, 1]) * shape[1] + idx[:, 2]) * shape[2] + idx[:, 3]


# ---------------------------------------------------------------------------
# rulebook
# ---------------------------------------------------------------------------
def _rulebook(fn_conv, fn_subm, indices, batch_size, in_shape, ksize, stride, padding, dilation,
              subm, need_grid, fn_deconv=None, transpose=False, out_padding=0):
    indices = _i32(indices)
    n = indices.shape[0]
    ks, st, pd, dl = _triple(ksize), _triple(stride), _triple(padding), _triple(dilation)
    # the reference refuses a stride and a dilation above 1 on the same axis
    # (ss_conv/sp_ops/conv.py:50-51); its candidate enumeration is only valid without
    if not subm and any(s > 1 and d > 1 for s, d in zip(st, dl)):
        raise ValueError("stride > 1 together with dilation > 1 is not supported")
    if subm:  # src/conv/indice_conv.h:70-74
        st, pd = [1, 1, 1], [k // 2 for k in ks]
        out_shape = list(in_shape)
    elif transpose:  # ss_conv/sp_ops/ops.py:65-68, src/conv/indice_conv.h:86-93
        out_shape = deconv_output_size(list(in_shape), ks, st, pd, dl, _triple(out_padding))
        fn_conv = fn_deconv
    else:
        out_shape = conv_output_size(list(in_shape), ks, st, pd, dl)
    K = ks[0] * ks[1] * ks[2]
    pairs = np.full((K, 2, n), -1, dtype=np.int32)
    num = np.zeros(K, dtype=np.int32)
    a = [_i32(x) for x in (ks, st, pd, dl, out_shape)]
    grid = None
    if need_grid:
        grid = np.full(batch_size * int(np.prod(out_shape)), -1, dtype=np.int32)
    if subm:
        args = [_i(indices), n, batch_size] + [_i(x) for x in a]
        if need_grid:
            args.append(_i(grid))
        n_out = fn_subm(*args, _i(pairs), _i(num))
        out_idx = indices.copy()
    else:
        out_idx = np.zeros((max(n * K, 1), 4), dtype=np.int32)
        args = [_i(indices), n, batch_size] + [_i(x) for x in a] + [_i(out_idx)]
        if need_grid:
            args.append(_i(grid))
        n_out = fn_conv(*args, _i(pairs), _i(num))
        out_idx = out_idx[:n_out].copy()
    assert n_out >= 0
    return out_idx, pairs, num, out_shape


def rulebook(indices, batch_size, in_shape, ksize, stride=1, padding=0, dilation=1, subm=False,
             transpose=False, out_padding=0):
    """CPU rulebook of the reference (first-touch output numbering):
    src/conv/geometry.h:140-189 (regular), 190-237 (transposed), 241-288 (submanifold), driven
    as in src/conv/indice_conv.h:21-131.  Returns (out_indices, pairs[K,2,N], num[K], out_shape)."""
    L = lib()
    return _rulebook(L.orc_rulebook_conv, L.orc_rulebook_subm, indices, batch_size, in_shape,
                     ksize, stride, padding, dilation, subm, need_grid=False,
                     fn_deconv=L.orc_rulebook_deconv, transpose=transpose,
                     out_padding=out_padding)


def ref_rulebook(indices, batch_size, in_shape, ksize, stride=1, padding=0, dilation=1,
                 subm=False, transpose=False, out_padding=0):
    """Same call into the compiled reference sources (oracle/_ref)."""
    R = ref_lib()
    assert R is not None, "oracle/_ref/libssc_ref.so not built"
    return _rulebook(R.ref_rulebook_conv, R.ref_rulebook_subm, indices, batch_size, in_shape,
                     ksize, stride, padding, dilation, subm, need_grid=True,
                     fn_deconv=R.ref_rulebook_deconv, transpose=transpose,
                     out_padding=out_padding)


def canonicalize(out_idx, pairs, num, out_shape):
    """Canonical rulebook order: outputs ascending by flat key (the reference's
    GPU order, src/conv/indice_conv.h:120), pairs of an offset ascending by
    input row (the reference's CPU order, src/conv/geometry.h:166-186)."""
    key = flat_key(out_idx, out_shape)
    order = np.argsort(key, kind="stable")
    rank = np.empty_like(order)
    rank[order] = np.arange(order.size)
    new_pairs = np.full_like(pairs, -1)
    for k in range(pairs.shape[0]):
        n = int(num[k])
        if n == 0:
            continue
        i = pairs[k, 0, :n]
        o = rank[pairs[k, 1, :n]]
        s = np.argsort(i, kind="stable")
        new_pairs[k, 0, :n] = i[s]
        new_pairs[k, 1, :n] = o[s]
    return out_idx[order].copy(), new_pairs, num.copy()


# ---------------------------------------------------------------------------
# conv / pool over a rulebook
# ---------------------------------------------------------------------------
def conv_fwd(features, filters, pairs, num, n_out, inverse=False, matmul=None):
    """src/conv/indice_conv.h:247-343, CPU branch: for every non-empty offset
    gather rows (reordering_cpp_functor.cpp:15-24), GEMM (torch::mm_out, :320)
    and scatter-add (reordering_cpp_functor.cpp:26-44), offsets ascending.
    filters is [K, Cin, Cout].  matmul=None uses the scalar C GEMM; pass
    np.matmul for a BLAS GEMM (what torch::mm is on a CPU)."""
    L = lib()
    features = _f32(features)
    filters = _f32(filters)
    K, cin, cout = filters.shape
    out = np.zeros((n_out, cout), dtype=np.float32)
    for k in range(K):
        n = int(num[k])
        if n <= 0:
            continue
        rows_g = _i32(pairs[k, 1 if inverse else 0, :n])
        rows_s = _i32(pairs[k, 0 if inverse else 1, :n])
        buf = np.empty((n, cin), dtype=np.float32)
        L.orc_gather_rows(_f(buf), _f(features), _i(rows_g), n, cin)
        if matmul is None:
            obuf = np.empty((n, cout), dtype=np.float32)
            L.orc_mm_f32(_f(obuf), _f(buf), _f(filters[k]), n, cin, cout)
        else:
            obuf = _f32(matmul(buf, filters[k]))
        L.orc_scatter_add_rows(_f(out), _f(obuf), _i(rows_s), n, cout)
    return out


def conv_bwd(features, filters, out_grad, pairs, num, inverse=False):
    """src/conv/indice_conv.h:344-426, CPU branch: for every non-empty offset gather the
    input rows and the output-gradient rows (:383-390), filters_grad[k] = in^T * out_grad
    (torch::mm_out, :407), in_buffer = out_grad * W[k]^T (:408), scatter-add into the
    input gradient (:409-413).  filters is [K, Cin, Cout]; products in float64, rounded
    once (the order of a BLAS reduction is not part of the reference's contract).
    Returns (input_grad [N_in, Cin], filters_grad [K, Cin, Cout])."""
    features, filters, out_grad = _f32(features), _f32(filters), _f32(out_grad)
    K, cin, cout = filters.shape
    d_in = np.zeros(features.shape, dtype=np.float64)
    d_w = np.zeros(filters.shape, dtype=np.float64)
    for k in range(K):
        n = int(num[k])
        if n <= 0:
            continue
        rows_i = pairs[k, 1 if inverse else 0, :n]
        rows_o = pairs[k, 0 if inverse else 1, :n]
        fin = features[rows_i].astype(np.float64)
        gout = out_grad[rows_o].astype(np.float64)
        d_w[k] = fin.T @ gout
        np.add.at(d_in, rows_i, gout @ filters[k].astype(np.float64).T)
    return d_in.astype(np.float32), d_w.astype(np.float32)


def ref_gather_scatter_conv(features, filters, pairs, num, n_out):
    """conv_fwd with the reference's own compiled gather / scatter functors and
    a NumPy GEMM in place of torch::mm."""
    R = ref_lib()
    features = _f32(features)
    filters = _f32(filters)
    K, cin, cout = filters.shape
    out = np.zeros((n_out, cout), dtype=np.float32)
    for k in range(K):
        n = int(num[k])
        if n <= 0:
            continue
        buf = np.empty((n, cin), dtype=np.float32)
        R.ref_gather_rows(_f(buf), n, _f(features), features.shape[0], cin,
                          _i(_i32(pairs[k, 0, :n])), n)
        obuf = _f32(buf @ filters[k])
        R.ref_scatter_add_rows(_f(out), n_out, _f(obuf), n, cout, _i(_i32(pairs[k, 1, :n])), n)
    return out


def maxpool_fwd(features, pairs, num, n_out):
    """src/pool/indice_maxpool.h:15-50 with the CPU functor
    src/pool/indice_maxpool_cpp_functor.cpp:16-35 (output zero-initialised)."""
    L = lib()
    features = _f32(features)
    c = features.shape[1]
    out = np.zeros((n_out, c), dtype=np.float32)
    for k in range(pairs.shape[0]):
        n = int(num[k])
        if n > 0:
            L.orc_maxpool_offset(_f(out), _f(features), _i(_i32(pairs[k, 0, :n])),
                                 _i(_i32(pairs[k, 1, :n])), n, c)
    return out


def ref_maxpool_fwd(features, pairs, num, n_out):
    R = ref_lib()
    features = _f32(features)
    pairs = _i32(pairs)
    c = features.shape[1]
    out = np.zeros((n_out, c), dtype=np.float32)
    stride = pairs.shape[2]
    for k in range(pairs.shape[0]):
        n = int(num[k])
        if n > 0:
            R.ref_maxpool_offset(_f(out), n_out, _f(features), features.shape[0], c,
                                 _i(pairs[k]), stride, n)
    return out


def maxpool_bwd(features, out_features, out_grad, pairs, num):
    """src/pool/indice_maxpool_cuda_functor.cu:426-455, offsets ascending: the gradient of an
    output row goes to every input of its window that equals the pooled value."""
    features, out_features, out_grad = _f32(features), _f32(out_features), _f32(out_grad)
    din = np.zeros_like(features)
    for k in range(pairs.shape[0]):
        n = int(num[k])
        if n <= 0:
            continue
        ri, ro = pairs[k, 0, :n], pairs[k, 1, :n]
        hit = features[ri] == out_features[ro]
        din[ri] = (din[ri] + np.where(hit, out_grad[ro], np.float32(0))).astype(np.float32)
    return din


def avgpool_bwd(out_grad, pairs, num, n_in, rf):
    """src/pool/indice_avgpool_cuda_functor.cu (backward kernels), offsets ascending:
    din[i] += dout[o] / (float)rf[o]."""
    out_grad = _f32(out_grad)
    din = np.zeros((n_in, out_grad.shape[1]), dtype=np.float32)
    rf = np.asarray(rf).astype(np.float32)
    for k in range(pairs.shape[0]):
        n = int(num[k])
        if n <= 0:
            continue
        ri, ro = pairs[k, 0, :n], pairs[k, 1, :n]
        din[ri] = (din[ri] + out_grad[ro] / rf[ro][:, None]).astype(np.float32)
    return din


def segment_avg_bwd(out_grad, offsets, n_rows):
    """src/pool/global_avgpool_cuda_kernel.cu:44-55."""
    out_grad = _f32(out_grad)
    din = np.zeros((n_rows, out_grad.shape[1]), dtype=np.float32)
    for s in range(len(offsets) - 1):
        a, b = int(offsets[s]), int(offsets[s + 1])
        if b > a:
            din[a:b] = out_grad[s] / np.float32(b - a)
    return din


def segment_max_bwd(out_grad, arg, n_rows):
    """src/pool/global_maxpool_cuda_kernel.cu:45-53."""
    out_grad = _f32(out_grad)
    din = np.zeros((n_rows, out_grad.shape[1]), dtype=np.float32)
    for s in range(out_grad.shape[0]):
        for c in range(out_grad.shape[1]):
            if arg[s, c] >= 0:
                din[arg[s, c], c] += out_grad[s, c]
    return din


def voxel_reduce_bwd(out_grad, maps, mode, n_point):
    """src/voxelize/voxelize_cuda_kernel.h:44-58."""
    out_grad = _f32(out_grad)
    din = np.zeros((n_point, out_grad.shape[1]), dtype=np.float32)
    for v in range(maps.shape[0]):
        na = int(maps[v, 0])
        mult = np.float32(1.0) / np.float32(na) if (mode == 4 and na > 0) else np.float32(1.0)
        for i in range(1, na + 1):
            din[maps[v, i]] += mult * out_grad[v]
    return din


def three_interp_bwd(out_grad, idx, weight, m):
    """src/voxelize/interpolate_cuda_kernel.cu:104-121 (accumulated in float64: the
    reference's atomic order is not fixed)."""
    out_grad, weight = _f32(out_grad), _f32(weight)
    g = np.zeros((m, out_grad.shape[1]), dtype=np.float64)
    for j in range(3):
        np.add.at(g, idx[:, j], out_grad.astype(np.float64) * weight[:, j:j + 1].astype(np.float64))
    return g.astype(np.float32)


def summary_rf(pairs, num, n_out):
    """src/ss_conv_ops.cu:116-145 + src/pool/indiceSummaryRF.cu:21-36."""
    L = lib()
    rf = np.zeros(n_out, dtype=np.int32)
    for k in range(pairs.shape[0]):
        n = int(num[k])
        if n > 0:
            L.orc_summary_rf_offset(_i(rf), _i(_i32(pairs[k, 1, :n])), n)
    return rf


def avgpool_fwd(features, pairs, num, n_out, rf=None):
    """ss_conv/sp_ops/functional.py:162-185 (rf = kernel volume when use_gs)
    + src/pool/indice_avgpool.h:17-52 with the arithmetic of the CUDA kernel
    src/pool/indice_avgpool_cuda_functor.cu:159-161."""
    L = lib()
    features = _f32(features)
    c = features.shape[1]
    if rf is None:
        rf = np.full(n_out, pairs.shape[0], dtype=np.int32)
    rf = _i32(rf)
    out = np.zeros((n_out, c), dtype=np.float32)
    for k in range(pairs.shape[0]):
        n = int(num[k])
        if n > 0:
            L.orc_avgpool_offset(_f(out), _f(features), _i(_i32(pairs[k, 0, :n])),
                                 _i(_i32(pairs[k, 1, :n])), n, c, _i(rf))
    return out


def _f16(a):
    return np.ascontiguousarray(a, dtype=np.float16)


def maxpool_fwd_half(features, pairs, num, n_out):
    """indiceMaxPool<at::Half> (src/pool/indice_maxpool.h:15-50, kernel statement
    src/pool/indice_maxpool_cuda_functor.cu:39-43: if (in > out) out = in, output starts at 0).
    Comparisons round nothing, so the order of the offsets does not matter."""
    features = _f16(features)
    out = np.zeros((n_out, features.shape[1]), dtype=np.float16)
    for k in range(pairs.shape[0]):
        n = int(num[k])
        if n > 0:
            ri, ro = pairs[k, 0, :n], pairs[k, 1, :n]
            out[ro] = np.maximum(out[ro], features[ri])
    return out


def avgpool_fwd_half(features, pairs, num, n_out, rf=None):
    """indiceAvgPool<at::Half> (src/pool/indice_avgpool.h:17-52), statement
    src/pool/indice_avgpool_cuda_functor.cu:46: out = out + in / (T)rf with T = at::Half,
    whose operators compute in float and round the result to half; offsets ascending (one
    launch per offset).  numpy's float16 operators round the same way."""
    features = _f16(features)
    if rf is None:
        rf = np.full(n_out, pairs.shape[0], dtype=np.int32)
    rf16 = np.asarray(rf).astype(np.float32).astype(np.float16)
    out = np.zeros((n_out, features.shape[1]), dtype=np.float16)
    for k in range(pairs.shape[0]):
        n = int(num[k])
        if n > 0:
            ri, ro = pairs[k, 0, :n], pairs[k, 1, :n]  # output rows are unique inside an offset
            out[ro] = out[ro] + features[ri] / rf16[ro][:, None]
    return out


def maxpool_bwd_half(features, out_features, out_grad, pairs, num):
    """src/pool/indice_maxpool_cuda_functor.cu:426-455 with T = at::Half:
    if (in == out) din = half(din + dout), offsets ascending."""
    features, out_features, out_grad = _f16(features), _f16(out_features), _f16(out_grad)
    din = np.zeros_like(features)
    for k in range(pairs.shape[0]):
        n = int(num[k])
        if n > 0:
            ri, ro = pairs[k, 0, :n], pairs[k, 1, :n]  # input rows are unique inside an offset
            hit = features[ri] == out_features[ro]
            din[ri] = np.where(hit, din[ri] + out_grad[ro], din[ri])
    return din


def avgpool_bwd_half(out_grad, pairs, num, n_in, rf):
    """src/pool/indice_avgpool_cuda_functor.cu:204 with T = at::Half:
    din = half(din + half(dout / half(rf))), offsets ascending."""
    out_grad = _f16(out_grad)
    rf16 = np.asarray(rf).astype(np.float32).astype(np.float16)
    din = np.zeros((n_in, out_grad.shape[1]), dtype=np.float16)
    for k in range(pairs.shape[0]):
        n = int(num[k])
        if n > 0:
            ri, ro = pairs[k, 0, :n], pairs[k, 1, :n]
            din[ri] = din[ri] + out_grad[ro] / rf16[ro][:, None]
    return din


def segment_avg(feats, offsets):
    """src/pool/global_avgpool_cuda_kernel.cu:16-34."""
    feats, offsets = _f32(feats), _i32(offsets)
    out = np.zeros((offsets.size - 1, feats.shape[1]), dtype=np.float32)
    with np.errstate(all="ignore"):
        lib().orc_segment_avg(_f(feats), _i(offsets), _f(out), offsets.size - 1, feats.shape[1])
    return out


def segment_max(feats, offsets):
    """src/pool/global_maxpool_cuda_kernel.cu:16-35.  Returns (max, argmax)."""
    feats, offsets = _f32(feats), _i32(offsets)
    out = np.zeros((offsets.size - 1, feats.shape[1]), dtype=np.float32)
    idx = np.zeros(out.shape, dtype=np.int32)
    lib().orc_segment_max(_f(feats), _i(offsets), _f(out), _i(idx), offsets.size - 1,
                          feats.shape[1])
    return out, idx


# ---------------------------------------------------------------------------
# point <-> voxel
# ---------------------------------------------------------------------------
def voxel_map(inverse, n_voxel, max_active, mode=4):
    """ss_conv/sp_ops/functional.py:329-355 + src/voxelize/voxel2point_cuda_kernel.cu:16-37."""
    inverse = _i32(inverse).reshape(-1)
    n = inverse.size
    ids = np.arange(n, dtype=np.int32)
    if mode in (3, 4):
        maps = np.zeros((n_voxel, max_active + 1), dtype=np.int32)
    elif mode == 2:
        maps = np.full((n_voxel, max_active + 1), -1, dtype=np.int32)
    elif mode == 1:
        maps = np.full((n_voxel, max_active + 1), n, dtype=np.int32)
    else:
        raise AssertionError
    lib().orc_voxel_map(_i(inverse), _i(ids), _i(maps), n, max_active, mode)
    return maps


def voxel_reduce(feats, maps, mode=4):
    """ss_conv/sp_ops/functional.py:297-316 + src/voxelize/voxelize_cuda_kernel.h:18-32."""
    feats, maps = _f32(feats), _i32(maps)
    out = np.zeros((maps.shape[0], feats.shape[1]), dtype=np.float32)
    lib().orc_voxel_reduce(_f(feats), _f(out), _i(maps), mode, maps.shape[0], maps.shape[1] - 1,
                           feats.shape[1])
    return out


def point2voxel(points, feats, batch_ids, voxel_num_limit, unit_voxel_extent, mode=4):
    """ss_conv/sp_ops/voxelize.py:29-99.  Returns a dict with valid_points,
    valid_feats, valid_ids, flag, indices[M,4], inverse, counts, maps, features[M,C].
    The batch sort is stable (the reference's torch.sort leaves ties unspecified)."""
    points = _f32(points)
    feats = _f32(feats)
    ids = np.asarray(batch_ids, dtype=np.int64)
    C = feats.shape[1]
    unit = np.asarray(unit_voxel_extent, dtype=np.float64).astype(np.float32).reshape(1, 3)
    limit = np.asarray(voxel_num_limit).astype(np.float32).reshape(1, 3)
    total = limit * unit
    half = np.float32(0.5) * total
    uniq_ids = np.unique(ids)
    B1 = uniq_ids.size
    ok = (np.abs(points) > half).sum(1) == 0
    if ok.sum() == 0:
        flag = np.zeros(B1, dtype=np.float32)
        vp = np.zeros((B1, 3), dtype=np.float32)
        vf = np.zeros((B1, C), dtype=np.float32)
        vi = uniq_ids
    else:
        vp, vf, vi = points[ok], feats[ok], ids[ok]
        uv = np.unique(vi)
        if uv.size == B1:
            flag = np.ones(B1, dtype=np.float32)
        else:
            flag = np.isin(uniq_ids, uv).astype(np.float32)
            missing = uniq_ids[flag == 0]
            vp = np.concatenate([vp, np.zeros((missing.size, 3), np.float32)])
            vf = np.concatenate([vf, np.zeros((missing.size, C), np.float32)])
            vi = np.concatenate([vi, missing])
        order = np.argsort(vi, kind="stable")
        vp, vf, vi = vp[order], vf[order], vi[order]
    vox = ((vp + half) / unit).astype(np.int32)  # fp32 add, fp32 divide, truncate
    table = np.concatenate([vi.astype(np.int32)[:, None], vox], axis=1)
    uniq, inverse, counts = np.unique(table, axis=0, return_inverse=True, return_counts=True)
    inverse = inverse.reshape(-1)
    max_active = 1 if mode in (1, 2) else int(counts.max())
    maps = voxel_map(inverse, uniq.shape[0], max_active, mode)
    out = voxel_reduce(vf, maps, mode)
    return dict(valid_points=vp, valid_feats=vf, valid_ids=vi, flag=flag,
                indices=uniq.astype(np.int32), inverse=inverse.astype(np.int32),
                counts=counts.astype(np.int32), maps=maps, features=out, batch_size=B1)


def three_nn(unknown, known):
    """ss_conv/sp_ops/functional.py:361-384 + src/voxelize/interpolate_cuda_kernel.cu:8-55.
    Returns (sqrt(dist2), idx)."""
    unknown, known = _f32(unknown), _f32(known)
    n, m = unknown.shape[0], known.shape[0]
    d2 = np.zeros((n, 3), dtype=np.float32)
    idx = np.zeros((n, 3), dtype=np.int32)
    lib().orc_three_nn(n, m, _f(unknown), _f(known), _f(d2), _i(idx))
    with np.errstate(all="ignore"):
        return np.sqrt(d2), idx


def three_interp(feats, idx, weight):
    """src/voxelize/interpolate_cuda_kernel.cu:79-101."""
    feats, idx, weight = _f32(feats), _i32(idx), _f32(weight)
    out = np.zeros((idx.shape[0], feats.shape[1]), dtype=np.float32)
    lib().orc_three_interp(feats.shape[1], feats.shape[0], idx.shape[0], _f(feats), _i(idx),
                           _f(weight), _f(out))
    return out


def voxel2point(indices, features, spatial_shape, points, batch_ids, voxel_extent=None,
                unit_voxel_extent=None):
    """ss_conv/sp_ops/voxelize.py:110-162: voxel centres, 3-NN, inverse-distance
    weights, interpolation."""
    shape = np.asarray(spatial_shape, dtype=np.float64)
    if voxel_extent is not None:
        unit = (np.asarray(voxel_extent, np.float64) / shape).astype(np.float32)
        ext = np.asarray(voxel_extent, np.float64).astype(np.float32)
    else:
        unit = np.asarray(unit_voxel_extent, np.float64).astype(np.float32)
        ext = (np.asarray(unit_voxel_extent, np.float64) * shape).astype(np.float32)
    centres = np.asarray(indices).astype(np.float32)
    centres[:, 1:] = centres[:, 1:] * unit - np.float32(0.5) * ext + np.float32(0.5) * unit
    target = np.concatenate([np.asarray(batch_ids).astype(np.float32)[:, None], _f32(points)], 1)
    dist, idx = three_nn(target, centres)
    recip = np.float32(1.0) / (dist + np.float32(1e-8))
    weight = recip / recip.sum(1, keepdims=True)
    return three_interp(features, idx, weight), idx, weight


# ---------------------------------------------------------------------------
# steerable kernel synthesis
# ---------------------------------------------------------------------------
def combine(weight, bases, mults_out, dims_out, mults_in, dims_in, size):
    """ss_conv/utils/kernel.py:267-299.  bases[i][j] is the [n_beta,d_o,d_i,k,k,k]
    buffer kernel_i_j or None.  Returns the dense kernel [Cout,Cin,k,k,k]."""
    weight = np.asarray(weight, dtype=np.float32)
    off = 0
    rows = []
    for i, mi in enumerate(mults_out):
        cols = []
        for j, mj in enumerate(mults_in):
            kij = bases[i][j]
            if kij is not None:
                nb = kij.shape[0]
                w = weight[off:off + mi * mj * nb].reshape(mi, mj, nb)
                off += mi * mj * nb
                ker = np.einsum("uvb,bijxyz->uivjxyz", w, np.asarray(kij, np.float32))
                ker = ker.reshape(mi * dims_out[i], mj * dims_in[j], size, size, size)
            else:
                ker = np.zeros((mi * dims_out[i], mj * dims_in[j], size, size, size), np.float32)
            cols.append(ker)
        rows.append(np.concatenate(cols, axis=1))
    assert off == weight.size
    return np.concatenate(rows, axis=0).astype(np.float32)


# ---- SE(3) batch norm and gated non-linearity ---------------------------------------------
_ACTS = {
    None: (lambda u: u, lambda u: np.ones_like(u)),
    "relu": (lambda u: np.maximum(u, 0.0), lambda u: (u > 0).astype(u.dtype)),
    "sigmoid": (lambda u: 1.0 / (1.0 + np.exp(-u)),
                lambda u: (1.0 / (1.0 + np.exp(-u))) * (1.0 - 1.0 / (1.0 + np.exp(-u)))),
    "tanh": (lambda u: np.tanh(u), lambda u: 1.0 - np.tanh(u) ** 2),
}


def batchnorm_fwd(x, Rs, weight=None, bias=None, running_mean=None, running_var=None, eps=1e-5,
                  momentum=0.1, training=True, dtype=np.float64):
    """The reference's field loop (ss_conv/batchnorm.py:49-136), field by field:
    scalars are centred by their (batch or running) mean, every field is divided by the root
    of its (batch or running) mean squared norm plus eps, then weight per field and bias per
    scalar.  Returns (y, running_mean', running_var'), the running statistics moved by
    `momentum` when training (batchnorm.py:45-46)."""
    x = np.asarray(x, dtype=dtype)
    n = x.shape[0]
    n_scalar = sum(m for m, l in Rs if l == 0)
    n_field = sum(m for m, l in Rs)
    rm = np.zeros(n_scalar, dtype) if running_mean is None else np.asarray(running_mean, dtype).copy()
    rv = np.ones(n_field, dtype) if running_var is None else np.asarray(running_var, dtype).copy()
    new_rm, new_rv = rm.copy(), rv.copy()
    out = []
    ix = irm = irv = iw = ib = 0
    for m, l in Rs:
        d = 2 * l + 1
        field = x[:, ix:ix + m * d].reshape(n, m, d)
        ix += m * d
        if d == 1:
            if training:
                mean = field.mean(0).reshape(-1)
                new_rm[irm:irm + m] = (1 - momentum) * rm[irm:irm + m] + momentum * mean
            else:
                mean = rm[irm:irm + m]
            irm += m
            field = field - mean.reshape(1, m, 1)
        if training:
            norm = (field ** 2).sum(2).mean(0)
            new_rv[irv:irv + m] = (1 - momentum) * rv[irv:irv + m] + momentum * norm
        else:
            norm = rv[irv:irv + m]
        irv += m
        scale = (norm + eps) ** -0.5
        if weight is not None:
            scale = scale * np.asarray(weight, dtype)[iw:iw + m]
            iw += m
        field = field * scale.reshape(1, m, 1)
        if bias is not None and d == 1:
            field = field + np.asarray(bias, dtype)[ib:ib + m].reshape(1, m, 1)
            ib += m
        out.append(field.reshape(n, m * d))
    assert ix == x.shape[1]
    return np.concatenate(out, axis=1), new_rm, new_rv


def gate_fwd(y, Rs, scalar_bias=None, gate_bias=None, act_scalar=None, act_gate=None,
             dtype=np.float64):
    """Activation._gate (ss_conv/activation.py:55-100): the first entry of Rs, if scalar, goes
    through act_scalar(y + scalar_bias); every non-scalar field is multiplied by
    act_gate(g + gate_bias) of its gate scalar, the gates being the columns after the
    fields.  An activation given as None leaves its columns unchanged (and, for the gates,
    drops the gate columns unused)."""
    y = np.asarray(y, dtype=dtype)
    n = y.shape[0]
    out_dim = sum(m * (2 * l + 1) for m, l in Rs)
    gates = None
    if act_gate is not None:
        g = y[:, out_dim:]
        if gate_bias is not None:
            g = g + np.asarray(gate_bias, dtype).reshape(1, -1)
        gates = _ACTS[act_gate][0](g)
    z = np.empty((n, out_dim), dtype)
    begin_y = begin_g = 0
    for i, (m, l) in enumerate(Rs):
        if m == 0:
            continue
        d = 2 * l + 1
        field = y[:, begin_y:begin_y + m * d]
        if l == 0:
            if act_scalar is not None and i == 0:
                if scalar_bias is not None:
                    field = field + np.asarray(scalar_bias, dtype).reshape(1, -1)
                field = _ACTS[act_scalar][0](field)
        elif gates is not None:
            fg = gates[:, begin_g:begin_g + m].reshape(n, m, 1)
            field = (field.reshape(n, m, d) * fg).reshape(n, m * d)
            begin_g += m
        z[:, begin_y:begin_y + m * d] = field
        begin_y += m * d
    return z


def bn_gate_fwd(x, Rs_bn, Rs_act, params, eps=1e-5, training=True, act_scalar="relu",
                act_gate="sigmoid", running=None):
    """gate_fwd(batchnorm_fwd(x)) with params = dict(weight, bias, scalar_bias, gate_bias);
    Rs_act None: batch norm alone; Rs_bn None: the gate alone."""
    y = np.asarray(x, dtype=np.float64)
    if Rs_bn is not None:
        rm, rv = running if running is not None else (None, None)
        y, _, _ = batchnorm_fwd(y, Rs_bn, params.get("weight"), params.get("bias"), rm, rv, eps,
                                0.1, training)
    if Rs_act is not None:
        y = gate_fwd(y, Rs_act, params.get("scalar_bias"), params.get("gate_bias"), act_scalar,
                     act_gate)
    return y


def bn_gate_bwd(x, dy, Rs_bn, Rs_act, params, eps=1e-5, training=True, act_scalar="relu",
                act_gate="sigmoid", running=None):
    """Gradients of sum(dy * bn_gate_fwd(x)) with respect to x and to every entry of params,
    by the chain rule through the two layers (what torch autograd computes for the
    reference's modules; pinned against central differences of bn_gate_fwd).
    Returns dict(x=..., weight=..., bias=..., scalar_bias=..., gate_bias=...)."""
    x = np.asarray(x, dtype=np.float64)
    dy = np.asarray(dy, dtype=np.float64)
    n, c_in = x.shape
    grads = {}
    # ---- forward pieces
    if Rs_bn is not None:
        cols = []
        for m, l in Rs_bn:
            for _ in range(m):
                cols.append(2 * l + 1)
        field_of = np.repeat(np.arange(len(cols)), cols)
        is_scalar = np.repeat(np.array(cols) == 1, cols)
        rm, rv = running if running is not None else (np.zeros(is_scalar.sum()), np.ones(len(cols)))
        shift = np.zeros(c_in)
        shift[is_scalar] = x[:, is_scalar].mean(0) if training else np.asarray(rm, np.float64)
        xc = x - shift
        if training:
            norm = np.zeros(len(cols))
            np.add.at(norm, field_of, (xc ** 2).mean(0))
        else:
            norm = np.asarray(rv, np.float64)
        rstd = (norm + eps) ** -0.5
        w = np.ones(len(cols)) if params.get("weight") is None else np.asarray(params["weight"], np.float64)
        scale = (rstd * w)[field_of]
        add = np.zeros(c_in)
        if params.get("bias") is not None:
            add[is_scalar] = np.asarray(params["bias"], np.float64)
        z = xc * scale + add
    else:
        z = x
    # ---- through the gate: dz
    if Rs_act is not None:
        out_dim = sum(m * (2 * l + 1) for m, l in Rs_act)
        dz = np.zeros_like(z)
        sb, gb = params.get("scalar_bias"), params.get("gate_bias")
        col = g = 0
        for i, (m, l) in enumerate(Rs_act):
            d = 2 * l + 1
            for _ in range(m):
                sl = slice(col, col + d)
                if l == 0:
                    if act_scalar is not None and i == 0:
                        u = z[:, sl] + (0.0 if sb is None else np.asarray(sb, np.float64)[col:col + d])
                        dz[:, sl] = dy[:, sl] * _ACTS[act_scalar][1](u)
                    else:
                        dz[:, sl] = dy[:, sl]
                elif act_gate is not None:
                    gc = out_dim + g
                    u = z[:, gc] + (0.0 if gb is None else np.asarray(gb, np.float64)[g])
                    dz[:, sl] = dy[:, sl] * _ACTS[act_gate][0](u)[:, None]
                    dz[:, gc] = (dy[:, sl] * z[:, sl]).sum(1) * _ACTS[act_gate][1](u)
                    g += 1
                else:
                    dz[:, sl] = dy[:, sl]
                col += d
        m0 = Rs_act[0][0] if (Rs_act[0][1] == 0 and act_scalar is not None) else 0
        if sb is not None:
            grads["scalar_bias"] = dz[:, :m0].sum(0)
        if gb is not None:
            grads["gate_bias"] = dz[:, out_dim:out_dim + g].sum(0)
    else:
        dz = dy
    # ---- through the batch norm
    if Rs_bn is not None:
        col_b = dz.sum(0)
        field_a = np.zeros(len(cols))
        np.add.at(field_a, field_of, (dz * xc).sum(0))
        if params.get("bias") is not None:
            grads["bias"] = col_b[is_scalar]
        if params.get("weight") is not None:
            grads["weight"] = rstd * field_a
        dx = dz * scale
        if training:
            dx = dx - np.where(is_scalar, col_b / n, 0.0) * scale
            dx = dx - (scale * (rstd ** 2 * field_a)[field_of] / n) * xc
        grads["x"] = dx
    else:
        grads["x"] = dz
    return grads
