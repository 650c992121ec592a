"""ssc_pool_max_static_f32, the entry point that allocates nothing: its pair table lives in
an array inside the library.  Called through the C ABI and compared, bit for bit, with
ssc_pool_max_f32 (caller-provided workspace) on two calls in a row, the second one on a
smaller input, so that entries the first call left in the shared table would show."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

STATIC_ENTRIES = 4 << 20  # SSC_POOL_STATIC_ENTRIES


def _pool_case(device, batch, grid, n, channels, seed):
    from ss_conv.sp_ops.ops import get_indice_pairs
    rng = np.random.default_rng(seed)
    cells = rng.choice(batch * grid ** 3, size=n, replace=False)
    cells.sort()
    idx = np.stack([cells // grid ** 3, cells // grid ** 2 % grid, cells // grid % grid,
                    cells % grid], axis=1).astype(np.int32)
    t = torch.from_numpy(idx).to(device)
    o_idx, pairs, num = get_indice_pairs(t, batch, [grid] * 3, 2, 2, 0)
    feats = torch.from_numpy(rng.normal(size=(n, channels)).astype(np.float32)).to(device)
    return feats, pairs, num, o_idx.shape[0]


def _both_ways(lib, feats, pairs, num, n_out):
    K, c = pairs.shape[0], feats.shape[1]
    dev = feats.device
    want = torch.full((n_out, c), -7.0, device=dev)
    ws = torch.empty(lib.ssc_pool_workspace_bytes(n_out, K), dtype=torch.uint8, device=dev)
    assert lib.ssc_pool_max_f32(feats.data_ptr(), c, pairs.data_ptr(), pairs.shape[2],
                                num.data_ptr(), K, want.data_ptr(), n_out, ws.data_ptr(),
                                ws.numel(), None) == 0
    got = torch.full((n_out, c), -9.0, device=dev)
    assert lib.ssc_pool_max_static_f32(feats.data_ptr(), c, pairs.data_ptr(), pairs.shape[2],
                                       num.data_ptr(), K, got.data_ptr(), n_out, None) == 0
    torch.cuda.synchronize()
    return got, want


def test_static_pool_equals_workspace_pool_twice(device):
    from ss_conv import _ext
    lib = _ext._lib
    print("static pool: first call, 3 x 24^3 grid, 9000 voxels, 48 channels", flush=True)
    big = _pool_case(device, 3, 24, 9000, 48, seed=1)
    got, want = _both_ways(lib, *big)
    assert got.shape[0] > 2000 and torch.equal(got, want)
    print("static pool: second call, 1 x 10^3 grid, 300 voxels, 5 channels", flush=True)
    small = _pool_case(device, 1, 10, 300, 5, seed=2)
    got, want = _both_ways(lib, *small)
    assert 0 < got.shape[0] < 300 and torch.equal(got, want)
    # and the first input once more, after the small one
    got, want = _both_ways(lib, *big)
    assert torch.equal(got, want)


def test_static_pool_rejects_what_does_not_fit(device):
    from ss_conv import _ext
    lib = _ext._lib
    feats, pairs, num, n_out = _pool_case(device, 1, 10, 300, 4, seed=3)
    too_many = STATIC_ENTRIES // pairs.shape[0] + 1
    rc = lib.ssc_pool_max_static_f32(feats.data_ptr(), 4, pairs.data_ptr(), pairs.shape[2],
                                     num.data_ptr(), pairs.shape[0], feats.data_ptr(), too_many,
                                     None)
    assert rc == _ext.SSC_EINVAL
    assert b"exceeds" in lib.ssc_last_error()
    # nothing to do: still sets the table's address up and succeeds
    assert lib.ssc_pool_max_static_f32(None, 4, None, 0, None, 8, None, 0, None) == 0
