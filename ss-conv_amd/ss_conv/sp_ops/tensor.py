"""Sparse tensor container (reference: ss_conv/sp_ops/tensor.py:22-69)."""
import numpy as np
import torch


def scatter_nd(indices, updates, shape):
    """Dense tensor of `shape` with updates written at integer `indices`
    (reference: tensor.py:6-19).  Repeated indices keep one of the updates."""
    dense = torch.zeros(*shape, dtype=updates.dtype, device=updates.device)
    nd = indices.shape[-1]
    flat = indices.reshape(-1, nd)
    tail = list(shape[nd:])
    dense[tuple(flat[:, a] for a in range(nd))] = updates.reshape([flat.shape[0]] + tail)
    return dense


class SparseTensor(object):
    """features [N, C] float32, indices [N, 4] int32 rows of (batch, x, y, z).

    ``indice_dict`` caches rulebooks under their ``indice_key`` as
    (outids, indices, pairs, pair_num, spatial_shape) (reference: sp_ops/conv.py:136);
    ``grid`` is carried for signature parity only: the rulebook needs no dense
    int32 grid here.  ``plan_dict`` holds, under the same keys, what the native
    convolution keeps with a rulebook (order promises and the plans built over it,
    ss_conv._ext.RulebookMeta); like ``indice_dict`` it is shared with the tensors a
    layer returns.
    """

    def __init__(self, features, indices, spatial_shape, batch_size, grid=None):
        self.features = features
        self.indices = indices
        self.spatial_shape = spatial_shape
        self.batch_size = batch_size
        self.indice_dict = {}
        self.plan_dict = {}
        self.grid = grid

    @property
    def spatial_size(self):
        return np.prod(self.spatial_shape)

    def find_indice_pair(self, key):
        if key is None:
            return None
        return self.indice_dict.get(key, None)

    def dense(self, channels_first=True):
        shape = [self.batch_size] + list(self.spatial_shape) + [self.features.shape[1]]
        res = scatter_nd(self.indices.long(), self.features, shape)
        if not channels_first:
            return res
        nd = len(self.spatial_shape)
        order = [0, nd + 1] + list(range(1, nd + 1))
        return res.permute(*order).contiguous()

    def get_offsets(self):
        """int32 [batch_size + 1] row offsets of the batch elements (rows must be
        grouped by batch index in ascending order).  One device-side bincount
        and a single host transfer instead of one sync per batch element."""
        counts = torch.bincount(self.indices[:, 0].long(), minlength=self.batch_size)
        offsets = torch.zeros(self.batch_size + 1, dtype=torch.int32, device=self.features.device)
        offsets[1:] = torch.cumsum(counts[:self.batch_size], 0).to(torch.int32)
        return offsets.detach()

    @property
    def sparity(self):
        return self.indices.shape[0] / np.prod(self.spatial_shape) / self.batch_size
