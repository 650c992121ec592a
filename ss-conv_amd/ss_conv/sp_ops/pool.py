"""Rulebook pooling modules (reference: ss_conv/sp_ops/pool.py:16-114)."""
import torch.nn as nn

from .tensor import SparseTensor
from .ops import get_conv_output_size, get_indice_pairs
from .functional import indice_avgpool, indice_maxpool


def _per_axis(v, ndim):
    return list(v) if isinstance(v, (list, tuple)) else [v] * ndim


class _SparsePool(nn.Module):
    _op = None

    def __init__(self, ndim, kernel_size, stride=1, padding=0, dilation=1, subm=False):
        super(_SparsePool, self).__init__()
        self.ndim = ndim
        self.kernel_size = _per_axis(kernel_size, ndim)
        self.stride = _per_axis(stride, ndim)
        self.padding = _per_axis(padding, ndim)
        self.dilation = _per_axis(dilation, ndim)
        self.subm = subm

    def forward(self, input):
        """The rulebook is rebuilt on every call (pooling layers carry no indice_key)."""
        assert isinstance(input, SparseTensor)
        features = input.features
        device = features.device
        spatial_shape = input.spatial_shape
        batch_size = input.batch_size
        if self.subm:
            out_spatial_shape = spatial_shape
        else:
            out_spatial_shape = get_conv_output_size(spatial_shape, self.kernel_size, self.stride,
                                                     self.padding, self.dilation)
        outids, indice_pairs, indice_pairs_num = get_indice_pairs(
            input.indices, batch_size, spatial_shape, self.kernel_size, self.stride, self.padding,
            self.dilation, 0, self.subm)
        out_features = type(self)._op(features, indice_pairs.to(device),
                                      indice_pairs_num.to(device), outids.shape[0])
        out_tensor = SparseTensor(out_features, outids, out_spatial_shape, batch_size)
        out_tensor.indice_dict = input.indice_dict
        out_tensor.plan_dict = getattr(input, "plan_dict", {})
        out_tensor.grid = input.grid
        return out_tensor


class SparseAvgPool(_SparsePool):
    """Sum of the active inputs of the window divided by the kernel volume."""
    _op = staticmethod(indice_avgpool)


class SparseMaxPool(_SparsePool):
    """max(0, maximum over the active inputs of the window)."""
    _op = staticmethod(indice_maxpool)
