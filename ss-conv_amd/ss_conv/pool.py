"""User-facing pooling layers (reference: ss_conv/pool.py:15-92)."""
import torch.nn as nn

from ss_conv.sp_ops.tensor import SparseTensor
from ss_conv.sp_ops.pool import SparseAvgPool, SparseMaxPool
from ss_conv.sp_ops.functional import global_avgpool, global_maxpool


class AvgPool(SparseAvgPool):
    def __init__(self, kernel_size, stride=1, padding=0, dilation=1, subm=False):
        super(AvgPool, self).__init__(ndim=3, kernel_size=kernel_size, stride=stride,
                                      padding=padding, dilation=dilation, subm=subm)


class MaxPool(SparseMaxPool):
    def __init__(self, kernel_size, stride=1, padding=0, dilation=1, subm=False):
        super(MaxPool, self).__init__(ndim=3, kernel_size=kernel_size, stride=stride,
                                      padding=padding, dilation=dilation, subm=subm)


class _GlobalPool(nn.Module):
    """forward(inputs, offsets=None): inputs is a dense [sum_n, C] feature tensor
    with `offsets` [B+1] int32, the calling convention the reference's users rely
    on (LineMOD/model.py:213-215); a SparseTensor is accepted as well and then
    supplies its own offsets."""
    func = None

    def forward(self, inputs, offsets=None):
        if isinstance(inputs, SparseTensor):
            feats = inputs.features
            offsets = inputs.get_offsets() if offsets is None else offsets
        else:
            assert offsets is not None
            feats = inputs
        return type(self).func(feats.contiguous(), offsets.detach().int().contiguous())


class GlobalAvgPool(_GlobalPool):
    func = staticmethod(global_avgpool)


class GlobalMaxPool(_GlobalPool):
    func = staticmethod(global_maxpool)
