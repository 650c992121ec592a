"""BatchNorm followed by the gated Activation as one pass over the feature rows.

The reference applies the two layers one after the other (each a chain of torch ops over
[N, C], e.g. Common_utils/ss_conv_backbones.py:30-46).  This wrapper owns the two reference
layers unchanged, so parameters, buffers and state-dict keys (`bn.*`, `act.*`) are theirs, and
computes both in `ssc_bnact_fwd_f32`: the normalised rows are never written to memory.
"""
import torch.nn as nn

from ss_conv import bnact
from ss_conv.activation import Activation
from ss_conv.batchnorm import BatchNorm


class BatchNormActivation(nn.Module):
    def __init__(self, bn, act):
        """bn: BatchNorm over the fields and gate scalars; act: Activation of the fields."""
        super().__init__()
        if not isinstance(bn, BatchNorm) or not isinstance(act, Activation):
            raise TypeError("BatchNormActivation(bn: BatchNorm, act: Activation)")
        self.bn = bn
        self.act = act

    def forward(self, input):  # pylint: disable=W
        x = input.features
        act = self.act
        fusable = (act._kernel_ok and (act.scalar_act is not None or act.gate_act is not None)
                   and bnact.usable(x) and x.size(0) > 0 and self.bn.reduce == 'mean'
                   and x.size(1) == self.bn.num_channels
                   and x.size(1) == act._c_out + act._n_gates)
        if not fusable:
            return self.act(self.bn(input))
        plan = act.fill_plan(self.bn.plan(x.device), x.device)
        sb, gb = act.biases()
        input.features = bnact.bn_act(x, self.bn.weight, self.bn.bias, sb, gb, plan)
        return input
