"""SE(3)-equivariant batch normalisation on sparse tensors
(reference: ss_conv/batchnorm.py:13-136).

Scalar fields are centred by their mean; every field (a block of 2l+1 channels)
is divided by the root of its mean squared norm.  Buffers and parameters keep
the reference's names and shapes: running_mean [scalars], running_var [fields],
weight [fields], bias [scalars].  The per-field loop of the reference is
replaced by index tables.  Float32 features on the GPU run on the library's kernels
(two reads of the rows for the statistics, one read and one write to normalise, and a
hand-written backward pass); anything else takes the torch ops below.
"""
import torch
import torch.nn as nn

from ss_conv import bnact


class BatchNorm(nn.Module):
    def __init__(self, Rs, eps=1e-5, momentum=0.1, affine=True, reduce='mean'):
        super().__init__()
        self.Rs = Rs
        self.eps = eps
        self.momentum = momentum
        self.affine = affine
        self.reduce = reduce

        num_scalar = sum(m for m, l in Rs if l == 0)
        num_features = sum(m for m, l in Rs)
        self.register_buffer('running_mean', torch.zeros(num_scalar))
        self.register_buffer('running_var', torch.ones(num_features))
        if affine:
            self.weight = nn.Parameter(torch.ones(num_features))
            self.bias = nn.Parameter(torch.zeros(num_scalar))
        else:
            self.register_parameter('weight', None)
            self.register_parameter('bias', None)

        field_of, scalar_cols = [], []
        f = c = 0
        for m, l in Rs:
            d = 2 * l + 1
            for u in range(m):
                field_of += [f] * d
                if d == 1:
                    scalar_cols.append(c)
                f += 1
                c += d
        self.num_channels = c
        self.register_buffer('_field_of', torch.tensor(field_of, dtype=torch.long),
                             persistent=False)
        self.register_buffer('_scalar_cols', torch.tensor(scalar_cols, dtype=torch.long),
                             persistent=False)
        self._layout_cpu = bnact.field_layout(Rs)
        self._layout_dev = {}

    def layout(self, device):
        """Channel tables of the kernels on `device`."""
        key = str(device)
        if key not in self._layout_dev:
            self._layout_dev[key] = bnact.to_device(self._layout_cpu, device)
        return self._layout_dev[key]

    def plan(self, device):
        """The batch-norm half of a bnact.BnActPlan."""
        p = bnact.BnActPlan()
        p.bn = self.layout(device)
        p.training = self.training
        p.eps = self.eps
        p.momentum = self.momentum
        p.running_mean = self.running_mean
        p.running_var = self.running_var
        p.c_out = self.num_channels
        return p

    def __repr__(self):
        return "{} (Rs={}, eps={}, momentum={})".format(self.__class__.__name__, self.Rs, self.eps,
                                                        self.momentum)

    def _roll_avg(self, curr, update):
        return (1 - self.momentum) * curr + self.momentum * update.detach()

    def forward(self, input):  # pylint: disable=W
        x = input.features
        if x.size(1) != self.num_channels:
            raise AssertionError("features have {} channels, Rs describes {}".format(
                x.size(1), self.num_channels))
        if self.reduce != 'mean':
            raise ValueError("Invalid reduce option {}".format(self.reduce))
        if bnact.usable(x) and x.size(0) > 0:
            input.features = bnact.bn_act(x, self.weight, self.bias, None, None,
                                          self.plan(x.device))
            return input
        n_fields = self.running_var.numel()
        shift = x.new_zeros(self.num_channels)
        if self._scalar_cols.numel() > 0:
            if self.training:
                mean = x[:, self._scalar_cols].mean(0)
                self.running_mean.copy_(self._roll_avg(self.running_mean, mean))
            else:
                mean = self.running_mean
            shift = shift.index_copy(0, self._scalar_cols, mean)
        x = x - shift
        if self.training:
            norm = x.new_zeros(n_fields).index_add(0, self._field_of, (x * x).mean(0))
            self.running_var.copy_(self._roll_avg(self.running_var, norm))
        else:
            norm = self.running_var
        scale = (norm + self.eps).pow(-0.5)
        if self.affine:
            scale = scale * self.weight
        x = x * scale[self._field_of]
        if self.affine and self._scalar_cols.numel() > 0:
            x = x + x.new_zeros(self.num_channels).index_copy(0, self._scalar_cols, self.bias)
        input.features = x
        return input
