"""Per-field dropout on sparse tensors (reference: ss_conv/dropout.py:25-46):
one Bernoulli mask per (row, field), shared by the field's 2l+1 components;
identity in eval mode."""
import torch
import torch.nn as nn


class Dropout(nn.Module):
    def __init__(self, Rs, p=0.5):
        super().__init__()
        self.Rs = [(m, l) for m, l in Rs if m > 0]
        self.p = p

    def __repr__(self):
        return "{} (p={})".format(self.__class__.__name__, self.p)

    def forward(self, input):
        if not self.training:
            return input
        x = input.features
        n = x.size(0)
        pieces = []
        begin = 0
        for m, l in self.Rs:
            d = 2 * l + 1
            field = x[:, begin:begin + m * d].reshape(n, m, d)
            begin += m * d
            if self.p == 1:
                keep = x.new_zeros(n, m, 1)
            elif self.p == 0:
                keep = x.new_ones(n, m, 1)
            else:
                keep = torch.bernoulli(x.new_full((n, m, 1), 1 - self.p)) / (1 - self.p)
            pieces.append((field * keep).reshape(n, m * d))
        assert begin == x.size(1)
        input.features = torch.cat(pieces, dim=1)
        return input
