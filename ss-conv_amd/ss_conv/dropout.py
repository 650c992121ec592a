"""Per-field dropout on sparse tensors (reference: ss_conv/dropout.py:25-46):
one Bernoulli mask per (row, field), shared by the field's 2l+1 components;
identity in eval mode.

The masks are drawn with the reference's own sequence of calls (one
``new_empty(n, m).bernoulli_(1 - p).div_(1 - p)`` per entry of Rs), so a given seed gives
the reference's masks.  Float32 features on the GPU are then multiplied by one kernel of
the library (``ssc_field_scale_f32``); anything else takes the expand / multiply below."""
import torch
import torch.nn as nn

from ss_conv import _ext


class _FieldScale(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, scale, field_of):
        ctx.save_for_backward(scale, field_of)
        return _ext.field_scale(x, scale, field_of)

    @staticmethod
    def backward(ctx, dy):
        scale, field_of = ctx.saved_tensors
        return _ext.field_scale(dy.contiguous(), scale, field_of), None, None


class Dropout(nn.Module):
    def __init__(self, Rs, p=0.5):
        super().__init__()
        self.Rs = [(m, l) for m, l in Rs if m > 0]
        self.p = p
        field_of, f = [], 0
        for m, l in self.Rs:
            for _ in range(m):
                field_of += [f] * (2 * l + 1)
                f += 1
        self.register_buffer('_field_of', torch.tensor(field_of, dtype=torch.int32),
                             persistent=False)

    def __repr__(self):
        return "{} (p={})".format(self.__class__.__name__, self.p)

    def _noise(self, x):
        """[n, fields]: 0 or 1 / (1 - p) per row and field."""
        n = x.size(0)
        noises = []
        for m, l in self.Rs:
            noise = x.new_empty(n, m)
            if self.p == 1:
                noise.fill_(0)
            elif self.p == 0:
                noise.fill_(1)
            else:
                noise.bernoulli_(1 - self.p).div_(1 - self.p)
            noises.append(noise)
        return noises[0] if len(noises) == 1 else torch.cat(noises, dim=1)

    def forward(self, input):
        if not self.training:
            return input
        x = input.features
        assert x.size(1) == self._field_of.numel()
        noise = self._noise(x)
        if x.is_cuda and x.dtype == torch.float32 and x.size(0) > 0:
            input.features = _FieldScale.apply(x, noise, self._field_of.to(x.device))
        else:
            input.features = x * noise[:, self._field_of.long()]
        return input
