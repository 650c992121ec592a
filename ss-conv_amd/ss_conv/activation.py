"""Gated non-linearity on sparse tensors (reference: ss_conv/activation.py:16-160).

Input rows hold Rs2dim(Rs) field channels followed by one gate scalar per
non-scalar field.  Scalars pass through act(x + b); every non-scalar field is
multiplied by gate_act(g + b) of its gate.  Parameters keep the reference's
names (scalar_act.bias, gate_act.bias)."""
import torch
import torch.nn as nn
import torch.utils.checkpoint

from ss_conv import bnact
from ss_conv.utils.utils import Rs2dim


class ScalarActivation(nn.Module):
    """enable: list of (width, activation or None); a bias is added before each
    activation (reference: activation.py:103-160)."""

    def __init__(self, enable, bias=True, inplace=False):
        super().__init__()
        self.inplace = inplace
        self.enable = []
        for d, act in enable:
            if d == 0:
                continue
            if self.enable and self.enable[-1][1] is act:
                self.enable[-1] = (self.enable[-1][0] + d, act)
            else:
                self.enable.append((d, act))
        nbias = sum(d for d, act in self.enable if act is not None)
        self.bias = torch.nn.Parameter(torch.zeros(nbias)) if bias and nbias > 0 else None

    def forward(self, input):  # pylint: disable=W
        pieces = []
        col = used = 0
        for d, act in self.enable:
            x = input[:, col:col + d]
            if act is not None:
                if self.bias is not None:
                    x = x + self.bias[used:used + d].view(1, d)
                    used += d
                x = act(x)
            pieces.append(x)
            col += d
        assert col == input.size(1)
        assert self.bias is None or used == self.bias.size(0)
        out = pieces[0] if len(pieces) == 1 else torch.cat(pieces, dim=1)
        if self.inplace:
            input.copy_(out)
            return input
        return out


class Activation(nn.Module):
    def __init__(self, Rs, activation=(None, None), bias=True, checkpoint=True):
        super().__init__()
        self.Rs = Rs
        self.multiplicities = [m for m, _ in self.Rs]
        self.orders = [l for _, l in self.Rs]
        self.checkpoint = checkpoint
        if type(activation) is tuple:
            scalar_activation, gate_activation = activation
        else:
            scalar_activation, gate_activation = activation, activation

        if scalar_activation is not None and self.multiplicities[0] > 0 and self.orders[0] == 0:
            self.scalar_act = ScalarActivation([(self.multiplicities[0], scalar_activation)],
                                               bias=bias)
        else:
            self.scalar_act = None
        n_non_scalar = sum(self.multiplicities[1:])
        if gate_activation is not None and n_non_scalar > 0:
            self.gate_act = ScalarActivation([(n_non_scalar, gate_activation)], bias=bias)
        else:
            self.gate_act = None

        # gate index of every non-scalar channel, in field order
        gate_of, g = [], 0
        for m, l in self.Rs:
            if m == 0 or l == 0:
                continue
            for u in range(m):
                gate_of += [g] * (2 * l + 1)
                g += 1
        self.register_buffer('_gate_of', torch.tensor(gate_of, dtype=torch.long),
                             persistent=False)

        # the library's kernel covers identity / relu / sigmoid / tanh on the usual layout
        # (scalars first); other layers keep the torch code below
        self._codes = (bnact.activation_code(scalar_activation if self.scalar_act is not None
                                             else None),
                       bnact.activation_code(gate_activation if self.gate_act is not None
                                             else None))
        self._kernel_ok = None not in self._codes and bnact.canonical(self.Rs)
        if self._kernel_ok:
            self._tables_cpu, self._c_out, self._n_gates = bnact.gate_layout(
                self.Rs, self.scalar_act is not None, self.gate_act is not None)
        self._tables_dev = {}

    def fill_plan(self, plan, device):
        """Add the activation half to a bnact.BnActPlan."""
        key = str(device)
        if key not in self._tables_dev:
            self._tables_dev[key] = bnact.to_device(self._tables_cpu, device)
        plan.act = self._tables_dev[key]
        plan.act_scalar, plan.act_gate = self._codes
        plan.c_out = self._c_out
        plan.n_scalar_act = self.multiplicities[0] if self.scalar_act is not None else 0
        plan.n_gates = self._n_gates
        return plan

    def biases(self):
        return (self.scalar_act.bias if self.scalar_act is not None else None,
                self.gate_act.bias if self.gate_act is not None else None)

    def forward(self, input):
        if self.scalar_act is not None or self.gate_act is not None:
            features = input.features
            if (self._kernel_ok and bnact.usable(features) and features.size(0) > 0
                    and features.size(1) == self._c_out + self._n_gates):
                sb, gb = self.biases()
                input.features = bnact.bn_act(features, None, None, sb, gb,
                                              self.fill_plan(bnact.BnActPlan(), features.device))
                return input
            if self.checkpoint and torch.is_grad_enabled() and features.requires_grad:
                features = torch.utils.checkpoint.checkpoint(self._gate, features,
                                                             use_reentrant=False)
            else:
                features = self._gate(features)
            input.features = features
        return input

    def _gate(self, y):
        out_dim = Rs2dim(self.Rs)
        gates = self.gate_act(y[:, out_dim:]) if self.gate_act is not None else None
        pieces = []
        col = gcol = 0
        for m, l in self.Rs:
            if m == 0:
                continue
            width = m * (2 * l + 1)
            field = y[:, col:col + width]
            if l == 0:
                if self.scalar_act is not None:
                    field = self.scalar_act(field)
            elif gates is not None:
                field = field * gates[:, self._gate_of[gcol:gcol + width]]
                gcol += width
            pieces.append(field)
            col += width
        return torch.cat(pieces, dim=1)
