"""Layers of the reference's blocks run as fewer passes over the feature rows.

The reference applies convolution, batch norm and gated activation one after the other, each
a pass (or a chain of torch ops) over [N, C] (Common_utils/ss_conv_modules.py:105-117,
Common_utils/ss_conv_backbones.py:30-46).  The wrappers here own the reference layers
unchanged, so parameters, buffers and state-dict keys are theirs:

  BatchNormActivation(bn, act)            both in `ssc_bnact_fwd_f32`: the normalised rows are
                                          never written to memory;
  ConvBatchNormActivation(conv, bn, act)  in evaluation mode the batch norm's per-column
                                          constants and the gate are applied by the convolution
                                          kernel while it stores its rows
                                          (`ssc_conv_run_epilogue_f32`): the convolution's own
                                          output is never written either.  In training mode
                                          (batch statistics need every row first) it is the
                                          convolution followed by BatchNormActivation.
"""
import torch
import torch.nn as nn

from ss_conv import _ext, bnact
from ss_conv.activation import Activation
from ss_conv.batchnorm import BatchNorm
from ss_conv.sp_ops.conv import SparseConvolution


def _bn_act(bn, act, input):
    """act(bn(input)), in one pass where the kernels cover both layers."""
    if bn is None or act is None:
        if bn is not None:
            input = bn(input)
        return act(input) if act is not None else input
    x = input.features
    fusable = (act._kernel_ok and (act.scalar_act is not None or act.gate_act is not None)
               and bnact.usable(x) and x.size(0) > 0 and bn.reduce == 'mean'
               and x.size(1) == bn.num_channels
               and x.size(1) == act._c_out + act._n_gates)
    if not fusable:
        return act(bn(input))
    plan = act.fill_plan(bn.plan(x.device), x.device)
    sb, gb = act.biases()
    input.features = bnact.bn_act(x, bn.weight, bn.bias, sb, gb, plan)
    return input


class BatchNormActivation(nn.Module):
    def __init__(self, bn, act):
        """bn: BatchNorm over the fields and gate scalars; act: Activation of the fields."""
        super().__init__()
        if not isinstance(bn, BatchNorm) or not isinstance(act, Activation):
            raise TypeError("BatchNormActivation(bn: BatchNorm, act: Activation)")
        self.bn = bn
        self.act = act

    def forward(self, input):  # pylint: disable=W
        return _bn_act(self.bn, self.act, input)


class ConvBatchNormActivation(nn.Module):
    """conv -> bn -> activation of a block (Common_utils/ss_conv_modules.py:60-117; attribute
    names as there).  bn and activation may be None, as in the reference's block."""

    def __init__(self, conv, bn=None, activation=None):
        super().__init__()
        if not isinstance(conv, SparseConvolution):
            raise TypeError("conv must be a (Sparse)Convolution layer")
        if bn is not None and not isinstance(bn, BatchNorm):
            raise TypeError("bn must be a BatchNorm layer or None")
        if activation is not None and not isinstance(activation, Activation):
            raise TypeError("activation must be an Activation layer or None")
        self.conv = conv
        self.bn = bn
        self.activation = activation
        self._layout = None  # epilogue_layout() of this block, or False: not expressible
        self._held = None    # (key, permuted filters, ConvEpilogue)

    def _has_act(self):
        act = self.activation
        return act is not None and (act.scalar_act is not None or act.gate_act is not None)

    def _block_layout(self):
        if self._layout is None:
            self._layout = False
            act, bn, c_conv = self.activation, self.bn, self.conv.out_channels
            ok = bn is not None or self._has_act()
            if bn is not None:
                ok = ok and bn.reduce == 'mean' and bn.num_channels == c_conv
            if self._has_act():
                ok = ok and act._kernel_ok and act._c_out + act._n_gates == c_conv
            if ok:
                try:
                    if self._has_act():
                        t = act._tables_cpu
                        self._layout = bnact.epilogue_layout(act._c_out, t["out_mode"].tolist(),
                                                             t["gate_col"].tolist())
                    else:
                        self._layout = bnact.epilogue_layout(c_conv)
                except ValueError:
                    pass
        return self._layout

    def _epilogue(self, weight):
        """Filters in the epilogue's column order and its tables; rebuilt when the filters,
        the running statistics or a parameter of the two layers changed."""
        bn, act, dev = self.bn, self.activation, weight.device
        sb, gb = act.biases() if self._has_act() else (None, None)
        watched = [weight] + ([bn.running_mean, bn.running_var, bn.weight, bn.bias]
                              if bn is not None else []) + [sb, gb]
        key = tuple((id(t), t._version) for t in watched if t is not None) + (str(dev),)
        if self._held is not None and self._held[0] == key:
            return self._held[1], self._held[2]
        lay = self._layout
        c_conv = self.conv.out_channels
        src = lay["src"].to(dev).long()
        valid = src >= 0
        with torch.no_grad():
            wp = weight.new_zeros(tuple(weight.shape[:-1]) + (src.numel(),))
            wp[..., valid] = weight.detach()[..., src[valid]]
            # the tables are float32 whatever the rows are
            f32 = lambda t: None if t is None else t.detach().float().contiguous()  # noqa: E731
            zeros = lambda *shape: torch.zeros(shape, dtype=torch.float32, device=dev)  # noqa: E731
            if bn is not None:
                shift, scale, add, _ = _ext.bn_prepare(
                    zeros(1, c_conv), bn.layout(dev), False, bn.eps, bn.momentum,
                    f32(bn.weight), f32(bn.bias), f32(bn.running_mean), f32(bn.running_var))
            else:
                shift, add = zeros(c_conv), zeros(c_conv)
                scale = torch.ones(c_conv, dtype=torch.float32, device=dev)
            pre = zeros(c_conv)
            codes = (_ext.ACT_NONE, _ext.ACT_NONE)
            c_dest = c_conv
            if self._has_act():
                codes, c_dest = act._codes, act._c_out
                if sb is not None:
                    pre[:act.multiplicities[0]] = sb.detach().float()
                if gb is not None:
                    pre[act._c_out:act._c_out + act._n_gates] = gb.detach().float()
            pick = src.clamp(min=0)
            epi = _ext.ConvEpilogue(shift[pick].contiguous(), scale[pick].contiguous(),
                                    add[pick].contiguous(), pre[pick].contiguous(),
                                    lay["mode"].to(dev), lay["gate"].to(dev), lay["dest"].to(dev),
                                    lay["gate_run"].to(dev), codes[0], codes[1], c_dest)
        self._held = (key, wp, epi)
        return wp, epi

    def _tail_wants_grad(self):
        """Whether autograd is on and a parameter of the batch norm or the activation asks for
        a gradient (fine-tuning affine or bias parameters on frozen statistics): the one-kernel
        path builds no graph, so such a call takes the separate layers."""
        if not torch.is_grad_enabled():
            return False
        return any(p.requires_grad for m in (self.bn, self.activation) if m is not None
                   for p in m.parameters())

    def forward(self, input):  # pylint: disable=W
        conv = self.conv
        if not self.training and input.features.is_cuda and self._block_layout() \
                and not self._tail_wants_grad():
            feats = input.features
            weight = conv.eval_weight(feats) if hasattr(conv, "eval_weight") else conv.weight
            if weight is not None and conv.epilogue_ok(input, weight):
                wp, epi = self._epilogue(weight)
                return conv._sparse_conv(input, wp, epilogue=epi)
        return _bn_act(self.bn, self.activation, conv(input))
