"""SE(3) batch normalisation and gated non-linearity on the HIP kernels of libssc
(`ssc_bn_prepare_f32`, `ssc_bnact_fwd_f32`, `ssc_bnact_bwd_sums_f32`, `ssc_bnact_bwd_f32`).

The arithmetic is the reference's (ss_conv/batchnorm.py:49-136, ss_conv/activation.py:55-100);
the modules BatchNorm and Activation call into this file for CUDA float32 features, each on its
own or, through `fused.BatchNormActivation`, as one pass over the rows.  Only the input rows
and a few per-column vectors are kept for the backward pass, which recomputes the normalised
values (what the reference gets from torch.utils.checkpoint).
"""
import torch

from ss_conv import _ext


def activation_code(fn):
    """Code of an activation callable for the kernels, or None when it is not one of
    identity / relu / sigmoid / tanh (such layers keep the torch code)."""
    if fn is None:
        return _ext.ACT_NONE
    if isinstance(fn, torch.nn.Module):
        table = ((torch.nn.ReLU, _ext.ACT_RELU), (torch.nn.Sigmoid, _ext.ACT_SIGMOID),
                 (torch.nn.Tanh, _ext.ACT_TANH), (torch.nn.Identity, _ext.ACT_NONE))
        for cls, code in table:
            if type(fn) is cls:
                return code
        return None
    names = {"relu": _ext.ACT_RELU, "sigmoid": _ext.ACT_SIGMOID, "tanh": _ext.ACT_TANH}
    known = (torch.relu, torch.nn.functional.relu, torch.sigmoid, torch.nn.functional.sigmoid,
             torch.tanh, torch.nn.functional.tanh)
    if any(fn is k for k in known):
        return names[getattr(fn, "__name__", "")]
    return None


def field_layout(Rs):
    """Tables of the batch norm's channel layout for Rs = [(multiplicity, order), ...]:
    field_of[c], scalar_idx[c], field_first[f], field_dim[f] (int32, CPU)."""
    field_of, scalar_idx, field_first, field_dim = [], [], [], []
    c = f = s = 0
    for m, l in Rs:
        d = 2 * l + 1
        for _ in range(m):
            field_first.append(c)
            field_dim.append(d)
            for _ in range(d):
                field_of.append(f)
                scalar_idx.append(s if d == 1 else -1)
            if d == 1:
                s += 1
            f += 1
            c += d
    as_t = lambda v: torch.tensor(v, dtype=torch.int32)  # noqa: E731
    return {"field_of": as_t(field_of), "scalar_idx": as_t(scalar_idx),
            "field_first": as_t(field_first), "field_dim": as_t(field_dim),
            # index tensors of the same layout for the few torch ops of the backward pass
            "field_of_long": torch.tensor(field_of, dtype=torch.long),
            "scalar_cols": torch.tensor([c for c, s in enumerate(scalar_idx) if s >= 0],
                                        dtype=torch.long)}


def gate_layout(Rs, has_scalar_act, has_gate_act):
    """Tables of the gated non-linearity for output fields Rs: out_mode[j], gate_col[j] for
    the c_out output columns and gated_first[c], gated_dim[c] for the c_in = c_out + gates
    input columns (int32, CPU).  Returns (tables, c_out, n_gates)."""
    c_out = sum(m * (2 * l + 1) for m, l in Rs)
    n_gates = sum(m for m, l in list(Rs)[1:]) if has_gate_act else 0
    out_mode, gate_col = [], []
    gated_first, gated_dim = [0] * (c_out + n_gates), [0] * (c_out + n_gates)
    col = g = 0
    for i, (m, l) in enumerate(Rs):
        d = 2 * l + 1
        for _ in range(m):
            if l == 0:
                out_mode += [1 if (has_scalar_act and i == 0) else 0] * d
                gate_col += [0] * d
            elif has_gate_act:
                out_mode += [2] * d
                gate_col += [c_out + g] * d
                gated_first[c_out + g] = col
                gated_dim[c_out + g] = d
                g += 1
            else:
                out_mode += [0] * d
                gate_col += [0] * d
            col += d
    # every entry of Rs after the first owns gates (reference: n_non_scalar =
    # sum(multiplicities[1:])), scalar entries among them included: their gates are read
    # by nothing, which the reference's loop does as well
    as_t = lambda v: torch.tensor(v, dtype=torch.int32)  # noqa: E731
    tables = {"out_mode": as_t(out_mode), "gate_col": as_t(gate_col),
              "gated_first": as_t(gated_first), "gated_dim": as_t(gated_dim)}
    return tables, c_out, n_gates


def epilogue_layout(c_out, out_mode=None, gate_col=None, block=64):
    """Column order in which a convolution computes its outputs when the evaluation-mode
    batch norm and gate are applied as its rows are stored (ssc_conv_run_epilogue_f32): the
    kernel works on blocks of `block` columns and a gate must sit in the block of the columns
    it gates.  Each block holds a run of output columns in their own order (a multiple of 4,
    so that a thread's four columns are four neighbours of the stored row), then the gates of
    the fields that run touches (at most 16 in a block) -- a gate is computed once per block
    that needs it, a gate no column reads not at all -- padded to the block size; the last
    block to a multiple of 4.

    out_mode / gate_col as in gate_layout() (None: no activation).  Returns CPU tensors
    src[c] (column of the convolution's own output order, -1 for padding), mode[c] (0 copy,
    1 scalar activation, 2 gated, 3 not stored), gate[c] (position of the gate of column c),
    dest[c] (output column), all int32 with one entry per computed column, and
    gate_run[2b], gate_run[2b+1]: first gate column and number of gates of block b."""
    pad4 = lambda n: (n + 3) // 4 * 4  # noqa: E731
    out_mode = [0] * c_out if out_mode is None else [int(v) for v in out_mode]
    gate_col = [0] * c_out if gate_col is None else [int(v) for v in gate_col]
    blocks, a = [], 0
    while a < c_out:
        b, gates = a, []
        while b < c_out:
            nb = min(b + 4, c_out)
            g2 = list(gates)
            for j in range(b, nb):
                if out_mode[j] == 2 and gate_col[j] not in g2:
                    g2.append(gate_col[j])
            if pad4(nb - a) + pad4(len(g2)) > block or len(g2) > 16:
                break
            b, gates = nb, g2
        if b == a:
            raise ValueError("a block of %d columns cannot hold four outputs and their gates" % block)
        blocks.append((a, b, gates))
        a = b
    src, mode, gate, dest, gate_run = [], [], [], [], []
    for i, (a, b, gates) in enumerate(blocks):
        base = len(src)
        first_gate = base + pad4(b - a)
        gate_run += [first_gate, len(gates)]
        for j in range(a, b):
            src.append(j)
            mode.append(out_mode[j])
            gate.append(first_gate + gates.index(gate_col[j]) if out_mode[j] == 2 else base + j - a)
            dest.append(j)
        end = base + (block if i + 1 < len(blocks) else pad4(b - a) + pad4(len(gates)))
        for pos in range(base + b - a, end):
            k = pos - first_gate
            src.append(gates[k] if 0 <= k < len(gates) else -1)
            mode.append(3)
            gate.append(pos)
            dest.append(0)
    as_t = lambda v: torch.tensor(v, dtype=torch.int32)  # noqa: E731
    return {"src": as_t(src), "mode": as_t(mode), "gate": as_t(gate), "dest": as_t(dest),
            "gate_run": as_t(gate_run)}


class BnActPlan:
    """What one call of the fused function needs besides tensors that carry gradients."""

    def __init__(self):
        self.bn = None            # tables of field_layout() on the device, or None: no batch norm
        self.training = False
        self.eps = 1e-5
        self.momentum = 0.1
        self.running_mean = None
        self.running_var = None
        self.act = None           # tables of gate_layout() on the device, or None: no activation
        self.act_scalar = _ext.ACT_NONE
        self.act_gate = _ext.ACT_NONE
        self.c_out = 0
        self.n_scalar_act = 0     # leading columns that carry a scalar-activation bias
        self.n_gates = 0


class _BnAct(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, scalar_bias, gate_bias, plan):
        x = x.contiguous()
        c_in = x.size(1)
        shift = scale = add = rstd = None
        if plan.bn is not None:
            shift, scale, add, rstd = _ext.bn_prepare(
                x, plan.bn, plan.training, plan.eps, plan.momentum,
                None if weight is None else weight.detach().contiguous(),
                None if bias is None else bias.detach().contiguous(), plan.running_mean,
                plan.running_var)
        pre_bias = None
        if scalar_bias is not None or gate_bias is not None:
            pre_bias = x.new_zeros(c_in)
            if scalar_bias is not None:
                pre_bias[:plan.n_scalar_act] = scalar_bias.detach()
            if gate_bias is not None:
                pre_bias[plan.c_out:plan.c_out + plan.n_gates] = gate_bias.detach()
        act = plan.act or {}
        y = _ext.bnact_forward(x, shift, scale, add, pre_bias, act.get("out_mode"),
                               act.get("gate_col"), plan.act_scalar, plan.act_gate, plan.c_out)
        ctx.plan = plan
        ctx.was_training = plan.bn is not None and plan.training
        ctx.has = (weight is not None, bias is not None, scalar_bias is not None,
                   gate_bias is not None)
        ctx.save_for_backward(x, shift, scale, add, rstd, pre_bias)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, shift, scale, add, rstd, pre_bias = ctx.saved_tensors
        plan = ctx.plan
        act = plan.act or {}
        args = (shift, scale, add, pre_bias, act.get("out_mode"), act.get("gate_col"),
                act.get("gated_first"), act.get("gated_dim"), plan.act_scalar, plan.act_gate)
        dy = dy.contiguous()
        n = x.size(0)
        has_w, has_b, has_sb, has_gb = ctx.has
        need_sums = ctx.was_training or any(ctx.has)
        d_weight = d_bias = d_sb = d_gb = None
        dz_mean = coef = None
        if need_sums:
            sums = _ext.bnact_backward_sums(x, dy, *args)
            col_b, col_a = sums[0], sums[1]
            if has_sb:
                d_sb = col_b[:plan.n_scalar_act].clone()
            if has_gb:
                d_gb = col_b[plan.c_out:plan.c_out + plan.n_gates].clone()
            if plan.bn is not None:
                field_of = plan.bn["field_of_long"]
                scalar_cols = plan.bn["scalar_cols"]
                field_a = torch.zeros_like(rstd).index_add_(0, field_of, col_a)
                if has_b:
                    d_bias = col_b[scalar_cols].clone()
                if has_w:
                    d_weight = rstd * field_a
                if ctx.was_training:
                    dz_mean = torch.zeros_like(col_b)
                    dz_mean[scalar_cols] = col_b[scalar_cols] / n
                    coef = scale * (rstd * rstd * field_a)[field_of] / n
        dx = _ext.bnact_backward(x, dy, *args, dz_mean, coef) if ctx.needs_input_grad[0] else None
        return dx, d_weight, d_bias, d_sb, d_gb, None


def bn_act(x, weight, bias, scalar_bias, gate_bias, plan):
    """y = gate(batch_norm(x)) for float32 CUDA rows x[n, c_in]; either half may be absent
    (plan.bn / plan.act None).  Differentiable in x and the four parameter vectors."""
    return _BnAct.apply(x, weight, bias, scalar_bias, gate_bias, plan)


MAX_CHANNELS = 1536  # the backward kernels hold their per-column tables in LDS


def usable(x):
    return (x.is_cuda and x.dtype == torch.float32 and x.dim() == 2
            and x.size(1) <= MAX_CHANNELS)


def canonical(Rs):
    """The layout the gate tables describe: a first entry of scalars (possibly with
    multiplicity 0), then non-scalar fields.  A first entry of order > 0 has no gates in the
    reference's count (n_non_scalar = sum(multiplicities[1:]), activation.py:44-52) although
    its loop asks for one per field: such a layer keeps the torch code, which fails at
    forward as the reference's does."""
    Rs = [(m, l) for m, l in Rs]
    if len(Rs) == 0:
        return False
    first_ok = Rs[0][1] == 0 or Rs[0][0] == 0
    return first_ok and all(l > 0 for m, l in Rs[1:] if m > 0)


def to_device(tables, device):
    return {k: v.to(device) for k, v in tables.items()}
