"""The oracle's batch norm and gated non-linearity (oracle.batchnorm_fwd, gate_fwd,
bn_gate_bwd) pinned by what the mathematics fixes, and the host logic of the layers
(channel tables, torch code path, parameter names) checked on the CPU."""
import numpy as np
import pytest
import torch

RS = [(3, 0), (2, 1), (2, 2)]
RS_BN = RS + [(4, 0)]           # fields + one gate scalar per non-scalar field
C_IN = 3 + 6 + 10 + 4
C_OUT = 3 + 6 + 10


def _params(rng):
    return dict(weight=rng.normal(size=11) + 1, bias=rng.normal(size=7),
                scalar_bias=rng.normal(size=3), gate_bias=rng.normal(size=4))


def test_batchnorm_training_statistics(oracle):
    rng = np.random.default_rng(1)
    x = rng.normal(size=(500, C_IN)) * 3 + 2
    y, rm, rv = oracle.batchnorm_fwd(x, RS_BN, eps=0.0, momentum=0.25, training=True)
    # scalars: zero mean, unit variance; every field: unit mean squared norm
    scalar_cols = [0, 1, 2, 19, 20, 21, 22]
    assert np.allclose(y[:, scalar_cols].mean(0), 0, atol=1e-12)
    assert np.allclose((y[:, scalar_cols] ** 2).mean(0), 1, atol=1e-12)
    assert np.allclose((y[:, 3:6] ** 2).sum(1).mean(), 1, atol=1e-12)
    assert np.allclose((y[:, 9:14] ** 2).sum(1).mean(), 1, atol=1e-12)
    # non-scalar fields are scaled, not shifted: directions are preserved
    ratio = y[:, 3:6] / x[:, 3:6]
    assert np.allclose(ratio, ratio[0, 0])
    # running statistics move by the momentum from (0, 1)
    assert np.allclose(rm, 0.25 * x[:, scalar_cols].mean(0))
    assert np.allclose(rv[3], 0.75 + 0.25 * (x[:, 3:6] ** 2).sum(1).mean())
    assert np.allclose(rv[0], 0.75 + 0.25 * x[:, 0].var())


def test_batchnorm_eval_and_affine(oracle):
    rng = np.random.default_rng(2)
    x = rng.normal(size=(50, C_IN))
    p = _params(rng)
    rm, rv = rng.normal(size=7), rng.uniform(0.5, 2, size=11)
    y, rm2, rv2 = oracle.batchnorm_fwd(x, RS_BN, p["weight"], p["bias"], rm, rv, eps=1e-5,
                                       training=False)
    assert np.array_equal(rm2, rm) and np.array_equal(rv2, rv)
    # column 1: scalar number 1, field number 1; column 4: field 3 (first l=1 field), no shift
    assert np.allclose(y[:, 1], (x[:, 1] - rm[1]) / np.sqrt(rv[1] + 1e-5) * p["weight"][1] + p["bias"][1])
    assert np.allclose(y[:, 4], x[:, 4] / np.sqrt(rv[3] + 1e-5) * p["weight"][3])
    # last gate scalar: scalar number 6, field number 10
    assert np.allclose(y[:, 22], (x[:, 22] - rm[6]) / np.sqrt(rv[10] + 1e-5) * p["weight"][10] + p["bias"][6])


def test_gate_known_answer(oracle):
    Rs = [(1, 0), (1, 1)]
    y = np.array([[-1.0, 1.0, 2.0, 3.0, 0.0],
                  [2.0, -1.0, 0.5, 4.0, np.log(3.0)]])
    z = oracle.gate_fwd(y, Rs, scalar_bias=[0.5], gate_bias=[0.0], act_scalar="relu",
                        act_gate="sigmoid")
    assert np.allclose(z[0], [0.0, 0.5, 1.0, 1.5])            # relu(-0.5) = 0, sigmoid(0) = 1/2
    assert np.allclose(z[1], [2.5, -0.75, 0.375, 3.0])        # sigmoid(log 3) = 3/4
    # no gate activation: gate columns are dropped, fields unchanged
    z = oracle.gate_fwd(y, Rs, act_scalar="tanh", act_gate=None)
    assert np.allclose(z[:, 1:], y[:, 1:4]) and np.allclose(z[:, 0], np.tanh(y[:, 0]))


@pytest.mark.parametrize("training", [True, False])
@pytest.mark.parametrize("acts", [("relu", "sigmoid"), ("tanh", "tanh"), (None, "sigmoid")])
def test_backward_matches_central_differences(oracle, training, acts):
    rng = np.random.default_rng(3)
    x = rng.normal(size=(6, C_IN)) * 2 + 0.5
    dy = rng.normal(size=(6, C_OUT))
    p = _params(rng)
    if acts[0] is None:
        p["scalar_bias"] = None
    running = (rng.normal(size=7), rng.uniform(0.5, 2, size=11))
    kw = dict(training=training, act_scalar=acts[0], act_gate=acts[1], running=running)

    def loss(xx, pp):
        return (dy * oracle.bn_gate_fwd(xx, RS_BN, RS, pp, **kw)).sum()

    g = oracle.bn_gate_bwd(x, dy, RS_BN, RS, p, **kw)
    h = 1e-6
    num = np.zeros_like(x)
    for i in range(x.shape[0]):
        for j in range(x.shape[1]):
            xp, xm = x.copy(), x.copy()
            xp[i, j] += h
            xm[i, j] -= h
            num[i, j] = (loss(xp, p) - loss(xm, p)) / (2 * h)
    assert np.abs(num - g["x"]).max() < 1e-7
    for k, v in p.items():
        if v is None:
            continue
        numk = np.zeros_like(v)
        for j in range(len(v)):
            pp = {a: (None if b is None else b.copy()) for a, b in p.items()}
            pm = {a: (None if b is None else b.copy()) for a, b in p.items()}
            pp[k][j] += h
            pm[k][j] -= h
            numk[j] = (loss(x, pp) - loss(x, pm)) / (2 * h)
        assert np.abs(numk - g[k]).max() < 1e-7, k


def test_layers_torch_path_equals_oracle(oracle):
    """BatchNorm and Activation on CPU tensors (the torch code of the layers)."""
    from ss_conv.activation import Activation
    from ss_conv.batchnorm import BatchNorm
    from ss_conv.sp_ops.tensor import SparseTensor
    rng = np.random.default_rng(4)
    x = rng.normal(size=(40, C_IN)).astype(np.float32)
    p = _params(rng)
    bn = BatchNorm(RS_BN)
    act = Activation(RS, (torch.relu, torch.sigmoid))
    with torch.no_grad():
        bn.weight.copy_(torch.from_numpy(p["weight"]))
        bn.bias.copy_(torch.from_numpy(p["bias"]))
        act.scalar_act.bias.copy_(torch.from_numpy(p["scalar_bias"]))
        act.gate_act.bias.copy_(torch.from_numpy(p["gate_bias"]))
    for training in (True, False):
        bn.train(training)
        running = (bn.running_mean.numpy().copy(), bn.running_var.numpy().copy())
        st = SparseTensor(torch.from_numpy(x), torch.zeros(40, 4, dtype=torch.int32), [4, 4, 4], 1)
        y = act(bn(st)).features.detach().numpy()
        want = oracle.bn_gate_fwd(x, RS_BN, RS, p, training=training, running=running)
        assert np.abs(y - want).max() < 1e-4
        if training:
            _, rm, rv = oracle.batchnorm_fwd(x, RS_BN, p["weight"], p["bias"], *running)
            assert np.allclose(bn.running_mean.numpy(), rm, atol=1e-5)
            assert np.allclose(bn.running_var.numpy(), rv, atol=1e-5)


def test_channel_tables():
    from ss_conv import bnact
    lay = bnact.field_layout(RS_BN)
    assert lay["field_of"].tolist() == [0, 1, 2, 3, 3, 3, 4, 4, 4, 5, 5, 5, 5, 5, 6, 6, 6, 6, 6, 7, 8, 9, 10]
    assert lay["scalar_idx"].tolist() == [0, 1, 2] + [-1] * 16 + [3, 4, 5, 6]
    assert lay["field_first"].tolist() == [0, 1, 2, 3, 6, 9, 14, 19, 20, 21, 22]
    assert lay["field_dim"].tolist() == [1, 1, 1, 3, 3, 5, 5, 1, 1, 1, 1]
    tab, c_out, n_gates = bnact.gate_layout(RS, True, True)
    assert (c_out, n_gates) == (C_OUT, 4)
    assert tab["out_mode"].tolist() == [1] * 3 + [2] * 16
    assert tab["gate_col"].tolist()[3:] == [19] * 3 + [20] * 3 + [21] * 5 + [22] * 5
    assert tab["gated_first"].tolist()[19:] == [3, 6, 9, 14]
    assert tab["gated_dim"].tolist()[19:] == [3, 3, 5, 5]
    # no scalar activation / no gates
    tab, c_out, n_gates = bnact.gate_layout(RS, False, False)
    assert n_gates == 0 and set(tab["out_mode"].tolist()) == {0}
    assert bnact.canonical(RS) and bnact.canonical([(0, 0), (2, 1)])
    assert not bnact.canonical([(2, 1), (2, 0)])
    assert bnact.activation_code(torch.relu) == 1 and bnact.activation_code(torch.sigmoid) == 2
    assert bnact.activation_code(torch.nn.Tanh()) == 3 and bnact.activation_code(None) == 0
    assert bnact.activation_code(torch.nn.functional.softplus) is None


def test_parameter_names_follow_the_reference():
    """State-dict keys of the layers are the reference's (batchnorm.py:27-36,
    activation.py:31-41,118, convolution.py:33-34, kernel.py:238-255), so its checkpoints load."""
    from ss_conv.activation import Activation
    from ss_conv.batchnorm import BatchNorm
    from ss_conv.convolution import Convolution
    from ss_conv.fused import BatchNormActivation
    bn = BatchNorm(RS_BN)
    act = Activation(RS, (torch.relu, torch.sigmoid))
    assert sorted(bn.state_dict()) == ["bias", "running_mean", "running_var", "weight"]
    assert sorted(act.state_dict()) == ["gate_act.bias", "scalar_act.bias"]
    assert bn.running_mean.shape == (7,) and bn.running_var.shape == (11,)
    assert bn.weight.shape == (11,) and bn.bias.shape == (7,)
    assert act.scalar_act.bias.shape == (3,) and act.gate_act.bias.shape == (4,)
    fused = BatchNormActivation(bn, act)
    assert sorted(fused.state_dict()) == ["act.gate_act.bias", "act.scalar_act.bias", "bn.bias",
                                          "bn.running_mean", "bn.running_var", "bn.weight"]
    conv = Convolution([(2, 0), (1, 1)], [(2, 0), (1, 1)], 3, padding=1)
    keys = sorted(conv.state_dict())
    assert "kernel.weight" in keys
    assert [k for k in keys if k.startswith("kernel.kernel_")] == [
        "kernel.kernel_0_0", "kernel.kernel_0_1", "kernel.kernel_1_0", "kernel.kernel_1_1"]
