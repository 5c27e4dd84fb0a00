"""Per-unit activation functions and steepnesses (the reference keeps them as per-unit arrays in struct AF_unit and reads
them per unit in Forward_Pass__FC_AF / Backward_Pass__FC__DF / Compute__Error).  CPU: the oracle against float64
autograd of a model that applies a different function to every column.  GPU: the HIP path against the oracle."""
import numpy as np
import pytest
import torch

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, oracle_desc, oracle_hyper, run_step
from tests.oracle_lib import OracleNetwork
from tests.test_oracle_fc import _t_act

NAMES = ["TANH", "SIGMOID", "RELU", "LINEAR", "LEAKY_RELU", "ELLIOT_SYMMETRIC", "SINE_SYMMETRIC", "GAUSSIAN", "ISRU"]
SPECS = [dict(units=7), dict(units=11, activation="TANH"), dict(type="residual", block_depth=2), dict(units=9, activation="TANH"),
         dict(units=11, activation="SIGMOID"), dict(units=5, activation="SIGMOID")]
B = 6


def _unit_types(n, seed):
    rng = np.random.default_rng(seed)
    names = [NAMES[i] for i in rng.integers(0, len(NAMES), n)]
    return names, np.array([mb.AF[x] for x in names], dtype=np.uint32)


def _setup(net_cls, desc, h, w):
    net = net_cls(desc, h)
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(w)
    names1, t1 = _unit_types(11, 1)          # plain hidden layer: 11 units
    names4, t4 = _unit_types(9, 2)           # second member of the block: activation units on its input side (fan-in 9)
    names5, t5 = _unit_types(5, 3)           # output layer
    net.set_unit_activations(1, t1)
    net.set_unit_activations(4, t4)
    net.set_unit_activations(5, t5)
    return net, (names1, names4, names5)


def _columns(names, x):
    return torch.stack([_t_act(n, x[:, j]) for j, n in enumerate(names)], dim=1)


def test_oracle_per_unit_functions_match_float64_autograd():
    desc = oracle_desc(SPECS, B)
    w = glorot_parameters(desc, 5, bias_range=0.3)
    rng = np.random.default_rng(6)
    X = rng.normal(0, 1, (B, 7)).astype(np.float32)
    Y = rng.normal(0, 1, (B, 5)).astype(np.float32)
    net, (n1, n4, n5) = _setup(OracleNetwork, desc, oracle_hyper(type_loss_function=mb.LOSS["MSE"]), w)
    run_step(net, B, X, Y, update=False)
    flat = torch.tensor(w.astype(np.float64), requires_grad=True)
    L = desc.layers
    lin = lambda li, x, out: x @ flat[L[li].first_connection_index:L[li].first_connection_index + out * x.shape[1]].view(out, x.shape[1]).t() \
        + flat[L[li].first_bias_connection_index:L[li].first_bias_connection_index + out]
    x = torch.tensor(X.astype(np.float64))
    h1 = _columns(n1, lin(1, x, 11))
    u3 = lin(3, h1, 9)                                   # first member: weights only
    u4 = lin(4, _columns(n4, u3), 11)                    # second member: per-unit activation of its input, then weights
    y = _columns(n5, lin(5, h1 + u4, 5))
    (0.5 * ((y - torch.tensor(Y.astype(np.float64))) ** 2).sum()).backward()
    assert_close(net.download_tensor(5, mb.TENSOR["OUTPUTS"]).reshape(B, 5), y.detach().numpy(), 3e-5, 3e-6, "outputs")
    assert_close(net.download_gradient(), flat.grad.numpy(), 3e-4, 3e-5, "gradient")


def test_oracle_per_unit_steepness_scales_the_derivative_only():
    """steepness multiplies act' and never the forward value (Activation_Functions.hpp): with steepness s_j on the hidden
    units the weight gradient of that layer's unit j is s_j times the gradient at steepness 1."""
    specs = [dict(units=4), dict(units=6, activation="TANH"), dict(units=3, activation="LINEAR")]
    desc = oracle_desc(specs, B)
    w = glorot_parameters(desc, 7, bias_range=0.3)
    rng = np.random.default_rng(8)
    X = rng.normal(0, 1, (B, 4)).astype(np.float32)
    Y = rng.normal(0, 1, (B, 3)).astype(np.float32)
    st = np.array([1.0, 0.5, 0.25, 1.0, 0.75, 0.1], dtype=np.float32)
    grads, outs = [], []
    for steep in (None, st):
        net = OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS["MSE"]))
        net.set_state_propagation(mb.STATE_TRAINING)
        net.upload_parameters(w)
        if steep is not None:
            net.set_unit_activations(1, None, steep)
        run_step(net, B, X, Y, update=False)
        grads.append(net.download_gradient())
        outs.append(net.download_tensor(2, mb.TENSOR["OUTPUTS"]))
    assert np.array_equal(outs[0], outs[1])
    l1 = desc.layers[1]
    g0 = grads[0][l1.first_connection_index:l1.last_connection_index].reshape(6, 4)
    g1 = grads[1][l1.first_connection_index:l1.last_connection_index].reshape(6, 4)
    assert_close(g1, g0 * st[:, None], 1e-5, 1e-7)
    l2 = desc.layers[2]
    assert np.array_equal(grads[0][l2.first_connection_index:l2.last_connection_index], grads[1][l2.first_connection_index:l2.last_connection_index])


@pytest.mark.gpu
@pytest.mark.parametrize("optimizer", ["GD", "ADAM"])
def test_gpu_per_unit_activations_match_oracle(optimizer):
    desc = mb.make_desc(SPECS, B)
    w = glorot_parameters(desc, 5, bias_range=0.3)
    rng = np.random.default_rng(6)
    X = rng.normal(0, 1, (B, 7)).astype(np.float32)
    Y = rng.normal(0, 1, (B, 5)).astype(np.float32)
    h = mb.default_hyper(type_loss_function=mb.LOSS["MSE"], type_optimizer_function=mb.OPTIMIZER[optimizer])
    gpu, _ = _setup(mb.HipNetwork, desc, h, w)
    cpu, _ = _setup(OracleNetwork, desc, h, w)
    st = rng.uniform(0.1, 1.0, 11).astype(np.float32)
    for n in (gpu, cpu):
        n.set_unit_activations(1, _unit_types(11, 1)[1], st)
        n.Clear_Training_Arrays()
    lib = mb.load_library()
    for step in range(2):
        for n in (gpu, cpu):
            n.Reset__Loss()
            run_step(n, B, X, Y, update=False)
        for li in range(1, desc.n_layers):
            width = lib.myea_net_desc_number_outputs(desc, li)
            for kind in ("OUTPUTS", "ERRORS"):
                assert_close(gpu.download_tensor(li, mb.TENSOR[kind], B * width), cpu.download_tensor(li, mb.TENSOR[kind], B * width), 1e-4, 1e-5, "layer %d %s" % (li, kind))
        assert_close(gpu.download_gradient(), cpu.download_gradient(), 1e-4, 1e-5, "gradient")
        for n in (gpu, cpu):
            n.Update_Parameter(B, B)
        gpu.upload_parameters(cpu.download_parameters())
        if optimizer == "ADAM":
            for k in (1, 2):
                gpu.upload_optimizer_state(k, cpu.download_optimizer_state(k))
    # back to the layer-wide function
    for n in (gpu, cpu):
        for li in (1, 4, 5):
            n.set_unit_activations(li, None, None)
        run_step(n, B, X, Y, update=False)
    assert_close(gpu.download_gradient(), cpu.download_gradient(), 1e-4, 1e-5, "gradient, layer-wide again")
    with pytest.raises(mb.MyeaError):
        gpu.set_unit_activations(1, np.zeros(10, dtype=np.uint32))      # wrong count
    with pytest.raises(mb.MyeaError):
        gpu.set_unit_activations(1, np.full(11, mb.AF["SOFTMAX"], dtype=np.uint32))
