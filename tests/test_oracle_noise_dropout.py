"""Pins the oracle's Gaussian (y *= g) and Uout (y += y u) dropout: neutral draws change nothing, constant draws scale the
layer's outputs, the inference pass ignores the draws, and the backward pass - which never sees them - against float64
autograd of a straight-through model.  The draws are an input of the oracle (the reference takes them from its host
generators inside the pass).  CPU only."""
import numpy as np
import pytest
import torch

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, oracle_desc, oracle_hyper
from tests.oracle_lib import OracleNetwork


def _net(specs, B, T=1, seed=1, state=mb.STATE_TRAINING):
    desc = oracle_desc(specs, B, T)
    net = OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS["MSE"]))
    w = glorot_parameters(desc, seed, bias_range=0.3)
    net.set_state_propagation(state)
    net.upload_parameters(w)
    net.Clear_Training_Arrays()
    return desc, net, w


@pytest.mark.parametrize("kind,const,factor", [("GAUSSIAN", 1.0, 1.0), ("GAUSSIAN", 0.5, 0.5), ("UOUT", 0.0, 1.0), ("UOUT", 0.25, 1.25), ("UOUT", -1.0, 0.0)])
def test_constant_draws_scale_the_outputs(kind, const, factor):
    B, T, H = 5, 3, 9
    plain = [dict(units=4), dict(units=H, activation="TANH"), dict(units=3, activation="LINEAR")]
    noisy = [dict(units=4), dict(units=H, activation="TANH", dropout=kind, keep=0.3), dict(units=3, activation="LINEAR")]
    X = np.random.default_rng(1).normal(0, 1, (B, T * 4)).astype(np.float32)
    _, a, _ = _net(plain, B, T)
    _, b, _ = _net(noisy, B, T)
    b.upload_dropout_noise(1, np.full(T * B * H, const, dtype=np.float32))
    a.Forward_Pass(B, X); b.Forward_Pass(B, X)
    ya, yb = a.download_tensor(1, mb.TENSOR["OUTPUTS"]), b.download_tensor(1, mb.TENSOR["OUTPUTS"])
    assert np.array_equal(yb, (ya * np.float32(factor)).astype(np.float32))
    # the inference state ignores the draws
    _, c, _ = _net(noisy, B, T, state=mb.STATE_INFERENCE)
    c.upload_dropout_noise(1, np.full(T * B * H, 7.0, dtype=np.float32))
    c.Forward_Pass(B, X)
    assert np.array_equal(c.download_tensor(1, mb.TENSOR["OUTPUTS"]), ya)


@pytest.mark.parametrize("kind", ["GAUSSIAN", "UOUT"])
def test_forward_uses_one_draw_per_example_and_unit_and_backward_ignores_them(kind):
    B, H = 6, 12
    specs = [dict(units=5), dict(units=H, activation="LEAKY_RELU", dropout=kind, keep=0.4), dict(units=3, activation="LINEAR")]
    desc, net, w = _net(specs, B, seed=2)
    rng = np.random.default_rng(2)
    X, Y = rng.normal(0, 1, (B, 5)).astype(np.float32), rng.normal(0, 1, (B, 3)).astype(np.float32)
    noise = (rng.normal(1, 0.6, (B, H)) if kind == "GAUSSIAN" else rng.uniform(-0.4, 0.4, (B, H))).astype(np.float32)
    net.upload_dropout_noise(1, noise)
    net.Forward_Pass(B, X); net.Compute__Error(B, Y); net.Backward_Pass(B); net.Update_Derivative_Weight(B)
    W = torch.tensor(w.astype(np.float64), requires_grad=True)
    l1, l2 = desc.layers[1], desc.layers[2]
    W1 = W[l1.first_connection_index:l1.last_connection_index].reshape(H, 5)
    W2 = W[l2.first_connection_index:l2.last_connection_index].reshape(3, H)
    b1 = W[l1.first_bias_connection_index:l1.first_bias_connection_index + H]
    b2 = W[l2.first_bias_connection_index:l2.first_bias_connection_index + 3]
    s = torch.tensor(X.astype(np.float64)) @ W1.T + b1
    a = torch.where(s < 0, 0.01 * s, s)
    g = torch.tensor(noise.astype(np.float64))
    noisy = a * g if kind == "GAUSSIAN" else a + a * g
    h = a + (noisy - a).detach()                       # forward: with the draws; backward: as if they were not there
    y = h @ W2.T + b2
    (0.5 * ((y - torch.tensor(Y.astype(np.float64))) ** 2).sum()).backward()
    assert_close(net.download_tensor(1, mb.TENSOR["OUTPUTS"], B * H), noisy.detach().numpy().ravel(), rel=1e-5, abs_=2e-6, what="layer outputs")
    assert_close(net.download_tensor(2, mb.TENSOR["OUTPUTS"], B * 3), y.detach().numpy().ravel(), rel=1e-5, abs_=2e-6, what="outputs")
    assert_close(net.download_gradient(), W.grad.numpy(), rel=3e-4, abs_=3e-6, what="gradient")
