"""Pins the oracle's average / max pooling layers (forward, backward, layout) with torch's pooling routines and float64
autograd through a stack FC -> pooling -> FC.  CPU only."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, oracle_desc, oracle_hyper
from tests.oracle_lib import OracleNetwork

POOLS = [
    dict(type="average_pooling", kernel=2, stride=2),
    dict(type="average_pooling", kernel=3, stride=2, padding=1),
    dict(type="average_pooling", kernel=4, stride=3, padding=2, ceil_mode=1),
    dict(type="max_pooling", kernel=2, stride=2),
    dict(type="max_pooling", kernel=3, stride=1, padding=1),
    dict(type="max_pooling", kernel=3, stride=2, padding=1, dilation=2),
    dict(type="max_pooling", kernel=2, stride=3, padding=1, ceil_mode=1),
]


def _torch_pool(spec, x):
    """the reference's semantics in torch terms: zeros stand in the padding (also for the maximum), the average always divides
    by the kernel size, ceil mode only changes the number of windows (a window hanging over the right edge sees zeros)"""
    k, s, p, d, ceil = (spec.get(n, dflt) for n, dflt in (("kernel", 0), ("stride", 1), ("padding", 0), ("dilation", 1), ("ceil_mode", 0)))
    In = x.shape[-1]
    if spec["type"] == "average_pooling":
        span = In + 2 * p - k
    else:
        span = In + 2 * p - d * (k - 1) - 1
    out = int(np.ceil(span / s + 1)) if ceil else int(np.floor(span / s + 1))
    need = (out - 1) * s + (k - 1) * d + 1                    # padded length the last window reaches
    right = max(need - (In + p), 0)
    xp = F.pad(x.unsqueeze(1), (p, right))                   # zero padding on both sides
    if spec["type"] == "average_pooling":
        y = F.avg_pool1d(xp, k, s, 0, ceil_mode=False, count_include_pad=True) if d == 1 else None
    else:
        y = F.max_pool1d(xp, k, s, 0, dilation=d, ceil_mode=False)
    return y.squeeze(1)[..., :out], out


@pytest.mark.parametrize("spec", POOLS, ids=lambda s: "%s-k%d-s%d-p%d-d%d-c%d" % (s["type"][:3], s["kernel"], s.get("stride", 1), s.get("padding", 0), s.get("dilation", 1), s.get("ceil_mode", 0)))
def test_pooling_layer_against_torch_forward_and_autograd(spec):
    In, B = 13, 5
    specs = [dict(units=7), dict(units=In, activation="TANH"), dict(spec), dict(units=4, activation="LINEAR")]
    desc = oracle_desc(specs, B)
    x0 = torch.zeros(1, In, dtype=torch.float64)
    _, out = _torch_pool(spec, x0)
    assert desc.layers[2].n_units == out                                  # the layout computes the width
    assert desc.layers[2].first_connection_index == desc.layers[2].last_connection_index
    assert desc.layers[3].last_connection_index - desc.layers[3].first_connection_index == 4 * out
    assert desc.total_bias == In + 4 and desc.total_mask_units == 7 + In + 4
    net = OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS["MSE"]))
    w = glorot_parameters(desc, 1, bias_range=0.3)
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(w)
    net.Clear_Training_Arrays()
    rng = np.random.default_rng(1)
    X, Y = rng.normal(0, 1, (B, 7)).astype(np.float32), rng.normal(0, 1, (B, 4)).astype(np.float32)
    net.Forward_Pass(B, X); net.Compute__Error(B, Y); net.Backward_Pass(B); net.Update_Derivative_Weight(B)
    # float64 model
    W = torch.tensor(w.astype(np.float64), requires_grad=True)
    l1, l3 = desc.layers[1], desc.layers[3]
    W1 = W[l1.first_connection_index:l1.last_connection_index].reshape(In, 7)
    W3 = W[l3.first_connection_index:l3.last_connection_index].reshape(4, out)
    b1 = W[desc.total_weights:desc.total_weights + In]; b3 = W[desc.total_weights + In:desc.total_weights + In + 4]
    h = torch.tanh(torch.tensor(X.astype(np.float64)) @ W1.T + b1)
    pooled, _ = _torch_pool(spec, h)
    y = pooled @ W3.T + b3
    loss = 0.5 * ((y - torch.tensor(Y.astype(np.float64))) ** 2).sum()
    loss.backward()
    assert_close(net.download_tensor(2, mb.TENSOR["OUTPUTS"], B * out), pooled.detach().numpy().ravel(), rel=1e-5, abs_=1e-6, what="pooled")
    assert_close(net.download_tensor(3, mb.TENSOR["OUTPUTS"], B * 4), y.detach().numpy().ravel(), rel=1e-5, abs_=1e-6, what="outputs")
    assert_close(net.download_gradient(), W.grad.numpy(), rel=2e-4, abs_=2e-6, what="gradient")


def test_average_pooling_with_dilation_follows_the_reference_window():
    """the width formula ignores the dilation while the window uses it: positions past the input count as zero"""
    specs = [dict(units=6), dict(units=8, activation="LINEAR"), dict(type="average_pooling", kernel=2, stride=2, dilation=3), dict(units=2, activation="LINEAR")]
    desc = oracle_desc(specs, 1)
    assert desc.layers[2].n_units == 4
    net = OracleNetwork(desc, oracle_hyper())
    w = np.zeros(desc.total_parameters, dtype=np.float32)
    l1 = desc.layers[1]
    w[l1.first_connection_index:l1.last_connection_index].reshape(8, 6)[np.arange(6), np.arange(6)] = 1     # h[0..5] = x, h[6..7] = 0
    w[desc.total_weights + 6] = 7.0; w[desc.total_weights + 7] = 9.0                                          # h[6] = 7, h[7] = 9
    net.upload_parameters(w)
    net.Forward_Pass(1, np.arange(1, 7, dtype=np.float32).reshape(1, 6))
    h = np.array([1, 2, 3, 4, 5, 6, 7, 9], dtype=np.float64)
    want = [(h[0] + h[3]) / 2, (h[2] + h[5]) / 2, (h[4] + h[7]) / 2, (h[6] + 0) / 2]                          # 6 + 3 = 9 is past the input
    assert_close(net.download_tensor(2, mb.TENSOR["OUTPUTS"], 4), np.array(want), rel=1e-6)


def test_pooling_layers_are_refused_where_this_path_has_none():
    with pytest.raises(ValueError):    # as the output layer
        oracle_desc([dict(units=6), dict(units=8, activation="TANH"), dict(type="max_pooling", kernel=2, stride=2)], 2)
    with pytest.raises(ValueError):    # window larger than the padded input
        oracle_desc([dict(units=6), dict(units=3, activation="TANH"), dict(type="average_pooling", kernel=9, stride=1), dict(units=2, activation="LINEAR")], 2)
