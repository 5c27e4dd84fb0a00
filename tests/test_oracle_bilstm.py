"""Pins the oracle's two-direction LSTM layer.  The reference's own bidirectional path overlays the two directions'
buffers and takes the sub-layers' bias indices before they are assigned, so it has no behaviour to match; the contract
here is: each direction is the reference's one-direction recurrence over its own blocks (second half of the layer's
blocks walks time backwards), the layer outputs the SUM of both cell outputs, both directions receive the same delta.
Each direction is pinned against the already pinned one-direction path, the combination against float64 autograd."""
import types

import numpy as np
import pytest
import torch

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, oracle_desc, oracle_hyper, run_step
from tests.oracle_lib import OracleNetwork
from tests.test_oracle_lstm import T64, lstm_forward, lstm_views


def _geom(l, In):
    K, cpb = l.n_units, l.n_cells_per_block
    C = K * cpb
    per_block = cpb * (In + C) + 3 * In + 3 * C + 3 * cpb
    return K, C, per_block, C + 3 * K


def _dir_layer(l, In, direction):
    """the descriptor entry as one direction sees it: its first block and its bias vectors"""
    K, C, per_block, G = _geom(l, In)
    return types.SimpleNamespace(n_units=l.n_units, n_cells_per_block=l.n_cells_per_block,
                                 first_connection_index=l.first_connection_index + direction * K * per_block,
                                 first_bias_connection_index=l.first_bias_connection_index + direction * G)


def _run(specs, B, T, w, X, Y, loss="MSE"):
    desc = oracle_desc(specs, B, T)
    net = OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS[loss]))
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(w)
    run_step(net, B, X, Y, update=False)
    return desc, net


BI = [dict(units=5), dict(type="lstm", units=4, cells_per_block=2, bidirectional=True), dict(units=9, activation="LINEAR")]
UNI = [dict(units=5), dict(type="lstm", units=4, cells_per_block=2), dict(units=9, activation="LINEAR")]
B, T = 3, 5


def _split(desc_bi, desc_uni):
    """index ranges: direction 0 / 1 weights and biases in the two-direction net, the one-direction net's, the heads'"""
    lb, lu = desc_bi.layers[1], desc_uni.layers[1]
    K, C, per_block, G = _geom(lu, 5)
    wn = K * per_block
    return dict(w0=slice(lb.first_connection_index, lb.first_connection_index + wn), w1=slice(lb.first_connection_index + wn, lb.first_connection_index + 2 * wn),
                b0=slice(lb.first_bias_connection_index, lb.first_bias_connection_index + G), b1=slice(lb.first_bias_connection_index + G, lb.first_bias_connection_index + 2 * G),
                wu=slice(lu.first_connection_index, lu.first_connection_index + wn), bu=slice(lu.first_bias_connection_index, lu.first_bias_connection_index + G))


def test_layout_of_a_two_direction_layer():
    d = oracle_desc(BI, B, T)
    K, C, per_block, G = _geom(d.layers[1], 5)
    assert d.layers[1].last_connection_index - d.layers[1].first_connection_index == 2 * K * per_block
    assert d.layers[1].first_bias_connection_index == d.total_weights          # the slice's start: no shift by the cell count
    assert d.layers[2].first_bias_connection_index == d.total_weights + 2 * G
    assert d.total_bias == 2 * G + 9


@pytest.mark.parametrize("direction", [0, 1])
def test_one_live_direction_is_the_one_direction_layer(direction):
    """All parameters of the other direction zero: its cell outputs are exactly 0 (z = tanh 0, c = i z), so the layer is
    the one-direction layer - on the time-reversed sequence when the live direction is the second one.  Outputs, the
    delta handed to the layer, every gradient of the live direction and of the head are those of the one-direction net."""
    d_bi, d_uni = oracle_desc(BI, B, T), oracle_desc(UNI, B, T)
    ix = _split(d_bi, d_uni)
    wu = glorot_parameters(d_uni, 7, bias_range=0.3)
    # the one-direction layer's bias index quirk shifts its vectors C entries into the head's biases; keep the head's biases
    # zero so that both nets have the same head
    hu, hb = d_uni.layers[2], d_bi.layers[2]
    wu[hu.first_bias_connection_index:hu.first_bias_connection_index + 9] = 0
    K, C, per_block, G = _geom(d_uni.layers[1], 5)
    wb = np.zeros(d_bi.total_parameters, dtype=np.float32)
    wb[ix["w1" if direction else "w0"]] = wu[ix["wu"]]
    wb[ix["b1" if direction else "b0"]] = wu[ix["bu"]]
    wb[hb.first_connection_index:hb.last_connection_index] = wu[hu.first_connection_index:hu.last_connection_index]
    rng = np.random.default_rng(8)
    X = rng.normal(0, 1, (B, T, 5)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T, 9)).astype(np.float32)
    Xu, Yu = (X[:, ::-1], Y[:, ::-1]) if direction else (X, Y)
    _, nb = _run(BI, B, T, wb, X.reshape(B, -1), Y.reshape(B, -1))
    _, nu = _run(UNI, B, T, wu, np.ascontiguousarray(Xu).reshape(B, -1), np.ascontiguousarray(Yu).reshape(B, -1))
    hb_out = nb.download_tensor(1, mb.TENSOR["OUTPUTS"]).reshape(T, B, C)
    hu_out = nu.download_tensor(1, mb.TENSOR["OUTPUTS"]).reshape(T, B, C)
    assert np.array_equal(hb_out, hu_out[::-1] if direction else hu_out)
    dead = nb.download_tensor(1, mb.TENSOR["LSTM_CELL_OUTPUT"] | (0 if direction else mb.TENSOR["DIRECTION_BACKWARD"]))
    assert np.all(dead == 0)
    gb, gu = nb.download_gradient(), nu.download_gradient()
    assert_close(gb[ix["w1" if direction else "w0"]], gu[ix["wu"]], 1e-6, 1e-7, "live direction weights")
    # head: weights and the 9 biases (the one-direction net's head biases also collect the LSTM's shifted bias gradients:
    # compare the part past the C overrun slots)
    assert_close(gb[hb.first_connection_index:hb.last_connection_index], gu[hu.first_connection_index:hu.last_connection_index], 1e-6, 1e-7, "head weights")
    assert_close(gb[hb.first_bias_connection_index + C:hb.first_bias_connection_index + 9], gu[hu.first_bias_connection_index + C:hu.first_bias_connection_index + 9], 1e-6, 1e-7)
    # LSTM biases: the one-direction vectors start at its (shifted) index
    assert_close(gb[ix["b1" if direction else "b0"]][:G - C], gu[ix["bu"]][:G - C], 1e-6, 1e-7, "live direction biases")


def test_two_directions_match_float64_autograd():
    specs = [dict(units=6), dict(units=7, activation="TANH"), dict(type="lstm", units=3, cells_per_block=2, bidirectional=True),
             dict(type="lstm", units=5, bidirectional=True), dict(units=4, activation="SOFTMAX")]
    Bb, Tt = 4, 6
    desc = oracle_desc(specs, Bb, Tt)
    w = glorot_parameters(desc, 9, bias_range=0.3)
    rng = np.random.default_rng(10)
    X = rng.normal(0, 1, (Bb, Tt, 6)).astype(np.float32)
    labels = rng.integers(0, 4, (Bb, Tt))
    Y = np.zeros((Bb, Tt, 4), dtype=np.float32)
    np.put_along_axis(Y, labels[..., None], 1.0, axis=2)
    _, net = _run(specs, Bb, Tt, w, X.reshape(Bb, -1), Y.reshape(Bb, -1), loss="CROSS_ENTROPY")
    flat = torch.tensor(w.astype(np.float64), dtype=T64, requires_grad=True)
    x = torch.tensor(X.astype(np.float64))
    l1 = desc.layers[1]
    x = torch.tanh(x @ flat[l1.first_connection_index:l1.first_connection_index + 42].view(7, 6).t() + flat[l1.first_bias_connection_index:l1.first_bias_connection_index + 7])
    widths = [6, 7, 6, 5, 4]
    taps = {}
    for li in (2, 3):
        l = desc.layers[li]
        fwd = lstm_forward(lstm_views(flat, _dir_layer(l, widths[li - 1], 0), widths[li - 1]), x)
        bwd = lstm_forward(lstm_views(flat, _dir_layer(l, widths[li - 1], 1), widths[li - 1]), torch.flip(x, dims=[1]))
        x = fwd + torch.flip(bwd, dims=[1])
        x.retain_grad()
        taps[li] = x
    l4 = desc.layers[4]
    y = torch.softmax(x @ flat[l4.first_connection_index:l4.first_connection_index + 20].view(4, 5).t() + flat[l4.first_bias_connection_index:l4.first_bias_connection_index + 4], dim=2)
    (-(torch.tensor(Y.astype(np.float64)) * torch.log(y)).sum()).backward()
    for li in (2, 3):
        got = net.download_tensor(li, mb.TENSOR["OUTPUTS"]).reshape(Tt, Bb, widths[li])
        assert_close(got, taps[li].detach().numpy().transpose(1, 0, 2), 3e-5, 3e-6, "outputs layer %d" % li)
    assert_close(net.download_gradient(), flat.grad.numpy(), 3e-4, 3e-5, "gradient")
    assert np.count_nonzero(flat.grad.numpy()) > 0.8 * desc.total_weights
