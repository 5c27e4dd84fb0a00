"""Pins the oracle's zoneout (Krueger et al. 2016: a zoned-out unit keeps its previous value) on LSTM layers: forward against
a float64 restatement with the same masks, the all-ones mask against the plain layer, inference against the plain layer,
and the mask buffer's layout.  The reference's BACKWARD pass does not read the masks (no zoneout branch exists in
Neural_Network__Recurrent_Backward_Pass__*.cpp) - parity unpinned there: the restated behaviour is fixed by
test_backward_ignores_the_masks_as_written below and shown to differ from the true gradient.  CPU only."""
import numpy as np
import pytest
import torch

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, oracle_desc, oracle_hyper
from tests.oracle_lib import OracleNetwork
from tests.test_oracle_lstm import T64, lstm_views

zone = lambda units, cpb=1, **kw: dict(type="lstm", units=units, cells_per_block=cpb, dropout="ZONEOUT", keep=0.3, keep_output=0.2, **kw)


def lstm_forward_zoneout(v, x, ms, mo):
    """x [B, T, In]; ms / mo [T, C] cell-state / cell-output masks (1 = update)."""
    B, T, _ = x.shape
    K, cpb, C = v["K"], v["cpb"], v["C"]
    h = torch.zeros(B, C, dtype=T64); c = torch.zeros(B, C, dtype=T64)
    per_block = lambda t_: t_.reshape(B, K, cpb).sum(2)
    spread = lambda g: g.repeat_interleave(cpb, dim=1)
    outs = []
    for t in range(T):
        xt = x[:, t]
        i = torch.sigmoid(xt @ v["W_in"][0].t() + h @ v["W_rec"][0].t() + per_block(c * v["peep"][0]) + v["bi"])
        f = torch.sigmoid(xt @ v["W_in"][1].t() + h @ v["W_rec"][1].t() + per_block(c * v["peep"][1]) + v["bf"])
        z = torch.tanh(xt @ v["Wz_in"].t() + h @ v["Wz_rec"].t() + v["bz"])
        c = ms[t] * (z * spread(i) + spread(f) * c) + (1 - ms[t]) * c
        o = torch.sigmoid(xt @ v["W_in"][2].t() + h @ v["W_rec"][2].t() + per_block(c * v["peep"][2]) + v["bo"])
        h = mo[t] * (spread(o) * torch.tanh(c)) + (1 - mo[t]) * h
        outs.append(h)
    return torch.stack(outs, dim=1)


def _net(specs, B, T, seed, state=mb.STATE_TRAINING):
    desc = oracle_desc(specs, B, T)
    net = OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS["MSE"]))
    w = glorot_parameters(desc, seed, bias_range=0.3)
    net.set_state_propagation(state)
    net.upload_parameters(w)
    net.Clear_Training_Arrays()
    return desc, net, w


def _masks(rng, T, cells):
    """[state | output] halves, per LSTM layer [T][cells]"""
    total = sum(cells)
    state = [(rng.uniform(0, 1, (T, c)) < 0.6).astype(np.uint8) for c in cells]
    out = [(rng.uniform(0, 1, (T, c)) < 0.6).astype(np.uint8) for c in cells]
    flat = np.concatenate([m.ravel() for m in state] + [m.ravel() for m in out])
    assert flat.size == 2 * T * total
    return state, out, flat


@pytest.mark.parametrize("cpb", [1, 2])
def test_zoneout_forward_matches_the_published_operator_on_two_stacked_layers(cpb):
    T, B = 6, 4
    specs = [dict(units=5), zone(4, cpb), zone(3, cpb), dict(units=3 * cpb, activation="LINEAR")]
    desc, net, w = _net(specs, B, T, 3)
    rng = np.random.default_rng(3)
    state, out, flat_masks = _masks(rng, T, [4 * cpb, 3 * cpb])
    net.upload_zoneout_masks(flat_masks)
    X = rng.normal(0, 1, (B, T * 5)).astype(np.float32)
    net.Forward_Pass(B, X)
    flat = torch.tensor(w.astype(np.float64))
    x = torch.tensor(X.astype(np.float64)).reshape(B, T, 5)
    h1 = lstm_forward_zoneout(lstm_views(flat, desc.layers[1], 5), x, torch.tensor(state[0], dtype=T64), torch.tensor(out[0], dtype=T64))
    h2 = lstm_forward_zoneout(lstm_views(flat, desc.layers[2], 4 * cpb), h1, torch.tensor(state[1], dtype=T64), torch.tensor(out[1], dtype=T64))
    for li, want in ((1, h1), (2, h2)):
        C_ = want.shape[2]
        got = net.download_tensor(li, mb.TENSOR["OUTPUTS"], T * B * C_).reshape(T, B, C_).transpose(1, 0, 2)
        assert_close(got, want.numpy(), rel=2e-5, abs_=2e-6, what="layer %d" % li)
    # zoned-out outputs really repeat the previous step (and are 0 on the first)
    got = net.download_tensor(1, mb.TENSOR["OUTPUTS"], T * B * 4 * cpb).reshape(T, B, 4 * cpb)
    for t in range(T):
        held = out[0][t] == 0
        assert held.any()
        assert np.array_equal(got[t][:, held], got[t - 1][:, held] if t else np.zeros_like(got[t][:, held]))


def test_all_ones_masks_and_the_inference_state_are_the_plain_layer():
    T, B = 5, 3
    plain = [dict(units=4), dict(type="lstm", units=6), dict(units=6, activation="LINEAR")]
    zoned = [dict(units=4), zone(6), dict(units=6, activation="LINEAR")]
    rng = np.random.default_rng(4)
    X = rng.normal(0, 1, (B, T * 4)).astype(np.float32)
    _, ref, _ = _net(plain, B, T, 4)
    ref.Forward_Pass(B, X)
    want = ref.download_tensor(2, mb.TENSOR["OUTPUTS"], T * B * 6)
    desc, net, _ = _net(zoned, B, T, 4)
    net.Forward_Pass(B, X)                                                   # masks are all ones after create
    assert np.array_equal(net.download_tensor(2, mb.TENSOR["OUTPUTS"], T * B * 6), want)
    net.upload_zoneout_masks(np.zeros(2 * T * 6, dtype=np.uint8))
    net.Forward_Pass(B, X)
    assert np.all(net.download_tensor(1, mb.TENSOR["OUTPUTS"], T * B * 6) == 0)    # everything zoned out: the state never leaves 0
    net.set_state_propagation(mb.STATE_INFERENCE)                            # the masks act in the training state only
    net.Forward_Pass(B, X)
    assert np.array_equal(net.download_tensor(2, mb.TENSOR["OUTPUTS"], T * B * 6), want)


def test_backward_ignores_the_masks_as_written():
    """same stored gates and states -> same deltas formulas: with masks the result is NOT the gradient of the zoned forward"""
    T, B = 4, 3
    specs = [dict(units=4), zone(5), dict(units=5, activation="LINEAR")]
    desc, net, w = _net(specs, B, T, 6)
    rng = np.random.default_rng(6)
    state, out, flat_masks = _masks(rng, T, [5])
    net.upload_zoneout_masks(flat_masks)
    X, Y = rng.normal(0, 1, (B, T * 4)).astype(np.float32), rng.normal(0, 1, (B, T * 5)).astype(np.float32)
    net.Forward_Pass(B, X); net.Compute__Error(B, Y); net.Backward_Pass(B); net.Update_Derivative_Weight(B)
    g = net.download_gradient().astype(np.float64)
    flat = torch.tensor(w.astype(np.float64), requires_grad=True)
    h = lstm_forward_zoneout(lstm_views(flat, desc.layers[1], 4), torch.tensor(X.astype(np.float64)).reshape(B, T, 4),
                             torch.tensor(state[0], dtype=T64), torch.tensor(out[0], dtype=T64))
    l2 = desc.layers[2]
    W2 = flat[l2.first_connection_index:l2.last_connection_index].reshape(5, 5)
    y = h @ W2.t() + flat[l2.first_bias_connection_index:l2.first_bias_connection_index + 5]
    (0.5 * ((y - torch.tensor(Y.astype(np.float64)).reshape(B, T, 5)) ** 2).sum()).backward()
    true = flat.grad.numpy()
    head = slice(l2.first_connection_index, l2.last_connection_index)
    assert_close(g[head], true[head], rel=1e-4, abs_=1e-6)                    # the head's gradient only needs the forward values
    lstm = slice(desc.layers[1].first_connection_index, desc.layers[1].last_connection_index)
    assert np.abs(g[lstm] - true[lstm]).max() > 1e-3                          # the LSTM's is the unmasked recursion, not the gradient
