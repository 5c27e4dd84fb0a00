"""Pins the oracle's independently recurrent layer, h[t] = AF(W x[t] + b + u * h[t-1]): forward, back-propagation through
time and the self-weight gradient against float64 autograd of an independent model; the connection layout against
Prepare__Connections__FC_Ind_RNN; the clip of the self weights after an update.  CPU only."""
import numpy as np
import pytest
import torch

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, oracle_desc, oracle_hyper
from tests.oracle_lib import OracleNetwork

ACT = {"TANH": torch.tanh, "SIGMOID": torch.sigmoid, "RELU": torch.relu, "LINEAR": lambda v: v}


def _with_self_weights(desc, w, seed, lo=-0.9, hi=0.9):
    """self weights large enough for the recurrent term to matter"""
    rng = np.random.default_rng(seed)
    for i in range(1, desc.n_layers):
        l = desc.layers[i]
        if l.type_layer == mb.LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT:
            w[l.last_connection_index - l.n_units:l.last_connection_index] = rng.uniform(lo, hi, l.n_units).astype(np.float32)
    return w


def _float64_model(desc, specs, w, X, masks, B, T, training=True):
    """forward of the stack in float64 torch, time-major; returns (outputs [B][T][Out], parameter tensor)"""
    W = torch.tensor(w.astype(np.float64), requires_grad=True)
    widths = [s["units"] for s in specs]
    x = torch.tensor(X.astype(np.float64)).reshape(B, T, widths[0])
    seq = [x[:, t, :] for t in range(T)]
    bias_at = desc.total_weights
    norm_at = desc.total_weights + desc.total_bias
    for i in range(1, len(specs)):
        s, l = specs[i], desc.layers[i]
        In, H = widths[i - 1], widths[i]
        Wm = W[l.first_connection_index:l.first_connection_index + H * In].reshape(H, In)
        normed = s.get("normalization", "NONE") != "NONE"
        before = s.get("norm_before", True)
        b = None
        if not normed:
            b = W[l.first_bias_connection_index:l.first_bias_connection_index + H]
        scale = shift = None
        if normed:
            at = norm_at + l.first_normalized_unit_index
            scale, shift = W[at:at + H], W[at + desc.total_normalized_units:at + desc.total_normalized_units + H]
        u = W[l.first_connection_index + H * In:l.first_connection_index + H * In + H] if s.get("type") == "ind_rnn" else None
        act = ACT[s.get("activation", "SIGMOID")]
        keep = s.get("keep", 1.0)
        m = None
        if s.get("dropout", "NONE") != "NONE":
            m = torch.tensor(masks[l.first_mask_index:l.first_mask_index + T * H].astype(np.float64)).reshape(T, H)
            if s["dropout"] == "BERNOULLI_INVERTED":
                m = m / keep

        def bn(v):
            mean = v.mean(0)
            var = ((v - mean) ** 2).mean(0)
            return scale * (v - mean) / torch.sqrt(var + 1e-5) + shift

        out, h = [], None
        for t in range(T):
            v = seq[t] @ Wm.T
            if b is not None:
                v = v + b
            if normed and before:
                v = bn(v)
            if u is not None and t > 0:
                v = v + u * h
            a = act(v)
            y = a
            if normed and not before:
                y = bn(a)
            if m is not None:
                y = y * m[t]
            h = y if not (normed and not before) else a      # the recurrence reads the activation array as the step left it
            out.append(y)
        seq = out
    return torch.stack(seq, 1), W


def _run_oracle(specs, B, T, seed, hyper=None, masks=None):
    desc = oracle_desc(specs, B, T)
    net = OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS["MSE"], **(hyper or {})))
    w = _with_self_weights(desc, glorot_parameters(desc, seed, bias_range=0.3), seed)
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(w)
    if masks is None:
        masks = np.ones(desc.total_mask_units, dtype=np.uint8)
    net.upload_masks(masks)
    net.Clear_Training_Arrays()
    rng = np.random.default_rng(seed + 100)
    X = rng.normal(0, 1, (B, T * specs[0]["units"])).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * specs[-1]["units"])).astype(np.float32)
    net.Forward_Pass(B, X); net.Compute__Error(B, Y); net.Backward_Pass(B); net.Update_Derivative_Weight(B)
    return desc, net, w, X, Y, masks


def test_layout_follows_prepare_connections():
    specs = [dict(units=5), dict(type="ind_rnn", units=7, activation="RELU"), dict(units=3, activation="LINEAR")]
    d = oracle_desc(specs, 4, 6)
    l = d.layers[1]
    assert l.type_layer == 5
    assert l.first_connection_index == 0 and l.last_connection_index == 7 * 5 + 7      # matrix, then one self weight per unit
    assert d.layers[2].first_connection_index == 42 and d.total_weights == 42 + 21
    assert l.first_bias_connection_index == d.total_weights and d.total_bias == 10
    assert d.total_mask_units == 6 * (5 + 7 + 3)
    # Compute__Regularization__Constraint_Recurrent_Weight__Default: MAG = clip(clip_gradient = 1, 2, 10) = 2
    assert l.constraint_recurrent_weight_upper_bound == pytest.approx(2.0 ** (1.0 / 6.0), rel=1e-6)
    assert l.constraint_recurrent_weight_lower_bound == pytest.approx(-2.0 ** (1.0 / 6.0), rel=1e-6)
    sym = oracle_desc([dict(units=5), dict(type="ind_rnn", units=7, activation="TANH"), dict(units=3, activation="LINEAR")], 4, 6).layers[1]
    assert sym.constraint_recurrent_weight_upper_bound == pytest.approx((2.0 / 0.9 ** 0.6) ** (1.0 / 6.0), rel=1e-6)
    # not as the first or the last layer
    with pytest.raises(ValueError):
        oracle_desc([dict(units=5), dict(type="ind_rnn", units=3, activation="TANH")], 4, 6)


@pytest.mark.parametrize("name,specs", [
    ("tanh", [dict(units=6), dict(type="ind_rnn", units=9, activation="TANH"), dict(units=4, activation="LINEAR")]),
    ("relu-stacked", [dict(units=6), dict(type="ind_rnn", units=9, activation="RELU"), dict(type="ind_rnn", units=8, activation="SIGMOID"), dict(units=4, activation="TANH")]),
    ("bn-before", [dict(units=6), dict(type="ind_rnn", units=9, activation="TANH", normalization="BATCH_NORMALIZATION", norm_before=True), dict(units=4, activation="LINEAR")]),
    ("bn-after", [dict(units=6), dict(type="ind_rnn", units=9, activation="TANH", normalization="BATCH_NORMALIZATION", norm_before=False), dict(units=4, activation="LINEAR")]),
    ("fc-below", [dict(units=6), dict(units=7, activation="TANH"), dict(type="ind_rnn", units=9, activation="TANH"), dict(units=5, activation="LINEAR")]),
])
def test_forward_and_bptt_against_float64_autograd(name, specs):
    B, T = 5, 6
    desc, net, w, X, Y, masks = _run_oracle(specs, B, T, seed=3)
    y, W = _float64_model(desc, specs, w, X, masks, B, T)
    loss = 0.5 * ((y - torch.tensor(Y.astype(np.float64)).reshape(y.shape)) ** 2).sum()
    loss.backward()     # delta = AF'(y) (y - d) at the outputs: the gradient of 0.5 sum (y - d)^2
    out = net.download_tensor(desc.n_layers - 1, mb.TENSOR["OUTPUTS"], T * B * specs[-1]["units"]).reshape(T, B, -1)
    assert_close(out.transpose(1, 0, 2).ravel(), y.detach().numpy().ravel(), rel=1e-5, abs_=2e-6, what="outputs")
    g, want = net.download_gradient(), W.grad.numpy()
    assert_close(g, want, rel=3e-4, abs_=2e-6 * float(np.abs(want).max()), what="gradient")   # entries that cancel: absolute, at the scale of the vector
    li = next(i for i, s in enumerate(specs) if s.get("type") == "ind_rnn")
    l, H = desc.layers[li], specs[li]["units"]
    du = want[l.last_connection_index - H:l.last_connection_index]
    assert np.abs(du).min() > 1e-4        # the self-weight gradient is exercised, not vacuous


def test_in_place_dropout_feeds_the_recurrence():
    """without a normalisation behind the activation the Bernoulli mask works in place on the activations, so the next
    time step's recurrent term reads the masked value"""
    B, T = 4, 5
    specs = [dict(units=6), dict(type="ind_rnn", units=8, activation="TANH", dropout="BERNOULLI_INVERTED", keep=0.6), dict(units=3, activation="LINEAR")]
    d0 = oracle_desc(specs, B, T)
    masks = (np.random.default_rng(5).uniform(0, 1, d0.total_mask_units) < 0.6).astype(np.uint8)
    desc, net, w, X, Y, masks = _run_oracle(specs, B, T, seed=7, masks=masks)
    y, W = _float64_model(desc, specs, w, X, masks, B, T)
    out = net.download_tensor(2, mb.TENSOR["OUTPUTS"], T * B * 3).reshape(T, B, -1)
    assert_close(out.transpose(1, 0, 2).ravel(), y.detach().numpy().ravel(), rel=1e-5, abs_=2e-6, what="outputs")


def test_self_weights_are_clipped_after_the_update():
    B, T = 4, 5
    specs = [dict(units=6), dict(type="ind_rnn", units=8, activation="RELU", recurrent_bounds=(-0.25, 0.5)), dict(units=3, activation="LINEAR")]
    desc, net, w, X, Y, _ = _run_oracle(specs, B, T, seed=9, hyper=dict(type_optimizer_function=mb.OPTIMIZER["GD"], learning_rate=1e-3))
    before = net.download_parameters().copy()
    net.Update_Parameter(B, B)
    after = net.download_parameters()
    l = desc.layers[1]
    u0, u1 = before[l.last_connection_index - 8:l.last_connection_index], after[l.last_connection_index - 8:l.last_connection_index]
    assert (np.abs(u0) > 0.5).any()                                   # some start outside the bounds
    assert u1.min() >= -0.25 and u1.max() <= 0.5
    inside = (u0 > -0.2) & (u0 < 0.45)
    assert inside.any() and np.all(u1[inside] != u0[inside])          # the others moved by the plain step
    # no bounds, no clip
    specs[1]["recurrent_bounds"] = (0.0, 0.0)
    desc, net, w, X, Y, _ = _run_oracle(specs, B, T, seed=9, hyper=dict(type_optimizer_function=mb.OPTIMIZER["GD"], learning_rate=1e-3))
    net.Update_Parameter(B, B)
    u2 = net.download_parameters()[l.last_connection_index - 8:l.last_connection_index]
    assert (np.abs(u2) > 0.5).any()
