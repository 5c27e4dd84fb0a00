"""Randomly drawn networks, seeded: the HIP path (through the C ABI) against the CPU oracle on stacks no hand-written case lists -
dense layers with and without dropout, pooling layers, residual blocks with dense and pooling members, at a recurrent depth of
one or several, with batches that do not fill the network's rows; and recurrent stacks of LSTM (one or two directions,
zoneout), independently recurrent, dense and pooling layers and residual blocks whose members are of all four kinds.  Every layer's outputs and deltas, the loss and the gradient of two steps
(the second accumulates onto the first), then a gradient-descent update.  Tolerance rel 1e-4 / abs 1e-5 (of the gradient's
largest magnitude for the sums over the batch and time).  Normalisation is left to the hand-written cases: over a handful of
examples its backward pass amplifies fp32 rounding beyond what a fixed tolerance can separate from an error."""
import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, one_hot
from tests.oracle_lib import OracleNetwork

pytestmark = pytest.mark.gpu

REL, ABS = 1e-4, 1e-5
SMOOTH = ["TANH", "SIGMOID", "ELLIOT_SYMMETRIC", "SINE_SYMMETRIC", "GAUSSIAN", "ISRU"]
KINKED = ["RELU", "LEAKY_RELU", "LINEAR"]


def _dense(rng, units, allow_dropout=True):
    spec = dict(units=int(units), activation=str(rng.choice(SMOOTH + KINKED)))
    if allow_dropout and rng.random() < 0.3:
        spec.update(dropout=str(rng.choice(["BERNOULLI", "BERNOULLI_INVERTED"])), keep=float(rng.choice([0.5, 0.7])))
    return spec


def _pool(rng, width):
    """a pooling layer that fits a `width` wide input, and the width it leaves"""
    kind = str(rng.choice(["average_pooling", "max_pooling"]))
    kernel, stride, padding = int(rng.integers(2, 4)), int(rng.integers(1, 3)), int(rng.integers(0, 2))
    dilation = int(rng.integers(1, 3)) if kind == "max_pooling" else 1
    span = width + 2 * padding - (kernel if kind == "average_pooling" else dilation * (kernel - 1) + 1)
    if span < 0:
        return None, width
    return dict(type=kind, kernel=kernel, stride=stride, padding=padding, dilation=dilation), span // stride + 1


def _feed_forward_specs(rng):
    width = int(rng.integers(5, 40))
    specs = [dict(units=width)]
    for _ in range(int(rng.integers(2, 5))):
        what = rng.random()
        if what < 0.35 and specs[-1].get("type", "fc") == "fc":            # a residual block of dense and pooling members
            depth = int(rng.integers(1, 4))
            members, w = [], width
            for k in range(depth):
                if rng.random() < 0.3:
                    p, w2 = _pool(rng, w)
                    if p is not None and w2 >= 2:
                        members.append(p)
                        w = w2
                        continue
                w = int(rng.integers(4, 40))
                m = _dense(rng, w, allow_dropout=k > 0)   # the first member has no activation unit to drop
                if m["activation"] == "SOFTMAX":
                    m["activation"] = "TANH"
                members.append(m)
            specs += [dict(type="residual", block_depth=depth)] + members
            width = max(width, w)
        elif what < 0.5 and specs[-1].get("type", "fc") in ("fc",) and len(specs) > 1:
            p, w2 = _pool(rng, width)
            if p is not None and w2 >= 2:
                specs.append(p)
                width = w2
                continue
            width = int(rng.integers(4, 40))
            specs.append(_dense(rng, width))
        else:
            width = int(rng.integers(4, 40))
            specs.append(_dense(rng, width))
    if specs[-1].get("type", "fc") != "fc" or rng.random() < 2:      # a consumer behind whatever came last
        softmax = rng.random() < 0.5
        specs.append(dict(units=int(rng.integers(2, 9)), activation="SOFTMAX" if softmax else str(rng.choice(["LINEAR", "TANH"]))))
    return specs


def _lstm(rng):
    spec = dict(type="lstm", units=int(rng.choice([8, 12, 32, 64, 128])), bidirectional=bool(rng.random() < 0.3))
    if rng.random() < 0.3:
        spec.update(dropout="ZONEOUT", keep=float(rng.choice([0.3, 0.6])), keep_output=float(rng.choice([0.2, 0.5])))
    return spec


def _outputs(spec):
    return spec["units"] * (2 if spec.get("bidirectional") else 1)


def _recurrent_specs(rng):
    """LSTM, independently recurrent and dense layers; pooling layers and residual blocks between them, the blocks' members
    drawn from all four kinds (an independently recurrent member behind another member is as wide as its input)"""
    width = int(rng.integers(3, 20))
    specs = [dict(units=width)]
    for _ in range(int(rng.integers(1, 4))):
        what = rng.random()
        if len(specs) == 1:
            what *= 0.7            # a layer with weights comes first
        if what < 0.4:
            specs.append(_lstm(rng))
            width = _outputs(specs[-1])
        elif what < 0.55:
            width = int(rng.integers(4, 30))
            specs.append(dict(type="ind_rnn", units=width, activation=str(rng.choice(["RELU", "TANH"]))))
        elif what < 0.7:
            width = int(rng.integers(4, 30))
            specs.append(_dense(rng, width))
        elif what < 0.8 and len(specs) > 1 and "pooling" not in specs[-1].get("type", ""):
            p, w2 = _pool(rng, width)
            if p is None or w2 < 2:
                p, w2 = dict(type="average_pooling", kernel=2, stride=1), width - 1
            specs.append(p)
            width = w2
        else:
            depth = int(rng.integers(1, 4))
            members, w = [], width
            for k in range(depth):
                kind = rng.random()
                if kind < 0.25:
                    members.append(_lstm(rng))
                    w = _outputs(members[-1])
                elif kind < 0.5:
                    if k > 0:                       # as wide as its input; the first member's width is free
                        members.append(dict(type="ind_rnn", units=w, activation=str(rng.choice(["SIGMOID", "TANH"]))))
                    else:
                        w = int(rng.integers(4, 30))
                        members.append(dict(type="ind_rnn", units=w, activation="TANH"))
                elif kind < 0.65:
                    p, w2 = _pool(rng, w)
                    if p is None or w2 < 2:
                        w = int(rng.integers(4, 30))
                        members.append(_dense(rng, w, allow_dropout=k > 0))
                    else:
                        members.append(p)
                        w = w2
                else:
                    w = int(rng.integers(4, 30))
                    members.append(_dense(rng, w, allow_dropout=k > 0))
            specs += [dict(type="residual", block_depth=depth)] + members
            width = max(width, w)
    specs.append(dict(units=int(rng.integers(2, 9)), activation=str(rng.choice(["LINEAR", "TANH"]))))
    return specs


def _room_for_lstm_bias(specs, Bmax, T):
    """An LSTM layer's four bias vectors start where Prepare__Bias__LSTM leaves the index - its cells past the layer's own
    slots - and reach into the slots of the layers behind it; past the end of the bias region the reference itself would be
    outside its parameter array.  The head is widened until every LSTM layer of the draw has that room."""
    while True:
        desc = mb.make_desc(specs, Bmax, T)
        end = desc.total_weights + desc.total_bias
        short = 0
        for i in range(desc.n_layers):
            l = desc.layers[i]
            if l.type_layer == mb.LAYER_LSTM:
                gates = l.n_units * l.n_cells_per_block + 3 * l.n_units
                short = max(short, l.first_bias_connection_index + (2 if l.use_bidirectional else 1) * gates - end)
        if short <= 0:
            return specs
        specs = specs[:-1] + [dict(specs[-1], units=specs[-1]["units"] + int(short))]


def _width(desc, lib, li):
    return int(lib.myea_net_desc_number_outputs(desc, li))


def _run(specs, T, Bmax, B, seed, loss):
    lib = mb.load_library()
    try:
        desc = mb.make_desc(specs, Bmax, T)
        h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["GD"], type_loss_function=mb.LOSS[loss], learning_momentum=0.9)
        gpu = mb.HipNetwork(desc, h)
    except (ValueError, mb.MyeaError) as e:   # the generators draw only what the path takes: a refusal is a failure
        raise AssertionError("refused: %s: %r" % (e, specs))
    cpu = OracleNetwork(desc, h)
    w = glorot_parameters(desc, seed, bias_range=0.3)
    rng = np.random.default_rng(seed + 1000)
    masks = (rng.uniform(0, 1, max(1, desc.total_mask_units)) < 0.6).astype(np.uint8)[:desc.total_mask_units]
    zone = None
    cells = sum(_width(desc, lib, i) * (2 if desc.layers[i].use_bidirectional else 1) for i in range(desc.n_layers) if desc.layers[i].type_layer == mb.LAYER_LSTM)
    if any(s.get("dropout") == "ZONEOUT" for s in specs):
        zone = (rng.uniform(0, 1, 2 * T * cells) < 0.6).astype(np.uint8)
    n_in, n_out = specs[0]["units"], specs[-1]["units"]
    X = rng.normal(0, 1, (B, T * n_in)).astype(np.float32)
    Y = one_hot(rng.integers(0, n_out, B * T), n_out).reshape(B, T * n_out) if loss == "CROSS_ENTROPY" else rng.normal(0, 1, (B, T * n_out)).astype(np.float32)
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        if desc.total_mask_units:
            n.upload_masks(masks)
        if zone is not None:
            n.upload_zoneout_masks(zone)
        n.Clear_Training_Arrays()
    what = "seed %d %r T=%d B=%d/%d" % (seed, [s.get("type", "fc") + str(s.get("units", "")) for s in specs], T, B, Bmax)
    for step in range(2):
        for n in (gpu, cpu):
            n.Reset__Loss()
            n.Forward_Pass(B, X)
            n.Compute__Error(B, Y)
            if n is gpu and step == 1:
                n.Backward_Pass__Update_Derivative_Weight(B)      # the combined call on the second step
            else:
                n.Backward_Pass(B)
                n.Update_Derivative_Weight(B)
        for li in range(1, desc.n_layers):
            W = _width(desc, lib, li)
            for kind in ("OUTPUTS", "ERRORS"):
                a = np.asarray(gpu.download_tensor(li, mb.TENSOR[kind], T * Bmax * W)).reshape(T, Bmax, W)[:, :B]
                b = np.asarray(cpu.download_tensor(li, mb.TENSOR[kind], T * Bmax * W)).reshape(T, Bmax, W)[:, :B]
                assert_close(a, b, REL, ABS * max(1.0, float(np.abs(b).max())), what="%s: step %d layer %d %s" % (what, step, li, kind))
        g = cpu.download_gradient()
        assert_close(gpu.download_gradient(), g, REL, ABS * max(1.0, float(np.abs(g).max())), what="%s: gradient, step %d" % (what, step))
        assert gpu.get_loss().loss_values == pytest.approx(cpu.get_loss().loss_values, rel=1e-4, abs=1e-6)
    for n in (gpu, cpu):
        n.Update_Parameter(B, 3 * B)
    p = cpu.download_parameters()
    assert_close(gpu.download_parameters(), p, REL, 2 * ABS * max(1.0, float(np.abs(p).max())), what=what + ": parameters")
    gpu.close()


@pytest.mark.parametrize("seed", range(48))
def test_random_feed_forward_stack(seed):
    rng = np.random.default_rng(5000 + seed)
    specs = _feed_forward_specs(rng)
    T = int(rng.choice([1, 1, 3]))
    Bmax = int(rng.integers(3, 40))
    B = int(rng.integers(1, Bmax + 1))
    _run(specs, T, Bmax, B, seed, "CROSS_ENTROPY" if specs[-1]["activation"] == "SOFTMAX" else "MSE")


@pytest.mark.parametrize("seed", range(48))
def test_random_recurrent_stack(seed):
    rng = np.random.default_rng(7000 + seed)
    T = int(rng.integers(2, 7))
    Bmax = int(rng.integers(2, 40))
    specs = _room_for_lstm_bias(_recurrent_specs(rng), Bmax, T)
    B = int(rng.integers(1, Bmax + 1))
    _run(specs, T, Bmax, B, 100 + seed, "MSE")
