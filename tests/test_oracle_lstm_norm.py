"""Pins the oracle's normalised LSTM path (one cell per block) on the CPU.  A float64 model of the forward pass, written from
the layer's definition (nine normalisations per time step: the eight gate sums and the cell state, each with its own batch
statistics per step), is differentiated by autograd.  What calculus fixes must agree: outputs, the deltas handed down, the
input and recurrent weights, the biases and the nine scale vectors.  What is the reference's own is checked against
quantities autograd provides: the peephole gradients are built from the deltas of the gate SUMS (after the normalisation's
backward pass) where calculus uses the gates' own deltas, and the shift vectors get no gradient at all."""
import numpy as np
import pytest
import torch

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, oracle_desc, oracle_hyper, run_step
from tests.oracle_lib import OracleError, OracleNetwork
from tests.test_oracle_lstm import T64, _widths, lstm_views

EPS = 1e-5   # normalization_epsilon of the hyper-parameters used here
GROUPS = ["z_in", "z_rec", "c", "i_in", "i_rec", "f_in", "f_rec", "o_in", "o_rec"]


def norm_views(flat, desc, l, direction=0):
    """scale / shift vectors of the nine groups: per direction [3 groups of C | 6 groups of K] in group order, scales first,
    shifts total_normalized_units further on"""
    K = l.n_units
    C = K * l.n_cells_per_block
    at = desc.total_weights + desc.total_bias + l.first_normalized_unit_index + direction * (3 * C + 6 * K)
    out = {}
    for g, name in enumerate(GROUPS):
        H = C if g < 3 else K
        out[name] = (at, H, flat[at:at + H], flat[at + desc.total_normalized_units:at + desc.total_normalized_units + H])
        at += H
    return out


def batch_norm(x, scale, shift):
    mean = x.mean(0)
    sigma = torch.sqrt((x * x).mean(0) - mean * mean + EPS)
    return scale * ((x - mean) / sigma) + shift


def lstm_norm_forward(v, nv, x, reverse=False, zone=None, taps=None):
    """x [B, T, In] -> h [B, T, C]; one cell per block.  zone: (state mask [T, C], output mask [T, C]) with 1 = update.
    taps: dict that receives the eight sums and the cell state per time step (leaves of the graph's interior)."""
    B, T, _ = x.shape
    C = v["C"]
    h = torch.zeros(B, C, dtype=T64)
    c = torch.zeros(B, C, dtype=T64)
    outs = [None] * T
    order = range(T - 1, -1, -1) if reverse else range(T)
    W = dict(z=(v["Wz_in"], v["Wz_rec"], v["bz"]), i=(v["W_in"][0], v["W_rec"][0], v["bi"]), f=(v["W_in"][1], v["W_rec"][1], v["bf"]),
             o=(v["W_in"][2], v["W_rec"][2], v["bo"]))
    for step, t in enumerate(order):
        first = step == 0
        xt = x[:, t]
        s = {}
        for g in "zifo":
            s[g + "_in"] = xt @ W[g][0].t()
            if not first:
                s[g + "_rec"] = h @ W[g][1].t()
        for name, val in s.items():
            val.retain_grad()
            if taps is not None:
                taps[(name, t)] = val

        def gate(g, peep_on):
            a = batch_norm(s[g + "_in"], *nv[g + "_in"][2:]) + W[g][2]
            if not first:
                a = a + batch_norm(s[g + "_rec"], *nv[g + "_rec"][2:])
            return a if peep_on is None else a + peep_on
        i = torch.sigmoid(gate("i", None if first else c * v["peep"][0]))
        z = torch.tanh(gate("z", None))
        if first:
            c_new = z * i
        else:
            f = torch.sigmoid(gate("f", c * v["peep"][1]))
            c_new = z * i + f * c
        if zone is not None:
            m = zone[0][t].to(T64)
            c_new = m * c_new + (1 - m) * c
        c_new.retain_grad()
        if taps is not None:
            taps[("c", t)] = c_new
        ca = torch.tanh(batch_norm(c_new, *nv["c"][2:]))
        o = torch.sigmoid(gate("o", c_new * v["peep"][2]))
        h_new = o * ca
        if zone is not None:
            m = zone[1][t].to(T64)
            h_new = m * h_new + (1 - m) * h
        c, h = c_new, h_new
        outs[t] = h
    return torch.stack(outs, dim=1)


def torch_net(desc, specs, flat_np, X, T, zone=None):
    flat = torch.tensor(np.asarray(flat_np, dtype=np.float64), dtype=T64, requires_grad=True)
    w = _widths(desc)
    B = X.shape[0]
    x = torch.tensor(np.asarray(X, dtype=np.float64), dtype=T64).reshape(B, T, w[0])
    outs, taps = {}, {}
    for i in range(1, desc.n_layers):
        l = desc.layers[i]
        if l.type_layer == mb.LAYER_LSTM:
            taps[i] = {}
            v = lstm_views(flat, l, w[i - 1])
            x = lstm_norm_forward(v, norm_views(flat, desc, l), x, zone=zone, taps=taps[i])
        else:
            W = flat[l.first_connection_index:l.first_connection_index + w[i] * w[i - 1]].view(w[i], w[i - 1])
            s = x @ W.t() + flat[l.first_bias_connection_index:l.first_bias_connection_index + w[i]]
            x = {"LINEAR": lambda q: q, "TANH": torch.tanh, "SIGMOID": torch.sigmoid}[specs[i].get("activation", "SIGMOID")](s)
        x.retain_grad()
        outs[i] = x
    return flat, x, outs, taps


def parameters(desc, seed):
    """weights and biases as for the other LSTM tests; scales around 1 and shifts around 0 so that every one of them matters"""
    w = glorot_parameters(desc, seed, bias_range=0.3)
    rng = np.random.default_rng(seed + 1000)
    base, N = desc.total_weights + desc.total_bias, desc.total_normalized_units
    w[base:base + N] = rng.uniform(0.5, 1.5, N).astype(np.float32)
    w[base + N:base + 2 * N] = rng.uniform(-0.3, 0.3, N).astype(np.float32)
    return w


def lstm(units, **kw):
    return dict(type="lstm", units=units, normalization=kw.pop("normalization", "BATCH_NORMALIZATION"), **kw)


def oracle(specs, B, T, seed, X, Y, Bmax=None, masks=None, **hyper):
    desc = oracle_desc(specs, Bmax or B, T)
    net = OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS["MSE"], type_optimizer_function=mb.OPTIMIZER["AMSGRAD"], **hyper))
    net.set_state_propagation(mb.STATE_TRAINING)
    w = parameters(desc, seed)
    net.upload_parameters(w)
    if masks is not None:
        net.upload_zoneout_masks(masks)
    net.Clear_Training_Arrays()
    run_step(net, B, X, Y, update=False)
    return desc, net, w


CASES = [   # name, layers, T, B, Bmax
    ("one-layer", [dict(units=6), lstm(5), dict(units=7, activation="LINEAR")], 4, 9, 9),
    ("stacked-on-a-dense-layer", [dict(units=5), dict(units=7, activation="TANH"), lstm(4), lstm(6), dict(units=6, activation="LINEAR")], 5, 7, 7),
    ("two-steps", [dict(units=3), lstm(4), dict(units=5, activation="LINEAR")], 2, 6, 6),
    ("batch-smaller-than-the-allocation", [dict(units=4), lstm(5), dict(units=5, activation="LINEAR")], 3, 6, 10),
]


def _peephole_slots(l, In):
    K = l.n_units
    per_block = (In + K) + 3 * In + 3 * K + 3
    return [[l.first_connection_index + k * per_block + per_block - 3 + g for k in range(K)] for g in range(3)]


@pytest.mark.parametrize("name,specs,T,B,Bmax", CASES, ids=[c[0] for c in CASES])
def test_normalised_lstm_against_autograd(name, specs, T, B, Bmax):
    seed = 23
    rng = np.random.default_rng(seed)
    n_in, n_out = specs[0]["units"], specs[-1]["units"]
    X = rng.normal(0, 1, (B, T * n_in)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * n_out)).astype(np.float32)
    desc, net, w = oracle(specs, B, T, seed, X, Y, Bmax=Bmax)
    flat, y, outs, taps = torch_net(desc, specs, w, X, T)
    (0.5 * ((y - torch.tensor(Y.astype(np.float64)).reshape(B, T, n_out)) ** 2).sum()).backward()
    widths = _widths(desc)
    for i in range(1, desc.n_layers):
        got = net.download_tensor(i, mb.TENSOR["OUTPUTS"]).reshape(T, Bmax, widths[i])[:, :B]
        assert_close(got, outs[i].detach().numpy().transpose(1, 0, 2), rel=1e-4, abs_=1e-5, what="outputs layer %d" % i)
    got, want = net.download_gradient().astype(np.float64), flat.grad.numpy().copy()
    N, base = desc.total_normalized_units, desc.total_weights + desc.total_bias
    excluded = np.zeros(desc.total_parameters, dtype=bool)
    excluded[base + N:base + 2 * N] = True   # shifts
    for i in range(1, desc.n_layers):
        l = desc.layers[i]
        if l.type_layer != mb.LAYER_LSTM:
            continue
        slots = _peephole_slots(l, widths[i - 1])
        for g in range(3):
            excluded[slots[g]] = True
        # the reference's peephole gradients: input and forget peepholes from the delta of the gate's RECURRENT sum of the next
        # step, the output peephole from the delta of the output gate's sum FROM BELOW, each times the cell state of the step
        tp = taps[i]
        c = lambda t: tp[("c", t)].detach()
        ref = [sum((tp[(gname + "_rec", t + 1)].grad * c(t)).sum(0) for t in range(T - 1)) for gname in "if"]
        ref.append(sum((tp[("o_in", t)].grad * c(t)).sum(0) for t in range(T)))
        for g in range(3):
            assert_close(got[slots[g]], ref[g].numpy(), rel=5e-4, abs_=5e-5, what="%s: peephole %d of layer %d" % (name, g, i))
        assert not np.allclose(got[slots[2]], want[slots[2]], rtol=1e-2, atol=1e-4), "the output peephole's gradient is not the calculus one"
    assert_close(got[~excluded], want[~excluded], rel=5e-4, abs_=5e-5, what="gradient " + name)
    # shifts: used by the forward pass, never given a gradient (the backward pass the LSTM path calls has no shift term)
    lstm_shift = np.zeros(desc.total_parameters, dtype=bool)
    for i in range(1, desc.n_layers):
        l = desc.layers[i]
        if l.type_layer == mb.LAYER_LSTM:
            for at, H, _, _ in norm_views(flat, desc, l).values():
                lstm_shift[at + N:at + N + H] = True
    assert np.all(got[lstm_shift] == 0.0) and np.count_nonzero(want[lstm_shift]) > 0.5 * lstm_shift.sum()
    assert np.count_nonzero(got[:desc.total_weights]) > 0.8 * desc.total_weights


def test_renormalisation_with_unit_corrections_is_normalisation():
    """r clipped to [1, 1] and d to [0, 0]: batch renormalisation computes what batch normalisation computes, forward and backward"""
    T, B = 4, 8
    rng = np.random.default_rng(5)
    X = rng.normal(0, 1, (B, T * 5)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * 6)).astype(np.float32)
    grads, outs = [], []
    for kind in ("BATCH_NORMALIZATION", "BATCH_RENORMALIZATION"):
        specs = [dict(units=5), lstm(4, normalization=kind), dict(units=6, activation="LINEAR")]
        desc, net, w = oracle(specs, B, T, 11, X, Y, batch_renormalization_r_correction_maximum=1.0, batch_renormalization_d_correction_maximum=0.0)
        grads.append(net.download_gradient())
        outs.append(net.download_tensor(1, mb.TENSOR["OUTPUTS"]))
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(grads[0], grads[1])


def test_renormalisation_corrections_enter_forward_and_backward():
    """with room for the corrections the renormalised layer differs, and its gradient is still the gradient of its forward pass
    with r and d held constant: checked through the scale gradients by finite differences of the loss in float32 would be too
    coarse, so the check is structural - x-hat = (x - mean) / sigma * r + d with the recorded statistics"""
    T, B = 3, 8
    rng = np.random.default_rng(6)
    X = rng.normal(0, 1, (B, T * 5)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * 6)).astype(np.float32)
    specs = [dict(units=5), lstm(4, normalization="BATCH_RENORMALIZATION"), dict(units=6, activation="LINEAR")]
    desc = oracle_desc(specs, B, T)
    net = OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS["MSE"], batch_renormalization_r_correction_maximum=3.0,
                                           batch_renormalization_d_correction_maximum=5.0, normalization_momentum_average=0.5))
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(parameters(desc, 4))
    net.Clear_Training_Arrays()
    for _ in range(2):   # the second pass sees running averages that differ from the batch statistics
        run_step(net, B, X, Y, update=False)
    g = mb.TENSOR_LSTM_NORM_GROUP(2)
    state = net.download_tensor(1, mb.TENSOR["LSTM_CELL_STATE"]).reshape(T, B, 4).astype(np.float64)
    hats = net.download_tensor(1, mb.TENSOR["NORM_HATS"] | g).reshape(T, B, 4)
    mean = net.download_tensor(1, mb.TENSOR["NORM_MEANS"] | g).reshape(T, 1, 4).astype(np.float64)
    sigma = net.download_tensor(1, mb.TENSOR["NORM_VARIANCES"] | g).reshape(T, 1, 4).astype(np.float64)
    mavg = net.download_tensor(1, mb.TENSOR["NORM_MEANS_AVERAGES"] | g).reshape(T, 1, 4).astype(np.float64)
    vavg = net.download_tensor(1, mb.TENSOR["NORM_VARIANCES_AVERAGES"] | g).reshape(T, 1, 4).astype(np.float64)
    assert_close(mean, state.mean(1, keepdims=True), rel=1e-5, abs_=1e-6, what="batch mean of the cell state")
    assert_close(sigma, np.sqrt((state ** 2).mean(1, keepdims=True) - state.mean(1, keepdims=True) ** 2 + EPS), rel=1e-4, abs_=1e-6, what="sigma")
    r = np.clip(sigma / vavg, 1 / 3.0, 3.0)
    d = np.clip((mean - mavg) / vavg, -5.0, 5.0)
    assert np.abs(r - 1).max() > 1e-3 and np.abs(d).max() > 1e-3
    assert_close(hats, (state - mean) / sigma * r + d, rel=1e-4, abs_=1e-5, what="renormalised cell state")


def test_first_step_runs_four_of_the_nine_groups():
    """at the direction's first step only the block input and input gate sums from below, the cell state and the output gate's
    sum from below are normalised: the other groups keep their initial statistics there (averages 0 and 1)"""
    T, B = 3, 6
    rng = np.random.default_rng(8)
    X = rng.normal(0, 1, (B, T * 4)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * 5)).astype(np.float32)
    desc, net, w = oracle([dict(units=4), lstm(5), dict(units=5, activation="LINEAR")], B, T, 2, X, Y)
    for g, name in enumerate(GROUPS):
        mavg = net.download_tensor(1, mb.TENSOR["NORM_MEANS_AVERAGES"] | mb.TENSOR_LSTM_NORM_GROUP(g)).reshape(T, 5)
        vavg = net.download_tensor(1, mb.TENSOR["NORM_VARIANCES_AVERAGES"] | mb.TENSOR_LSTM_NORM_GROUP(g)).reshape(T, 5)
        ran_first = name in ("z_in", "i_in", "c", "o_in")
        assert (np.all(mavg[0] == 0) and np.all(vavg[0] == 1)) != ran_first, name
        assert np.any(mavg[1:] != 0) and np.all(vavg[1:] != 1), name


def test_inference_uses_the_running_averages():
    T, B = 3, 7
    rng = np.random.default_rng(9)
    X = rng.normal(0, 1, (B, T * 4)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * 5)).astype(np.float32)
    specs = [dict(units=4), lstm(5), dict(units=5, activation="LINEAR")]
    desc, net, w = oracle(specs, B, T, 3, X, Y, normalization_momentum_average=0.4)
    avgs = {name: (net.download_tensor(1, mb.TENSOR["NORM_MEANS_AVERAGES"] | mb.TENSOR_LSTM_NORM_GROUP(g)).reshape(T, 5).astype(np.float64),
                   net.download_tensor(1, mb.TENSOR["NORM_VARIANCES_AVERAGES"] | mb.TENSOR_LSTM_NORM_GROUP(g)).reshape(T, 5).astype(np.float64))
            for g, name in enumerate(GROUPS)}
    net.set_state_propagation(mb.STATE_INFERENCE)
    net.Forward_Pass(B, X)
    got = net.download_tensor(1, mb.TENSOR["OUTPUTS"]).reshape(T, B, 5)
    # the same recurrence with every normalisation replaced by scale * (x - average mean) / average sigma + shift of its time step
    flat = torch.tensor(w.astype(np.float64))
    l = desc.layers[1]
    v, nv = lstm_views(flat, l, 4), norm_views(flat, desc, l)
    x = torch.tensor(X.astype(np.float64)).reshape(B, T, 4)
    h = torch.zeros(B, 5, dtype=T64)
    c = torch.zeros(B, 5, dtype=T64)
    W = dict(z=(v["Wz_in"], v["Wz_rec"], v["bz"]), i=(v["W_in"][0], v["W_rec"][0], v["bi"]), f=(v["W_in"][1], v["W_rec"][1], v["bf"]),
             o=(v["W_in"][2], v["W_rec"][2], v["bo"]))
    fixed = lambda name, t, val: nv[name][2] * ((val - torch.tensor(avgs[name][0][t])) / torch.tensor(avgs[name][1][t])) + nv[name][3]
    for t in range(T):
        def gate(g):
            a = fixed(g + "_in", t, x[:, t] @ W[g][0].t()) + W[g][2]
            return a if t == 0 else a + fixed(g + "_rec", t, h @ W[g][1].t())
        i = torch.sigmoid(gate("i") + (0 if t == 0 else c * v["peep"][0]))
        z = torch.tanh(gate("z"))
        c = z * i if t == 0 else z * i + torch.sigmoid(gate("f") + c * v["peep"][1]) * c
        h = torch.sigmoid(gate("o") + c * v["peep"][2]) * torch.tanh(fixed("c", t, c))
        assert_close(got[t], h.numpy(), rel=1e-4, abs_=1e-5, what="inference step %d" % t)


def test_zoneout_forward():
    """zoneout masks on the normalised layer, a batch smaller than the allocation: the forward pass against the model with the
    same masks.  (The backward pass does not know the masks, in the normalised layer as in the plain one: it is the reference's
    own and is not compared with calculus.)"""
    T, B, Bmax = 4, 6, 9
    specs = [dict(units=4), lstm(5, dropout="ZONEOUT", keep=0.5, keep_output=0.5), dict(units=5, activation="LINEAR")]
    rng = np.random.default_rng(12)
    X = rng.normal(0, 1, (B, T * 4)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * 5)).astype(np.float32)
    masks = (rng.uniform(0, 1, 2 * T * 5) < 0.6).astype(np.uint8)
    desc, net, w = oracle(specs, B, T, 14, X, Y, Bmax=Bmax, masks=masks)
    zone = (torch.tensor(masks[:T * 5].reshape(T, 5)), torch.tensor(masks[T * 5:].reshape(T, 5)))
    flat, y, outs, taps = torch_net(desc, specs, w, X, T, zone=zone)
    for i in (1, 2):
        got = net.download_tensor(i, mb.TENSOR["OUTPUTS"]).reshape(T, Bmax, 5)[:, :B]
        assert_close(got, outs[i].detach().numpy().transpose(1, 0, 2), rel=1e-4, abs_=1e-5, what="outputs of layer %d under zoneout" % i)


def test_more_cells_per_block_are_refused():
    specs = [dict(units=4), lstm(3, cells_per_block=2), dict(units=6, activation="LINEAR")]
    with pytest.raises(OracleError) as e:
        OracleNetwork(oracle_desc(specs, 4, 3), oracle_hyper())
    assert e.value.code == mb.E_UNSUPPORTED
