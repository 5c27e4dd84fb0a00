"""Pins the oracle's LSTM-with-peephole path (forward, BPTT, dW) on the CPU: float64 autograd of an independently
written forward model, torch.nn.LSTM for the peephole-free special case, and explicit checks of the boundary-step
behaviour that is the reference's rather than calculus."""
import numpy as np
import pytest
import torch

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, oracle_desc, oracle_hyper, run_step
from tests.oracle_lib import OracleNetwork

T64 = torch.float64


def _widths(desc):
    return [desc.layers[i].n_units * (desc.layers[i].n_cells_per_block if desc.layers[i].type_layer == mb.LAYER_LSTM else 1)
            for i in range(desc.n_layers)]


def lstm_views(flat, l, In):
    """Gate matrices of one LSTM layer as gathers from the flat vector: per block [z_in | z_rec] per cell, then i/f/o
    input rows, i/f/o recurrent rows, i/f/o peepholes."""
    K, cpb = l.n_units, l.n_cells_per_block
    C = K * cpb
    per_block = cpb * (In + C) + 3 * In + 3 * C + 3 * cpb
    base = l.first_connection_index
    idx = lambda start, n: torch.arange(start, start + n)
    Wz_in = torch.stack([flat[idx(base + k * per_block + j * (In + C), In)] for k in range(K) for j in range(cpb)])
    Wz_rec = torch.stack([flat[idx(base + k * per_block + j * (In + C) + In, C)] for k in range(K) for j in range(cpb)])
    g0 = lambda k: base + k * per_block + cpb * (In + C)
    W_in = [torch.stack([flat[idx(g0(k) + g * In, In)] for k in range(K)]) for g in range(3)]
    W_rec = [torch.stack([flat[idx(g0(k) + 3 * In + g * C, C)] for k in range(K)]) for g in range(3)]
    peep = [torch.stack([flat[idx(g0(k) + 3 * In + 3 * C + g * cpb, cpb)] for k in range(K)]).reshape(C) for g in range(3)]
    b0 = l.first_bias_connection_index
    bz, bi, bf, bo = flat[idx(b0, C)], flat[idx(b0 + C, K)], flat[idx(b0 + C + K, K)], flat[idx(b0 + C + 2 * K, K)]
    return dict(K=K, cpb=cpb, C=C, Wz_in=Wz_in, Wz_rec=Wz_rec, W_in=W_in, W_rec=W_rec, peep=peep, bz=bz, bi=bi, bf=bf, bo=bo)


def lstm_forward(v, x):
    """x [B, T, In] -> h [B, T, C].  h_{-1} = c_{-1} = 0; the gates of a block are shared by its cells."""
    B, T, _ = x.shape
    K, cpb, C = v["K"], v["cpb"], v["C"]
    h = torch.zeros(B, C, dtype=T64)
    c = torch.zeros(B, C, dtype=T64)
    per_block = lambda t_: t_.reshape(B, K, cpb).sum(2)
    spread = lambda g: g.repeat_interleave(cpb, dim=1)
    outs = []
    for t in range(T):
        xt = x[:, t]
        i = torch.sigmoid(xt @ v["W_in"][0].t() + h @ v["W_rec"][0].t() + per_block(c * v["peep"][0]) + v["bi"])
        f = torch.sigmoid(xt @ v["W_in"][1].t() + h @ v["W_rec"][1].t() + per_block(c * v["peep"][1]) + v["bf"])
        z = torch.tanh(xt @ v["Wz_in"].t() + h @ v["Wz_rec"].t() + v["bz"])
        c = z * spread(i) + spread(f) * c
        o = torch.sigmoid(xt @ v["W_in"][2].t() + h @ v["W_rec"][2].t() + per_block(c * v["peep"][2]) + v["bo"])
        h = spread(o) * torch.tanh(c)
        outs.append(h)
    return torch.stack(outs, dim=1)


def torch_net(desc, specs, flat_np, X, T):
    """float64 model of a recurrent stack (FC layers applied per time step); returns (flat leaf, outputs [B,T,Out], taps)."""
    flat = torch.tensor(np.asarray(flat_np, dtype=np.float64), dtype=T64, requires_grad=True)
    w = _widths(desc)
    B = X.shape[0]
    x = torch.tensor(np.asarray(X, dtype=np.float64), dtype=T64).reshape(B, T, w[0])
    taps = {}
    for i in range(1, desc.n_layers):
        l = desc.layers[i]
        if l.type_layer == mb.LAYER_LSTM:
            x = lstm_forward(lstm_views(flat, l, w[i - 1]), x)
        else:
            W = flat[l.first_connection_index:l.first_connection_index + w[i] * w[i - 1]].view(w[i], w[i - 1])
            s = x @ W.t() + flat[l.first_bias_connection_index:l.first_bias_connection_index + w[i]]
            act = specs[i].get("activation", "SIGMOID")
            x = {"LINEAR": lambda q: q, "TANH": torch.tanh, "SIGMOID": torch.sigmoid,
                 "SOFTMAX": lambda q: torch.softmax(q, dim=2)}[act](s)
        x.retain_grad()
        taps[i] = x
    return flat, x, taps


def _oracle(specs, B, T, seed, X, Y, loss="MSE", Bmax=None):
    desc = oracle_desc(specs, Bmax or B, T)
    net = OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS[loss], type_optimizer_function=mb.OPTIMIZER["AMSGRAD"]))
    net.set_state_propagation(mb.STATE_TRAINING)
    w = glorot_parameters(desc, seed, bias_range=0.3)
    net.upload_parameters(w)
    run_step(net, B, X, Y, update=False)
    return desc, net, w


CASES = [
    # (the layers after the last LSTM own at least C bias slots: its bias index overrun must stay inside the vector)
    ("one-cell-per-block", [dict(units=6), dict(type="lstm", units=5), dict(units=7, activation="LINEAR")], 4),
    ("two-cells-per-block", [dict(units=4), dict(type="lstm", units=3, cells_per_block=2), dict(units=6, activation="TANH")], 5),
    ("config3-shape-shrunk", [dict(units=8), dict(type="lstm", units=12), dict(type="lstm", units=12), dict(units=12, activation="LINEAR")], 6),
    ("fc-below-lstm", [dict(units=5), dict(units=7, activation="TANH"), dict(type="lstm", units=4, cells_per_block=3), dict(units=9, activation="SIGMOID"),
                       dict(units=4, activation="LINEAR")], 3),
    ("two-steps", [dict(units=3), dict(type="lstm", units=4), dict(units=5, activation="LINEAR")], 2),
]


@pytest.mark.parametrize("name,specs,T", CASES, ids=[c[0] for c in CASES])
def test_bptt_gradient_matches_autograd(name, specs, T):
    """For T >= 2 the reference's BPTT is the exact gradient of its forward pass: all parameter classes (input,
    recurrent, peephole, the four bias vectors, FC weights) agree with float64 autograd, as do the layer outputs and
    the delta handed to each layer.  The parameter index table (including the LSTM bias index as the reference leaves
    it) is taken from the descriptor on both sides."""
    B, seed = 5, 17
    rng = np.random.default_rng(seed)
    n_in, n_out = specs[0]["units"], specs[-1]["units"]
    X = rng.normal(0, 1, (B, T * n_in)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * n_out)).astype(np.float32)
    desc, net, w = _oracle(specs, B, T, seed, X, Y)
    flat, y, taps = torch_net(desc, specs, w, X, T)
    t = torch.tensor(Y.astype(np.float64)).reshape(B, T, n_out)
    (0.5 * ((y - t) ** 2).sum()).backward()
    widths = _widths(desc)
    for i in range(1, desc.n_layers):
        got = net.download_tensor(i, mb.TENSOR["OUTPUTS"]).reshape(T, B, widths[i])          # [T][Bmax][H]
        assert_close(got, taps[i].detach().numpy().transpose(1, 0, 2), rel=3e-5, abs_=3e-6, what="outputs layer %d" % i)
    assert_close(net.download_gradient(), flat.grad.numpy(), rel=3e-4, abs_=3e-5, what="gradient " + name)
    assert np.count_nonzero(flat.grad.numpy()) > 0.8 * desc.total_weights


def test_peephole_free_case_is_the_textbook_lstm():
    """peepholes = 0: the forward pass equals torch.nn.LSTM (gate order i, f, g, o; zero initial state)."""
    In, H, T, B = 5, 7, 6, 4
    specs = [dict(units=In), dict(type="lstm", units=H), dict(units=H, activation="LINEAR")]
    desc = oracle_desc(specs, B, T)
    w = glorot_parameters(desc, 3, bias_range=0.3)
    l = desc.layers[1]
    per_block = (In + H) + 3 * In + 3 * H + 3
    for k in range(H):
        w[l.first_connection_index + k * per_block + per_block - 3: l.first_connection_index + (k + 1) * per_block] = 0
    # the FC head: identity, zero bias, so that the net's output is h
    l2 = desc.layers[2]
    w[l2.first_connection_index:l2.last_connection_index] = np.eye(H, dtype=np.float32).ravel()
    w[l2.first_bias_connection_index:l2.first_bias_connection_index + H] = 0   # also the slots the LSTM's b_o overruns into
    net = OracleNetwork(desc, oracle_hyper())
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(w)
    X = np.random.default_rng(3).normal(0, 1, (B, T * In)).astype(np.float32)
    net.Forward_Pass(B, X)
    v = lstm_views(torch.tensor(w.astype(np.float64)), l, In)
    ref = torch.nn.LSTM(In, H, batch_first=True).double()
    with torch.no_grad():
        ref.weight_ih_l0.copy_(torch.cat([v["W_in"][0], v["W_in"][1], v["Wz_in"], v["W_in"][2]]))
        ref.weight_hh_l0.copy_(torch.cat([v["W_rec"][0], v["W_rec"][1], v["Wz_rec"], v["W_rec"][2]]))
        ref.bias_ih_l0.copy_(torch.cat([v["bi"], v["bf"], v["bz"], v["bo"]]))
        ref.bias_hh_l0.zero_()
        want, _ = ref(torch.tensor(X.astype(np.float64)).reshape(B, T, In))
    got = net.download_tensor(2, mb.TENSOR["OUTPUTS"]).reshape(T, B, H)
    assert_close(got, want.numpy().transpose(1, 0, 2), rel=3e-5, abs_=3e-6)


def test_lstm_bias_index_overrun_aliases_the_next_layers_bias():
    """Prepare__Bias__LSTM leaves first_bias_connection_index one cell-count past the layer's slice, so the last C
    entries of the LSTM's output-gate bias ARE the first entries of the next layer's bias: both uses read the same
    parameter and both write its gradient.  (Pinned by reading only.)"""
    T, B, In, K = 3, 2, 3, 4
    specs = [dict(units=In), dict(type="lstm", units=K), dict(units=5, activation="LINEAR")]
    desc = oracle_desc(specs, B, T)
    l1, l2 = desc.layers[1], desc.layers[2]
    assert l1.first_bias_connection_index == desc.total_weights + K
    assert l1.first_bias_connection_index + 4 * K == l2.first_bias_connection_index + K    # b_o's last K entries overlap the head's bias
    rng = np.random.default_rng(0)
    X = rng.normal(0, 1, (B, T * In)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * 5)).astype(np.float32)
    desc, net, w = _oracle(specs, B, T, 1, X, Y)
    flat, y, _ = torch_net(desc, specs, w, X, T)
    (0.5 * ((y - torch.tensor(Y.astype(np.float64)).reshape(B, T, 5)) ** 2).sum()).backward()
    g = net.download_gradient()
    assert_close(g, flat.grad.numpy(), rel=3e-4, abs_=3e-5)
    shared = slice(l2.first_bias_connection_index, l2.first_bias_connection_index + K)
    head_only = (y.detach().numpy() - Y.reshape(B, T, 5)).sum((0, 1))[:K]
    assert np.abs(g[shared] - head_only).max() > 1e-3        # the LSTM's output-gate term is in there too
    assert np.all(g[desc.total_weights:desc.total_weights + K] == 0)   # the first C bias slots of the slice are never used


def test_single_time_step_computes_no_gate_deltas():
    """T == 1: no branch of Backward_Pass__LSTM_Derivative__Gates_CIF_AF_State matches, so delta z / i / f stay zero and
    only the output-gate path (weights, peephole, bias) and the layers above get a gradient."""
    B, In, K = 4, 3, 5
    specs = [dict(units=In), dict(type="lstm", units=K), dict(units=6, activation="LINEAR")]
    rng = np.random.default_rng(2)
    X = rng.normal(0, 1, (B, In)).astype(np.float32)
    Y = rng.normal(0, 1, (B, 6)).astype(np.float32)
    desc, net, w = _oracle(specs, B, 1, 4, X, Y)
    for kind in ("LSTM_DELTA_CELL_INPUT", "LSTM_DELTA_INPUT_GATE", "LSTM_DELTA_FORGET_GATE"):
        assert np.all(net.download_tensor(1, mb.TENSOR[kind]) == 0)
    assert np.abs(net.download_tensor(1, mb.TENSOR["LSTM_DELTA_OUTPUT_GATE"])).max() > 0
    flat, y, _ = torch_net(desc, specs, w, X, 1)
    (0.5 * ((y - torch.tensor(Y.astype(np.float64)).reshape(B, 1, 6)) ** 2).sum()).backward()
    g, t = net.download_gradient(), flat.grad.numpy()
    l = desc.layers[1]
    per_block = (In + K) + 3 * In + 3 * K + 3
    for k in range(K):
        b = l.first_connection_index + k * per_block
        o_in = slice(b + (In + K) + 2 * In, b + (In + K) + 3 * In)
        assert_close(g[o_in], t[o_in], rel=3e-4, abs_=3e-5)                       # output-gate input weights: exact
        assert_close(g[b + per_block - 1], t[b + per_block - 1], rel=3e-4, abs_=3e-5)   # output-gate peephole: exact
        assert np.all(g[b:b + (In + K) + 2 * In] == 0)                            # z, i, f input/recurrent rows: untouched
        assert np.abs(t[b:b + In]).max() > 0                                      # ... though the true gradient is not zero


def test_first_step_forget_gate_and_partial_batch():
    """delta f of the first step stays zero (its forget gate is never evaluated); B < Bmax leaves the rows past B alone."""
    B, Bmax, T, In, K = 3, 5, 4, 3, 4
    specs = [dict(units=In), dict(type="lstm", units=K, cells_per_block=2), dict(units=8, activation="LINEAR")]
    rng = np.random.default_rng(6)
    X = rng.normal(0, 1, (B, T * In)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * 8)).astype(np.float32)
    desc, net, w = _oracle(specs, B, T, 8, X, Y, Bmax=Bmax)
    df = net.download_tensor(1, mb.TENSOR["LSTM_DELTA_FORGET_GATE"]).reshape(T, Bmax, K)
    assert np.all(df[0] == 0) and np.abs(df[1:, :B]).min() > 0 and np.all(df[:, B:] == 0)
    flat, y, _ = torch_net(oracle_desc(specs, B, T), specs, w, X, T)
    (0.5 * ((y - torch.tensor(Y.astype(np.float64)).reshape(B, T, 8)) ** 2).sum()).backward()
    assert_close(net.download_gradient(), flat.grad.numpy(), rel=3e-4, abs_=3e-5)


def test_rnn_head_reads_the_first_units_pre_activation():
    """RNN__Compute__Error does not advance the pre-activation pointer per unit (Recurrent_Compute__Error__OpenMP.cpp:97-99):
    harmless for linear / tanh / sigmoid / softmax heads, visible for a ReLU head.  (Pinned by reading only.)"""
    B, T = 3, 2
    specs = [dict(units=4), dict(units=5, activation="RELU")]
    desc = oracle_desc(specs, B, T)
    net = OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS["MSE"]))
    net.set_state_propagation(mb.STATE_TRAINING)
    w = glorot_parameters(desc, 2, bias_range=0.5)
    net.upload_parameters(w)
    rng = np.random.default_rng(9)
    X = rng.normal(0, 1, (B, T * 4)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * 5)).astype(np.float32)
    net.Forward_Pass(B, X)
    net.Compute__Error(B, Y)
    s = net.download_tensor(1, mb.TENSOR["SUMMATIONS"]).reshape(T, B, 5)
    y = net.download_tensor(1, mb.TENSOR["OUTPUTS"]).reshape(T, B, 5)
    err = net.download_tensor(1, mb.TENSOR["ERRORS"]).reshape(T, B, 5)
    want = (s[:, :, :1] >= 0) * (y - Y.reshape(B, T, 5).transpose(1, 0, 2))
    assert_close(err, want, rel=1e-6, abs_=1e-7)
    assert not np.allclose(err, (s >= 0) * (y - Y.reshape(B, T, 5).transpose(1, 0, 2)))


def test_time_delays_skip_the_first_steps_and_directional_accuracy():
    B, T = 2, 4
    specs = [dict(units=3), dict(type="lstm", units=2), dict(units=2, activation="TANH")]
    desc = oracle_desc(specs, B, T)
    net = OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS["MSE"], type_accuracy_function=mb.ACCURACY["DIRECTIONAL"], number_time_delays=2))
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(glorot_parameters(desc, 1))
    rng = np.random.default_rng(1)
    X = rng.normal(0, 1, (B, T * 3)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * 2)).astype(np.float32)
    net.Reset__Loss()
    net.Forward_Pass(B, X)
    net.Compute__Error(B, Y)
    st = net.get_loss()
    assert st.number_loss == B * 2 * 2
    err = net.download_tensor(2, mb.TENSOR["ERRORS"]).reshape(T, B, 2)
    assert np.all(err[:2] == 0) and np.abs(err[2:]).min() > 0
    y = net.download_tensor(2, mb.TENSOR["OUTPUTS"]).reshape(T, B, 2).transpose(1, 0, 2)
    d = Y.reshape(B, T, 2)
    want = sum(np.sign(d[:, t] - d[:, t - 1]) == np.sign(y[:, t] - d[:, t - 1]) for t in (2, 3)).sum()
    assert st.accuracy_value == float(want)


def test_bias_overrun_past_the_parameter_vector_is_rejected():
    """a head narrower than the last LSTM would make the reference read/write past its parameter array"""
    with pytest.raises(Exception):
        OracleNetwork(oracle_desc([dict(units=3), dict(type="lstm", units=6), dict(units=2, activation="LINEAR")], 2, 3))
