"""Pins the oracle's recurrent stacks that mix layer kinds - residual blocks whose members are independently recurrent layers,
LSTM layers, dense and pooling layers (the member switch of Recurrent__Forward_Pass__Residual__Layer,
Neural_Network__Recurrent_Forward_Pass__OpenMP.cpp:711-771; the reference's own example network, LW/debug.cpp `simple_debug`,
is residual blocks of independently recurrent members with pooling), and residual / pooling layers next to LSTM layers -
against float64 automatic differentiation through time of an independently written model.  Also the member-level dropouts
and the k-sparse filter (closed forms with supplied draws) and ShakeDrop with one mask per (time step, example).  CPU only."""
import types
import zlib

import numpy as np
import pytest
import torch

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, oracle_desc, oracle_hyper, run_step
from tests.oracle_lib import OracleNetwork
from tests.test_oracle_lstm import lstm_forward, lstm_views
from tests.test_oracle_pooling import _torch_pool

T64 = torch.float64
ACT = {"TANH": torch.tanh, "SIGMOID": torch.sigmoid, "LINEAR": lambda v: v, "ISRU": lambda v: v / torch.sqrt(1 + v * v),
       "SOFTMAX": lambda v: torch.softmax(v, dim=-1), "SINE_SYMMETRIC": torch.sin}


def fc(units, act="TANH", **kw): return dict(units=units, activation=act, **kw)
def ind(units, act="TANH", **kw): return dict(type="ind_rnn", units=units, activation=act, **kw)
def lstm(units, **kw): return dict(type="lstm", units=units, **kw)
def res(depth, **kw): return dict(type="residual", block_depth=depth, **kw)
def avg(k, s, **kw): return dict(type="average_pooling", kernel=k, stride=s, **kw)
def mx(k, s, **kw): return dict(type="max_pooling", kernel=k, stride=s, **kw)


class Model:
    """Tensors are [B][T][width].  A dense layer acts per time step; an independently recurrent one adds u * (its own activation
    of the step before) in front of its activation; an LSTM layer is the peephole recurrence of tests/test_oracle_lstm.py, the
    second direction on the time-reversed sequence, both summed; pooling acts per time step.  A residual block over the
    shortcut source x: member 1 applies its weights to x as it is, member k > 1 applies activation (with its recurrence,
    for an independently recurrent member: on its INPUT side, fan-in wide) and then its weights; an LSTM or pooling member is
    the layer itself; y = pad(x) + pad(last member's output)."""

    def __init__(self, desc, specs, flat, T, eps=1e-5):
        self.d, self.specs, self.T, self.eps = desc, specs, T, eps
        self.flat = torch.tensor(np.asarray(flat, dtype=np.float64), dtype=T64, requires_grad=True)
        self.taps = {}

    def width(self, li):
        l = self.d.layers[li]
        return l.n_units * (l.n_cells_per_block if l.type_layer == mb.LAYER_LSTM else 1)

    def linear(self, li, x):
        l, H, In = self.d.layers[li], self.specs[li]["units"], x.shape[-1]
        W = self.flat[l.first_connection_index:l.first_connection_index + H * In].view(H, In)
        s = x @ W.t()
        if self.specs[li].get("normalization", "NONE") == "NONE":
            s = s + self.flat[l.first_bias_connection_index:l.first_bias_connection_index + H]
        return s

    def bn(self, li, x):
        """training-state batch normalisation with the statistics of each time step's batch"""
        n = x.shape[-1]
        base = self.d.total_weights + self.d.total_bias + self.d.layers[li].first_normalized_unit_index
        scale, shift = self.flat[base:base + n], self.flat[base + self.d.total_normalized_units:base + self.d.total_normalized_units + n]
        mu = x.mean(0, keepdim=True)
        sd = torch.sqrt((x * x).mean(0, keepdim=True) - mu * mu + self.eps)
        return scale * (x - mu) / sd + shift

    def recur(self, li, x, units_at):
        """h[t] = act(x[t] + u * h[t-1]) with the layer's self weights at flat index units_at"""
        act = ACT[self.specs[li]["activation"]]
        u = self.flat[units_at:units_at + x.shape[-1]]
        h, out = None, []
        for t in range(self.T):
            h = act(x[:, t] if t == 0 else x[:, t] + u * h)
            out.append(h)
        return torch.stack(out, 1)

    def lstm(self, li, x):
        l, In = self.d.layers[li], x.shape[-1]
        K, cpb = l.n_units, l.n_cells_per_block
        C = K * cpb
        per_block, G = cpb * (In + C) + 3 * In + 3 * C + 3 * cpb, C + 3 * K
        view = lambda direction: types.SimpleNamespace(n_units=K, n_cells_per_block=cpb, first_connection_index=l.first_connection_index + direction * K * per_block,
                                                       first_bias_connection_index=l.first_bias_connection_index + direction * G)
        y = lstm_forward(lstm_views(self.flat, view(0), In), x)
        if l.use_bidirectional:
            y = y + torch.flip(lstm_forward(lstm_views(self.flat, view(1), In), torch.flip(x, dims=[1])), dims=[1])
        return y

    def pool(self, li, x):
        B, T, W = x.shape
        y, out = _torch_pool(self.specs[li], x.reshape(B * T, W))
        return y.reshape(B, T, out)

    def layer(self, li, x):
        sp, kind = self.specs[li], self.specs[li].get("type", "fc")
        if kind == "lstm": return self.lstm(li, x)
        if kind.endswith("pooling"): return self.pool(li, x)
        s = self.linear(li, x)
        if sp.get("normalization", "NONE") != "NONE": s = self.bn(li, s)
        if kind == "ind_rnn":
            l = self.d.layers[li]
            return self.recur(li, s, l.first_connection_index + sp["units"] * x.shape[-1])
        return ACT[sp["activation"]](s)

    def member(self, li, u, first):
        sp, kind = self.specs[li], self.specs[li].get("type", "fc")
        if kind == "lstm": return self.lstm(li, u)
        if kind.endswith("pooling"): return self.pool(li, u)
        if sp.get("normalization", "NONE") != "NONE": u = self.bn(li, u)
        if not first:
            if kind == "ind_rnn":
                l = self.d.layers[li]
                u = self.recur(li, u, l.first_connection_index + sp["units"] * u.shape[-1])
            else:
                u = ACT[sp["activation"]](u)
        return self.linear(li, u)

    def forward(self, X):
        B = X.shape[0]
        x = torch.tensor(np.asarray(X, dtype=np.float64), dtype=T64).reshape(B, self.T, self.specs[0]["units"])
        li = 1
        while li < len(self.specs):
            sp = self.specs[li]
            if sp.get("type") == "residual":
                u = x
                for k in range(1, sp["block_depth"] + 1):
                    u = self.member(li + k, u, k == 1)
                    if u.requires_grad:
                        u.retain_grad()
                        self.taps[li + k] = u
                if sp.get("normalization", "NONE") != "NONE": u = self.bn(li, u)
                na, nb = x.shape[-1], u.shape[-1]
                pad = (abs(na - nb) + 1) // 2
                x = x + torch.nn.functional.pad(u, (pad, na - nb - pad)) if na >= nb else u + torch.nn.functional.pad(x, (pad, nb - na - pad))
                x.retain_grad()
                self.taps[li] = x
                li += sp["block_depth"] + 1
            else:
                x = self.layer(li, x)
                x.retain_grad()
                self.taps[li] = x
                li += 1
        return x


def _self_weights(desc, specs, w, seed):
    """self weights of the independently recurrent layers large enough for the recurrence to matter (glorot leaves them tiny)"""
    import ctypes as C
    from tests.oracle_lib import load_oracle
    lib = load_oracle()
    rng = np.random.default_rng(seed)
    for i in range(1, desc.n_layers):
        l = desc.layers[i]
        if l.type_layer != mb.LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT:
            continue
        fan_in = lib.myea_net_desc_number_outputs(C.byref(desc), lib.myea_net_desc_previous_layer(C.byref(desc), i))
        n_self = l.last_connection_index - l.first_connection_index - l.n_units * fan_in     # behind the [units][fan-in] matrix
        w[l.last_connection_index - n_self:l.last_connection_index] = rng.uniform(-0.9, 0.9, n_self).astype(np.float32)
    return w


CASES = {
    # the reference's example network in small: residual blocks of independently recurrent members with pooling, T > 1
    "ind_rnn_members_with_pooling": ([fc(6), fc(8, "TANH"), res(3), ind(8, "TANH"), ind(8, "SIGMOID"), ind(8, "TANH"), avg(2, 2),
                                      res(2), ind(4, "TANH"), ind(4, "TANH"), fc(3, "LINEAR")], 5, 4),
    # members of three kinds in one block; the independently recurrent one normalised on its input side
    "mixed_members_normalised": ([fc(5), fc(7, "SIGMOID"), res(3), fc(9, "TANH"), ind(9, "TANH", normalization="BATCH_NORMALIZATION"), mx(3, 1, padding=1),
                                  fc(4, "SOFTMAX")], 4, 6),
    # an LSTM as the block's last member (its output meets the shortcut), a dense member in front of it
    "lstm_last_member": ([fc(6), fc(7, "TANH"), res(2), fc(5, "TANH"), lstm(7), fc(7, "LINEAR")], 4, 5),
    # an LSTM as the block's first member: the layer in front of the block gets dG Win and the shortcut's share
    "lstm_first_member": ([fc(5), fc(6, "TANH"), res(2), lstm(4, cells_per_block=2), fc(6, "TANH"), fc(6, "LINEAR")], 3, 4),
    # a two-direction LSTM as the first member: both directions' dG Win and the shortcut's share meet in the layer in front of the block
    "two_directions_first_member": ([fc(5), fc(8, "TANH"), res(2), lstm(4, bidirectional=True), fc(8, "SIGMOID"), fc(3, "LINEAR")], 4, 3),
    # an LSTM between two dense members, two directions
    "lstm_middle_member_two_directions": ([fc(5), fc(8, "TANH"), res(3), fc(6, "TANH"), lstm(5, bidirectional=True), ind(5, "TANH"), fc(10, "LINEAR")], 4, 3),
    # residual blocks and pooling layers next to LSTM layers, outside blocks
    "blocks_and_pooling_beside_lstm": ([fc(6), lstm(8), avg(2, 2), res(2), fc(6, "TANH"), fc(4, "SIGMOID"), lstm(9), mx(3, 2, padding=1), fc(9, "LINEAR")], 4, 4),
    # the block directly on an LSTM layer (the LSTM is the shortcut source), block-level normalisation
    "block_on_lstm": ([fc(4), lstm(6), res(2, normalization="BATCH_NORMALIZATION"), fc(5, "TANH"), ind(5, "TANH"), fc(6, "LINEAR")], 3, 5),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_recurrent_stack_matches_float64_autograd(name):
    specs, T, B = CASES[name]
    desc = oracle_desc(specs, B, T)
    seed = zlib.crc32(name.encode()) % 1000
    rng = np.random.default_rng(seed)
    w = _self_weights(desc, specs, glorot_parameters(desc, seed, bias_range=0.3), seed)
    n_in, n_out = specs[0]["units"], specs[-1]["units"]
    X = rng.normal(0, 1, (B, T * n_in)).astype(np.float32)
    softmax = specs[-1]["activation"] == "SOFTMAX"
    if softmax:
        Y = np.zeros((B, T, n_out), np.float32)
        np.put_along_axis(Y, rng.integers(0, n_out, (B, T))[..., None], 1.0, axis=2)
        Y = Y.reshape(B, -1)
    else:
        Y = rng.normal(0, 1, (B, T * n_out)).astype(np.float32)
    net = OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS["CROSS_ENTROPY" if softmax else "MSE"]))
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(w)
    net.Clear_Training_Arrays()
    run_step(net, B, X, Y, update=False)
    model = Model(desc, specs, w, T)
    y = model.forward(X)
    t = torch.tensor(Y.astype(np.float64)).reshape(B, T, n_out)
    loss = -(t * torch.log(y)).sum() if softmax else 0.5 * ((y - t) ** 2).sum()
    loss.backward()
    got = net.download_tensor(desc.n_layers - 1, mb.TENSOR["OUTPUTS"]).reshape(T, B, n_out)
    assert_close(got, y.detach().numpy().transpose(1, 0, 2), 3e-5, 3e-6, "outputs")
    for li, tap in model.taps.items():
        width = tap.shape[-1]
        assert_close(net.download_tensor(li, mb.TENSOR["OUTPUTS"]).reshape(T, B, width), tap.detach().numpy().transpose(1, 0, 2), 3e-5, 3e-6, "outputs of layer %d" % li)
    g = model.flat.grad.numpy()
    assert np.count_nonzero(g[:desc.total_weights]) > 0.9 * desc.total_weights
    # the bias slots an LSTM's shifted bias index leaves unused carry no gradient on either side
    assert_close(net.download_gradient(), g, 3e-4, 3e-5, "gradient")


def test_layout_of_independently_recurrent_members():
    """Prepare__Connections__FC_Ind_RNN inside a block: one self weight per recurrent activation unit - fan-in many on a member,
    none on the block's first member, whose activation units do not exist (Assign__Post__Residual_Layer)."""
    specs = [fc(5), fc(7), res(3), ind(6), ind(6), ind(6), fc(3)]
    d = oracle_desc(specs, 2, 3)
    sizes = [d.layers[i].last_connection_index - d.layers[i].first_connection_index for i in range(7)]
    assert sizes == [0, 35, 0, 7 * 6, 6 * 6 + 6, 6 * 6 + 6, 7 * 3]
    masks = [d.layers[i].first_mask_index for i in range(7)]
    assert masks == [0, 15, 36, 36, 36, 54, 72] and d.total_mask_units == 72 + 9


def test_an_independently_recurrent_member_must_be_as_wide_as_its_input():
    with pytest.raises(Exception):
        OracleNetwork(oracle_desc([fc(5), fc(7), res(2), fc(6), ind(4), fc(3)], 2, 3))


def _run(specs, T, B, seed, state=mb.STATE_TRAINING, noise=None, masks=None):
    desc = oracle_desc(specs, B, T)
    net = OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS["MSE"]))
    net.set_state_propagation(state)
    net.upload_parameters(glorot_parameters(desc, seed, bias_range=0.3))
    if masks is not None:
        net.upload_masks(masks)
    for li, draws in (noise or {}).items():
        net.upload_dropout_noise(li, draws)
    rng = np.random.default_rng(seed)
    X = rng.normal(0, 1, (B, T * specs[0]["units"])).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * specs[-1]["units"])).astype(np.float32)
    net.Forward_Pass(B, X)
    return desc, net, X, Y


@pytest.mark.parametrize("kind", ["GAUSSIAN", "UOUT"])
def test_noise_dropout_on_a_member_acts_on_its_input_side_activations(kind):
    """Constant draws c: a Gaussian member's activations are multiplied by c, a Uout member's by (1 + c), so the member's
    output is that of the plain block fed activations scaled that way - for a tanh member, the plain block whose member
    weights are scaled by the factor (biases untouched).  Draws are [T][B][fan-in]; outside the training state nothing happens."""
    T, B, c = 3, 4, 0.37
    base = [fc(5), fc(6, "TANH"), res(2), fc(7, "TANH"), fc(6, "TANH"), fc(3, "LINEAR")]
    noisy = [dict(s) for s in base]
    noisy[4].update(dropout=kind, keep=0.5)
    factor = c if kind == "GAUSSIAN" else 1.0 + c
    d0, plain, X, _ = _run(base, T, B, 3)
    w = glorot_parameters(d0, 3, bias_range=0.3)
    l4 = d0.layers[4]
    w[l4.first_connection_index:l4.last_connection_index] *= factor
    plain.upload_parameters(w)
    plain.Forward_Pass(B, X)
    want = plain.download_tensor(5, mb.TENSOR["OUTPUTS"])
    d1, net, X1, _ = _run(noisy, T, B, 3, noise={4: np.full(T * B * 7, c, np.float32)})
    assert np.array_equal(X, X1)
    assert_close(net.download_tensor(5, mb.TENSOR["OUTPUTS"]), want, 1e-5, 1e-6)
    _, off, _, _ = _run(noisy, T, B, 3, state=mb.STATE_INFERENCE, noise={4: np.full(T * B * 7, c, np.float32)})
    d0b, plain2, _, _ = _run(base, T, B, 3, state=mb.STATE_INFERENCE)
    assert np.array_equal(off.download_tensor(5, mb.TENSOR["OUTPUTS"]), plain2.download_tensor(5, mb.TENSOR["OUTPUTS"]))


def test_bernoulli_inference_scaling_and_k_sparse_filter_on_a_member():
    """Outside the training state a Bernoulli member's activations are scaled by the retention probability (a tanh member: its
    weights scaled); a k-sparse member keeps the k largest of its fan-in activations per example and time step."""
    T, B = 2, 5
    base = [fc(5), fc(6, "TANH"), res(2), fc(8, "TANH"), fc(6, "TANH"), fc(3, "LINEAR")]
    drop = [dict(s) for s in base]
    drop[4].update(dropout="BERNOULLI", keep=0.6)
    d0, plain, X, _ = _run(base, T, B, 5, state=mb.STATE_INFERENCE)
    w = glorot_parameters(d0, 5, bias_range=0.3)
    l4 = d0.layers[4]
    w[l4.first_connection_index:l4.last_connection_index] *= np.float32(0.6)
    plain.upload_parameters(w)
    plain.Forward_Pass(B, X)
    _, net, _, _ = _run(drop, T, B, 5, state=mb.STATE_INFERENCE)
    assert_close(net.download_tensor(5, mb.TENSOR["OUTPUTS"]), plain.download_tensor(5, mb.TENSOR["OUTPUTS"]), 1e-5, 1e-6)
    sparse = [dict(s) for s in base]
    sparse[4].update(k_sparsity=3)
    d2, net2, X2, _ = _run(sparse, T, B, 5)
    w2 = glorot_parameters(d2, 5, bias_range=0.3)
    # the member's activations before the filter: tanh of the first member's sums; recompute the member's output from the 3 largest
    u = net2.download_tensor(3, mb.TENSOR["OUTPUTS"]).reshape(T, B, 8).astype(np.float64)
    a = np.tanh(u)
    cut = np.sort(a, axis=2)[:, :, -3][..., None]
    a = np.where(a >= cut, a, 0.0)
    l = d2.layers[4]
    W = w2[l.first_connection_index:l.last_connection_index].reshape(6, 8).astype(np.float64)
    b = w2[l.first_bias_connection_index:l.first_bias_connection_index + 6].astype(np.float64)
    assert_close(net2.download_tensor(4, mb.TENSOR["OUTPUTS"]).reshape(T, B, 6), a @ W.T + b, 1e-5, 1e-6)


def test_shakedrop_has_a_mask_per_time_step_and_example():
    """[T][B] masks, then [T][B][width] forward draws, then the backward draws: a perturbed (time step, example) has its block
    output multiplied value by value going forward and its delta by the backward draws going back; the others are the plain
    block's.  Checked against the plain block's tensors."""
    T, B, W = 3, 4, 6
    base = [fc(5), fc(6, "TANH"), res(2), fc(7, "TANH"), fc(6, "TANH"), fc(3, "LINEAR")]
    shake = [dict(s) for s in base]
    shake[2].update(dropout="SHAKEDROP", keep=0.5)
    rng = np.random.default_rng(9)
    mask = (rng.uniform(0, 1, (T, B)) < 0.5).astype(np.float32)
    alpha, beta = rng.uniform(-1, 1, (T, B, W)).astype(np.float32), rng.uniform(0, 1, (T, B, W)).astype(np.float32)
    assert 0 < mask.sum() < T * B
    draws = np.concatenate([mask.ravel(), alpha.ravel(), beta.ravel()])
    d0, plain, X, Y = _run(base, T, B, 9)
    d1, net, _, _ = _run(shake, T, B, 9, noise={2: draws})
    f_plain = plain.download_tensor(4, mb.TENSOR["OUTPUTS"]).reshape(T, B, W)     # the last member's sums: the block's output
    x_plain = plain.download_tensor(1, mb.TENSOR["OUTPUTS"]).reshape(T, B, W)
    want = x_plain + np.where(mask[..., None] != 0, f_plain * alpha, f_plain)
    assert_close(net.download_tensor(2, mb.TENSOR["OUTPUTS"]).reshape(T, B, W), want, 1e-6, 1e-7)
    for n in (net,):
        n.Compute__Error(B, Y)
        n.Backward_Pass(B)
    d_res = net.download_tensor(2, mb.TENSOR["ERRORS"]).reshape(T, B, W)
    d_last = net.download_tensor(4, mb.TENSOR["ERRORS"]).reshape(T, B, W)
    assert_close(d_last, np.where(mask[..., None] != 0, d_res * beta, d_res), 1e-6, 1e-7)
