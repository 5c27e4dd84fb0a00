"""Pins the oracle's residual-block path (pre-activation members, block-level normalisation, zero-padded identity
shortcut) without the reference build: the descriptor layout against hand-counted offsets, the forward/backward
against automatic differentiation of an independent float64 model, and a block that computes zero against the same
stack without the block.  CPU only."""
import zlib

import numpy as np
import pytest
import torch

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, one_hot, oracle_desc, oracle_hyper, run_step
from tests.oracle_lib import OracleNetwork, load_oracle
from tests.test_oracle_pooling import _torch_pool

T64 = torch.float64


def fc(units, act="TANH", **kw):
    return dict(units=units, activation=act, **kw)


def res(depth, **kw):
    return dict(type="residual", block_depth=depth, **kw)


# ------------------------------------------------------------------------------------------------
# layout
# ------------------------------------------------------------------------------------------------
def test_layout_of_a_residual_stack_hand_counted():
    """[0 in 5][1 fc 6][2 residual d=2][3 fc 9 BN][4 fc 4][5 residual d=1 BN][6 fc 7][7 fc 3], T=1.
    connections: prev(3) = 1 (the shortcut source), prev(4) = 3, prev(5) = 2, prev(6) = 2, prev(7) = 5.
    widths: residual 2 = max(6, 4) = 6; residual 5 = max(6, 7) = 7.
    weights: 5*6 | 6*9 | 9*4 | 6*7 | 7*3; biases: 6 | (3 normalised: none... keeps its slot) ..."""
    specs = [fc(5), fc(6), res(2), fc(9, normalization="BATCH_NORMALIZATION"), fc(4), res(1, normalization="BATCH_NORMALIZATION"), fc(7), fc(3)]
    d = oracle_desc(specs, 4)
    lib = load_oracle()
    prev = [lib.myea_net_desc_previous_layer(d, i) for i in range(8)]
    assert prev == [0, 0, 1, 1, 3, 2, 2, 5]
    outs = [lib.myea_net_desc_number_outputs(d, i) for i in range(8)]
    assert outs == [5, 6, 6, 9, 4, 7, 7, 3]
    first = [d.layers[i].first_connection_index for i in range(8)]
    assert first[1] == 0 and first[3] == 30 and first[4] == 30 + 54 and first[6] == 30 + 54 + 36 and first[7] == 30 + 54 + 36 + 42
    assert d.total_weights == 30 + 54 + 36 + 42 + 21
    # every FC layer keeps a bias slot, normalised or not (Prepare__Bias__FC), residual layers own none
    assert d.total_bias == 6 + 9 + 4 + 7 + 3
    bias = [d.layers[i].first_bias_connection_index - d.total_weights for i in (1, 3, 4, 6, 7)]
    assert bias == [0, 6, 15, 19, 26]
    # normalised units: input 5, fc 6, residual 2 -> its last member's width 4, member 3 -> fan-in 6, member 4 -> fan-in 9,
    # residual 5 -> 7, member 6 -> fan-in 6, fc 3
    norm = [d.layers[i].first_normalized_unit_index for i in range(8)]
    assert norm == [0, 5, 11, 15, 21, 30, 37, 43]
    assert d.total_normalized_units == 46
    assert d.total_parameters == d.total_weights + d.total_bias + 2 * 46
    # masks follow the activation units: input 5, fc 6, residual 0, first member 0, member 4 -> fan-in 9, residual 0,
    # first member 0, fc 3
    mask = [d.layers[i].first_mask_index for i in range(8)]
    assert mask == [0, 5, 11, 11, 11, 20, 20, 20]
    assert d.total_mask_units == 23


def test_layout_rejects_malformed_blocks():
    lib = load_oracle()
    for specs in ([fc(4), res(0), fc(3), fc(2)],                 # empty block
                  [fc(4), res(2), fc(3), fc(2)],                 # block runs to the end: nothing consumes it
                  [fc(4), res(3), fc(3), fc(2)]):                # block runs past the end
        with pytest.raises(ValueError):
            mb.make_desc(specs, 2, lib=lib)


# ------------------------------------------------------------------------------------------------
# float64 autograd model
# ------------------------------------------------------------------------------------------------
def _act(name, x):
    if name == "TANH": return torch.tanh(x)
    if name == "SIGMOID": return torch.sigmoid(x)
    if name == "LINEAR": return x
    if name == "ISRU": return x / torch.sqrt(1 + x * x)
    if name == "ELLIOT_SYMMETRIC": return x / (1 + x.abs())
    if name == "SINE_SYMMETRIC": return torch.sin(x)
    if name == "SOFTMAX": return torch.softmax(x, dim=1)
    if name == "RELU": return torch.relu(x)
    if name == "LEAKY_RELU": return torch.where(x < 0, 0.01 * x, x)
    if name == "GAUSSIAN": return torch.exp(-x * x)
    raise KeyError(name)


class _DroppedActivation(torch.autograd.Function):
    """v = act(u) * mask * scale with the reference's backward: no mask or scale on the way back, and the activation's
    derivative as the reference writes it, on the pre-activation u and the STORED (masked, rescaled) value v
    (Activation_Functions.hpp: tanh' = 1 - v^2, sigmoid' = v (1 - v), gaussian' = -2 u v, isru' = (v / u)^3, ...)."""

    @staticmethod
    def forward(ctx, u, name, mult):
        v = _act(name, u) * mult
        ctx.save_for_backward(u, v)
        ctx.name = name
        return v

    @staticmethod
    def backward(ctx, grad):
        u, v = ctx.saved_tensors
        name = ctx.name
        if name == "RELU": d = (u >= 0).to(T64)
        elif name == "LEAKY_RELU": d = torch.where(u < 0, torch.full_like(u, 0.01), torch.ones_like(u))
        elif name == "TANH": d = 1 - v * v
        elif name == "SIGMOID": d = v * (1 - v)
        elif name == "GAUSSIAN": d = -2 * u * v
        elif name == "ISRU": d = (v / u) ** 3
        elif name == "ELLIOT_SYMMETRIC": d = 1 / (1 + u.abs()) ** 2
        elif name == "SINE_SYMMETRIC": d = torch.cos(u)
        else: raise KeyError(name)
        return grad * d, None, None


class TorchResidualNet:
    """Independent model.  Plain layer: y = act(BN(x W^T + b)).  Residual block over the shortcut source x:
    u_1 = BN_1(x) W_1^T (+ b_1), u_k = drop(act_k(BN_k(u_{k-1}))) W_k^T (+ b_k), y = pad(x) + pad(BN_R(u_d)) where the
    narrower operand starts at column (|difference| + 1) // 2 of the wider one.  A normalised layer has no bias."""

    def __init__(self, desc, specs, flat, eps=1e-5, r_max=1.0, d_max=0.0, momentum=0.999, running=None):
        """running: {layer: (mean averages, std averages)} before the step, for batch renormalisation (default: the
        initial 0 / 1); its corrections r, d are constants of the backward pass."""
        self.d, self.specs, self.eps = desc, specs, eps
        self.r_max, self.d_max, self.momentum, self.running = r_max, d_max, momentum, running or {}
        self.flat = torch.tensor(np.asarray(flat, dtype=np.float64), dtype=T64, requires_grad=True)
        self.taps = {}

    def _norm_params(self, li, n):
        d = self.d
        base = d.total_weights + d.total_bias + d.layers[li].first_normalized_unit_index
        return self.flat[base:base + n], self.flat[base + d.total_normalized_units:base + d.total_normalized_units + n]

    def _bn(self, li, z):
        scale, shift = self._norm_params(li, z.shape[1])
        mu = z.mean(0)
        sd = torch.sqrt((z * z).mean(0) - mu * mu + self.eps)
        hat = (z - mu) / sd
        if self.specs[li].get("normalization") == "BATCH_RENORMALIZATION":
            n = z.shape[1]
            m0, v0 = self.running.get(li, (np.zeros(n), np.ones(n)))
            mavg = torch.tensor(np.asarray(m0, dtype=np.float64)) + self.momentum * (mu.detach() - torch.tensor(np.asarray(m0, dtype=np.float64)))
            vavg = torch.tensor(np.asarray(v0, dtype=np.float64)) + self.momentum * (sd.detach() - torch.tensor(np.asarray(v0, dtype=np.float64)))
            r = torch.clamp(sd.detach() / vavg, 1.0 / self.r_max, self.r_max)
            dd = torch.clamp((mu.detach() - mavg) / vavg, -self.d_max, self.d_max)
            hat = hat * r + dd
        return scale * hat + shift

    def _linear(self, li, x, width):
        l = self.d.layers[li]
        fan = x.shape[1]
        W = self.flat[l.first_connection_index:l.first_connection_index + width * fan].view(width, fan)
        s = x @ W.t()
        if self.specs[li].get("normalization", "NONE") == "NONE":
            s = s + self.flat[l.first_bias_connection_index:l.first_bias_connection_index + width]
        return s

    def forward(self, X, masks=None):
        specs = self.specs
        outs = {0: torch.tensor(np.asarray(X, dtype=np.float64), dtype=T64)}
        last, li = 0, 1
        while li < len(specs):
            sp = specs[li]
            if sp.get("type") == "residual":
                x = outs[last]
                u = x
                for k in range(1, sp["block_depth"] + 1):
                    m = li + k
                    if specs[m].get("type", "").endswith("pooling"):   # a pooling member: windows over the member before it
                        u, _ = _torch_pool(specs[m], u)
                        if u.requires_grad:   # not when the block hangs on the input layer and this is its first member
                            u.retain_grad()
                            self.taps[m] = u
                        continue
                    if specs[m].get("normalization", "NONE") != "NONE":
                        u = self._bn(m, u)
                    if k > 1:
                        if masks is not None and specs[m].get("dropout", "NONE") != "NONE":
                            off = self.d.layers[m].first_mask_index
                            mk = torch.tensor(masks[off:off + u.shape[1]].astype(np.float64))
                            mult = mk * (1.0 / specs[m]["keep"] if specs[m]["dropout"] == "BERNOULLI_INVERTED" else 1.0)
                            u = _DroppedActivation.apply(u, specs[m]["activation"], mult)
                        else:
                            u = _act(specs[m]["activation"], u)
                    u = self._linear(m, u, specs[m]["units"])
                    u.retain_grad()
                    self.taps[m] = u
                if sp.get("normalization", "NONE") != "NONE":
                    u = self._bn(li, u)
                na, nb = x.shape[1], u.shape[1]
                pad = (abs(na - nb) + 1) // 2
                if na >= nb:
                    y = x + torch.nn.functional.pad(u, (pad, na - nb - pad))
                else:
                    y = u + torch.nn.functional.pad(x, (pad, nb - na - pad))
                y.retain_grad()
                self.taps[li] = y
                outs[li] = y
                last = li
                li += sp["block_depth"] + 1
            else:
                s = self._linear(li, outs[last], sp["units"])
                if sp.get("normalization", "NONE") != "NONE":
                    s = self._bn(li, s)
                s.retain_grad()
                self.taps[("pre", li)] = s
                y = _act(sp["activation"], s)
                outs[li] = y
                last = li
                li += 1
        return outs[last]

    def loss(self, y, Y):
        t = torch.tensor(np.asarray(Y, dtype=np.float64), dtype=T64)
        if self.specs[-1]["activation"] == "SOFTMAX":
            return -(t * torch.log(y)).sum()
        return 0.5 * ((y - t) ** 2).sum()


CASES = {
    # equal widths, no normalisation: y = x + F(x)
    "equal_plain": ([fc(6), fc(8, "TANH"), res(2), fc(8, "TANH"), fc(8, "SIGMOID"), fc(4, "SOFTMAX")], 7),
    # block wider than the shortcut (6 -> 9, offset 2), normalised members and block-level normalisation, depth 3
    "wider_bn": ([fc(5), fc(6, "SIGMOID"), res(3, normalization="BATCH_NORMALIZATION"), fc(7, "TANH", normalization="BATCH_NORMALIZATION"),
                  fc(5, "ISRU", normalization="BATCH_NORMALIZATION"), fc(9, "TANH"), fc(3, "LINEAR")], 9),
    # block narrower than the shortcut (10 -> 7, offset 2); the block hangs directly off the input layer; first member plain,
    # second normalised; a second block follows the first (its shortcut source is the first residual layer)
    "narrower_two_blocks": ([fc(10), res(2), fc(6, "TANH"), fc(7, "ELLIOT_SYMMETRIC", normalization="BATCH_NORMALIZATION"),
                             res(1, normalization="BATCH_NORMALIZATION"), fc(13, "TANH"), fc(5, "SINE_SYMMETRIC"), fc(4, "SOFTMAX")], 8),
    # odd difference of one: offset (1 + 1) // 2 = 1, so the narrower operand lands on the LAST column
    "difference_of_one": ([fc(4), fc(5, "TANH"), res(1), fc(6, "TANH"), fc(2, "LINEAR")], 5),
    # pooling members (Forward_Pass__Residual__Layer's switch, NN/Neural_Network__Forward_Pass__OpenMP.cpp:4005-4030): an average
    # pooling between two dense members (12 -> 6), a normalised member behind it
    "average_pooling_member": ([fc(6), fc(8, "TANH"), res(3), fc(12, "TANH"), dict(type="average_pooling", kernel=2, stride=2),
                                fc(8, "SIGMOID", normalization="BATCH_NORMALIZATION"), fc(4, "SOFTMAX")], 7),
    # a max pooling as the block's LAST member (11 -> 6 with padding: narrower than the 9-wide shortcut) under a block-level
    # normalisation, and two pooling members in a row
    "max_pooling_last_member": ([fc(5), fc(9, "TANH"), res(2, normalization="BATCH_NORMALIZATION"), fc(11, "TANH"),
                                 dict(type="max_pooling", kernel=3, stride=2, padding=1), fc(3, "LINEAR")], 6),
    # a pooling layer as the block's FIRST member: the layer in front of the block receives its share and the shortcut's
    "pooling_first_member": ([fc(6), fc(12, "TANH"), res(2), dict(type="average_pooling", kernel=2, stride=2), fc(9, "TANH"), fc(3, "LINEAR")], 6),
    "max_pooling_first_member_on_the_input": ([fc(10), res(3), dict(type="max_pooling", kernel=3, stride=1, padding=1),
                                               fc(7, "SIGMOID"), fc(12, "TANH"), fc(4, "SOFTMAX")], 7),
    "two_pooling_members": ([fc(5), fc(7, "SIGMOID"), res(4), fc(16, "TANH"), dict(type="max_pooling", kernel=2, stride=2),
                             dict(type="average_pooling", kernel=3, stride=1, padding=1), fc(7, "TANH"), fc(2, "LINEAR")], 6),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_residual_forward_and_gradients_match_float64_autograd(name):
    specs, B = CASES[name]
    desc = oracle_desc(specs, B)
    rng = np.random.default_rng(zlib.crc32(name.encode()) % 1000)   # str hashes change from process to process
    w = glorot_parameters(desc, 11, bias_range=0.3)
    X = rng.normal(0, 1, (B, specs[0]["units"])).astype(np.float32)
    n_out = specs[-1]["units"]
    softmax = specs[-1]["activation"] == "SOFTMAX"
    Y = one_hot(rng.integers(0, n_out, B), n_out) if softmax else rng.normal(0, 1, (B, n_out)).astype(np.float32)
    net = OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS["CROSS_ENTROPY" if softmax else "MSE"]))
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(w)
    run_step(net, B, X, Y, update=False)
    model = TorchResidualNet(desc, specs, w)
    y = model.forward(X)
    model.loss(y, Y).backward()
    assert_close(net.download_tensor(desc.n_layers - 1, mb.TENSOR["OUTPUTS"]).reshape(B, n_out), y.detach().numpy(), 2e-5, 2e-6, "outputs")
    for key, t in model.taps.items():
        if isinstance(key, tuple):
            continue
        kind = "ERRORS"
        width = t.shape[1]
        got_v = net.download_tensor(key, mb.TENSOR["OUTPUTS"]).reshape(B, width)
        assert_close(got_v, t.detach().numpy(), 3e-5, 3e-6, "values of layer %d" % key)
        got_e = net.download_tensor(key, mb.TENSOR[kind]).reshape(B, width)
        # fp32 against float64: entries that are small differences of O(1) terms carry the terms' rounding
        assert_close(got_e, t.grad.numpy(), 3e-4, 1e-5, "delta of layer %d" % key)
    assert_close(net.download_gradient(), model.flat.grad.numpy(), 3e-4, 3e-5, "gradient")


def test_block_that_computes_zero_is_the_stack_without_it():
    """Equal widths, all-zero member weights and biases: y = x + 0, so every other layer sees exactly what it sees in
    the plain stack (an already pinned path): same outputs, same deltas, same gradients for the shared parameters; the
    members' own gradients are those of a linear probe: dW_last = delta_y^T act(u), with u = 0."""
    B = 6
    with_block = [fc(5), fc(7, "TANH"), res(2), fc(7, "TANH"), fc(7, "TANH"), fc(3, "SOFTMAX")]
    plain = [fc(5), fc(7, "TANH"), fc(3, "SOFTMAX")]
    d1, d2 = oracle_desc(with_block, B), oracle_desc(plain, B)
    w2 = glorot_parameters(d2, 3, bias_range=0.3)
    w1 = np.zeros(d1.total_parameters, dtype=np.float32)
    for a, b in ((1, 1), (5, 2)):
        n = d2.layers[b].last_connection_index - d2.layers[b].first_connection_index
        w1[d1.layers[a].first_connection_index:d1.layers[a].first_connection_index + n] = w2[d2.layers[b].first_connection_index:d2.layers[b].last_connection_index]
        nb = with_block[a]["units"]
        w1[d1.layers[a].first_bias_connection_index:d1.layers[a].first_bias_connection_index + nb] = \
            w2[d2.layers[b].first_bias_connection_index:d2.layers[b].first_bias_connection_index + nb]
    rng = np.random.default_rng(4)
    X = rng.normal(0, 1, (B, 5)).astype(np.float32)
    Y = one_hot(rng.integers(0, 3, B), 3)
    nets = []
    for d, w in ((d1, w1), (d2, w2)):
        net = OracleNetwork(d, oracle_hyper(type_loss_function=mb.LOSS["CROSS_ENTROPY"]))
        net.set_state_propagation(mb.STATE_TRAINING)
        net.upload_parameters(w)
        run_step(net, B, X, Y, update=False)
        nets.append(net)
    n1, n2 = nets
    assert np.array_equal(n1.download_tensor(2, mb.TENSOR["OUTPUTS"]), n2.download_tensor(1, mb.TENSOR["OUTPUTS"]))
    assert np.array_equal(n1.download_tensor(5, mb.TENSOR["OUTPUTS"]), n2.download_tensor(2, mb.TENSOR["OUTPUTS"]))
    g1, g2 = n1.download_gradient(), n2.download_gradient()
    for a, b in ((1, 1), (5, 2)):
        la, lb = d1.layers[a], d2.layers[b]
        n = lb.last_connection_index - lb.first_connection_index
        assert_close(g1[la.first_connection_index:la.first_connection_index + n], g2[lb.first_connection_index:lb.last_connection_index], 1e-6, 1e-7)
    # delta of the block's last member = delta of the residual layer = what the head sends down
    e_res = n1.download_tensor(2, mb.TENSOR["ERRORS"])
    assert np.array_equal(n1.download_tensor(4, mb.TENSOR["ERRORS"]), e_res)
    # zero weights: nothing flows through the members, their weight gradients see act(0) = 0 for tanh
    l4 = d1.layers[4]
    assert np.all(g1[l4.first_connection_index:l4.last_connection_index] == 0)
    assert np.all(n1.download_tensor(3, mb.TENSOR["ERRORS"]) == 0)
    # bias gradient of the last member = column sums of its delta
    assert_close(g1[l4.first_bias_connection_index:l4.first_bias_connection_index + 7], e_res.reshape(B, 7).sum(0), 1e-6, 1e-7)


def test_member_dropout_acts_on_the_input_side_and_is_not_replayed_backward():
    """Reference behaviour, not calculus: a member's dropout masks its input-side activation values (fan-in wide, mask
    shared by the batch); backward applies act' to the stored, already masked value and never the mask itself
    (Backward_Pass__Gradient__Residual__FC has no dropout step).  With tanh: a dropped unit has value 0, so act' = 1 and the
    delta passes through unscaled; a kept unit sees (1 - v^2) of the rescaled value."""
    B = 5
    specs = [fc(6), fc(8, "TANH"), res(2), fc(7, "TANH"), fc(8, "TANH", dropout="BERNOULLI_INVERTED", keep=0.5), fc(3, "LINEAR")]
    desc = oracle_desc(specs, B)
    w = glorot_parameters(desc, 5, bias_range=0.3)
    rng = np.random.default_rng(6)
    X = rng.normal(0, 1, (B, 6)).astype(np.float32)
    Y = rng.normal(0, 1, (B, 3)).astype(np.float32)
    masks = np.ones(desc.total_mask_units, dtype=np.uint8)
    off = desc.layers[4].first_mask_index
    assert desc.layers[5].first_mask_index - off == 7           # fan-in wide
    masks[off:off + 7] = [1, 0, 1, 1, 0, 0, 1]
    net = OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS["MSE"]))
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(w)
    net.upload_masks(masks)
    run_step(net, B, X, Y, update=False)
    # forward equals the float64 model with the mask applied to the activation values
    model = TorchResidualNet(desc, specs, w)
    y = model.forward(X, masks=masks)
    assert_close(net.download_tensor(5, mb.TENSOR["OUTPUTS"]).reshape(B, 3), y.detach().numpy(), 2e-5, 2e-6)
    # backward: input-side errors of member 4 from its own delta and weights, mask not replayed
    d4 = net.download_tensor(4, mb.TENSOR["ERRORS"]).reshape(B, 8).astype(np.float64)
    l4 = desc.layers[4]
    W4 = w[l4.first_connection_index:l4.last_connection_index].reshape(8, 7).astype(np.float64)
    u3 = net.download_tensor(3, mb.TENSOR["OUTPUTS"]).reshape(B, 7).astype(np.float64)
    v = np.tanh(u3) * masks[off:off + 7] * 2.0
    want = (d4 @ W4) * (1 - v * v)
    assert_close(net.download_tensor(4, mb.TENSOR["INPUT_SIDE_ERRORS"]).reshape(B, 7), want, 2e-4, 2e-6)
    # ... and they are what member 3 receives as its delta (a copy, not an accumulation)
    assert np.array_equal(net.download_tensor(3, mb.TENSOR["ERRORS"]), net.download_tensor(4, mb.TENSOR["INPUT_SIDE_ERRORS"]))
    # the weight gradient of member 4 sees the masked values
    g = net.download_gradient()
    assert_close(g[l4.first_connection_index:l4.last_connection_index].reshape(8, 7), d4.T @ v, 2e-4, 2e-6)


RECURRENT_SPECS = [fc(5), fc(6, "TANH", normalization="BATCH_NORMALIZATION", norm_before=True),
                   res(2, normalization="BATCH_NORMALIZATION"),
                   fc(7, "TANH", normalization="BATCH_NORMALIZATION"), fc(8, "SIGMOID", dropout="BERNOULLI_INVERTED", keep=0.5),
                   res(1), fc(8, "TANH"),
                   fc(3, "LINEAR")]


# the same with pooling members: a max pooling between two dense members (10 -> 5), an average pooling as the last one (6 -> 7)
RECURRENT_POOLING_SPECS = [fc(5), fc(6, "TANH"), res(4), fc(10, "TANH"), dict(type="max_pooling", kernel=2, stride=2),
                           fc(6, "SIGMOID", dropout="BERNOULLI_INVERTED", keep=0.5), dict(type="average_pooling", kernel=2, stride=1, padding=1),
                           fc(3, "LINEAR")]


def check_recurrent_depth_is_the_block_time_step_by_time_step(make_net, make_desc, rel=2e-5, abs_=2e-6, specs=None):
    """A stack of dense layers and residual blocks has no recurrence: with a recurrent depth T every layer, every batch
    normalisation (its own statistics and running averages per time step) and every dropout mask (its own per time step) works
    on the time steps one by one (Recurrent__Forward_Pass__Residual*, NN/Neural_Network__Recurrent_Forward_Pass__OpenMP.cpp:563-817;
    the backward walks them in descending order).  So time step t of the T-deep network IS the feed-forward network on
    the t-th slice of the inputs, targets, masks and normalisation parameters, and the weight gradients are the sums over the
    time steps - the feed-forward path is pinned by float64 differentiation above."""
    T, B, Bmax = 3, 5, 6
    specs = specs or RECURRENT_SPECS
    deep, flat = make_desc(specs, Bmax, T), make_desc(specs, Bmax, 1)
    rng = np.random.default_rng(17)
    X = rng.normal(0, 1, (B, T, 5)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T, 3)).astype(np.float32)
    w = glorot_parameters(deep, 17, bias_range=0.3)
    masks = (rng.uniform(0, 1, deep.total_mask_units) < 0.6).astype(np.uint8)
    assert deep.total_parameters == flat.total_parameters and deep.total_mask_units == T * flat.total_mask_units
    net = make_net(deep)
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(w)
    net.upload_masks(masks)
    net.Clear_Training_Arrays()
    run_step(net, B, X.reshape(B, T * 5), Y.reshape(B, T * 3), update=False)
    g_deep = net.download_gradient().astype(np.float64)
    g_sum = np.zeros_like(g_deep)
    last = deep.n_layers - 1
    out = net.download_tensor(last, mb.TENSOR["OUTPUTS"]).reshape(T, Bmax, 3)
    for t in range(T):
        m = np.ones(flat.total_mask_units, dtype=np.uint8)
        for li in range(flat.n_layers):
            a0 = flat.layers[li].first_mask_index
            a1 = flat.layers[li + 1].first_mask_index if li + 1 < flat.n_layers else flat.total_mask_units
            u = a1 - a0
            m[a0:a1] = masks[deep.layers[li].first_mask_index + t * u:deep.layers[li].first_mask_index + (t + 1) * u]
        one = make_net(flat)
        one.set_state_propagation(mb.STATE_TRAINING)
        one.upload_parameters(w)
        one.upload_masks(m)
        one.Clear_Training_Arrays()
        run_step(one, B, X[:, t], Y[:, t], update=False)
        assert_close(out[t, :B], one.download_tensor(last, mb.TENSOR["OUTPUTS"]).reshape(Bmax, 3)[:B], rel, abs_, what="outputs of time step %d" % t)
        for li in (1, 2, 3):   # the running averages of time step t are the feed-forward network's
            if specs[li].get("normalization", "NONE") == "NONE":
                continue
            nh = deep.layers[li + 1].first_normalized_unit_index - deep.layers[li].first_normalized_unit_index
            for kind in ("NORM_MEANS_AVERAGES", "NORM_VARIANCES_AVERAGES"):
                assert_close(net.download_tensor(li, mb.TENSOR[kind], T * nh).reshape(T, nh)[t], one.download_tensor(li, mb.TENSOR[kind], nh).reshape(nh), rel, abs_,
                             what="layer %d %s at time step %d" % (li, kind, t))
        g_sum += one.download_gradient().astype(np.float64)
    assert_close(g_deep, g_sum, 10 * rel, 10 * abs_, what="gradient = sum over the time steps")


def test_recurrent_depth_is_the_block_time_step_by_time_step():
    check_recurrent_depth_is_the_block_time_step_by_time_step(
        lambda desc: OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS["MSE"])), oracle_desc)


def test_recurrent_depth_with_pooling_members_is_the_block_time_step_by_time_step():
    check_recurrent_depth_is_the_block_time_step_by_time_step(
        lambda desc: OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS["MSE"])), oracle_desc, specs=RECURRENT_POOLING_SPECS)


def test_float64_model_reproduces_the_dropout_and_renormalisation_cases_of_the_oracle():
    """The float64 model with the reference's dropout backward and batch renormalisation (corrections held constant)
    against the oracle's gradient: the model is the arbiter of the GPU parity tests for these cases."""
    B = 16
    specs = [fc(12), fc(20, "TANH"), res(3, normalization="BATCH_RENORMALIZATION"), fc(17, "TANH", normalization="BATCH_RENORMALIZATION"),
             fc(24, "GAUSSIAN", dropout="BERNOULLI", keep=0.7), fc(15, "ISRU", normalization="BATCH_NORMALIZATION", dropout="BERNOULLI_INVERTED", keep=0.5),
             fc(6, "SOFTMAX")]
    desc = oracle_desc(specs, B)
    w = glorot_parameters(desc, 31, bias_range=0.3)
    rng = np.random.default_rng(32)
    X = rng.normal(0, 1, (B, 12)).astype(np.float32)
    Y = one_hot(rng.integers(0, 6, B), 6)
    masks = (rng.uniform(0, 1, desc.total_mask_units) < 0.6).astype(np.uint8)
    h = oracle_hyper(type_loss_function=mb.LOSS["CROSS_ENTROPY"], batch_renormalization_r_correction_maximum=1.5, batch_renormalization_d_correction_maximum=0.5)
    net = OracleNetwork(desc, h)
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(w)
    net.upload_masks(masks)
    run_step(net, B, X, Y, update=False)
    model = TorchResidualNet(desc, specs, w, r_max=1.5, d_max=0.5)
    model.loss(model.forward(X, masks=masks), Y).backward()
    assert_close(net.download_gradient(), model.flat.grad.numpy(), 5e-4, 5e-5, "gradient")
