"""GPU parity of independently recurrent layers, h[t] = AF(W x[t] + b + u * h[t-1]): the HIP library (through its C ABI)
against the CPU oracle on the same seeded inputs - layer tensors, gradient (with the self weights' slice looked at on its
own), the clipped update and the inference pass.  Tolerance rel 1e-4 / abs 1e-5."""
import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, one_hot, run_step
from tests.oracle_lib import OracleNetwork

pytestmark = pytest.mark.gpu
REL, ABS = 1e-4, 1e-5

ind = lambda units, act, **kw: dict(type="ind_rnn", units=units, activation=act, **kw)
CASES = [
    ("relu", [dict(units=12), ind(40, "RELU"), dict(units=5, activation="LINEAR")], 7, 9, 9),
    ("tanh-partial-batch", [dict(units=12), ind(33, "TANH"), dict(units=5, activation="TANH")], 6, 5, 8),
    ("stacked-with-fc-softmax-head", [dict(units=10), dict(units=24, activation="TANH"), ind(48, "RELU"), ind(32, "SIGMOID"), dict(units=6, activation="SOFTMAX")], 8, 16, 16),
    ("bn-before-dropout", [dict(units=10), ind(64, "RELU", normalization="BATCH_NORMALIZATION", norm_before=True, dropout="BERNOULLI_INVERTED", keep=0.7),
                           dict(units=4, activation="LINEAR")], 5, 16, 16),
    ("renorm-after-dropout", [dict(units=10), ind(40, "TANH", normalization="BATCH_RENORMALIZATION", norm_before=False, dropout="BERNOULLI", keep=0.8),
                              dict(units=4, activation="LINEAR")], 5, 12, 16),
    ("in-place-dropout", [dict(units=10), ind(40, "TANH", dropout="BERNOULLI_INVERTED", keep=0.6), dict(units=4, activation="LINEAR")], 6, 8, 8),
    ("between-lstm-layers", [dict(units=8), dict(type="lstm", units=12), ind(20, "RELU"), dict(type="lstm", units=6), dict(units=12, activation="LINEAR")], 5, 6, 6),
    ("single-time-step", [dict(units=12), ind(16, "RELU"), dict(units=5, activation="LINEAR")], 1, 4, 4),
    ("wide", [dict(units=64), ind(512, "RELU"), ind(512, "RELU"), dict(units=10, activation="SOFTMAX")], 12, 64, 64),
    # layers of at most 32 units over 640 rows: their weight gradients take the kernel that feeds the matrix unit from memory,
    # the self weights' gradient comes from the shares the backward time loop leaves; T > 32: two rounds of staged operands
    ("narrow-long", [dict(units=28), ind(31, "ISRLU", normalization="BATCH_NORMALIZATION", norm_before=True), ind(30, "ISRLU"), ind(17, "TANH"),
                     dict(units=10, activation="SOFTMAX")], 8, 80, 80),
    ("narrow-long-partial-batch", [dict(units=28), ind(31, "ISRLU"), ind(32, "RELU"), dict(units=10, activation="SOFTMAX")], 8, 70, 80),
    ("narrow-many-steps", [dict(units=9), ind(24, "ISRLU"), ind(11, "SIGMOID"), dict(units=3, activation="LINEAR")], 40, 16, 16),
]


def _self_weights(desc, w, seed):
    rng = np.random.default_rng(seed)
    for i in range(1, desc.n_layers):
        l = desc.layers[i]
        if l.type_layer == mb.LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT:
            w[l.last_connection_index - l.n_units:l.last_connection_index] = rng.uniform(-0.95, 0.95, l.n_units).astype(np.float32)
    return w


@pytest.mark.parametrize("name,specs,T,B,Bmax", CASES, ids=[c[0] for c in CASES])
def test_ind_rnn_stack_parity(name, specs, T, B, Bmax):
    desc = mb.make_desc(specs, Bmax, T)
    head = specs[-1]["activation"]
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["ADAM"], learning_rate=0.05,
                         type_loss_function=mb.LOSS["CROSS_ENTROPY" if head == "SOFTMAX" else "MSE"])
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h)
    w = _self_weights(desc, glorot_parameters(desc, 11, bias_range=0.3), 11)
    rng = np.random.default_rng(11)
    masks = (rng.uniform(0, 1, desc.total_mask_units) < 0.7).astype(np.uint8)
    n_in, n_out = specs[0]["units"], specs[-1]["units"]
    X = rng.normal(0, 1, (B, T * n_in)).astype(np.float32)
    Y = (one_hot(rng.integers(0, n_out, B * T), n_out).reshape(B, T * n_out) if head == "SOFTMAX" else rng.normal(0, 1, (B, T * n_out)).astype(np.float32))
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.upload_masks(masks)
        n.Clear_Training_Arrays()
    for step in range(2):
        for n in (gpu, cpu):
            n.Reset__Loss()
            run_step(n, B, X, Y, update=False)
        for li in range(1, desc.n_layers):
            l = desc.layers[li]
            if l.type_layer == mb.LAYER_LSTM:
                continue
            W = l.n_units
            for kind in ("OUTPUTS", "ERRORS"):
                a = gpu.download_tensor(li, mb.TENSOR[kind], T * Bmax * W).reshape(T, Bmax, W)[:, :B]
                b = cpu.download_tensor(li, mb.TENSOR[kind], T * Bmax * W).reshape(T, Bmax, W)[:, :B]
                assert_close(a, b, REL, ABS * max(1.0, float(np.abs(b).max())), what="step %d layer %d %s" % (step, li, kind))
        g, want = gpu.download_gradient(), cpu.download_gradient()
        scale = max(1.0, float(np.abs(want).max()))
        assert_close(g, want, REL, ABS * scale, what="gradient step %d" % step)
        for li in range(1, desc.n_layers):
            l = desc.layers[li]
            if l.type_layer != mb.LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT:
                continue
            sl = slice(l.last_connection_index - l.n_units, l.last_connection_index)
            if T > 1:
                assert np.abs(want[sl]).max() > 1e-3, "self-weight gradient vacuous"
            else:
                assert not want[sl].any() and not g[sl].any()            # no previous time step, no gradient
            assert_close(g[sl], want[sl], REL, ABS * scale, what="self-weight gradient layer %d step %d" % (li, step))
        for n in (gpu, cpu):
            n.Update_Parameter(B, B)
        got, ref = gpu.download_parameters(), cpu.download_parameters()
        for li in range(1, desc.n_layers):
            l = desc.layers[li]
            if l.type_layer != mb.LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT:
                continue
            sl = slice(l.last_connection_index - l.n_units, l.last_connection_index)
            assert got[sl].max() <= l.constraint_recurrent_weight_upper_bound and got[sl].min() >= l.constraint_recurrent_weight_lower_bound
            # Adam's first steps move every entry by about the learning rate whatever the gradient's size: compare where the
            # two sides agree on the gradient's sign beyond rounding
            firm = np.abs(want[sl]) > 1e-4 * scale
            assert_close(got[sl][firm], ref[sl][firm], REL, ABS, what="self weights after the update, layer %d" % li)
        gpu.upload_parameters(ref)
    assert gpu.get_loss().loss_values == pytest.approx(cpu.get_loss().loss_values, rel=1e-4)
    # inference pass (running averages, dropout scaling) from the same state
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_INFERENCE)
        n.Forward_Pass(B, X)
    lo = desc.n_layers - 1
    a = gpu.download_tensor(lo, mb.TENSOR["OUTPUTS"], T * Bmax * n_out).reshape(T, Bmax, n_out)[:, :B]
    b = cpu.download_tensor(lo, mb.TENSOR["OUTPUTS"], T * Bmax * n_out).reshape(T, Bmax, n_out)[:, :B]
    assert_close(a, b, REL, ABS, what="inference outputs")


def test_self_weight_clip_uses_the_layer_bounds():
    specs = [dict(units=6), ind(24, "RELU", recurrent_bounds=(-0.25, 0.5)), dict(units=3, activation="LINEAR")]
    B, T = 4, 5
    desc = mb.make_desc(specs, B, T)
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["GD"], learning_rate=1e-3, type_loss_function=mb.LOSS["MSE"])
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h)
    w = _self_weights(desc, glorot_parameters(desc, 4, bias_range=0.3), 4)
    rng = np.random.default_rng(4)
    X, Y = rng.normal(0, 1, (B, T * 6)).astype(np.float32), rng.normal(0, 1, (B, T * 3)).astype(np.float32)
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
        run_step(n, B, X, Y)
    got, ref = gpu.download_parameters(), cpu.download_parameters()
    l = desc.layers[1]
    u = got[l.last_connection_index - 24:l.last_connection_index]
    assert u.min() >= -0.25 and u.max() <= 0.5 and (u == 0.5).any() and (u == -0.25).any()
    assert_close(got, ref, REL, ABS, what="parameters")


def test_refusals():
    with pytest.raises(mb.MyeaError):      # softmax on a recurrent hidden layer
        mb.HipNetwork(mb.make_desc([dict(units=6), ind(8, "SOFTMAX"), dict(units=3, activation="LINEAR")], 4, 3))
    with pytest.raises(ValueError):        # as the output layer
        mb.make_desc([dict(units=6), ind(8, "TANH")], 4, 3)


def test_gradient_sums_of_many_layers_follow_the_batch_size():
    """A narrow normalised stack over 640 rows adds its per-layer partial results - the normalisations' per-time-step shares,
    the narrow weight gradients' slabs, the self weights' per-example shares - in one launch per pass when the batch fills the
    network's rows, and layer by layer when it does not: full, partial and full batches in turn give the oracle's gradient each
    time."""
    specs = [dict(units=20), ind(31, "ISRLU", normalization="BATCH_NORMALIZATION", norm_before=True),
             ind(29, "TANH", normalization="BATCH_NORMALIZATION", norm_before=True), dict(units=7, activation="LINEAR")]
    T, Bmax = 8, 80
    desc = mb.make_desc(specs, Bmax, T)
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["GD"], learning_rate=1e-5, type_loss_function=mb.LOSS["MSE"])
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h)
    w = _self_weights(desc, glorot_parameters(desc, 21, bias_range=0.3), 21)
    rng = np.random.default_rng(21)
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
    for step, B in enumerate((80, 64, 80, 80, 33)):
        X = rng.normal(0, 1, (B, T * 20)).astype(np.float32)
        Y = rng.normal(0, 1, (B, T * 7)).astype(np.float32)
        for n in (gpu, cpu):
            n.Reset__Loss()
            run_step(n, B, X, Y, update=False)
        g, want = gpu.download_gradient(), cpu.download_gradient()
        assert 1e-3 < float(np.abs(want).max()) < 1e4, "the steps stay small: the gradient is neither vacuous nor blown up"
        assert_close(g, want, REL, ABS * max(1.0, float(np.abs(want).max())), what="gradient, step %d with %d examples" % (step, B))
        for n in (gpu, cpu):
            n.Update_Parameter(B, B)
        gpu.upload_parameters(cpu.download_parameters())
