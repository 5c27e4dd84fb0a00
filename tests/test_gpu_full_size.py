"""The benchmark configurations at their full sizes.

First the headline configuration (fully-connected 4096 x 4 -> 1000 softmax, batch 1024, Adam: 71.2 M parameters) through
properties that do not depend on the size: every stage is recomputed in float64 on sampled entries straight from the tensors
the device holds (a forward unit is a dot product of the layer below, a delta is the weighted deltas above times the
activation's derivative, a weight gradient entry is a column-by-column product over the batch, a bias gradient a column
sum), a second pass without an update doubles the gradient exactly, and the Adam step follows the scalar closed form on
every 5th parameter.  Then the same configuration, the two-direction LSTM-1024 and the normalised FC-2048 stack against the
CPU oracle itself, one whole step each (the oracle's step takes 4 to 20 s on the host's cores).
Tolerance: rel 1e-4 / abs 1e-5 (of the vector's largest magnitude for sums over 1024 or 4096 terms in the sampled checks)."""
import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, one_hot
from tests.full_size_support import GradientTerms, assert_first_adam_type_step_matches, assert_sums_match

pytestmark = pytest.mark.gpu

WIDTHS = [4096, 4096, 4096, 4096, 4096, 1000]
B = 1024
SAMPLES = 48


def _weights(desc, w, li):
    l = desc.layers[li]
    W = w[l.first_connection_index:l.last_connection_index].reshape(WIDTHS[li], WIDTHS[li - 1])
    b = w[l.first_bias_connection_index:l.first_bias_connection_index + WIDTHS[li]]
    return W, b


@pytest.fixture(scope="module")
def trained():
    specs = [dict(units=4096)] + [dict(units=4096, activation="RELU")] * 4 + [dict(units=1000, activation="SOFTMAX")]
    desc = mb.make_desc(specs, B)
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["ADAM"], type_loss_function=mb.LOSS["CROSS_ENTROPY"])
    net = mb.HipNetwork(desc, h)
    w = glorot_parameters(desc, 11, bias_range=0.2)
    rng = np.random.default_rng(11)
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(w)
    net.Clear_Training_Arrays()
    X = rng.normal(0, 1, (B, 4096)).astype(np.float32)
    Y = one_hot(rng.integers(0, 1000, B), 1000)
    net.Forward_Pass(B, X)
    net.Compute__Error(B, Y)
    net.Backward_Pass__Update_Derivative_Weight(B)
    outs = [X] + [net.download_tensor(li, mb.TENSOR["OUTPUTS"]).reshape(B, WIDTHS[li]) for li in range(1, 6)]
    deltas = [None] + [net.download_tensor(li, mb.TENSOR["ERRORS"]).reshape(B, WIDTHS[li]) for li in range(1, 6)]
    g1 = net.download_gradient()
    return dict(net=net, desc=desc, h=h, w=w, X=X, Y=Y, outs=outs, deltas=deltas, g1=g1, rng=rng)


def test_forward_units_are_dot_products_of_the_layer_below(trained):
    desc, w, outs, rng = trained["desc"], trained["w"], trained["outs"], trained["rng"]
    for li in range(1, 5):
        W, b = _weights(desc, w, li)
        rows, cols = rng.integers(0, B, SAMPLES), rng.integers(0, WIDTHS[li], SAMPLES)
        want = np.einsum("sk,sk->s", outs[li - 1][rows].astype(np.float64), W[cols].astype(np.float64)) + b[cols]
        want = np.maximum(want, 0.0)
        assert_close(outs[li][rows, cols], want, 1e-4, 1e-5 * max(1.0, float(np.abs(want).max())), what="layer %d outputs" % li)
    W, b = _weights(desc, w, 5)                      # the head: whole softmax rows
    rows = rng.integers(0, B, 8)
    z = outs[4][rows].astype(np.float64) @ W.astype(np.float64).T + b
    e = np.exp(z - z.max(axis=1, keepdims=True))
    assert_close(outs[5][rows], e / e.sum(axis=1, keepdims=True), 1e-4, 1e-6, what="softmax rows")
    assert_close(outs[5].sum(axis=1), np.ones(B), 1e-5, 0, what="softmax rows sum to one")


def test_deltas_follow_the_chain_rule(trained):
    desc, w, outs, deltas, Y, rng = trained["desc"], trained["w"], trained["outs"], trained["deltas"], trained["Y"], trained["rng"]
    assert_close(deltas[5], outs[5].astype(np.float64) - Y, 1e-5, 1e-7, what="softmax + cross-entropy delta = y - t")
    for li in range(4, 0, -1):
        W_up, _ = _weights(desc, w, li + 1)
        rows, cols = rng.integers(0, B, SAMPLES), rng.integers(0, WIDTHS[li], SAMPLES)
        want = np.einsum("so,os->s", deltas[li + 1][rows].astype(np.float64), W_up[:, cols].astype(np.float64)) * (outs[li][rows, cols] > 0)
        scale = float(np.abs(deltas[li]).max())
        assert_close(deltas[li][rows, cols], want, 1e-4, 1e-5 * scale, what="layer %d deltas" % li)


def test_gradient_entries_are_products_over_the_batch(trained):
    desc, outs, deltas, g1, rng = trained["desc"], trained["outs"], trained["deltas"], trained["g1"], trained["rng"]
    for li in range(1, 6):
        l = desc.layers[li]
        G = g1[l.first_connection_index:l.last_connection_index].reshape(WIDTHS[li], WIDTHS[li - 1])
        o, i = rng.integers(0, WIDTHS[li], SAMPLES), rng.integers(0, WIDTHS[li - 1], SAMPLES)
        want = np.einsum("bs,bs->s", deltas[li][:, o].astype(np.float64), outs[li - 1][:, i].astype(np.float64))
        assert_close(G[o, i], want, 1e-4, 1e-5 * float(np.abs(G).max()), what="layer %d weight gradient" % li)
        gb = g1[l.first_bias_connection_index:l.first_bias_connection_index + WIDTHS[li]]
        want_b = deltas[li].astype(np.float64).sum(axis=0)
        assert_close(gb, want_b, 1e-4, 1e-5 * float(np.abs(want_b).max()), what="layer %d bias gradient" % li)


def test_second_pass_doubles_the_gradient_then_adam_follows_its_closed_form(trained):
    net, desc, h, w, X, Y, g1 = (trained[k] for k in ("net", "desc", "h", "w", "X", "Y", "g1"))
    net.Forward_Pass(B, X)
    net.Compute__Error(B, Y)
    net.Backward_Pass(B)
    net.Update_Derivative_Weight(B)                 # the two separate calls on top of the combined one
    g2 = net.download_gradient()
    assert np.array_equal(g2, g1 + g1)
    net.Update_Parameter(B, B)
    w1 = net.download_parameters()
    assert not net.download_gradient().any(), "the update leaves the gradient zeroed"
    # Update_Parameters__Adam (NN/Neural_Network__Adam.cpp:43-97) at its first step from zero moments, float64
    sel = slice(0, desc.total_parameters, 5)
    g = g2[sel].astype(np.float64)
    b1, b2, eps = float(h.adam_beta1), float(h.adam_beta2), float(h.adam_epsilon)
    lr_t = float(h.adam_learning_rate) * (np.sqrt(1.0 - b2) / (1.0 - b1) if h.use_adam_bias_correction else 1.0)
    m, v = (1.0 - b1) * g, (1.0 - b2) * g * g
    want = w[sel].astype(np.float64) - lr_t * m / (np.sqrt(v) + eps)
    # a first Adam step has the size lr_t (1 - b1) / sqrt(1 - b2) whatever |g| is; where the gradient is rounding noise
    # its direction is the noise's, so those entries are only held to that size
    solid = np.abs(g) > 1e-6
    assert solid.mean() > 0.2
    assert_close(w1[sel][solid], want[solid], 1e-4, 1e-6, what="Adam step")
    full_step = lr_t * (1.0 - b1) / np.sqrt(1.0 - b2)
    assert float(np.abs(w1[sel][~solid] - w[sel][~solid]).max(initial=0.0)) <= 1.05 * full_step
    assert_close(net.download_optimizer_state(mb.OPT_STATE["FIRST_MOMENT"])[sel], m, 1e-5, 1e-12, what="first moment")
    assert_close(net.download_optimizer_state(mb.OPT_STATE["SECOND_MOMENT"])[sel], v, 1e-5, 1e-20, what="second moment")


def test_the_one_call_step_updates_the_wide_layers_early_and_equals_the_separate_calls(trained):
    """Backward_Pass + Update_Derivative_Weight + Update_Parameter as one call: the four 4096 x 4096 layers take their Adam step on
    the second stream beside the contractions below them (five update launches a step: four layers, then the head with the
    biases), and parameters and moments equal those of the separate calls bit for bit"""
    desc, h, w, X, Y = (trained[k] for k in ("desc", "h", "w", "X", "Y"))
    nets = [mb.HipNetwork(desc, h) for _ in range(2)]
    for n in nets:
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
    apart, one = nets
    one.profile_enable(True)
    for step in range(2):
        for n in nets:
            n.Forward_Pass(B, X)
            n.Compute__Error(B, Y)
        apart.Backward_Pass__Update_Derivative_Weight(B)
        apart.Update_Parameter(B, 8 * B)
        one.Backward_Pass__Update_Derivative_Weight__Update_Parameter(B, 8 * B)
    assert one.profile_read(3)[0] == 2 * 5
    one.profile_enable(False)
    assert np.array_equal(apart.download_parameters(), one.download_parameters())
    for kind in ("FIRST_MOMENT", "SECOND_MOMENT"):
        assert np.array_equal(apart.download_optimizer_state(mb.OPT_STATE[kind]), one.download_optimizer_state(mb.OPT_STATE[kind])), kind
    assert not one.download_gradient().any()
    for n in nets:
        n.close()


def test_config5_full_size_sampled_examples_and_batch_additivity():
    """Bidirectional LSTM, 1024 cells per direction, input 256, T = 512, batch 64, per-step 32-class softmax (the largest
    recurrent configuration).  Without normalisation an example's forward values and deltas do not depend on the rest of
    the batch: two of the 64 examples are walked by the CPU oracle alone (a batch of two) and compared at every time step,
    both directions.  The weight gradient is a sum over examples: the full batch against its two halves accumulated."""
    import os
    from tests.oracle_lib import OracleNetwork
    T, Bfull, picks = 512, 64, [5, 41]
    specs = [dict(units=256), dict(type="lstm", units=1024, bidirectional=True), dict(units=32, activation="SOFTMAX")]
    hyper = dict(type_optimizer_function=mb.OPTIMIZER["ADABOUND"], type_loss_function=mb.LOSS["CROSS_ENTROPY"])
    desc = mb.make_desc(specs, Bfull, T)
    small = mb.make_desc(specs, len(picks), T)
    assert desc.total_parameters == small.total_parameters
    gpu = mb.HipNetwork(desc, mb.default_hyper(**hyper))
    cpu = OracleNetwork(small, mb.default_hyper(**hyper), threads=min(2, os.cpu_count() or 1))
    w = glorot_parameters(desc, 17, bias_range=0.2)
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
    rng = np.random.default_rng(17)
    X = rng.uniform(-1, 1, (Bfull, T * 256)).astype(np.float32)
    Y = one_hot(rng.integers(0, 32, Bfull * T), 32).reshape(Bfull, T * 32)

    def step(net, B, x, y):
        net.Forward_Pass(B, x)
        net.Compute__Error(B, y)
        net.Backward_Pass(B)
        net.Update_Derivative_Weight(B)

    step(gpu, Bfull, X, Y)
    step(cpu, len(picks), np.ascontiguousarray(X[picks]), np.ascontiguousarray(Y[picks]))
    for li, width in ((1, 1024), (2, 32)):
        for kind in ("OUTPUTS", "ERRORS"):
            a = gpu.download_tensor(li, mb.TENSOR[kind]).reshape(T, Bfull, width)[:, picks]
            b = np.asarray(cpu.download_tensor(li, mb.TENSOR[kind])).reshape(T, len(picks), width)
            assert_close(a, b, 1e-4, 1e-5 * max(1.0, float(np.abs(b).max())), what="layer %d %s of examples %r" % (li, kind, picks))
    for direction in (0, mb.TENSOR["DIRECTION_BACKWARD"]):
        for kind in ("LSTM_CELL_STATE", "LSTM_DELTA_CELL_STATE", "LSTM_DELTA_CELL_INPUT"):
            a = gpu.download_tensor(1, mb.TENSOR[kind] | direction).reshape(T, Bfull, 1024)[:, picks]
            b = np.asarray(cpu.download_tensor(1, mb.TENSOR[kind] | direction)).reshape(T, len(picks), 1024)
            assert_close(a, b, 1e-4, 1e-5 * max(1.0, float(np.abs(b).max())), what="%s direction %d" % (kind, int(direction != 0)))
    g_full = gpu.download_gradient().astype(np.float64)
    gpu.Clear_Training_Arrays()
    half = Bfull // 2
    step(gpu, half, np.ascontiguousarray(X[:half]), np.ascontiguousarray(Y[:half]))
    step(gpu, half, np.ascontiguousarray(X[half:]), np.ascontiguousarray(Y[half:]))
    g_halves = gpu.download_gradient().astype(np.float64)
    scale = float(np.abs(g_full).max())
    assert scale > 0
    assert float(np.abs(g_full - g_halves).max()) <= 1e-4 * scale


def _relu_stack_float64(desc, w, X, Y=None):
    """float64 model of the ReLU stack with a softmax head: pre-activations and outputs per layer; with Y also the deltas and
    the flat gradient (softmax + cross-entropy: delta = y - t, no 1 / batch factor, as Compute__Error leaves it)"""
    w64 = w.astype(np.float64)
    outs, pres = [X.astype(np.float64)], [None]
    mats = [None]
    for li in range(1, 6):
        l = desc.layers[li]
        Wm = w64[l.first_connection_index:l.last_connection_index].reshape(WIDTHS[li], WIDTHS[li - 1])
        mats.append(Wm)
        z = outs[-1] @ Wm.T + w64[l.first_bias_connection_index:l.first_bias_connection_index + WIDTHS[li]]
        pres.append(z)
        if li < 5:
            outs.append(np.maximum(z, 0.0))
        else:
            e = np.exp(z - z.max(axis=1, keepdims=True))
            outs.append(e / e.sum(axis=1, keepdims=True))
    if Y is None:
        return pres, outs
    deltas = [None] * 6
    deltas[5] = outs[5] - Y
    g = np.zeros(desc.total_parameters)
    mags = np.zeros(desc.total_parameters)
    for li in range(5, 0, -1):
        l = desc.layers[li]
        g[l.first_connection_index:l.last_connection_index] = (deltas[li].T @ outs[li - 1]).ravel()
        mags[l.first_connection_index:l.last_connection_index] = (np.abs(deltas[li]).T @ np.abs(outs[li - 1])).ravel()
        b0 = l.first_bias_connection_index
        g[b0:b0 + WIDTHS[li]] = deltas[li].sum(axis=0)
        mags[b0:b0 + WIDTHS[li]] = np.abs(deltas[li]).sum(axis=0)
        if li > 1:
            deltas[li - 1] = (deltas[li] @ mats[li]) * (pres[li - 1] > 0)
    return pres, outs, deltas, g, mags


def test_config2_full_size_one_step_against_the_oracle():
    """One whole step of the headline configuration on the device and on the CPU oracle: every layer's outputs and deltas, the
    whole gradient, then the Adam-stepped parameters and both moments.

    ReLU' is a step function of the pre-activation: a unit whose pre-activation lies within fp32 rounding (about 5e-7 here)
    of zero gets derivative 0 from one fp32 implementation and 1 from another, and that one unit changes its example's whole
    row of deltas in every layer below and with it every entry of those layers' gradients by 1e-4 of their size (measured:
    three such units among 4.2 M in the top hidden layer moved 79 % of the first layer's gradient entries out of tolerance -
    the oracle's, by float64).  A batch of N(0, 1) inputs has one or two such units per layer.  The examples here are drawn
    N(0, 1) and kept when, in a float64 forward pass, every hidden pre-activation stays at least 1e-5 away from zero (about
    13 % are redrawn): then the derivative is the same in any fp32 implementation and all tensors are comparable entry by
    entry.  What is summed over the batch is held as tests/full_size_support.py says, against the float64 model's gradient."""
    import os
    from tests.oracle_lib import OracleNetwork
    specs = [dict(units=4096)] + [dict(units=4096, activation="RELU")] * 4 + [dict(units=1000, activation="SOFTMAX")]
    desc = mb.make_desc(specs, B)
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["ADAM"], type_loss_function=mb.LOSS["CROSS_ENTROPY"])
    threads = min(16, os.cpu_count() or 1)
    gpu, cpu, twin = mb.HipNetwork(desc, h), OracleNetwork(desc, h, threads=threads), OracleNetwork(desc, h, threads=threads)
    w = glorot_parameters(desc, 29, bias_range=0.2)
    rng = np.random.default_rng(29)
    X = np.zeros((0, 4096), dtype=np.float32)
    while len(X) < B:
        cand = rng.normal(0, 1, (B // 2, 4096)).astype(np.float32)
        pres, _ = _relu_stack_float64(desc, w, cand)
        clear = np.min([np.abs(pres[li]).min(axis=1) for li in range(1, 5)], axis=0) >= 1e-5
        X = np.concatenate([X, cand[clear]])[:B]
    Y = one_hot(rng.integers(0, 1000, B), 1000)
    for n in (gpu, cpu, twin):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
    for n in (gpu, cpu):
        n.Forward_Pass(B, X)
        n.Compute__Error(B, Y)
        n.Backward_Pass(B)
        n.Update_Derivative_Weight(B)
    pres, outs, deltas, g64, mags = _relu_stack_float64(desc, w, X, Y)
    for li in range(1, 6):
        for kind, exact in (("OUTPUTS", outs[li]), ("ERRORS", deltas[li])):
            a, b = gpu.download_tensor(li, mb.TENSOR[kind]), np.asarray(cpu.download_tensor(li, mb.TENSOR[kind]))
            assert_close(a, b, 1e-4, 1e-5, what="layer %d %s against the oracle" % (li, kind))
            assert_close(a, exact.ravel(), 1e-4, 1e-5, what="layer %d %s against float64" % (li, kind))
            if kind == "OUTPUTS" and li < 5:
                assert np.array_equal(a == 0, b == 0), "layer %d: the same units are rectified on both sides" % li
    g_gpu, g_cpu = gpu.download_gradient(), cpu.download_gradient()
    report = {}
    assert_sums_match(g_gpu, g_cpu, lambda idx: (g64[idx], mags[idx]), "gradient", report=report)
    print("config 2 gradient:", report["gradient"])
    print("config 2 update:", assert_first_adam_type_step_matches(gpu, cpu, twin, w, g_gpu, g_cpu, B, h, ("FIRST_MOMENT", "SECOND_MOMENT"), "Adam step"))
    assert gpu.get_hyper().optimizer_time_step == 1.0 and not gpu.download_gradient().any()
    for n in (gpu, cpu, twin):
        n.close()


def test_config5_full_size_one_step_against_the_oracle():
    """Bidirectional LSTM, 1024 cells per direction, input 256, T = 512, batch 64, per-step 32-class softmax cross-entropy,
    clipping at norm 1, AdaBound: the whole batch through the CPU oracle once (about 20 s on 16 cores) - outputs and deltas of
    both layers, cell states and the gate deltas of both directions at every time step, the whole gradient (entries outside the
    tolerance of the oracle go to a float64 sum of their 32768 products, tests/full_size_support.py), the clipped AdaBound step
    and both moments."""
    import os
    from tests.oracle_lib import OracleNetwork
    T, Bn = 512, 64
    specs = [dict(units=256), dict(type="lstm", units=1024, bidirectional=True), dict(units=32, activation="SOFTMAX")]
    hyper = dict(type_optimizer_function=mb.OPTIMIZER["ADABOUND"], type_loss_function=mb.LOSS["CROSS_ENTROPY"], use_clip_gradient=1, clip_gradient=1.0)
    desc = mb.make_desc(specs, Bn, T)
    h = mb.default_hyper(**hyper)
    threads = min(16, os.cpu_count() or 1)
    gpu, cpu, twin = mb.HipNetwork(desc, h), OracleNetwork(desc, h, threads=threads), OracleNetwork(desc, h, threads=threads)
    w = glorot_parameters(desc, 19, bias_range=0.2)
    rng = np.random.default_rng(19)
    X = rng.uniform(-1, 1, (Bn, T * 256)).astype(np.float32)
    Y = one_hot(rng.integers(0, 32, Bn * T), 32).reshape(Bn, T * 32)
    for n in (gpu, cpu, twin):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
    for n in (gpu, cpu):
        n.Reset__Loss()
        n.Forward_Pass(Bn, X)
        n.Compute__Error(Bn, Y)
        n.Backward_Pass(Bn)
        n.Update_Derivative_Weight(Bn)
    for li in (1, 2):
        for kind in ("OUTPUTS", "ERRORS"):
            assert_close(gpu.download_tensor(li, mb.TENSOR[kind]), np.asarray(cpu.download_tensor(li, mb.TENSOR[kind])), 1e-4, 1e-5, what="layer %d %s" % (li, kind))
    for direction in (0, mb.TENSOR["DIRECTION_BACKWARD"]):
        for kind in ("LSTM_CELL_STATE", "LSTM_CELL_OUTPUT", "LSTM_DELTA_CELL_STATE", "LSTM_DELTA_CELL_INPUT", "LSTM_DELTA_INPUT_GATE", "LSTM_DELTA_FORGET_GATE", "LSTM_DELTA_OUTPUT_GATE"):
            assert_close(gpu.download_tensor(1, mb.TENSOR[kind] | direction), np.asarray(cpu.download_tensor(1, mb.TENSOR[kind] | direction)), 1e-4, 1e-5,
                         what="%s direction %d" % (kind, int(direction != 0)))
    lg, lc = gpu.get_loss(), cpu.get_loss()
    assert lg.number_loss == lc.number_loss and lg.loss_values == pytest.approx(lc.loss_values, rel=1e-5)
    g_gpu, g_cpu = gpu.download_gradient(), cpu.download_gradient()
    report = {}
    assert_sums_match(g_gpu, g_cpu, GradientTerms(desc, cpu, X, Bn).exact, "gradient", report=report)
    print("config 5 gradient:", report["gradient"])
    print("config 5 update:", assert_first_adam_type_step_matches(gpu, cpu, twin, w, g_gpu, g_cpu, Bn, h, ("FIRST_MOMENT", "SECOND_MOMENT"), "clipped AdaBound step"))
    for n in (gpu, cpu, twin):
        n.close()


def test_config4_full_size_forward_against_the_oracle_backward_layer_by_layer():
    """8 x [FC 2048, BatchNorm before the activation, ReLU, inverted Bernoulli dropout keep 0.5] -> 100-class softmax,
    batch 512, Nesterov, at full size.  The forward pass is compared with the CPU oracle directly (the host's cores share
    the examples), zero patterns included.  The backward pass is not comparable that way, and says so: eight layers up
    the two fp32 forward passes differ by 1e-5, a handful of the million pre-activations per layer lie that near to zero,
    ReLU' of those differs between ANY two fp32 implementations, and BatchNorm's backward spreads each such unit over its
    whole column and from there over everything below.  So every layer's backward step is recomputed in float64 from the
    device's own forward state and the device's own delta of the layer above (sampled columns, all 512 rows), the
    gradient from the device's own deltas, and the Nesterov step by the oracle fed the device's gradient."""
    import os
    from tests.oracle_lib import OracleNetwork
    width, depth, Bn = 2048, 8, 512
    layer = dict(units=width, activation="RELU", normalization="BATCH_NORMALIZATION", norm_before=True, dropout="BERNOULLI_INVERTED", keep=0.5)
    specs = [dict(units=width)] + [dict(layer) for _ in range(depth)] + [dict(units=100, activation="SOFTMAX")]
    kw = dict(type_optimizer_function=mb.OPTIMIZER["GD"], use_Nesterov=1, learning_rate=0.01, learning_momentum=0.9, type_loss_function=mb.LOSS["CROSS_ENTROPY"])
    desc = mb.make_desc(specs, Bn)
    h = mb.default_hyper(**kw)
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h, threads=min(16, os.cpu_count() or 1))
    w = glorot_parameters(desc, 23)
    rng = np.random.default_rng(23)
    masks = (rng.uniform(0, 1, desc.total_mask_units) < 0.5).astype(np.uint8)
    X = rng.normal(0, 1, (Bn, width)).astype(np.float32)
    Y = one_hot(rng.integers(0, 100, Bn), 100)
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
        n.upload_masks(masks)
        n.Forward_Pass(Bn, X)
        n.Compute__Error(Bn, Y)
    gpu.Backward_Pass__Update_Derivative_Weight(Bn)
    widths = [width] * (depth + 1) + [100]
    outs, hats, deltas = [X], [None], [None]
    for li in range(1, desc.n_layers):
        H = widths[li]
        for kind in ("OUTPUTS", "SUMMATIONS") + (("NORM_HATS",) if li <= depth else ()):
            a = gpu.download_tensor(li, mb.TENSOR[kind], Bn * H)
            b = np.asarray(cpu.download_tensor(li, mb.TENSOR[kind], Bn * H))
            assert_close(a, b, 1e-4, 1e-5 * max(1.0, float(np.abs(b).max())), what="layer %d %s" % (li, kind))
            if kind == "OUTPUTS" and li <= depth:
                differ = int(np.count_nonzero((a == 0) != (b == 0)))
                assert differ <= 16, "layer %d: %d units rectified or dropped on one side only" % (li, differ)
        outs.append(gpu.download_tensor(li, mb.TENSOR["OUTPUTS"], Bn * H).reshape(Bn, H))
        hats.append(gpu.download_tensor(li, mb.TENSOR["NORM_HATS"], Bn * H).reshape(Bn, H).astype(np.float64) if li <= depth else None)
        deltas.append(gpu.download_tensor(li, mb.TENSOR["ERRORS"], Bn * H).reshape(Bn, H))
    assert_close(deltas[-1], outs[-1].astype(np.float64) - Y, 1e-5, 1e-7, what="head delta = y - t")
    g = gpu.download_gradient()
    scales = w[desc.total_weights + desc.total_bias:desc.total_weights + desc.total_bias + 2 * desc.total_normalized_units]   # scales, then shifts
    for li in range(depth, 0, -1):
        l, up = desc.layers[li], desc.layers[li + 1]
        cols = rng.choice(width, 24, replace=False)
        W_up = w[up.first_connection_index:up.last_connection_index].reshape(widths[li + 1], width)
        # Backward_Pass__FC: delta of the layer's output; the backward pass has no dropout operator and ReLU' reads the
        # pre-activation (here the normalised value), so a dropped unit with a positive pre-activation passes its delta on
        d_out = deltas[li + 1].astype(np.float64) @ W_up[:, cols].astype(np.float64)
        shift = scales[desc.total_normalized_units + l.first_normalized_unit_index + cols].astype(np.float64)
        pre = hats[li][:, cols] * scales[l.first_normalized_unit_index + cols].astype(np.float64) + shift
        kept = masks[l.first_mask_index + cols] != 0
        positive = np.where(kept[None, :], outs[li][:, cols] > 0, pre >= 0)      # kept units: exactly what the device rectified
        gact = d_out * positive
        # Backward_Pass__Batch_Normalization (NN/Neural_Network__Backward_Pass__OpenMP.cpp:1346-1467) with x - mean = hat * sigma
        sigma = gpu.download_tensor(li, mb.TENSOR["NORM_VARIANCES"], width)[cols].astype(np.float64)
        scale = scales[l.first_normalized_unit_index + cols].astype(np.float64)
        xh = hats[li][:, cols]
        gs = gact * scale
        d_mean = (-gs / sigma).sum(axis=0)
        d_var = (-gs * xh / sigma).sum(axis=0)
        want = gs / sigma + d_var * xh / Bn + d_mean / Bn
        assert_close(deltas[li][:, cols], want, 1e-4, 1e-5 * float(np.abs(want).max()), what="layer %d deltas" % li)
        base = desc.total_weights + desc.total_bias + l.first_normalized_unit_index
        assert_close(g[base + cols], (gact * xh).sum(axis=0), 1e-4, 1e-5 * float(np.abs(gact).sum(axis=0).max()), what="layer %d scale gradient" % li)
        assert_close(g[base + desc.total_normalized_units + cols], gact.sum(axis=0), 1e-4, 1e-5 * float(np.abs(gact).sum(axis=0).max()), what="layer %d shift gradient" % li)
        G = g[l.first_connection_index:l.last_connection_index].reshape(width, width)
        want_w = deltas[li][:, cols].astype(np.float64).T @ outs[li - 1].astype(np.float64)
        assert_close(G[cols], want_w, 1e-4, 1e-5 * float(np.abs(want_w).max()), what="layer %d weight gradient" % li)
    # the Nesterov step: the oracle takes the device's gradient and both update
    cpu.upload_gradient(g)
    for n in (gpu, cpu):
        n.Update_Parameter(Bn, Bn)
    assert_close(gpu.download_parameters(), cpu.download_parameters(), 1e-5, 1e-7, what="parameters after the Nesterov step")
