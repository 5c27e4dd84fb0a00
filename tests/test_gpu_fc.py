"""GPU parity of the feed-forward path: the HIP library (through its C ABI) against the CPU oracle on the
same seeded inputs.  Tolerance of north_star: rel 1e-4 / abs 1e-5 on gradients and updated weights (fp32);
masks and indexing bit-exact."""
import ctypes as C

import numpy as np
import pytest

from myea_amd import binding as mb
import torch

from tests.common import assert_close, assert_close_or_nearer_truth, glorot_parameters, one_hot, run_step
from tests.test_oracle_fc import TorchMLP
from tests.oracle_lib import OracleNetwork

pytestmark = pytest.mark.gpu

REL, ABS = 1e-4, 1e-5


def _pair(specs, B, hyper_kw, T=1, seed=0, masks=None):
    desc = mb.make_desc(specs, B, T)
    h = mb.default_hyper(**hyper_kw)
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h)
    w = glorot_parameters(desc, seed)
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
        if masks is not None:
            n.upload_masks(masks)
    return desc, gpu, cpu


def _compare_layers(desc, gpu, cpu, B, kinds=("OUTPUTS", "ERRORS")):
    for li in range(1, desc.n_layers):
        H = desc.layers[li].n_units
        for kind in kinds:
            a = gpu.download_tensor(li, mb.TENSOR[kind], B * H)
            b = cpu.download_tensor(li, mb.TENSOR[kind], B * H)
            assert_close(a, b, REL, ABS, what="layer %d %s" % (li, kind))


def _data(specs, B, seed, head):
    rng = np.random.default_rng(seed)
    n_in, n_out = specs[0]["units"], specs[-1]["units"]
    X = rng.normal(0, 1, (B, n_in)).astype(np.float32)
    Y = one_hot(rng.integers(0, n_out, B), n_out) if head == "SOFTMAX" else rng.uniform(0, 1, (B, n_out)).astype(np.float32)
    return X, Y


def test_c1_mlp_784_256_10_sgd_momentum_10_steps():
    """BASELINE config 1 at full size: tanh hidden, sigmoid output, MSE, SGD lr .01 momentum .9, 10 steps."""
    specs = [dict(units=784), dict(units=256, activation="TANH"), dict(units=10, activation="SIGMOID")]
    B = 128
    desc, gpu, cpu = _pair(specs, B, dict(type_optimizer_function=mb.OPTIMIZER["GD"], type_loss_function=mb.LOSS["MSE"],
                                          learning_rate=0.01, learning_momentum=0.9), seed=1)
    rng = np.random.default_rng(1)
    X = rng.uniform(0, 1, (B, 784)).astype(np.float32)
    Y = one_hot(rng.integers(0, 10, B), 10)
    for step in range(10):
        for n in (gpu, cpu):
            n.Reset__Loss()
            run_step(n, B, X, Y, update=False)
        if step in (0, 9):
            _compare_layers(desc, gpu, cpu, B)
            assert_close(gpu.download_gradient(), cpu.download_gradient(), REL, ABS, what="gradient step %d" % step)
        lg, lc = gpu.get_loss(), cpu.get_loss()
        assert lg.number_loss == lc.number_loss == B * 10
        assert lg.loss_values == pytest.approx(lc.loss_values, rel=1e-4)
        assert lg.accuracy_value == lc.accuracy_value
        for n in (gpu, cpu):
            n.Update_Parameter(B, B)
        assert_close(gpu.download_parameters(), cpu.download_parameters(), REL, ABS, what="parameters step %d" % step)
    assert_close(gpu.download_optimizer_state(mb.OPT_STATE["PREVIOUS_DELTA"]), cpu.download_optimizer_state(mb.OPT_STATE["PREVIOUS_DELTA"]), REL, ABS)
    assert gpu.get_hyper().optimizer_time_step == 10


@pytest.mark.parametrize("optimizer,extra", [
    ("ADAM", {}), ("AMSGRAD", {}), ("ADABOUND", dict(use_clip_gradient=1, clip_gradient=1.0)),
    ("GD", dict(learning_momentum=0.0)), ("GD", dict(use_Nesterov=1)), ("ADAM", dict(regularization__weight_decay=1e-3, use_clip_gradient=1, clip_gradient=0.5)),
])
def test_c2_shape_relu_softmax_ce_shrunk(optimizer, extra):
    """BASELINE config 2 shrunk (deep ReLU MLP, softmax + cross-entropy), 3 steps per optimizer."""
    specs = [dict(units=192)] + [dict(units=256, activation="RELU")] * 4 + [dict(units=100, activation="SOFTMAX")]
    B = 96
    kw = dict(type_optimizer_function=mb.OPTIMIZER[optimizer], type_loss_function=mb.LOSS["CROSS_ENTROPY"],
              type_accuracy_function=mb.ACCURACY["CROSS_ENTROPY"])
    kw.update(extra)
    desc, gpu, cpu = _pair(specs, B, kw, seed=2)
    X, Y = _data(specs, B, 2, "SOFTMAX")
    # The Adam family divides by sqrt(v): a parameter whose gradient is within rounding noise of zero (|g| < 1e-5
    # here, against summation noise of ~1e-8) gets a step of up to lr whose value is decided by that noise, on any
    # two summation orders (the reference's own __Loop and __OpenMP variants included).  Such entries are few; they
    # are held to the bound |dw| <= 2.1 lr per step instead of the elementwise tolerance.
    adam_like = optimizer != "GD"
    noisy = np.zeros(desc.total_parameters, dtype=bool)
    for step in range(3):
        for n in (gpu, cpu):
            n.Reset__Loss()
            run_step(n, B, X, Y, update=False)
        _compare_layers(desc, gpu, cpu, B)
        g_cpu = cpu.download_gradient()
        assert_close(gpu.download_gradient(), g_cpu, REL, ABS, what="gradient step %d" % step)
        assert gpu.get_loss().accuracy_value == cpu.get_loss().accuracy_value
        if adam_like:
            noisy |= (np.abs(g_cpu) < 1e-5) & (g_cpu != 0)
            assert noisy.mean() < 0.01
        for n in (gpu, cpu):
            n.Update_Parameter(B, B)
        wg, wc = gpu.download_parameters(), cpu.download_parameters()
        assert_close(wg[~noisy], wc[~noisy], REL, ABS, what="parameters step %d" % step)
        if noisy.any():   # keep the two trajectories on the same point for the next step
            wg[noisy] = wc[noisy]
            gpu.upload_parameters(wg)
        assert np.all(np.abs(wg[noisy].astype(np.float64) - wc[noisy]) <= 2.1 * 0.1 * (step + 1) if optimizer == "ADABOUND" else
                      np.abs(wg[noisy].astype(np.float64) - wc[noisy]) <= 2.1e-3 * (step + 1))
        assert np.all(gpu.download_gradient() == 0)
    for kind in range(4):
        assert_close(gpu.download_optimizer_state(kind), cpu.download_optimizer_state(kind), REL, ABS, what="optimizer state %d" % kind)


@pytest.mark.parametrize("B,Bmax", [(1, 1), (5, 8), (33, 33)])
def test_ragged_shapes_use_the_guarded_path(B, Bmax):
    """widths that are not multiples of 4 (unaligned weight slices), batch smaller than the allocated batch"""
    specs = [dict(units=13), dict(units=31, activation="SIGMOID"), dict(units=7, activation="LEAKY_RELU"),
             dict(units=66, activation="ELLIOT_SYMMETRIC"), dict(units=3, activation="LINEAR")]
    desc, gpu, cpu = _pair(specs, Bmax, dict(type_optimizer_function=mb.OPTIMIZER["ADAM"], type_loss_function=mb.LOSS["MSE"]), seed=5)
    X, Y = _data(specs, B, 5, "LINEAR")
    for n in (gpu, cpu):
        run_step(n, B, X, Y, update=False)
    _compare_layers(desc, gpu, cpu, B)
    assert_close(gpu.download_gradient(), cpu.download_gradient(), REL, ABS)
    for n in (gpu, cpu):
        n.Update_Derivative_Weight(B, 1, desc.n_layers)   # accumulates: doubles the gradient
    assert_close(gpu.download_gradient(), cpu.download_gradient(), REL, ABS)
    for n in (gpu, cpu):
        n.Update_Parameter(B, B)
    assert_close(gpu.download_parameters(), cpu.download_parameters(), REL, ABS)


@pytest.mark.parametrize("act", ["COSINE", "ELU", "GAUSSIAN", "ISRLU", "SELU", "SINE_SYMMETRIC", "TANH_STEPWISE", "THRESHOLD_SYMMETRIC", "LINEAR_PIECE"])
def test_unfused_activations(act):
    specs = [dict(units=24), dict(units=40, activation=act, steepness=1.5), dict(units=12, activation="TANH")]
    B = 16
    desc, gpu, cpu = _pair(specs, B, dict(type_optimizer_function=mb.OPTIMIZER["GD"], type_loss_function=mb.LOSS["MSE"]), seed=6)
    X, Y = _data(specs, B, 6, "TANH")
    for n in (gpu, cpu):
        run_step(n, B, X, Y, update=False)
    _compare_layers(desc, gpu, cpu, B)
    assert_close(gpu.download_gradient(), cpu.download_gradient(), REL, ABS)


NORM_CASES = {
    "bn-before-relu": dict(normalization="BATCH_NORMALIZATION", norm_before=True, activation="RELU"),
    "bn-after-tanh": dict(normalization="BATCH_NORMALIZATION", norm_before=False, activation="TANH"),
    "brn-before-sine": dict(normalization="BATCH_RENORMALIZATION", norm_before=True, activation="SINE_SYMMETRIC"),
    "brn-after-sigmoid": dict(normalization="BATCH_RENORMALIZATION", norm_before=False, activation="SIGMOID"),
}


@pytest.mark.parametrize("case", sorted(NORM_CASES))
def test_batch_normalisation_and_renormalisation(case):
    """The reference computes sigma = sqrt(E[x^2] - mean^2 + eps) in fp32, which loses digits when |mean| >> sigma and
    then depends on the summation order (also between its own __Loop and __OpenMP variants); the cases keep the
    normalised inputs roughly centred so that the comparison stays inside rel 1e-4 / abs 1e-5."""
    layer = dict(units=96, **NORM_CASES[case])
    specs = [dict(units=48), layer, dict(layer), dict(units=10, activation="SOFTMAX")]
    B = 64
    kw = dict(type_optimizer_function=mb.OPTIMIZER["GD"], use_Nesterov=1, type_loss_function=mb.LOSS["CROSS_ENTROPY"],
              batch_renormalization_r_correction_maximum=2.0, batch_renormalization_d_correction_maximum=1.0)
    desc, gpu, cpu = _pair(specs, B, kw, seed=7)
    X, Y = _data(specs, B, 7, "SOFTMAX")
    for step in range(3):
        # float64 arbiter for the gradient: autograd of the independent forward model, from the oracle's state
        w_now = cpu.download_parameters()
        running = {li: (torch.tensor(cpu.download_tensor(li, mb.TENSOR["NORM_MEANS_AVERAGES"], 96).astype(np.float64)),
                        torch.tensor(cpu.download_tensor(li, mb.TENSOR["NORM_VARIANCES_AVERAGES"], 96).astype(np.float64))) for li in (1, 2)}
        model = TorchMLP(desc, specs, w_now, r_max=2.0, d_max=1.0)
        model.loss(model.forward(X, running=running), Y, "SOFTMAX").backward()
        for n in (gpu, cpu):
            run_step(n, B, X, Y, update=False)
        _compare_layers(desc, gpu, cpu, B, kinds=("OUTPUTS",))
        for li in (1, 2):
            assert_close(gpu.download_tensor(li, mb.TENSOR["NORM_HATS"], B * 96), cpu.download_tensor(li, mb.TENSOR["NORM_HATS"], B * 96), REL, ABS)
            for kind in ("NORM_MEANS", "NORM_VARIANCES", "NORM_MEANS_AVERAGES", "NORM_VARIANCES_AVERAGES"):
                assert_close(gpu.download_tensor(li, mb.TENSOR[kind], 96), cpu.download_tensor(li, mb.TENSOR[kind], 96), REL, ABS, what=kind)
        assert_close_or_nearer_truth(gpu.download_gradient(), cpu.download_gradient(), model.flat.grad.numpy(), REL, ABS, what="gradient step %d" % step)
        for n in (gpu, cpu):
            n.Update_Parameter(B, B)
        assert_close(gpu.download_parameters(), cpu.download_parameters(), REL, ABS, what="parameters step %d" % step)
        gpu.upload_parameters(cpu.download_parameters())   # identical inputs for the next step
    # inference uses the running statistics
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_INFERENCE)
        n.Forward_Pass(B, X)
    _compare_layers(desc, gpu, cpu, B, kinds=("OUTPUTS",))


def test_c4_shape_bn_relu_inverted_dropout_nesterov_shrunk():
    """BASELINE config 4 shrunk: [FC, BN before activation, ReLU, inverted Bernoulli keep .5] x 4 + softmax head,
    SGD-Nesterov; masks come from one seeded host buffer written to both sides (bit-exact by construction) and are
    redrawn every step."""
    width, depth, B = 128, 4, 48
    layer = dict(units=width, activation="RELU", normalization="BATCH_NORMALIZATION", norm_before=True, dropout="BERNOULLI_INVERTED", keep=0.5)
    specs = [dict(units=width)] + [dict(layer) for _ in range(depth)] + [dict(units=20, activation="SOFTMAX")]
    kw = dict(type_optimizer_function=mb.OPTIMIZER["GD"], use_Nesterov=1, learning_rate=0.01, learning_momentum=0.9,
              type_loss_function=mb.LOSS["CROSS_ENTROPY"])
    desc, gpu, cpu = _pair(specs, B, kw, seed=4)
    X, Y = _data(specs, B, 4, "SOFTMAX")
    rng = np.random.default_rng(4)
    for step in range(3):
        masks = (rng.uniform(0, 1, desc.total_mask_units) < 0.5).astype(np.uint8)
        for n in (gpu, cpu):
            n.upload_masks(masks)
            run_step(n, B, X, Y, update=False)
        for li in range(1, depth + 1):
            m = masks[desc.layers[li].first_mask_index:desc.layers[li].first_mask_index + width]
            out = gpu.download_tensor(li, mb.TENSOR["OUTPUTS"], B * width).reshape(B, width)
            assert np.all(out[:, m == 0] == 0)                      # dropped units are exactly zero
            assert np.array_equal(out == 0, cpu.download_tensor(li, mb.TENSOR["OUTPUTS"], B * width).reshape(B, width) == 0)
        _compare_layers(desc, gpu, cpu, B)
        assert_close(gpu.download_gradient(), cpu.download_gradient(), REL, ABS, what="gradient step %d" % step)
        for n in (gpu, cpu):
            n.Update_Parameter(B, B)
        assert_close(gpu.download_parameters(), cpu.download_parameters(), REL, ABS, what="parameters step %d" % step)


def test_plain_bernoulli_dropout_with_input_layer_dropout_and_inference_scaling():
    specs = [dict(units=40, dropout="BERNOULLI", keep=0.8), dict(units=64, activation="TANH", dropout="BERNOULLI", keep=0.6),
             dict(units=64, activation="SIGMOID", dropout="BERNOULLI_INVERTED", keep=0.7), dict(units=8, activation="SIGMOID")]
    B = 24
    desc, gpu, cpu = _pair(specs, B, dict(type_optimizer_function=mb.OPTIMIZER["GD"], type_loss_function=mb.LOSS["MSE"]), seed=8)
    masks = (np.random.default_rng(8).uniform(0, 1, desc.total_mask_units) < 0.7).astype(np.uint8)
    X, Y = _data(specs, B, 8, "SIGMOID")
    for n in (gpu, cpu):
        n.upload_masks(masks)
        run_step(n, B, X, Y, update=False)
    assert_close(gpu.download_tensor(0, mb.TENSOR["OUTPUTS"], B * 40), cpu.download_tensor(0, mb.TENSOR["OUTPUTS"], B * 40), 0, 0)
    _compare_layers(desc, gpu, cpu, B)
    assert_close(gpu.download_gradient(), cpu.download_gradient(), REL, ABS)
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_INFERENCE)
        n.Forward_Pass(B, X)
    _compare_layers(desc, gpu, cpu, B, kinds=("OUTPUTS",))


def test_loss_functions_and_accuracy_counters():
    specs = [dict(units=16), dict(units=9, activation="SIGMOID")]
    B = 37
    for loss in ("MSE", "MAE", "L1", "CROSS_ENTROPY", "SMAPE", "MAPE", "BIT"):
        for acc in ("DISTANCE", "SIGN", "DIRECTIONAL", "CROSS_ENTROPY"):
            desc, gpu, cpu = _pair(specs, B, dict(type_loss_function=mb.LOSS[loss], type_accuracy_function=mb.ACCURACY[acc]), seed=9)
            X, Y = _data(specs, B, 9, "SOFTMAX")
            for n in (gpu, cpu):
                n.Reset__Loss()
                n.Forward_Pass(B, X)
                n.Compute__Error(B, Y)
                n.Compute__Error(B, Y)   # accumulates until reset
            g, c = gpu.get_loss(), cpu.get_loss()
            assert g.number_loss == c.number_loss and g.number_bit_fail == c.number_bit_fail, (loss, acc)
            assert g.loss_values == pytest.approx(c.loss_values, rel=1e-4, abs=1e-6), (loss, acc)
            assert g.accuracy_value == c.accuracy_value, (loss, acc)


def test_error_paths_return_codes_and_keep_the_net_usable():
    specs = [dict(units=8), dict(units=8, activation="TANH"), dict(units=2, activation="SIGMOID")]
    desc, gpu, cpu = _pair(specs, 4, dict(type_optimizer_function=mb.OPTIMIZER["GD"], type_loss_function=mb.LOSS["MSE"]))
    X = np.zeros((5, 8), dtype=np.float32)
    with pytest.raises(mb.MyeaError) as e:
        gpu.Forward_Pass(5, X)                      # batch > allocated batch (Forward_Pass__OpenMP.cpp:33-43)
    assert e.value.code == mb.E_BATCH and "batch size" in str(e.value)
    gpu.set_state_propagation(mb.STATE_INFERENCE)
    with pytest.raises(mb.MyeaError) as e:
        gpu.Backward_Pass(4)                        # backward in inference mode (Backward_Pass__OpenMP.cpp:41-51)
    assert e.value.code == mb.E_STATE
    h = mb.default_hyper(type_optimizer_function=7)  # iRPROP-: not on this path
    gpu.set_hyper(h)
    with pytest.raises(mb.MyeaError) as e:
        gpu.Update_Parameter(4, 4)
    assert e.value.code == mb.E_UNSUPPORTED and gpu.get_hyper().optimizer_time_step == 0
    bad = mb.make_desc(specs, 4)
    bad.layers[1].type_layer = 2                    # convolution: unmanaged layer type
    with pytest.raises(mb.MyeaError) as e:
        mb.HipNetwork(bad)
    assert e.value.code == mb.E_UNSUPPORTED
    bad = mb.make_desc(specs, 4)
    bad.layers[2].first_connection_index = bad.total_weights  # slice leaves the weight region
    with pytest.raises(mb.MyeaError) as e:
        mb.HipNetwork(bad)
    assert e.value.code == mb.E_INVALID
    # still usable
    gpu.set_hyper(mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["GD"], type_loss_function=mb.LOSS["MSE"]))
    gpu.set_state_propagation(mb.STATE_TRAINING)
    Xs, Ys = _data(specs, 4, 1, "SIGMOID")
    for n in (gpu, cpu):
        run_step(n, 4, Xs, Ys)
    assert_close(gpu.download_parameters(), cpu.download_parameters(), REL, ABS)


def test_device_resident_inputs_match_host_inputs():
    import torch
    specs = [dict(units=32), dict(units=48, activation="RELU"), dict(units=6, activation="SOFTMAX")]
    B = 20
    desc, gpu, cpu = _pair(specs, B, dict(type_optimizer_function=mb.OPTIMIZER["ADAM"], type_loss_function=mb.LOSS["CROSS_ENTROPY"]), seed=3)
    X, Y = _data(specs, B, 3, "SOFTMAX")
    xd, yd = torch.from_numpy(X).cuda(), torch.from_numpy(Y).cuda()
    torch.cuda.synchronize()
    gpu.Forward_Pass(B, xd, on_device=True)
    gpu.Compute__Error(B, yd, on_device=True)
    gpu.Backward_Pass(B)
    gpu.Update_Derivative_Weight(B)
    run_step(cpu, B, X, Y, update=False)
    assert_close(gpu.download_gradient(), cpu.download_gradient(), REL, ABS)


def test_forward_contraction_that_splits_a_tile_between_two_workgroups():
    """A forward contraction with at most one 64 x 64 tile per compute unit (here 512 x 1024 outputs over k = 512 and 1024) splits
    each tile's k between two workgroups that combine their halves inside the launch: against the oracle, and bit for bit
    the same from run to run (the combined sum is half 0 + half 1 whichever workgroup finishes first)."""
    specs = [dict(units=512), dict(units=1024, activation="TANH"), dict(units=1024, activation="SIGMOID", normalization="BATCH_NORMALIZATION"),
             dict(units=64, activation="LINEAR")]
    B = 512
    desc = mb.make_desc(specs, B, 1)
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["GD"], type_loss_function=mb.LOSS["MSE"])
    w = glorot_parameters(desc, 5)
    rng = np.random.default_rng(5)
    X = rng.normal(0, 1, (B, 512)).astype(np.float32)
    Y = rng.normal(0, 1, (B, 64)).astype(np.float32)
    outs = []
    for cls in (mb.HipNetwork, mb.HipNetwork, OracleNetwork):
        n = cls(desc, h)
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
        run_step(n, B, X, Y, update=False)
        outs.append([n.download_tensor(li, mb.TENSOR["OUTPUTS"], B * desc.layers[li].n_units) for li in (1, 2, 3)] + [n.download_gradient()])
    for a, b in zip(outs[0], outs[1]):
        assert np.array_equal(a, b)
    for k, (a, b) in enumerate(zip(outs[0], outs[2])):
        assert_close(a, b, 1e-4, 1e-5 * max(1.0, float(np.abs(b).max())), what="tensor %d" % k)


def test_forward_contraction_that_splits_a_128_tile_between_two_workgroups():
    """One size up: at most one 128 x 128 tile per compute unit and k >= 2048 (here 1024 x 2048 outputs over k = 2048; the layer
    behind it has half the tiles and takes the 64 x 64 form): outputs held against float64 on sampled entries - the oracle
    would take minutes at this size - and bit for bit the same from run to run."""
    specs = [dict(units=2048), dict(units=2048, activation="TANH"), dict(units=1024, activation="RELU"), dict(units=16, activation="LINEAR")]
    B = 1024
    desc = mb.make_desc(specs, B, 1)
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["GD"], type_loss_function=mb.LOSS["MSE"])
    w = glorot_parameters(desc, 8, bias_range=0.2)
    rng = np.random.default_rng(8)
    X = rng.normal(0, 1, (B, 2048)).astype(np.float32)
    runs = []
    for _ in range(2):
        n = mb.HipNetwork(desc, h)
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Forward_Pass(B, X)
        runs.append([n.download_tensor(li, mb.TENSOR["OUTPUTS"], B * desc.layers[li].n_units) for li in (1, 2)])
        n.close()
    for a, b in zip(*runs):
        assert np.array_equal(a, b)
    l = desc.layers[1]
    W = w[l.first_connection_index:l.first_connection_index + 2048 * 2048].reshape(2048, 2048).astype(np.float64)
    bias = w[l.first_bias_connection_index:l.first_bias_connection_index + 2048].astype(np.float64)
    rows, cols = rng.integers(0, B, 256), rng.integers(0, 2048, 256)
    want = np.tanh(np.einsum("sk,sk->s", X[rows].astype(np.float64), W[cols]) + bias[cols])
    got = runs[0][0].reshape(B, 2048)[rows, cols]
    assert_close(got, want, 1e-4, 1e-5, what="outputs of the split 128 x 128 tiles")
