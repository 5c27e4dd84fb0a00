"""The C++ adaptor `Neural_Network_HIP` (include/myea_nn_hip.hpp) driven like the reference's class by a compiled host
program (tests/cpp/adaptor_check.cpp, built by `python -m myea_amd.build`), checked against the CPU oracle."""
import os
import subprocess

import numpy as np
import pytest

from myea_amd import binding as mb
from myea_amd.dataset import get_loss
from tests.common import assert_close, glorot_parameters, one_hot, run_step
from tests.oracle_lib import OracleNetwork

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "cpp", "adaptor_check")


def _run(tmp_path, kind, specs, B, T, hyper, X, Y, masks, seed, gradient_close=None):
    desc = mb.make_desc(specs, B, T)
    w = glorot_parameters(desc, seed, bias_range=0.3)
    for name, arr in (("w", w), ("x", X), ("y", Y), ("mask", masks.astype(np.float32))):
        np.asarray(arr, dtype=np.float32).tofile(str(tmp_path / (name + ".bin")))
    out = subprocess.run([BIN, str(tmp_path), kind], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    cpu = OracleNetwork(desc, mb.default_hyper(**hyper))
    cpu.set_state_propagation(mb.STATE_TRAINING)
    cpu.upload_parameters(w)
    cpu.upload_masks(masks)
    losses = []
    for step in range(3):
        cpu.Reset__Loss()
        run_step(cpu, B, X, Y, update=False)
        g = cpu.download_gradient()
        losses.append(get_loss(cpu, specs[-1]["units"]))
        cpu.Update_Parameter(B, B)
    got_losses = [float(l.split()[-1]) for l in out.stdout.splitlines() if l.startswith("step ")]
    assert got_losses == pytest.approx(losses, rel=1e-4)
    assert "time step 3.0" in out.stdout and "ERROR" in out.stdout     # the oversized batch printed and returned
    (gradient_close or (lambda a, b: assert_close(a, b, 1e-4, 1e-5, what="gradient")))(np.fromfile(str(tmp_path / "grad.bin"), dtype=np.float32), g)
    return np.fromfile(str(tmp_path / "params.bin"), dtype=np.float32), cpu.download_parameters(), g


def test_adaptor_mlp_bn_dropout_nesterov(tmp_path):
    specs = [dict(units=20), dict(units=32, activation="RELU", normalization="BATCH_NORMALIZATION", norm_before=True, dropout="BERNOULLI_INVERTED", keep=0.5),
             dict(units=24, activation="TANH"), dict(units=6, activation="SOFTMAX")]
    B = 16
    rng = np.random.default_rng(1)
    X = rng.normal(0, 1, (B, 20)).astype(np.float32)
    Y = one_hot(rng.integers(0, 6, B), 6)
    desc = mb.make_desc(specs, B)
    masks = (rng.uniform(0, 1, desc.total_mask_units) < 0.5).astype(np.uint8)
    hyper = dict(type_optimizer_function=mb.OPTIMIZER["GD"], use_Nesterov=1, type_loss_function=mb.LOSS["CROSS_ENTROPY"],
                 type_accuracy_function=mb.ACCURACY["CROSS_ENTROPY"])
    got, want, _ = _run(tmp_path, "mlp", specs, B, 1, hyper, X, Y, masks, seed=1)
    assert_close(got, want, 1e-4, 1e-5, what="parameters")


def test_adaptor_lstm_amsgrad_clip(tmp_path):
    specs = [dict(units=8), dict(type="lstm", units=12), dict(type="lstm", units=6, cells_per_block=2), dict(units=12, activation="LINEAR")]
    B, T = 6, 5
    rng = np.random.default_rng(2)
    X = rng.normal(0, 1, (B, T * 8)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * 12)).astype(np.float32)
    desc = mb.make_desc(specs, B, T)
    masks = np.ones(desc.total_mask_units, dtype=np.uint8)
    hyper = dict(type_optimizer_function=mb.OPTIMIZER["AMSGRAD"], type_loss_function=mb.LOSS["MSE"], use_clip_gradient=1, clip_gradient=1.0)
    got, want, g = _run(tmp_path, "lstm", specs, B, T, hyper, X, Y, masks, seed=2)
    # three AMSGrad steps without re-synchronisation: entries driven by rounding-noise gradients may move by up to lr per step
    close = np.abs(got.astype(np.float64) - want) <= 1e-5 + 1e-4 * np.abs(want)
    assert close.mean() > 0.99 and np.max(np.abs(got.astype(np.float64) - want)) <= 3 * 2.1e-3


def test_adaptor_ind_rnn_default_bounds_and_clip(tmp_path):
    """Compile's defaults for independently recurrent layers (rectifier, bounds that follow the activation and the clip value
    until they are set by hand) are asserted inside the host program; the training steps against the oracle here"""
    specs = [dict(units=8), dict(type="ind_rnn", units=16, activation="RELU"), dict(type="ind_rnn", units=12, activation="TANH", recurrent_bounds=(-0.5, 0.75)),
             dict(units=4, activation="LINEAR")]
    B, T = 6, 5
    rng = np.random.default_rng(3)
    X = rng.normal(0, 1, (B, T * 8)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * 4)).astype(np.float32)
    desc = mb.make_desc(specs, B, T)
    masks = np.ones(desc.total_mask_units, dtype=np.uint8)
    hyper = dict(type_optimizer_function=mb.OPTIMIZER["GD"], type_loss_function=mb.LOSS["MSE"])
    got, want, _ = _run(tmp_path, "indrnn", specs, B, T, hyper, X, Y, masks, seed=3)
    assert_close(got, want, 1e-4, 1e-5, what="parameters")
    l = desc.layers[2]
    u = got[l.last_connection_index - 12:l.last_connection_index]
    assert u.min() >= -0.5 and u.max() <= 0.75


def test_adaptor_builds_and_trains_the_reference_example_network(tmp_path):
    """The host program makes the calls of the reference's worked example in its order (residual blocks of independently
    recurrent members, pooling between the groups, normalisation set on every hidden layer, AMSGrad, max-norm constraint, the
    label read at the last time step); the description it arrives at must be the builder's, its three steps the oracle's."""
    from myea_amd.synthetic import simple_debug_layers
    specs = simple_debug_layers()
    B, T = 12, 5
    rng = np.random.default_rng(5)
    X = rng.uniform(0, 1, (B, T * 28)).astype(np.float32)
    Y = np.zeros((B, T, 10), np.float32)
    np.put_along_axis(Y, rng.integers(0, 10, (B, T))[..., None], 1.0, axis=2)
    Y = Y.reshape(B, T * 10)
    desc = mb.make_desc(specs, B, T, network=mb.NETWORK_FEEDFORWARD)
    masks = np.ones(max(1, desc.total_mask_units), dtype=np.uint8)[:desc.total_mask_units]
    hyper = dict(type_optimizer_function=mb.OPTIMIZER["AMSGRAD"], type_loss_function=mb.LOSS["CROSS_ENTROPY"], type_accuracy_function=mb.ACCURACY["CROSS_ENTROPY"],
                 regularization__max_norm_constraints=8.0, normalization_momentum_average=1.0, normalization_epsilon=0.1, number_time_delays=T - 1)
    def mostly_close(a, b):
        """rel 1e-4 / abs 1e-5, up to 1 % of the entries off by up to 1 %: 28 normalisations over 12 examples amplify fp32 rounding"""
        err = np.abs(a.astype(np.float64) - b)
        bad = err > 1e-4 * np.abs(b) + 1e-5
        assert bad.mean() <= 0.01 and np.all(err[bad] <= 1e-2 * np.abs(b[bad]) + 1e-4), "gradient: %d / %d out of tolerance" % (int(bad.sum()), a.size)
    got, want, _ = _run(tmp_path, "example", specs, B, T, hyper, X, Y, masks, seed=5, gradient_close=mostly_close)
    # three AMSGrad steps without re-synchronisation: entries driven by rounding-noise gradients may move by up to lr per step
    close = np.abs(got.astype(np.float64) - want) <= 1e-5 + 1e-4 * np.abs(want)
    assert close.mean() > 0.98 and np.max(np.abs(got.astype(np.float64) - want)) <= 3 * 2.1e-3
