"""The C++ epoch loops `Dataset_Mini_Batch_HIP` / `Dataset_HIP` (include/myea_dataset_hip.hpp) driven by a compiled host
program (tests/cpp/dataset_check.cpp, built by `python -m myea_amd.build`) over a dataset resident in HBM, checked
against the CPU oracle walked through the same mini-batch order by the Python mirror of the same loops."""
import os
import re
import subprocess

import numpy as np
import pytest

from myea_amd import binding as mb
from myea_amd.dataset import Dataset_Mini_Batch
from tests.common import assert_close, glorot_parameters, one_hot
from tests.oracle_lib import OracleNetwork

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "cpp", "dataset_check")


def _run(tmp_path, kind, specs, bmax, T, hyper, X, Y, per_batch, seed):
    desc = mb.make_desc(specs, bmax, T)
    w = glorot_parameters(desc, seed, bias_range=0.3)
    for name, arr in (("w", w), ("x", X), ("y", Y)):
        np.asarray(arr, dtype=np.float32).tofile(str(tmp_path / (name + ".bin")))
    out = subprocess.run([BIN, str(tmp_path), kind], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    N = X.shape[0]
    order = np.fromfile(str(tmp_path / "order.bin"), dtype=np.float32).astype(np.uint64).reshape(-1, N)
    assert all(sorted(o.tolist()) == list(range(N)) for o in order) and not np.array_equal(order[0], np.arange(N))
    cpu = OracleNetwork(desc, mb.default_hyper(**hyper))
    cpu.upload_parameters(w)
    cpu.Clear_Training_Arrays()
    data = Dataset_Mini_Batch(X, Y, False, per_batch, recurrent_depth=T)
    lines = out.stdout.splitlines()
    m = re.match(r"mini-batches (\d+) of (\d+) last (\d+)", lines[0])
    assert tuple(int(g) for g in m.groups()) == (data.number_mini_batch, data.number_examples_per_iteration, data.number_examples_last_iteration)
    for e in range(order.shape[0]):
        data.stochastic_index = order[e].copy()
        loss = data.Training(cpu)
        got = re.match(r"epoch %d training loss (\S+) accuracy (\S+)" % e, lines[1 + e])
        assert float(got.group(1)) == pytest.approx(loss, rel=1e-4), "epoch %d" % e
        assert float(got.group(2)) == pytest.approx(data.accuracy_training, rel=1e-4, abs=1e-4), "epoch %d" % e
    loss = data.Testing(cpu)
    got = re.match(r"testing loss (\S+) accuracy (\S+)", lines[1 + order.shape[0]])
    assert float(got.group(1)) == pytest.approx(loss, rel=1e-4)
    assert float(got.group(2)) == pytest.approx(data.accuracy_testing, rel=1e-4, abs=1e-4)
    h = cpu.get_hyper()
    assert "time step %.1f epoch %.1f" % (h.optimizer_time_step, h.epoch_time_step) in out.stdout
    assert "mismatch returns max: 1" in out.stdout and "ERROR" in out.stdout
    return np.fromfile(str(tmp_path / "params.bin"), dtype=np.float32), cpu.download_parameters()


def test_mini_batch_classifier_epochs(tmp_path):
    specs = [dict(units=11), dict(units=20, activation="TANH"), dict(units=14, activation="RELU"), dict(units=5, activation="SOFTMAX")]
    rng = np.random.default_rng(21)
    X = rng.normal(0, 1, (103, 11)).astype(np.float32)
    Y = one_hot(rng.integers(0, 5, 103), 5)
    hyper = dict(type_optimizer_function=mb.OPTIMIZER["GD"], learning_rate=0.01, learning_momentum=0.9, regularization__weight_decay=0.02,
                 type_loss_function=mb.LOSS["CROSS_ENTROPY"], type_accuracy_function=mb.ACCURACY["CROSS_ENTROPY"])
    got, want = _run(tmp_path, "classify", specs, 16, 1, hyper, X, Y, 24, seed=21)
    assert_close(got, want, 1e-4, 1e-5, what="parameters")


def test_mini_batch_lstm_regression_epochs_with_r_accuracy(tmp_path):
    specs = [dict(units=6), dict(type="lstm", units=9), dict(type="lstm", units=7), dict(units=7, activation="LINEAR")]
    rng = np.random.default_rng(22)
    X = rng.normal(0, 1, (60, 5 * 6)).astype(np.float32)
    Y = (np.tanh(X.reshape(60, 5, 6)[:, :, :1]) * 0.5 + rng.normal(0, 0.3, (60, 5, 7))).astype(np.float32).reshape(60, -1)
    hyper = dict(type_optimizer_function=mb.OPTIMIZER["NOSADAM"], type_loss_function=mb.LOSS["RMSE"], type_accuracy_function=mb.ACCURACY["R"],
                 number_time_delays=1)
    got, want = _run(tmp_path, "regress", specs, 8, 5, hyper, X, Y, 20, seed=22)
    close = np.abs(got.astype(np.float64) - want) <= 1e-5 + 1e-4 * np.abs(want)
    # six Adam-type steps without re-synchronisation: entries driven by rounding-noise gradients may move by up to lr per step
    assert close.mean() > 0.99 and np.max(np.abs(got.astype(np.float64) - want)) <= 6 * 2.1e-3
