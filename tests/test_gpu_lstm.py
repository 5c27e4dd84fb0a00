"""GPU parity of the LSTM-with-peephole path (forward, BPTT, dW, AMSGrad) against the CPU oracle, through the C ABI.
Tolerance: rel 1e-4 / abs 1e-5."""
import os

import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, run_step
from tests.oracle_lib import OracleNetwork

pytestmark = pytest.mark.gpu
REL, ABS = 1e-4, 1e-5

LSTM_TAPS = ["LSTM_CELL_INPUT", "LSTM_CELL_STATE", "LSTM_INPUT_GATE", "LSTM_FORGET_GATE", "LSTM_OUTPUT_GATE",
             "LSTM_DELTA_CELL_INPUT", "LSTM_DELTA_CELL_STATE", "LSTM_DELTA_INPUT_GATE", "LSTM_DELTA_FORGET_GATE", "LSTM_DELTA_OUTPUT_GATE"]


def _width(l):
    return l.n_units * (l.n_cells_per_block if l.type_layer == mb.LAYER_LSTM else 1)


def _pair(specs, Bmax, T, hyper_kw, seed, threads=1):
    desc = mb.make_desc(specs, Bmax, T)
    h = mb.default_hyper(**hyper_kw)
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h, threads=threads)
    w = glorot_parameters(desc, seed, bias_range=0.3)
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
    return desc, gpu, cpu


def _rows(a, T, Bmax, B, W):
    """first B rows of every time step of a [T][Bmax][W] tensor"""
    return np.asarray(a).reshape(T, Bmax, W)[:, :B]


def _compare(desc, gpu, cpu, B, T, what=""):
    Bmax = desc.batch_size
    for li in range(1, desc.n_layers):
        l = desc.layers[li]
        W = _width(l)
        kinds = ["OUTPUTS", "ERRORS"] + (LSTM_TAPS if l.type_layer == mb.LAYER_LSTM else [])
        for kind in kinds:
            Wk = l.n_units if (kind.endswith("_GATE")) else W
            a = gpu.download_tensor(li, mb.TENSOR[kind], T * Bmax * Wk)
            b = cpu.download_tensor(li, mb.TENSOR[kind], T * Bmax * Wk)
            assert_close(_rows(a, T, Bmax, B, Wk), _rows(b, T, Bmax, B, Wk), REL, ABS, what="%s layer %d %s" % (what, li, kind))


CASES = [
    ("one-cell-per-block", [dict(units=6), dict(type="lstm", units=5), dict(units=7, activation="LINEAR")], 4, 5, 5),
    ("two-cells-per-block", [dict(units=4), dict(type="lstm", units=3, cells_per_block=2), dict(units=6, activation="TANH")], 5, 3, 3),
    ("config3-shape-shrunk", [dict(units=16), dict(type="lstm", units=64), dict(type="lstm", units=64), dict(units=64, activation="LINEAR")], 8, 32, 32),
    ("fc-below-lstm", [dict(units=5), dict(units=7, activation="TANH"), dict(type="lstm", units=4, cells_per_block=3), dict(units=9, activation="SIGMOID"),
                       dict(units=4, activation="LINEAR")], 3, 6, 6),
    ("partial-batch", [dict(units=12), dict(type="lstm", units=20), dict(type="lstm", units=8, cells_per_block=2), dict(units=16, activation="LINEAR")], 6, 5, 9),
    ("single-step", [dict(units=3), dict(type="lstm", units=5), dict(units=6, activation="LINEAR")], 1, 4, 4),
    ("two-steps", [dict(units=3), dict(type="lstm", units=4), dict(units=5, activation="LINEAR")], 2, 7, 7),
    ("unfused-activation-below", [dict(units=8), dict(units=12, activation="ELU"), dict(type="lstm", units=12), dict(units=12, activation="LINEAR")], 4, 8, 8),
    # one cell per block and a multiple of 32 cells: the one-launch-per-step kernels (k groups per wavefront 1, 3, 5; ragged rows)
    ("fused-step-32-cells", [dict(units=9), dict(type="lstm", units=32), dict(units=32, activation="LINEAR")], 5, 7, 7),
    ("fused-step-96-cells-partial-batch", [dict(units=20), dict(type="lstm", units=96), dict(units=96, activation="TANH")], 4, 37, 40),
    ("fused-step-160-cells-two-steps", [dict(units=6), dict(type="lstm", units=160), dict(units=160, activation="LINEAR")], 2, 33, 33),
    # enough (row tile, cell tile) pairs for the full-size tiles of the one-launch-per-step kernels, last row tile ragged
    ("fused-step-full-size-tiles-512-cells-ragged", [dict(units=12), dict(type="lstm", units=512), dict(units=512, activation="LINEAR")], 3, 130, 136),
    ("fused-step-full-size-tiles-256-cells-ragged", [dict(units=7), dict(type="lstm", units=256), dict(units=256, activation="TANH")], 2, 270, 270),
    ("fused-step-stacked-on-generic", [dict(units=10), dict(type="lstm", units=24), dict(type="lstm", units=64), dict(type="lstm", units=32),
                                       dict(units=32, activation="LINEAR")], 3, 12, 16),
]


@pytest.mark.parametrize("name,specs,T,B,Bmax", CASES, ids=[c[0] for c in CASES])
def test_lstm_parity_three_amsgrad_steps(name, specs, T, B, Bmax):
    desc, gpu, cpu = _pair(specs, Bmax, T, dict(type_optimizer_function=mb.OPTIMIZER["AMSGRAD"], type_loss_function=mb.LOSS["MSE"]), seed=3)
    rng = np.random.default_rng(3)
    X = rng.normal(0, 1, (B, T * specs[0]["units"])).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * specs[-1]["units"])).astype(np.float32)
    for step in range(3):
        for n in (gpu, cpu):
            n.Reset__Loss()
            run_step(n, B, X, Y, update=False)
        _compare(desc, gpu, cpu, B, T, what="step %d" % step)
        g_cpu = cpu.download_gradient()
        # sums over T x B terms of either sign: the absolute floor follows the gradient's scale where that exceeds 1
        assert_close(gpu.download_gradient(), g_cpu, REL, ABS * max(1.0, float(np.abs(g_cpu).max())), what="gradient step %d" % step)
        lg, lc = gpu.get_loss(), cpu.get_loss()
        assert lg.number_loss == lc.number_loss and lg.loss_values == pytest.approx(lc.loss_values, rel=1e-4)
        for n in (gpu, cpu):
            n.Update_Parameter(B, B)
        # entries whose gradient is rounding noise get a step decided by that noise under any Adam-type rule
        noisy = (np.abs(g_cpu) < 1e-5) & (g_cpu != 0)
        wg, wc = gpu.download_parameters(), cpu.download_parameters()
        assert noisy.mean() < 0.02
        assert_close(wg[~noisy], wc[~noisy], REL, ABS, what="parameters step %d" % step)
        assert np.all(np.abs(wg[noisy].astype(np.float64) - wc[noisy]) <= 2.1e-3)
        gpu.upload_parameters(wc)   # identical inputs for the next step
    for kind in (1, 2, 3):
        a, b = gpu.download_optimizer_state(kind), cpu.download_optimizer_state(kind)
        assert_close(a, b, REL, ABS, what="optimizer state %d" % kind)


def test_fused_time_step_matches_the_generic_path_on_the_gpu():
    """the same step through one launch per time step and through contraction + gate kernel per step (MYEA_LSTM_FUSED=0)"""
    T, B, Bmax = 7, 70, 72
    specs = [dict(units=24), dict(type="lstm", units=128), dict(type="lstm", units=64), dict(units=64, activation="LINEAR")]
    desc = mb.make_desc(specs, Bmax, T)
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["ADAM"], type_loss_function=mb.LOSS["MSE"])
    w = glorot_parameters(desc, 8, bias_range=0.3)
    rng = np.random.default_rng(8)
    X = rng.normal(0, 1, (B, T * 24)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * 64)).astype(np.float32)
    nets = []
    for flag in ("1", "0"):
        os.environ["MYEA_LSTM_FUSED"] = flag
        try:
            n = mb.HipNetwork(desc, h)
        finally:
            del os.environ["MYEA_LSTM_FUSED"]
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
        n.Reset__Loss()
        run_step(n, B, X, Y, update=False)
        nets.append(n)
    fused, generic = nets
    for li in (1, 2):
        for kind in ["OUTPUTS", "ERRORS"] + LSTM_TAPS:
            a = fused.download_tensor(li, mb.TENSOR[kind], T * Bmax * _width(desc.layers[li]))
            b = generic.download_tensor(li, mb.TENSOR[kind], T * Bmax * _width(desc.layers[li]))
            assert_close(_rows(a, T, Bmax, B, _width(desc.layers[li])), _rows(b, T, Bmax, B, _width(desc.layers[li])), REL, ABS, what="layer %d %s" % (li, kind))
    assert_close(fused.download_gradient(), generic.download_gradient(), REL, ABS, what="gradient")
    assert fused.get_loss().loss_values == pytest.approx(generic.get_loss().loss_values, rel=1e-5)


def test_lstm_softmax_head_cross_entropy_clip_and_adabound():
    """per-step softmax + cross-entropy head with gradient clipping at norm 1 and AdaBound (config 5's head and
    optimizer on a one-direction LSTM)"""
    T, B = 6, 10
    specs = [dict(units=12), dict(type="lstm", units=24), dict(units=24, activation="SOFTMAX")]
    kw = dict(type_optimizer_function=mb.OPTIMIZER["ADABOUND"], type_loss_function=mb.LOSS["CROSS_ENTROPY"],
              type_accuracy_function=mb.ACCURACY["CROSS_ENTROPY"], use_clip_gradient=1, clip_gradient=1.0)
    desc, gpu, cpu = _pair(specs, B, T, kw, seed=5)
    rng = np.random.default_rng(5)
    X = rng.uniform(-1, 1, (B, T * 12)).astype(np.float32)
    Y = np.zeros((B, T, 24), dtype=np.float32)
    lab = rng.integers(0, 24, (B, T))
    for b in range(B):
        Y[b, np.arange(T), lab[b]] = 1
    for n in (gpu, cpu):
        n.Reset__Loss()
        run_step(n, B, X, Y.reshape(B, -1), update=False)
    _compare(desc, gpu, cpu, B, T)
    assert_close(gpu.download_gradient(), cpu.download_gradient(), REL, ABS)
    assert gpu.get_loss().accuracy_value == cpu.get_loss().accuracy_value


def test_lstm_error_paths():
    with pytest.raises(mb.MyeaError) as e:   # head narrower than the last LSTM: its bias index overrun would leave the vector
        mb.HipNetwork(mb.make_desc([dict(units=3), dict(type="lstm", units=6), dict(units=2, activation="LINEAR")], 2, 3))
    assert e.value.code == mb.E_INVALID and "bias" in str(e.value)
    with pytest.raises(mb.MyeaError) as e:
        # a normalised layer with more than one cell per block: the reference's own indexing of the normalised units breaks there
        mb.HipNetwork(mb.make_desc([dict(units=3), dict(type="lstm", units=2, cells_per_block=2, normalization="BATCH_NORMALIZATION"), dict(units=8, activation="LINEAR")], 2, 3))
    assert e.value.code == mb.E_UNSUPPORTED


def test_config3_full_size_one_step():
    """BASELINE config 3 at full size: 2 x LSTM-512 (peephole), input 128, T = 64, batch 256, linear FC-512 head, MSE,
    AMSGrad; one whole step on both sides (the oracle runs on the host's cores): outputs, deltas and every LSTM tap of all
    layers at every time step, the whole gradient - entries outside the tolerance of the oracle go to a float64 sum of their
    16384 products (tests/full_size_support.py) - then the AMSGrad-stepped parameters and the three optimizer vectors."""
    from tests.full_size_support import GradientTerms, assert_first_adam_type_step_matches, assert_sums_match
    T, B = 64, 256
    specs = [dict(units=128), dict(type="lstm", units=512), dict(type="lstm", units=512), dict(units=512, activation="LINEAR")]
    threads = min(16, os.cpu_count() or 1)
    hyper = dict(type_optimizer_function=mb.OPTIMIZER["AMSGRAD"], type_loss_function=mb.LOSS["MSE"])
    desc, gpu, cpu = _pair(specs, B, T, hyper, seed=3, threads=threads)
    twin = OracleNetwork(desc, mb.default_hyper(**hyper), threads=threads)
    w = gpu.download_parameters()
    twin.set_state_propagation(mb.STATE_TRAINING)
    twin.upload_parameters(w)
    twin.Clear_Training_Arrays()
    rng = np.random.default_rng(3)
    X = rng.normal(0, 1, (B, T * 128)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * 512)).astype(np.float32)
    for n in (gpu, cpu):
        n.Reset__Loss()
        run_step(n, B, X, Y, update=False)
    _compare(desc, gpu, cpu, B, T, what="full size")
    lg, lc = gpu.get_loss(), cpu.get_loss()
    assert lg.number_loss == lc.number_loss and lg.loss_values == pytest.approx(lc.loss_values, rel=1e-5)
    g_gpu, g_cpu = gpu.download_gradient(), cpu.download_gradient()
    report = {}
    assert_sums_match(g_gpu, g_cpu, GradientTerms(desc, cpu, X, B).exact, "gradient", report=report)
    print("config 3 gradient:", report["gradient"])
    print("config 3 update:", assert_first_adam_type_step_matches(gpu, cpu, twin, w, g_gpu, g_cpu, B, mb.default_hyper(**hyper),
                                                                  ("FIRST_MOMENT", "SECOND_MOMENT", "SECOND_MOMENT_HAT"), "AMSGrad step"))
