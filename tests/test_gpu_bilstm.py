"""GPU parity of the two-direction LSTM layer (each direction the reference's one-direction recurrence over its own
blocks, the second walking time backwards; summed outputs; shared delta) against the CPU oracle through the C ABI.
Tolerance rel 1e-4 / abs 1e-5."""
import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, run_step
from tests.oracle_lib import OracleNetwork
from tests.test_gpu_lstm import LSTM_TAPS, _rows, _width

pytestmark = pytest.mark.gpu
REL, ABS = 1e-4, 1e-5
BACK = mb.TENSOR["DIRECTION_BACKWARD"]


def _compare(desc, gpu, cpu, B, T, what=""):
    Bmax = desc.batch_size
    for li in range(1, desc.n_layers):
        l = desc.layers[li]
        W = _width(l)
        kinds = [("OUTPUTS", 0), ("ERRORS", 0)]
        if l.type_layer == mb.LAYER_LSTM:
            for flag in ((0, BACK) if l.use_bidirectional else (0,)):
                kinds += [(k, flag) for k in LSTM_TAPS + ["LSTM_CELL_OUTPUT", "LSTM_DELTA_CELL_OUTPUT"]]
        for kind, flag in kinds:
            Wk = l.n_units if kind.endswith("_GATE") else W
            a = gpu.download_tensor(li, mb.TENSOR[kind] | flag, T * Bmax * Wk)
            b = cpu.download_tensor(li, mb.TENSOR[kind] | flag, T * Bmax * Wk)
            assert_close(_rows(a, T, Bmax, B, Wk), _rows(b, T, Bmax, B, Wk), REL, ABS, what="%s layer %d %s%s" % (what, li, kind, " (backward)" if flag else ""))


bi = lambda units, cpb=1: dict(type="lstm", units=units, cells_per_block=cpb, bidirectional=True)

CASES = [
    ("single-layer", [dict(units=6), bi(5), dict(units=7, activation="LINEAR")], 4, 5, 5, "MSE"),
    ("two-cells-per-block-partial-batch", [dict(units=4), bi(3, 2), dict(units=6, activation="TANH")], 5, 3, 7, "MSE"),
    ("stacked-with-fc-below", [dict(units=5), dict(units=12, activation="TANH"), bi(8), bi(4, 3), dict(units=9, activation="LINEAR")], 6, 6, 6, "MSE"),
    ("unfused-activation-below-and-mixed-directions", [dict(units=8), dict(units=12, activation="ELU"), bi(12), dict(type="lstm", units=10),
                                                       dict(units=10, activation="LINEAR")], 4, 8, 8, "MSE"),
    ("single-step", [dict(units=3), bi(5), dict(units=6, activation="LINEAR")], 1, 4, 4, "MSE"),
    ("two-steps", [dict(units=3), bi(4), dict(units=5, activation="LINEAR")], 2, 7, 7, "MSE"),
    ("config5-shape-shrunk", [dict(units=32), bi(64), dict(units=32, activation="SOFTMAX")], 24, 16, 16, "CROSS_ENTROPY"),
]


@pytest.mark.parametrize("name,specs,T,B,Bmax,loss", CASES, ids=[c[0] for c in CASES])
def test_two_direction_lstm_parity_adabound_clip(name, specs, T, B, Bmax, loss):
    """three steps of config 5's recipe: gradient clipping at norm 1, AdaBound"""
    desc = mb.make_desc(specs, Bmax, T)
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["ADABOUND"], type_loss_function=mb.LOSS[loss],
                         type_accuracy_function=mb.ACCURACY["CROSS_ENTROPY" if loss == "CROSS_ENTROPY" else "DISTANCE"], use_clip_gradient=1, clip_gradient=1.0)
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h)
    w = glorot_parameters(desc, 13, bias_range=0.3)
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
    rng = np.random.default_rng(14)
    n_in, n_out = specs[0]["units"], specs[-1]["units"]
    X = rng.uniform(-1, 1, (B, T * n_in)).astype(np.float32)
    if loss == "CROSS_ENTROPY":
        Y = np.zeros((B, T, n_out), dtype=np.float32)
        np.put_along_axis(Y, rng.integers(0, n_out, (B, T))[..., None], 1.0, axis=2)
        Y = Y.reshape(B, -1)
    else:
        Y = rng.normal(0, 1, (B, T * n_out)).astype(np.float32)
    for step in range(3):
        for n in (gpu, cpu):
            n.Reset__Loss()
            run_step(n, B, X, Y, update=False)
        _compare(desc, gpu, cpu, B, T, what="step %d" % step)
        g_cpu = cpu.download_gradient()
        assert_close(gpu.download_gradient(), g_cpu, REL, ABS, what="gradient step %d" % step)
        lg, lc = gpu.get_loss(), cpu.get_loss()
        assert lg.number_loss == lc.number_loss and lg.loss_values == pytest.approx(lc.loss_values, rel=1e-4)
        assert lg.accuracy_value == lc.accuracy_value
        for n in (gpu, cpu):
            n.Update_Parameter(B, B)
        noisy = (np.abs(g_cpu) < 1e-5) & (g_cpu != 0)
        wg, wc = gpu.download_parameters(), cpu.download_parameters()
        assert noisy.mean() < 0.02
        assert_close(wg[~noisy], wc[~noisy], REL, ABS, what="parameters step %d" % step)
        assert np.all(np.abs(wg[noisy].astype(np.float64) - wc[noisy]) <= 2.1e-3)
        gpu.upload_parameters(wc)
