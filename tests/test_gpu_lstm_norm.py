"""Normalised LSTM layers (batch normalisation / renormalisation of the eight gate sums and of the cell state at every time
step; one cell per block) through the C ABI against the CPU oracle: activations, deltas, the deltas of the nine normalised
groups, the gradient including the scale vectors, the running statistics, training over several updates, inference.
Tolerance rel 1e-4 / abs 1e-5 of the tensor's largest magnitude (the statistics divide by sigma: errors scale with it)."""
import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import assert_close, environment, run_step
from tests.oracle_lib import OracleNetwork
from tests.test_gpu_lstm import LSTM_TAPS, _rows, _width
from tests.test_oracle_lstm_norm import lstm, parameters

pytestmark = pytest.mark.gpu
REL, ABS = 1e-4, 1e-5
BACK = mb.TENSOR["DIRECTION_BACKWARD"]


def _pair(specs, Bmax, T, seed, masks=None, **hyper):
    desc = mb.make_desc(specs, Bmax, T)
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["ADAM"], type_loss_function=mb.LOSS["MSE"], **hyper)
    w = parameters(desc, seed)
    nets = []
    for cls in (mb.HipNetwork, OracleNetwork):
        n = cls(desc, h)
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        if masks is not None:
            n.upload_zoneout_masks(masks)
        n.Clear_Training_Arrays()
        nets.append(n)
    return desc, nets[0], nets[1]


def _close(a, b, what):
    scale = max(1.0, float(np.abs(b).max()))
    assert_close(a, b, REL, ABS * scale, what=what)


def _compare(desc, gpu, cpu, B, T, what, backward=True):
    Bmax = desc.batch_size
    for li in range(1, desc.n_layers):
        l = desc.layers[li]
        W = _width(l)
        kinds = [("OUTPUTS", 0)] + ([("ERRORS", 0)] if backward else [])
        if l.type_layer == mb.LAYER_LSTM:
            forward_taps = ["LSTM_CELL_INPUT", "LSTM_CELL_STATE", "LSTM_INPUT_GATE", "LSTM_FORGET_GATE", "LSTM_OUTPUT_GATE", "LSTM_CELL_OUTPUT"]
            for flag in ((0, BACK) if l.use_bidirectional else (0,)):
                kinds += [(k, flag) for k in (LSTM_TAPS + ["LSTM_CELL_OUTPUT", "LSTM_DELTA_CELL_OUTPUT"] if backward else forward_taps)]
        for kind, flag in kinds:
            a = gpu.download_tensor(li, mb.TENSOR[kind] | flag, T * Bmax * W)
            b = cpu.download_tensor(li, mb.TENSOR[kind] | flag, T * Bmax * W)
            _close(_rows(a, T, Bmax, B, W), _rows(b, T, Bmax, B, W), "%s: layer %d %s/%d" % (what, li, kind, flag))
        if l.type_layer != mb.LAYER_LSTM or l.type_normalization == mb.NORMALIZATION["NONE"]:
            continue
        for flag in ((0, BACK) if l.use_bidirectional else (0,)):
            for g in range(9):
                sel = mb.TENSOR_LSTM_NORM_GROUP(g) | flag
                for kind in ("NORM_MEANS", "NORM_VARIANCES", "NORM_MEANS_AVERAGES", "NORM_VARIANCES_AVERAGES"):
                    _close(gpu.download_tensor(li, mb.TENSOR[kind] | sel, T * W), cpu.download_tensor(li, mb.TENSOR[kind] | sel, T * W),
                           "%s: layer %d group %d %s/%d" % (what, li, g, kind, flag))
                for kind in ("NORM_HATS",) + (("ERRORS",) if backward else ()):
                    a = gpu.download_tensor(li, mb.TENSOR[kind] | sel, T * Bmax * W)
                    b = cpu.download_tensor(li, mb.TENSOR[kind] | sel, T * Bmax * W)
                    _close(_rows(a, T, Bmax, B, W), _rows(b, T, Bmax, B, W), "%s: layer %d group %d %s/%d" % (what, li, g, kind, flag))
    if backward:
        _close(gpu.download_gradient(), cpu.download_gradient(), what + ": gradient")


zone = dict(dropout="ZONEOUT", keep=0.4, keep_output=0.3)
CASES = [   # name, layers, T, B, Bmax
    ("one-layer", [dict(units=10), lstm(24), dict(units=24, activation="LINEAR")], 6, 19, 24),
    ("renormalised", [dict(units=10), lstm(24, normalization="BATCH_RENORMALIZATION"), dict(units=24, activation="TANH")], 5, 16, 16),
    ("stacked-on-a-dense-layer", [dict(units=7), dict(units=12, activation="TANH"), lstm(16), lstm(20), dict(units=20, activation="LINEAR")], 5, 13, 13),
    ("two-directions", [dict(units=9), lstm(16, bidirectional=True), dict(units=32, activation="LINEAR")], 4, 11, 12),
    ("zoneout", [dict(units=8), lstm(20, **zone), dict(units=20, activation="LINEAR")], 5, 14, 14),
    ("two-steps-wide", [dict(units=33), lstm(130), dict(units=130, activation="LINEAR")], 2, 70, 70),
    ("one-step", [dict(units=6), lstm(12), dict(units=12, activation="LINEAR")], 1, 9, 9),
    ("beside-a-plain-layer", [dict(units=8), dict(type="lstm", units=12), lstm(12), dict(units=12, activation="LINEAR")], 4, 10, 10),
]


@pytest.fixture(params=["one-launch-per-step", "launch-per-kernel"], autouse=True)
def step_form(request):
    """every test runs with a time step's work behind its recurrent contraction as one launch (the default) and as the sequence
    of statistics / apply / gate launches"""
    with environment(MYEA_LSTM_NORM_FUSED="1" if request.param == "one-launch-per-step" else "0"):
        yield request.param


@pytest.mark.parametrize("name,specs,T,B,Bmax", CASES, ids=[c[0] for c in CASES])
def test_training_steps_match_the_oracle(name, specs, T, B, Bmax):
    hyper = dict(batch_renormalization_r_correction_maximum=2.0, batch_renormalization_d_correction_maximum=3.0, normalization_momentum_average=0.3)
    rng = np.random.default_rng(31)
    masks = None
    desc0 = mb.make_desc(specs, Bmax, T)
    if any(s.get("dropout") == "ZONEOUT" for s in specs):
        cells = sum(_width(desc0.layers[i]) * (2 if desc0.layers[i].use_bidirectional else 1)
                    for i in range(desc0.n_layers) if desc0.layers[i].type_layer == mb.LAYER_LSTM)
        masks = (rng.uniform(0, 1, 2 * T * cells) < 0.6).astype(np.uint8)
    desc, gpu, cpu = _pair(specs, Bmax, T, 41, masks=masks, **hyper)
    X = rng.normal(0, 1, (B, T * specs[0]["units"])).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * specs[-1]["units"])).astype(np.float32)
    for step in range(3):
        for n in (gpu, cpu):
            n.Reset__Loss()
            run_step(n, B, X, Y, update=False)
        _compare(desc, gpu, cpu, B, T, "%s step %d" % (name, step))
        assert gpu.get_loss().loss_values == pytest.approx(cpu.get_loss().loss_values, rel=1e-4)
        for n in (gpu, cpu):
            n.Update_Parameter(B, B)
        _close(gpu.download_parameters(), cpu.download_parameters(), "%s step %d: parameters" % (name, step))
        gpu.upload_parameters(cpu.download_parameters())   # both sides continue from the same point


def test_inference_uses_the_running_statistics():
    specs = [dict(units=8), lstm(16), lstm(16, normalization="BATCH_RENORMALIZATION"), dict(units=16, activation="LINEAR")]
    T, B = 5, 12
    desc, gpu, cpu = _pair(specs, B, T, 43, normalization_momentum_average=0.5)
    rng = np.random.default_rng(2)
    X = rng.normal(0, 1, (B, T * 8)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * 16)).astype(np.float32)
    for n in (gpu, cpu):
        for _ in range(2):
            run_step(n, B, X, Y, update=False)
        n.set_state_propagation(mb.STATE_INFERENCE)
        n.Forward_Pass(7, X[:7])
    _compare(desc, gpu, cpu, 7, T, "inference", backward=False)


def test_running_statistics_can_be_restored():
    """the running mean and sigma of a group, written through the tensor upload a checkpoint uses, are what inference reads"""
    specs = [dict(units=6), lstm(12), dict(units=12, activation="LINEAR")]
    T, B = 3, 8
    desc, gpu, cpu = _pair(specs, B, T, 47)
    rng = np.random.default_rng(3)
    X = rng.normal(0, 1, (B, T * 6)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * 12)).astype(np.float32)
    run_step(cpu, B, X, Y, update=False)   # only the oracle trains; its statistics go to the GPU network
    for g in range(9):
        for kind in ("NORM_MEANS_AVERAGES", "NORM_VARIANCES_AVERAGES"):
            gpu.upload_tensor(1, mb.TENSOR[kind] | mb.TENSOR_LSTM_NORM_GROUP(g), cpu.download_tensor(1, mb.TENSOR[kind] | mb.TENSOR_LSTM_NORM_GROUP(g), T * 12))
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_INFERENCE)
        n.Forward_Pass(B, X)
    _close(gpu.download_tensor(2, mb.TENSOR["OUTPUTS"], T * B * 12), cpu.download_tensor(2, mb.TENSOR["OUTPUTS"], T * B * 12), "outputs from restored statistics")


def test_a_time_step_is_two_launches_per_pass(step_form):
    """behind its recurrent contraction a time step's normalisations and gate math are one launch (forward and backward); as
    separate kernels the same step takes six resp. six launches, which the library's own launch counter shows"""
    specs = [dict(units=8), lstm(32), dict(units=32, activation="LINEAR")]
    T, B = 6, 16
    desc, gpu, cpu = _pair(specs, B, T, 53)
    rng = np.random.default_rng(4)
    X = rng.normal(0, 1, (B, T * 8)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * 32)).astype(np.float32)
    gpu.profile_enable(True)
    run_step(gpu, B, X, Y, update=False)
    launches = gpu.profile_read(7)[0]       # the normalisation family's timed regions: one per launch group
    gpu.profile_enable(False)
    if step_form == "one-launch-per-step":
        assert launches == 2 * T
    else:
        assert launches > 2 * T
