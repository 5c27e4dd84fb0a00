"""The LSTM time loop as one resident launch per layer and pass (C = 128, 256, 512 cells; 1024 forward only), through the
C ABI: against the same library with one launch per time step (MYEA_LSTM_RESIDENT=0), against the CPU oracle, and the
bounded wait's give-up path.  Tolerance rel 1e-4 / abs 1e-5 (the resident kernels use the exp2 and reciprocal
instructions in the gate functions, the per-step kernels expf and a division: a few ulp apart)."""
import os

import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import assert_close, environment, glorot_parameters, run_step
from tests.oracle_lib import OracleNetwork
from tests.test_gpu_lstm import LSTM_TAPS, _rows, _width

pytestmark = pytest.mark.gpu
REL, ABS = 1e-4, 1e-5
BACK = mb.TENSOR["DIRECTION_BACKWARD"]
FORWARD_LOOP, BACKWARD_LOOP = 5, 6   # profile families of the time loops


lstm = lambda units, **kw: dict(type="lstm", units=units, **kw)
zone = lambda units, **kw: dict(type="lstm", units=units, dropout="ZONEOUT", keep=0.3, keep_output=0.2, **kw)

# name, layers, T, B, Bmax, resident backward loop too
CASES = [
    ("128-cells-last-chain-ragged", [dict(units=24), lstm(128), dict(units=128, activation="LINEAR")], 9, 70, 72, True),
    ("128-cells-second-chain-empty", [dict(units=8), lstm(128), dict(units=128, activation="LINEAR")], 5, 13, 16, True),
    ("256-cells-two-directions", [dict(units=12), lstm(256, bidirectional=True), dict(units=256, activation="TANH")], 5, 33, 40, True),
    ("512-cells-zoneout-stacked", [dict(units=16), zone(512), lstm(128), dict(units=128, activation="LINEAR")], 4, 48, 48, True),
    ("512-cells-two-directions-ragged", [dict(units=9), lstm(512, bidirectional=True), dict(units=512, activation="LINEAR")], 4, 41, 44, True),
    ("1024-cells-two-directions", [dict(units=10), lstm(1024, bidirectional=True), dict(units=1024, activation="LINEAR")], 3, 40, 40, True),
    ("1024-cells-ragged-seven-steps", [dict(units=6), lstm(1024), dict(units=1024, activation="LINEAR")], 7, 45, 48, True),
    ("1024-cells-two-steps", [dict(units=5), lstm(1024), dict(units=1024, activation="LINEAR")], 2, 33, 33, True),
    ("1024-cells-twelve-steps-zoneout", [dict(units=7), zone(1024, bidirectional=True), dict(units=1024, activation="LINEAR")], 12, 64, 64, True),
    ("two-steps", [dict(units=6), lstm(256), dict(units=256, activation="LINEAR")], 2, 32, 32, True),
]


def _net(desc, h, w, masks):
    n = mb.HipNetwork(desc, h)
    n.set_state_propagation(mb.STATE_TRAINING)
    n.upload_parameters(w)
    if masks is not None:
        n.upload_zoneout_masks(masks)
    n.Clear_Training_Arrays()
    return n


def _setup(specs, T, B, Bmax, seed):
    desc = mb.make_desc(specs, Bmax, T)
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["ADAM"], type_loss_function=mb.LOSS["MSE"])
    w = glorot_parameters(desc, seed, bias_range=0.3)
    rng = np.random.default_rng(seed)
    masks = None
    if any(s.get("dropout") == "ZONEOUT" for s in specs):
        cells = sum(_width(desc.layers[i]) * (2 if desc.layers[i].use_bidirectional else 1)
                    for i in range(desc.n_layers) if desc.layers[i].type_layer == mb.LAYER_LSTM)
        masks = (rng.uniform(0, 1, 2 * T * cells) < 0.6).astype(np.uint8)
    X = rng.normal(0, 1, (B, T * specs[0]["units"])).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * specs[-1]["units"])).astype(np.float32)
    return desc, h, w, masks, X, Y


def _compare(desc, a_net, b_net, B, T, what):
    Bmax = desc.batch_size
    for li in range(1, desc.n_layers):
        l = desc.layers[li]
        W = _width(l)
        kinds = [("OUTPUTS", 0), ("ERRORS", 0)]
        if l.type_layer == mb.LAYER_LSTM:
            for flag in ((0, BACK) if l.use_bidirectional else (0,)):
                kinds += [(k, flag) for k in LSTM_TAPS + ["LSTM_CELL_OUTPUT", "LSTM_DELTA_CELL_OUTPUT"]]
        for kind, flag in kinds:
            a = a_net.download_tensor(li, mb.TENSOR[kind] | flag, T * Bmax * W)
            b = b_net.download_tensor(li, mb.TENSOR[kind] | flag, T * Bmax * W)
            assert_close(_rows(a, T, Bmax, B, W), _rows(b, T, Bmax, B, W), REL, ABS, what="%s layer %d %s/%d" % (what, li, kind, flag))
    g = b_net.download_gradient()
    assert_close(a_net.download_gradient(), g, REL, ABS * max(1.0, float(np.abs(g).max())), what=what + " gradient")


def _loop_launches(net):
    return net.profile_read(FORWARD_LOOP)[0], net.profile_read(BACKWARD_LOOP)[0]


# the backward loop has two resident forms: split along k (members exchange partial sums; the default) and split along the
# columns of dh (members read each other's gate deltas; MYEA_LSTM_BACKWARD_KSPLIT=0); at 512 cells the column form runs a
# member's two chains in two sets of wavefronts, or (MYEA_LSTM_BACKWARD_SETS=0) in one instruction stream as at other widths
FORMS = [("backward-split-along-k", "1", "1"), ("backward-split-along-columns", "0", "1")]
LOOP_CASES = [c + f[1:] for c in CASES for f in FORMS] + [c + ("0", "0") for c in CASES if "512-cells" in c[0]]
LOOP_IDS = ["%s-%s" % (f[0], c[0]) for c in CASES for f in FORMS] + ["backward-split-along-columns-one-stream-" + c[0] for c in CASES if "512-cells" in c[0]]


@pytest.mark.parametrize("name,specs,T,B,Bmax,backward,ksplit,sets", LOOP_CASES, ids=LOOP_IDS)
def test_resident_loop_matches_one_launch_per_step_and_the_oracle(name, specs, T, B, Bmax, backward, ksplit, sets):
    desc, h, w, masks, X, Y = _setup(specs, T, B, Bmax, seed=21)
    resident = _net(desc, h, w, masks)
    stepwise = _net(desc, h, w, masks)
    cpu = OracleNetwork(desc, h)
    cpu.set_state_propagation(mb.STATE_TRAINING)
    cpu.upload_parameters(w)
    if masks is not None:
        cpu.upload_zoneout_masks(masks)
    cpu.Clear_Training_Arrays()
    layers = [desc.layers[i] for i in range(desc.n_layers) if desc.layers[i].type_layer == mb.LAYER_LSTM]
    wide = [l for l in layers]   # every LSTM layer of these cases has a resident form
    per_step = sum((2 if l.use_bidirectional else 1) * (T - 1) for l in layers)
    for step in range(2):
        with environment(MYEA_LSTM_BACKWARD_KSPLIT=ksplit, MYEA_LSTM_BACKWARD_SETS=sets):
            resident.profile_enable(True)
            resident.Reset__Loss()
            run_step(resident, B, X, Y, update=False)
            fwd, bwd = _loop_launches(resident)
            resident.profile_enable(False)
        assert fwd == len(wide), "the forward time loops did not run as one launch per layer"
        if backward:
            assert bwd == len(wide), "the backward time loops did not run as one launch per layer"
        with environment(MYEA_LSTM_RESIDENT=0):
            stepwise.profile_enable(True)
            stepwise.Reset__Loss()
            run_step(stepwise, B, X, Y, update=False)
            assert _loop_launches(stepwise) == (per_step, per_step)
            stepwise.profile_enable(False)
        cpu.Reset__Loss()
        run_step(cpu, B, X, Y, update=False)
        _compare(desc, resident, stepwise, B, T, "step %d, resident vs per-step" % step)
        _compare(desc, resident, cpu, B, T, "step %d, resident vs oracle" % step)
        assert resident.get_loss().loss_values == pytest.approx(cpu.get_loss().loss_values, rel=1e-4)
        for n in (resident, stepwise, cpu):
            n.Update_Parameter(B, B)
        wc = cpu.download_parameters()
        resident.upload_parameters(wc)
        stepwise.upload_parameters(wc)


@pytest.mark.parametrize("ksplit", ["1", "0"], ids=["backward-split-along-k", "backward-split-along-columns"])
def test_bias_and_peephole_gradients_summed_inside_the_backward_loop(ksplit):
    """the resident backward loop sums the bias and peephole gradients of its layer as it goes; MYEA_LSTM_RESIDENT_SUMS=0 has the
    weight-gradient pass read the gate deltas once more instead: the same gradient either way, with examples missing from the last
    group, in both directions, and when a smaller batch follows a larger one"""
    specs = [dict(units=12), lstm(256, bidirectional=True), lstm(128), dict(units=128, activation="LINEAR")]
    T, Bmax = 7, 80
    desc, h, w, masks, X, Y = _setup(specs, T, Bmax, Bmax, seed=33)
    inside, apart = _net(desc, h, w, None), _net(desc, h, w, None)
    for B in (80, 45):
        with environment(MYEA_LSTM_BACKWARD_KSPLIT=ksplit):
            inside.profile_enable(True)
            run_step(inside, B, X[:B], Y[:B], update=False)
            assert _loop_launches(inside)[1] == 2, "the backward time loops did not run as one launch per layer"
            inside.profile_enable(False)
            with environment(MYEA_LSTM_RESIDENT_SUMS="0"):
                run_step(apart, B, X[:B], Y[:B], update=False)
        g = apart.download_gradient()
        assert np.abs(g).max() > 0
        assert_close(inside.download_gradient(), g, 2e-5, 2e-6 * float(np.abs(g).max()), what="batch %d: sums inside the loop against the separate pass" % B)
        for n in (inside, apart):
            n.Update_Parameter(B, B)


@pytest.mark.parametrize("name,specs,T,B,Bmax", [(c[0], c[1], c[2], c[3], c[4]) for c in CASES if "512-cells" in c[0] or "1024-cells" in c[0]],
                         ids=[c[0] for c in CASES if "512-cells" in c[0] or "1024-cells" in c[0]])
def test_the_path_of_a_late_group(name, specs, T, B, Bmax):
    """At 512 and 1024 cells a unit requests the next unit's first tiles between its own last MFMAs if the other chain's
    counter is complete by then, behind them if not; which of the two happens depends on timing.  Here the second is forced
    (every unit is told "not yet") and held against the oracle."""
    desc, h, w, masks, X, Y = _setup(specs, T, B, Bmax, seed=23)
    zone_masks = masks if any(s.get("dropout") == "ZONEOUT" for s in specs) else None
    gpu = _net(desc, h, w, zone_masks)
    cpu = OracleNetwork(desc, h)
    cpu.set_state_propagation(mb.STATE_TRAINING)
    cpu.upload_parameters(w)
    if zone_masks is not None:
        cpu.upload_zoneout_masks(zone_masks)
    cpu.Clear_Training_Arrays()
    # the backward form that stages tiles, with a member's two chains in one instruction stream (the form that has the two paths)
    with environment(MYEA_LSTM_RESIDENT_TEST_NEVER_EARLY=1, MYEA_LSTM_BACKWARD_KSPLIT=0, MYEA_LSTM_BACKWARD_SETS=0):
        gpu.profile_enable(True)
        for n in (gpu, cpu):
            n.Reset__Loss()
            run_step(n, B, X[:B], Y[:B], update=False)
        fwd, bwd = _loop_launches(gpu)
        gpu.profile_enable(False)
    layers = sum(1 for i in range(desc.n_layers) if desc.layers[i].type_layer == mb.LAYER_LSTM)
    assert fwd == layers and bwd == layers, "the time loops did not run as one launch per layer"
    _compare(desc, gpu, cpu, B, T, "late path")


def test_a_smaller_batch_after_a_larger_one():
    """rows beyond the batch keep what the larger batch left there; the rows of the batch do not depend on them"""
    specs = [dict(units=8), lstm(128), dict(units=128, activation="LINEAR")]
    T, Bmax = 6, 64
    desc, h, w, masks, X, Y = _setup(specs, T, Bmax, Bmax, seed=5)
    gpu = _net(desc, h, w, None)
    cpu = OracleNetwork(desc, h)
    cpu.set_state_propagation(mb.STATE_TRAINING)
    cpu.upload_parameters(w)
    cpu.Clear_Training_Arrays()
    for B in (64, 19, 33):
        for n in (gpu, cpu):
            n.Clear_Training_Arrays()
            n.Reset__Loss()
            run_step(n, B, X[:B], Y[:B], update=False)
        _compare(desc, gpu, cpu, B, T, "batch %d" % B)


def test_a_wait_that_gives_up_is_reported_once_and_the_network_carries_on_per_step():
    """Every group is told to expect a member that does not exist: the first wait between time steps runs out of polls,
    every wavefront leaves through the give-up path, the next call that looks reports MYEA_E_DEVICE, and from then on the
    network uses one launch per time step."""
    specs = [dict(units=8), lstm(128), dict(units=128, activation="LINEAR")]
    T, B = 5, 32
    desc, h, w, masks, X, Y = _setup(specs, T, B, B, seed=7)
    gpu = _net(desc, h, w, None)
    with environment(MYEA_LSTM_RESIDENT_TEST_ABSENT_MEMBER=1, MYEA_LSTM_RESIDENT_SPIN_POLLS=64):
        gpu.Forward_Pass(B, X)
        with pytest.raises(mb.MyeaError) as e:
            gpu.synchronize()
    assert e.value.code == mb.E_DEVICE and "gave up" in str(e.value)
    gpu.synchronize()   # reported once
    cpu = OracleNetwork(desc, h)
    cpu.set_state_propagation(mb.STATE_TRAINING)
    cpu.upload_parameters(w)
    cpu.Clear_Training_Arrays()
    gpu.profile_enable(True)
    for n in (gpu, cpu):
        n.Clear_Training_Arrays()
        n.Reset__Loss()
        run_step(n, B, X, Y, update=False)
    assert _loop_launches(gpu) == (T - 1, T - 1), "after a give-up the time loops run one launch per step"
    gpu.profile_enable(False)
    _compare(desc, gpu, cpu, B, T, "after the give-up")


@pytest.mark.parametrize("cells,ksplit", [(128, "1"), (128, "0"), (512, "0"), (1024, "0")],
                         ids=["backward-split-along-k", "backward-split-along-columns", "512-cells-a-set-of-wavefronts-per-chain", "1024-cells-across-two-xcds"])
def test_a_backward_wait_that_gives_up_is_reported_too(cells, ksplit):
    """the same forced give-up in the backward loop, in each of its forms (at 1024 cells with tile loads into LDS in flight
    when the wait begins; at 512 cells every wait of the two sets of wavefronts - for the group, for the turn, for each other -
    runs out on its own): the forward pass runs normally, the backward loop's first wait between steps runs out of polls and
    every wavefront leaves"""
    specs = [dict(units=8), lstm(cells), dict(units=cells, activation="LINEAR")]
    T, B = 5, 32
    desc, h, w, masks, X, Y = _setup(specs, T, B, B, seed=9)
    gpu = _net(desc, h, w, None)
    gpu.Forward_Pass(B, X)
    gpu.Compute__Error(B, Y)
    gpu.synchronize()
    with environment(MYEA_LSTM_RESIDENT_TEST_ABSENT_MEMBER=1, MYEA_LSTM_RESIDENT_SPIN_POLLS=64, MYEA_LSTM_BACKWARD_KSPLIT=ksplit):
        gpu.Backward_Pass(B)
        with pytest.raises(mb.MyeaError) as e:
            gpu.synchronize()
    assert e.value.code == mb.E_DEVICE and "gave up" in str(e.value)
    cpu = OracleNetwork(desc, h)
    cpu.set_state_propagation(mb.STATE_TRAINING)
    cpu.upload_parameters(w)
    cpu.Clear_Training_Arrays()
    for n in (gpu, cpu):
        n.Clear_Training_Arrays()
        n.Reset__Loss()
        run_step(n, B, X, Y, update=False)
    _compare(desc, gpu, cpu, B, T, "after the backward give-up")


def test_weight_contractions_beside_the_backward_loop_change_nothing():
    """the combined backward + weight-gradient call runs the weight contractions of the layer above on a second stream beside an
    LSTM layer's backward time loop (and picks the loop's form that leaves them room): same gradient as the two separate calls
    within the tolerance the two resident forms are held to, and the same as the oracle"""
    specs = [dict(units=16), lstm(128), lstm(128), dict(units=128, activation="LINEAR")]
    T, B = 6, 64
    desc, h, w, masks, X, Y = _setup(specs, T, B, B, seed=13)
    combined, separate = _net(desc, h, w, None), _net(desc, h, w, None)
    cpu = OracleNetwork(desc, h)
    cpu.set_state_propagation(mb.STATE_TRAINING)
    cpu.upload_parameters(w)
    cpu.Clear_Training_Arrays()
    for step in range(2):
        combined.Forward_Pass(B, X)
        combined.Compute__Error(B, Y)
        combined.Backward_Pass__Update_Derivative_Weight(B)
        run_step(separate, B, X, Y, update=False)
        run_step(cpu, B, X, Y, update=False)
        g = cpu.download_gradient()
        tol = ABS * max(1.0, float(np.abs(g).max()))
        assert_close(combined.download_gradient(), separate.download_gradient(), REL, tol, what="step %d: combined against separate calls" % step)
        assert_close(combined.download_gradient(), g, REL, tol, what="step %d: combined against the oracle" % step)
        for n in (combined, separate, cpu):
            n.Update_Parameter(B, B)
        wc = cpu.download_parameters()
        combined.upload_parameters(wc)
        separate.upload_parameters(wc)
