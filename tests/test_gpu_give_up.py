"""What a bounded wait inside a kernel leaves behind when it gives up, through the C ABI.  Two kinds of kernels wait for
another workgroup: a contraction whose tiles two workgroups share (each half of k; the second waits for the first one's
half) and the resident LSTM time loops (a barrier between time steps).  The give-up is forced from the host - a poll
budget of zero, a member that does not exist - so that every kernel still exits normally.  Held here: the next call that
looks reports MYEA_E_DEVICE once; no Update_Parameter enqueued behind the incomplete pass has changed parameters or
optimizer state; the optimizer's time step is taken back; the gradient is cleared; the following step, on the plain form
of the kernel, matches the CPU oracle (rel 1e-4 / abs 1e-5)."""
import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import assert_close, environment, glorot_parameters, one_hot, run_step
from tests.oracle_lib import OracleNetwork

pytestmark = pytest.mark.gpu
REL, ABS = 1e-4, 1e-5


def _pair(specs, B, T, hyper, seed):
    desc = mb.make_desc(specs, B, T)
    h = mb.default_hyper(**hyper)
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h, threads=8)
    w = glorot_parameters(desc, seed, bias_range=0.2)
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
    return desc, gpu, cpu, w


def _state_untouched(gpu, w, kinds):
    assert np.array_equal(gpu.download_parameters(), w), "an update behind the incomplete pass changed the parameters"
    for kind in kinds:
        assert not gpu.download_optimizer_state(mb.OPT_STATE[kind]).any(), "optimizer state %s changed" % kind
    assert not gpu.download_gradient().any(), "the gradient is cleared"
    assert gpu.get_hyper().optimizer_time_step == 0.0, "the optimizer's time step is taken back"


def _steps_match(gpu, cpu, B, X, Y, steps=2):
    for step in range(steps):
        for n in (gpu, cpu):
            run_step(n, B, X, Y, update=False)
        g = cpu.download_gradient()
        assert_close(gpu.download_gradient(), g, REL, ABS * max(1.0, float(np.abs(g).max())), what="gradient, step %d after the give-up" % step)
        for n in (gpu, cpu):
            n.Update_Parameter(B, B)
        noisy = (np.abs(g) < 1e-5) & (g != 0)     # an Adam-type step of a gradient that is rounding noise follows the noise
        wg, wc = gpu.download_parameters(), cpu.download_parameters()
        assert noisy.mean() < 0.02
        assert_close(wg[~noisy], wc[~noisy], REL, ABS, what="parameters, step %d after the give-up" % step)
        gpu.upload_parameters(wc)
    assert gpu.get_hyper().optimizer_time_step == float(steps)


def test_a_shared_tile_wait_that_gives_up_is_reported_and_nothing_is_updated():
    """512 x 2048 x 2048 forward contractions run as 256 tiles of 64 x 64, each shared by two workgroups.  With a poll budget
    of zero the second workgroup of every tile gives up at once and stores nothing, so the pass is incomplete; a whole step
    including Update_Parameter is enqueued behind it before anything looks."""
    B = 512
    specs = [dict(units=2048), dict(units=2048, activation="SIGMOID"), dict(units=2048, activation="TANH"), dict(units=64, activation="SOFTMAX")]
    hyper = dict(type_optimizer_function=mb.OPTIMIZER["ADAM"], type_loss_function=mb.LOSS["CROSS_ENTROPY"])
    desc, gpu, cpu, w = _pair(specs, B, 1, hyper, seed=31)
    rng = np.random.default_rng(31)
    X = rng.normal(0, 1, (B, 2048)).astype(np.float32)
    Y = one_hot(rng.integers(0, 64, B), 64)
    with environment(MYEA_GEMM_PAIR_SPIN_POLLS=0):
        gpu.Forward_Pass(B, X)
    gpu.Compute__Error(B, Y)
    gpu.Backward_Pass__Update_Derivative_Weight__Update_Parameter(B, B)
    with pytest.raises(mb.MyeaError) as e:
        gpu.synchronize()
    assert e.value.code == mb.E_DEVICE and "gave up" in str(e.value) and "1 update" in str(e.value)
    gpu.synchronize()     # reported once
    _state_untouched(gpu, w, ("FIRST_MOMENT", "SECOND_MOMENT"))
    _steps_match(gpu, cpu, B, X, Y)


def test_two_updates_behind_a_give_up_are_both_skipped_and_counted():
    """the host may run several mini-batches ahead of the device: every update between the incomplete pass and the call that
    reports it is left out, and the time step goes back to where the last update that ran left it"""
    B = 512
    specs = [dict(units=2048), dict(units=2048, activation="TANH"), dict(units=32, activation="SOFTMAX")]
    hyper = dict(type_optimizer_function=mb.OPTIMIZER["AMSGRAD"], type_loss_function=mb.LOSS["CROSS_ENTROPY"])
    desc, gpu, cpu, w = _pair(specs, B, 1, hyper, seed=37)
    rng = np.random.default_rng(37)
    X = rng.normal(0, 1, (B, 2048)).astype(np.float32)
    Y = one_hot(rng.integers(0, 32, B), 32)
    for n in (gpu, cpu):                       # one good step first
        run_step(n, B, X, Y)
    gpu.synchronize()
    w1 = gpu.download_parameters()
    m1 = gpu.download_optimizer_state(mb.OPT_STATE["FIRST_MOMENT"])
    with environment(MYEA_GEMM_PAIR_SPIN_POLLS=0):
        gpu.Forward_Pass(B, X)      # the incomplete pass
    gpu.Compute__Error(B, Y)
    gpu.Backward_Pass(B)
    gpu.Update_Derivative_Weight(B)
    gpu.Update_Parameter(B, B)
    # the next mini-batch's Forward_Pass may or may not see the word already: either way it or the synchronize reports it
    with pytest.raises(mb.MyeaError) as e:
        gpu.Forward_Pass(B, X)
        gpu.Compute__Error(B, Y)
        gpu.Backward_Pass(B)
        gpu.Update_Derivative_Weight(B)
        gpu.Update_Parameter(B, B)
        gpu.synchronize()
    assert e.value.code == mb.E_DEVICE
    assert np.array_equal(gpu.download_parameters(), w1)
    assert np.array_equal(gpu.download_optimizer_state(mb.OPT_STATE["FIRST_MOMENT"]), m1)
    assert gpu.get_hyper().optimizer_time_step == 1.0
    assert not gpu.download_gradient().any()
    gpu.upload_parameters(cpu.download_parameters())
    for kind in ("FIRST_MOMENT", "SECOND_MOMENT", "SECOND_MOMENT_HAT"):
        gpu.upload_optimizer_state(mb.OPT_STATE[kind], cpu.download_optimizer_state(mb.OPT_STATE[kind]))
    for n in (gpu, cpu):
        run_step(n, B, X, Y)
    noisy = np.abs(cpu.download_optimizer_state(mb.OPT_STATE["FIRST_MOMENT"])) < 1e-6
    assert_close(gpu.download_parameters()[~noisy], cpu.download_parameters()[~noisy], REL, ABS, what="parameters of the step after the give-up")


@pytest.mark.parametrize("where", ["forward", "backward"])
def test_a_time_loop_that_gives_up_leaves_parameters_and_optimizer_state_alone(where):
    """the resident LSTM time loop's give-up (every group expects a member that does not exist), with the rest of the step and
    its Update_Parameter enqueued behind it before anything looks"""
    T, B = 5, 32
    specs = [dict(units=8), dict(type="lstm", units=128), dict(units=128, activation="LINEAR")]
    hyper = dict(type_optimizer_function=mb.OPTIMIZER["AMSGRAD"], type_loss_function=mb.LOSS["MSE"])
    desc, gpu, cpu, w = _pair(specs, B, T, hyper, seed=41)
    rng = np.random.default_rng(41)
    X = rng.normal(0, 1, (B, T * 8)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * 128)).astype(np.float32)
    forced = dict(MYEA_LSTM_RESIDENT_TEST_ABSENT_MEMBER=1, MYEA_LSTM_RESIDENT_SPIN_POLLS=64)
    if where == "forward":
        with environment(**forced):
            gpu.Forward_Pass(B, X)
        gpu.Compute__Error(B, Y)
        gpu.Backward_Pass(B)
    else:
        gpu.Forward_Pass(B, X)
        gpu.Compute__Error(B, Y)
        with environment(**forced):
            gpu.Backward_Pass(B)
    gpu.Update_Derivative_Weight(B)
    gpu.Update_Parameter(B, B)
    with pytest.raises(mb.MyeaError) as e:
        gpu.synchronize()
    assert e.value.code == mb.E_DEVICE and "gave up" in str(e.value)
    _state_untouched(gpu, w, ("FIRST_MOMENT", "SECOND_MOMENT", "SECOND_MOMENT_HAT"))
    _steps_match(gpu, cpu, B, X, Y)
