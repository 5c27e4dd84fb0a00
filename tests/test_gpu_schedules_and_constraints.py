"""GPU parity of Update_Parameter's remaining branches: AMSBound, NosAdam, iRPROP+, the max-norm constraint, normalized
weight decay and cosine warm restarts - the HIP library (through its C ABI) against the CPU oracle, fed the same
gradient sequence.  Tolerance: rel 1e-4 / abs 1e-5 on weights and optimizer state (fp32); iRPROP+ is sign logic and
must agree bit for bit; the scalar state the update advances (time steps, cycle length, running sums) exactly."""
import numpy as np
import pytest
import torch   # before the library first touches the device: imported later, torch finds no GPU in this process

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters
from tests.oracle_lib import OracleNetwork

pytestmark = pytest.mark.gpu

REL, ABS = 1e-4, 1e-5
FC = [dict(units=37), dict(units=53, activation="TANH"), dict(units=19, activation="SIGMOID")]   # P % 4 != 0
STATE_FIELDS = ("optimizer_time_step", "epoch_time_step", "adam_previous_beta2", "loss_rprop", "previous_loss_rprop",
                "warm_restarts_T_i", "warm_restarts_maximum_learning_rate")


def _pair(specs, hyper_kw, T=1, B=4, seed=0):
    desc = mb.make_desc(specs, B, T)
    h = mb.default_hyper(**hyper_kw)
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h)
    w = glorot_parameters(desc, seed)
    for n in (gpu, cpu):
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
    return desc, gpu, cpu


def _check(desc, gpu, cpu, what, exact=False):
    pairs = [("parameters", gpu.download_parameters(), cpu.download_parameters())]
    pairs += [(k, gpu.download_optimizer_state(v), cpu.download_optimizer_state(v)) for k, v in mb.OPT_STATE.items()]
    for name, a, b in pairs:
        if exact:
            assert np.array_equal(a, b), "%s: %s differs" % (what, name)
        else:
            assert_close(a, b, REL, ABS, what="%s %s" % (what, name))
    assert np.all(gpu.download_gradient() == 0)
    hg, hc = gpu.get_hyper(), cpu.get_hyper()
    for f in STATE_FIELDS:
        a, b = getattr(hg, f), getattr(hc, f)
        assert a == b or abs(a - b) <= 1e-6 * abs(b), "%s: hyper.%s %r != %r" % (what, f, a, b)


def _grads(P, steps, seed, scale=None):
    rng = np.random.default_rng(seed)
    out = [rng.normal(0, 0.5, P).astype(np.float32) for _ in range(steps)]
    if scale:
        out = [g * s for g, s in zip(out, scale)]
    return out


@pytest.mark.parametrize("kind,kw", [
    ("AMSBOUND", dict(learning_rate_final=0.1, learning_gamma=0.5)),
    ("AMSBOUND", dict(regularization__weight_decay=0.01, use_clip_gradient=1, clip_gradient=0.7)),
    ("NOSADAM", dict(adam_gamma=0.1)),
    ("NOSADAM", dict(adam_gamma=0.6, regularization__weight_decay=0.02, use_adam_bias_correction=0)),
])
def test_amsbound_and_nosadam(kind, kw):
    desc, gpu, cpu = _pair(FC, dict(type_optimizer_function=mb.OPTIMIZER[kind], **kw))
    grads = _grads(desc.total_parameters, 6, 1, scale=(4, 2, 1, 0.05, 0.02, 3))
    for k, g in enumerate(grads):
        for n in (gpu, cpu):
            n.upload_gradient(g)
            n.Update_Parameter(4, 64)
        _check(desc, gpu, cpu, "%s step %d" % (kind, k))


def test_irprop_plus_is_bit_exact_over_sign_changes_and_loss_flags():
    desc, gpu, cpu = _pair(FC, dict(type_optimizer_function=mb.OPTIMIZER["IRPROP_PLUS"], rprop_delta_zero=0.07, rprop_delta_max=0.2, rprop_delta_min=0.03))
    P = desc.total_parameters
    grads = _grads(P, 9, 2)
    grads[4][::5] = 0.0                                              # exact zeros take the third branch
    losses = [(3.0, 4.0), (2.5, 3.0), (2.7, 2.5), (2.6, 2.7), (2.9, 2.6), (2.9, 2.9), (1.0, 2.9), (1.5, 1.0), (1.2, 1.5)]
    for k, g in enumerate(grads):
        for n in (gpu, cpu):
            h = n.get_hyper(); h.loss_rprop, h.previous_loss_rprop = losses[k]; n.set_hyper(h)
            n.upload_gradient(g)
            n.Update_Parameter(4, 4)
        _check(desc, gpu, cpu, "iRPROP+ step %d" % k, exact=True)
    steps = gpu.download_optimizer_state(mb.OPT_STATE["PREVIOUS_STEPS"])
    assert steps.min() >= np.float32(0.03) and steps.max() <= np.float32(0.2) and len(np.unique(steps)) > 3
    for n in (gpu, cpu):
        n.Clear_Training_Arrays()
    _check(desc, gpu, cpu, "after Clear_Training_Arrays", exact=True)
    assert np.all(gpu.download_optimizer_state(mb.OPT_STATE["PREVIOUS_STEPS"]) == np.float32(0.07))


@pytest.mark.parametrize("kind,kw", [
    ("GD", dict(learning_rate=0.02, learning_momentum=0.9, use_Nesterov=1, regularization__weight_decay=0.05)),
    ("GD", dict(learning_rate=0.02, learning_momentum=0.0, regularization__weight_decay=0.05)),
    ("ADAM", dict(regularization__weight_decay=0.05)),
    ("ADABOUND", dict(learning_rate_final=0.05, learning_gamma=0.3)),
])
def test_warm_restarts_with_normalized_weight_decay(kind, kw):
    """three restarts inside the run (T_i 3 -> 6 -> 12); batch 4 of a set of 100 at epoch 2 scales the decay by sqrt(4/200)"""
    sched = dict(use_Warm_Restarts=1, warm_restarts_minimum_learning_rate=1e-4, warm_restarts_maximum_learning_rate=0.05,
                 warm_restarts_T_i=3.0, warm_restarts_multiplier=2.0, warm_restarts_decay_learning_rate=0.7)
    desc, gpu, cpu = _pair(FC, dict(type_optimizer_function=mb.OPTIMIZER[kind], **kw, **sched))
    for n in (gpu, cpu):
        h = n.get_hyper(); h.epoch_time_step = 2.0; n.set_hyper(h)
    grads = _grads(desc.total_parameters, 14, 3)
    for k, g in enumerate(grads):
        for n in (gpu, cpu):
            n.upload_gradient(g)
            n.Update_Parameter(4, 100)
        _check(desc, gpu, cpu, "%s update %d" % (kind, k))
    assert gpu.get_hyper().warm_restarts_T_i == 12.0 and gpu.get_hyper().epoch_time_step == 1.0


def _row_norms(desc, w, li, fan_in):
    l = desc.layers[li]
    return np.linalg.norm(w[l.first_connection_index:l.last_connection_index].reshape(-1, fan_in).astype(np.float64), axis=1)


@pytest.mark.parametrize("widths", [(37, 53, 19), (1030, 24, 2048, 8)], ids=["wave-per-neuron", "workgroup-per-neuron"])
def test_max_norm_constraint_on_fully_connected_layers(widths):
    specs = [dict(units=widths[0])] + [dict(units=u, activation="TANH") for u in widths[1:]]
    c = 0.9
    desc, gpu, cpu = _pair(specs, dict(type_optimizer_function=mb.OPTIMIZER["ADAM"], adam_learning_rate=0.02, regularization__max_norm_constraints=c))
    before = gpu.download_parameters()
    assert max(_row_norms(desc, before, li, widths[li - 1]).max() for li in range(1, len(widths))) > c
    for k, g in enumerate(_grads(desc.total_parameters, 3, 4)):
        for n in (gpu, cpu):
            n.upload_gradient(g)
            n.Update_Parameter(4, 4)
        _check(desc, gpu, cpu, "max-norm step %d" % k)
        w = gpu.download_parameters()
        norms = np.concatenate([_row_norms(desc, w, li, widths[li - 1]) for li in range(1, len(widths))])
        assert norms.max() <= c * (1 + 1e-5)
        assert (norms < c * (1 - 1e-3)).any() and (np.abs(norms - c) < 1e-5 * c).any()      # both branches were taken


@pytest.mark.parametrize("bidirectional", [False, True])
def test_max_norm_constraint_on_lstm_gate_vectors(bidirectional):
    specs = [dict(units=6), dict(type="lstm", units=5, cells_per_block=2, bidirectional=bidirectional), dict(units=24, activation="LINEAR")]
    c = 0.5
    desc, gpu, cpu = _pair(specs, dict(type_optimizer_function=mb.OPTIMIZER["GD"], learning_rate=0.05, learning_momentum=0.0,
                                       regularization__max_norm_constraints=c), T=3)
    w0 = gpu.download_parameters()
    for k, g in enumerate(_grads(desc.total_parameters, 2, 5)):
        for n in (gpu, cpu):
            n.upload_gradient(g)
            n.Update_Parameter(4, 4)
        _check(desc, gpu, cpu, "lstm max-norm step %d" % k)
    w = gpu.download_parameters()
    assert np.linalg.norm(w[:6]) > c                     # the vector at flat index 0 is never projected
    assert np.linalg.norm(w[6:16]) <= c * (1 + 1e-5)     # the recurrent vector after it is
    assert not np.array_equal(w, w0)
    # the projected weights are the ones the next forward pass multiplies with
    X = np.random.default_rng(0).normal(0, 1, (4, 3, 6)).astype(np.float32)
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.Forward_Pass(4, X)
    assert_close(gpu.download_tensor(2, mb.TENSOR["OUTPUTS"], 3 * 4 * 24), cpu.download_tensor(2, mb.TENSOR["OUTPUTS"], 3 * 4 * 24), REL, ABS)


def test_normalized_weight_decay_needs_the_training_set_size():
    desc, gpu, _ = _pair(FC, dict(type_optimizer_function=mb.OPTIMIZER["ADAM"], regularization__weight_decay=0.01))
    gpu.upload_gradient(np.ones(desc.total_parameters, dtype=np.float32))
    with pytest.raises(mb.MyeaError) as e:
        gpu.Update_Parameter(4, 0)
    assert e.value.code == mb.E_INVALID
    assert gpu.get_hyper().optimizer_time_step == 0
    gpu.Update_Parameter(4, 4)
    assert gpu.get_hyper().optimizer_time_step == 1


def test_clear_optimizer_touches_the_current_optimizers_state_only_on_the_gpu():
    from tests.test_oracle_optimizers import SPECS, check_clear_optimizer_touches_the_current_optimizers_state_only

    def make(**kw):
        desc = mb.make_desc(SPECS, 2)
        return desc, mb.HipNetwork(desc, mb.default_hyper(**kw))
    check_clear_optimizer_touches_the_current_optimizers_state_only(make)


def test_irprop_minus_through_the_kernel_level_entry_is_bit_exact():
    """iRPROP- (Neural_Network__iRPROP_minus.cpp:21-67) has no case in the reference's Update_Parameter, so it is reached the way
    the reference leaves it reachable: as a function of its own, myea_hip_optimizer_update on raw device vectors, against the
    oracle's restatement fed the same gradients (sign changes, zeros, steps at the cap and at the floor; a length that is not a
    multiple of four)."""
    import ctypes as C
    from tests.oracle_lib import load_oracle
    lib, olib = mb.load_library(), load_oracle()
    n = 100003
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["IRPROP_MINUS"], rprop_delta_max=0.15, rprop_delta_min=0.02)
    rng = np.random.default_rng(12)
    w = rng.normal(0, 1, n).astype(np.float32)
    steps, slopes = np.full(n, 0.1, np.float32), np.zeros(n, np.float32)
    dev = [torch.from_numpy(a.copy()).cuda() for a in (w, np.zeros(n, np.float32), steps, slopes)]
    for k in range(8):
        g = rng.normal(0, 1, n).astype(np.float32) * (rng.uniform(0, 1, n) > 0.1)    # a tenth exact zeros
        if k % 3 == 2:
            g = np.abs(g) * np.sign(slopes + (slopes == 0))                           # mostly the sign of before: steps reach the cap
        dev[1].copy_(torch.from_numpy(g))
        gc = g.copy()
        olib.myea_oracle_irprop_minus(C.byref(h), n, *(C.c_void_p(a.ctypes.data) for a in (w, gc, steps, slopes)))
        rc = lib.myea_hip_optimizer_update(None, C.byref(h), n, n, 1.0, C.c_void_p(dev[0].data_ptr()), C.c_void_p(dev[1].data_ptr()), None,
                                           C.c_void_p(dev[2].data_ptr()), C.c_void_p(dev[3].data_ptr()))
        assert rc == 0, lib.myea_hip_last_error()
        torch.cuda.synchronize()
        assert np.array_equal(dev[0].cpu().numpy(), w), "weights, update %d" % k
        assert np.array_equal(dev[2].cpu().numpy(), steps) and np.array_equal(dev[3].cpu().numpy(), slopes)
        assert not dev[1].cpu().numpy().any()
    assert steps.max() == np.float32(0.15) and steps.min() == np.float32(0.02)
    # the network-level update refuses it, as the reference's switch does
    desc, gpu, cpu = _pair(FC, dict(type_optimizer_function=mb.OPTIMIZER["IRPROP_MINUS"]))
    with pytest.raises(mb.MyeaError) as e:
        gpu.Update_Parameter(4, 4)
    assert e.value.code == mb.E_UNSUPPORTED
