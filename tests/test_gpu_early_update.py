"""myea_hip_backward_pass_update_derivative_weight_and_update_parameter against the calls it stands for: the same parameters,
optimizer state and time step, bit for bit, after several steps - on a stack wide enough for the weights of its layers to take
their step beside the contractions below them (checked through the profiling taps: one update launch per range instead of
one per step), on small stacks of every kind, and where the update's scalars are not known up front (clipping, iRPROP+) and
the calls simply run in turn.  (The separate calls are the ones the other tests hold against the oracle.)"""
import contextlib
import os

import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import glorot_parameters, one_hot

pytestmark = pytest.mark.gpu

UPDATE_FAMILY = 3


@contextlib.contextmanager
def environment(**kv):
    old = {k: os.environ.get(k) for k in kv}
    os.environ.update({k: str(v) for k, v in kv.items()})
    try:
        yield
    finally:
        for k, v in old.items():
            if v is None:
                del os.environ[k]
            else:
                os.environ[k] = v


def _step(net, B, X, Y, training_size, combined):
    net.Forward_Pass(B, X)
    net.Compute__Error(B, Y)
    if combined:
        net.Backward_Pass__Update_Derivative_Weight__Update_Parameter(B, training_size)
    else:
        net.Backward_Pass__Update_Derivative_Weight(B)
        net.Update_Parameter(B, training_size)


def _setup(specs, B, T, optimizer, loss, seed, Bmax=None, **hyper):
    desc = mb.make_desc(specs, Bmax or B, T)
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER[optimizer], type_loss_function=mb.LOSS[loss], **hyper)
    nets = [mb.HipNetwork(desc, h) for _ in range(2)]
    w = glorot_parameters(desc, seed, bias_range=0.3)
    rng = np.random.default_rng(seed)
    masks = (rng.uniform(0, 1, desc.total_mask_units) < 0.7).astype(np.uint8)
    for n in nets:
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        if desc.total_mask_units:
            n.upload_masks(masks)
        n.Clear_Training_Arrays()
    n_in, n_out = specs[0]["units"], specs[-1]["units"]
    X = rng.normal(0, 1, (B, T * n_in)).astype(np.float32)
    Y = one_hot(rng.integers(0, n_out, B * T), n_out).reshape(B, T * n_out) if loss == "CROSS_ENTROPY" else rng.normal(0, 1, (B, T * n_out)).astype(np.float32)
    return desc, nets, X, Y


def _same_state(a, b, kinds, what):
    assert np.array_equal(a.download_parameters(), b.download_parameters()), what + ": parameters"
    assert np.array_equal(a.download_gradient(), b.download_gradient()), what + ": gradient (zero after the update)"
    for kind in kinds:
        assert np.array_equal(a.download_optimizer_state(mb.OPT_STATE[kind]), b.download_optimizer_state(mb.OPT_STATE[kind])), what + ": " + kind
    assert a.get_hyper().optimizer_time_step == b.get_hyper().optimizer_time_step


@pytest.mark.parametrize("optimizer,kinds,hyper", [
    ("ADAM", ["FIRST_MOMENT", "SECOND_MOMENT"], dict(regularization__weight_decay=1e-3)),
    ("AMSGRAD", ["FIRST_MOMENT", "SECOND_MOMENT", "SECOND_MOMENT_HAT"], {}),
    ("GD", ["PREVIOUS_DELTA"], dict(learning_momentum=0.9, use_Nesterov=1)),
], ids=["adam-weight-decay", "amsgrad", "nesterov"])
def test_layers_step_beside_the_contractions_below_them(optimizer, kinds, hyper):
    specs = [dict(units=1024), dict(units=2048, activation="RELU"), dict(units=2048, activation="TANH"), dict(units=2048, activation="RELU"), dict(units=1000, activation="SOFTMAX")]
    B = 1024
    desc, (a, b), X, Y = _setup(specs, B, 1, optimizer, "CROSS_ENTROPY", seed=11, **hyper)
    b.profile_enable(True)
    steps = 3
    for step in range(steps):
        _step(a, B, X, Y, 4 * B, combined=False)
        with environment(MYEA_EARLY_UPDATE_MIN=0):   # layers of every size (by default only those of 8 M weights and more)
            _step(b, B, X, Y, 4 * B, combined=True)
        _same_state(a, b, kinds, "step %d" % step)
    launches = b.profile_read(UPDATE_FAMILY)[0]
    # every layer's weights on their own (4 ranges) and what is left (the biases) in one more launch
    assert launches == 5 * steps, "the update did not run layer by layer: %d launches in %d steps" % (launches, steps)
    # the default least size: none of these layers is large enough, one launch
    _step(b, B, X, Y, 4 * B, combined=True)
    _step(a, B, X, Y, 4 * B, combined=False)
    assert b.profile_read(UPDATE_FAMILY)[0] == 1   # reading the taps clears them
    b.profile_enable(False)
    _same_state(a, b, kinds, "default least size")


CASES = [
    ("mlp-bn-dropout-nesterov", [dict(units=20), dict(units=64, activation="RELU", normalization="BATCH_NORMALIZATION", dropout="BERNOULLI_INVERTED", keep=0.7),
                                 dict(units=48, activation="TANH"), dict(units=5, activation="SOFTMAX")], 1, 16, "CROSS_ENTROPY", "GD",
     dict(learning_momentum=0.9, use_Nesterov=1), ["PREVIOUS_DELTA"]),
    ("lstm-ind-rnn-adabound", [dict(units=8), dict(type="lstm", units=16), dict(type="ind_rnn", units=24, activation="RELU"), dict(units=16, activation="LINEAR")], 5, 6, "MSE",
     "ADABOUND", {}, ["FIRST_MOMENT", "SECOND_MOMENT"]),
    ("residual-pool-adam-max-norm", [dict(units=12), dict(units=32, activation="TANH"), dict(type="residual", block_depth=2), dict(units=24, activation="RELU"),
                                     dict(units=32, activation="RELU"), dict(type="max_pooling", kernel=2, stride=2), dict(units=4, activation="LINEAR")], 1, 9, "MSE",
     "ADAM", dict(regularization__max_norm_constraints=0.8), ["FIRST_MOMENT", "SECOND_MOMENT"]),
    ("mlp-odd-widths-adam", [dict(units=7), dict(units=13, activation="TANH"), dict(units=9, activation="RELU"), dict(units=3, activation="LINEAR")], 1, 5, "MSE",
     "ADAM", {}, ["FIRST_MOMENT", "SECOND_MOMENT"]),
    ("mlp-clipped-adam", [dict(units=16), dict(units=32, activation="TANH"), dict(units=8, activation="LINEAR")], 1, 12, "MSE",
     "ADAM", dict(use_clip_gradient=1, clip_gradient=0.05), ["FIRST_MOMENT", "SECOND_MOMENT"]),
    ("mlp-irprop", [dict(units=16), dict(units=32, activation="TANH"), dict(units=8, activation="LINEAR")], 1, 12, "MSE",
     "IRPROP_PLUS", {}, ["PREVIOUS_DELTA", "PREVIOUS_STEPS", "PREVIOUS_DERIVATIVES"]),
]


@pytest.mark.parametrize("name,specs,T,B,loss,optimizer,hyper,kinds", CASES, ids=[c[0] for c in CASES])
def test_one_call_equals_the_calls_it_stands_for(name, specs, T, B, loss, optimizer, hyper, kinds):
    desc, (a, b), X, Y = _setup(specs, B, T, optimizer, loss, seed=5, **hyper)
    with environment(MYEA_EARLY_UPDATE_MIN=0):
        for step in range(3):
            _step(a, B, X, Y, 3 * B, combined=False)
            _step(b, B, X, Y, 3 * B, combined=True)
            _same_state(a, b, kinds, "step %d" % step)
        # a smaller batch, then the error behaviour of Backward_Pass: not in the inference state
        small = max(1, B // 2)
        _step(a, small, X[:small], Y[:small], 3 * B, combined=False)
        _step(b, small, X[:small], Y[:small], 3 * B, combined=True)
        _same_state(a, b, kinds, "smaller batch")
    with pytest.raises(mb.MyeaError):
        b.set_state_propagation(mb.STATE_INFERENCE)
        b.Backward_Pass__Update_Derivative_Weight__Update_Parameter(B, B)
    assert a.get_hyper().optimizer_time_step == b.get_hyper().optimizer_time_step, "a refused call must not advance the optimizer's time step"
