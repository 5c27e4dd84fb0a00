"""GPU parity of myea_hip_update_derivative_weight_no_alloc (scratch memory in the library's static device array)
against myea_hip_update_derivative_weight, through the C ABI: same launches, so the gradients must be bit-identical.
Two calls in a row on each network, the second with a smaller batch, so that whatever the first call left in the
shared array is there when the second runs."""
import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import glorot_parameters, one_hot

pytestmark = pytest.mark.gpu


def _gradients(net, B, X, Y):
    """gradient through the existing entry point, then through the allocation-free one, from the same deltas"""
    P = net.desc.total_parameters
    net.Forward_Pass(B, X)
    net.Compute__Error(B, Y)
    net.Backward_Pass(B)
    net.upload_gradient(np.zeros(P, dtype=np.float32))
    net.Update_Derivative_Weight(B, 1, net.desc.n_layers)
    want = net.download_gradient()
    net.upload_gradient(np.zeros(P, dtype=np.float32))
    net.Update_Derivative_Weight__No_Alloc(B, 1, net.desc.n_layers)
    got = net.download_gradient()
    return got, want


def test_dense_stack_two_calls_second_smaller():
    # biases (column reductions through the scratch) and a narrow head over many rows (split-K slabs)
    specs = [dict(units=96), dict(units=160, activation="RELU"), dict(units=128, activation="TANH", normalization="BATCH_NORMALIZATION"),
             dict(units=10, activation="SOFTMAX")]
    Bmax = 192
    desc = mb.make_desc(specs, Bmax)
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["ADAM"], type_loss_function=mb.LOSS["CROSS_ENTROPY"])
    net = mb.HipNetwork(desc, h)
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(glorot_parameters(desc, 11))
    rng = np.random.default_rng(11)
    for B in (Bmax, 57):
        X = rng.normal(0, 1, (B, 96)).astype(np.float32)
        Y = one_hot(rng.integers(0, 10, B), 10)
        got, want = _gradients(net, B, X, Y)
        assert np.abs(want).max() > 0
        assert np.array_equal(got, want), "batch %d: %d entries differ" % (B, int((got != want).sum()))


def test_lstm_stack_two_calls_second_smaller():
    # packed weight-gradient slabs, peephole and bias partial sums of two LSTM layers, a dense head over T x batch rows
    T, Bmax, In = 12, 48, 24
    specs = [dict(units=In), dict(type="lstm", units=32), dict(type="lstm", units=32), dict(units=32, activation="LINEAR")]
    desc = mb.make_desc(specs, Bmax, T)
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["AMSGRAD"], type_loss_function=mb.LOSS["MSE"])
    net = mb.HipNetwork(desc, h)
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(glorot_parameters(desc, 12))
    rng = np.random.default_rng(12)
    for B in (Bmax, 20):
        X = rng.normal(0, 1, (B, T * In)).astype(np.float32)
        Y = rng.normal(0, 1, (B, T * 32)).astype(np.float32)
        got, want = _gradients(net, B, X, Y)
        assert np.abs(want).max() > 0
        assert np.array_equal(got, want), "batch %d: %d entries differ" % (B, int((got != want).sum()))


def test_rejects_a_network_beyond_the_static_buffer():
    # 16 slabs of 2048 x 640 packed gradients are 84 MB: more than the 32 MiB array
    desc = mb.make_desc([dict(units=128), dict(type="lstm", units=512), dict(units=512, activation="LINEAR")], 4, 3)
    net = mb.HipNetwork(desc, mb.default_hyper())
    net.set_state_propagation(mb.STATE_TRAINING)
    with pytest.raises(mb.MyeaError) as e:
        net.Update_Derivative_Weight__No_Alloc(4, 1, desc.n_layers)
    assert e.value.code == mb.E_INVALID and "static buffer holds" in str(e.value)
