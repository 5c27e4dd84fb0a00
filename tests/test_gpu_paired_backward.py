"""myea_hip_backward_pass_and_update_derivative_weight against the two calls it stands for: same deltas, same gradient, bit
for bit - at a batch of 1024 with 2048-wide layers, where a layer's weight-gradient contraction rides in the launch that sends
its delta down (checked through the profiling taps), and on small stacks of every kind, where it does not."""
import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, one_hot

pytestmark = pytest.mark.gpu


def _step(net, B, X, Y, fused):
    net.Forward_Pass(B, X)
    net.Compute__Error(B, Y)
    if fused:
        net.Backward_Pass__Update_Derivative_Weight(B)
    else:
        net.Backward_Pass(B)
        net.Update_Derivative_Weight(B)


def _pair(specs, B, T=1, seed=3, loss="MSE", Bmax=None):
    desc = mb.make_desc(specs, Bmax or B, T)
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["ADAM"], type_loss_function=mb.LOSS[loss])
    nets = [mb.HipNetwork(desc, h) for _ in range(2)]
    w = glorot_parameters(desc, seed, bias_range=0.3)
    rng = np.random.default_rng(seed)
    masks = (rng.uniform(0, 1, desc.total_mask_units) < 0.7).astype(np.uint8)
    for n in nets:
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.upload_masks(masks)
        n.Clear_Training_Arrays()
    n_in, n_out = specs[0]["units"], specs[-1]["units"]
    X = rng.normal(0, 1, (B, T * n_in)).astype(np.float32)
    Y = one_hot(rng.integers(0, n_out, B * T), n_out).reshape(B, T * n_out) if loss == "CROSS_ENTROPY" else rng.normal(0, 1, (B, T * n_out)).astype(np.float32)
    return desc, nets, X, Y, w


@pytest.mark.parametrize("B", [1024, 999])
def test_weight_gradient_rides_with_the_delta_at_batch_1024(B):
    specs = [dict(units=2048), dict(units=2048, activation="RELU"), dict(units=2048, activation="TANH"), dict(units=2048, activation="RELU"), dict(units=1000, activation="SOFTMAX")]
    desc, (a, b), X, Y, w = _pair(specs, B, loss="CROSS_ENTROPY", Bmax=1024)
    b.profile_enable(True)
    for step in range(2):                     # the second step accumulates onto a non-zero gradient
        _step(a, B, X, Y, fused=False)
        _step(b, B, X, Y, fused=True)
    pairs = b.profile_read(4)
    b.profile_enable(False)
    assert pairs[0] >= 4, "no paired launch happened: %r" % (pairs,)       # two per step: into layers 2 and 1... the head's pair too
    ga, gb = a.download_gradient(), b.download_gradient()
    assert np.array_equal(ga, gb)
    for li in range(1, desc.n_layers):
        assert np.array_equal(a.download_tensor(li, mb.TENSOR["ERRORS"]), b.download_tensor(li, mb.TENSOR["ERRORS"]))
    # and both agree with float64 on a slice of the largest layer's gradient: dW = delta^T X, accumulated twice
    l = desc.layers[2]
    delta = a.download_tensor(2, mb.TENSOR["ERRORS"]).reshape(1024, 2048)[:B].astype(np.float64)
    x = a.download_tensor(1, mb.TENSOR["OUTPUTS"]).reshape(1024, 2048)[:B].astype(np.float64)
    want = 2.0 * (delta[:, :64].T @ x)
    got = ga[l.first_connection_index:l.first_connection_index + 64 * 2048].reshape(64, 2048)
    assert_close(got, want, 1e-4, 1e-5 * float(np.abs(want).max()), what="dW rows 0..63 of layer 2")


CASES = [
    ("mlp-bn-dropout", [dict(units=20), dict(units=64, activation="RELU", normalization="BATCH_NORMALIZATION", dropout="BERNOULLI_INVERTED", keep=0.7),
                        dict(units=48, activation="TANH"), dict(units=5, activation="SOFTMAX")], 1, 16, "CROSS_ENTROPY"),
    ("lstm-ind-rnn", [dict(units=8), dict(type="lstm", units=16), dict(type="ind_rnn", units=24, activation="RELU"), dict(units=16, activation="LINEAR")], 5, 6, "MSE"),
    ("residual-pool", [dict(units=12), dict(units=32, activation="TANH"), dict(type="residual", block_depth=2), dict(units=24, activation="RELU"), dict(units=32, activation="RELU"),
                       dict(type="max_pooling", kernel=2, stride=2), dict(units=4, activation="LINEAR")], 1, 9, "MSE"),
]


@pytest.mark.parametrize("name,specs,T,B,loss", CASES, ids=[c[0] for c in CASES])
def test_one_call_equals_the_two_calls(name, specs, T, B, loss):
    desc, (a, b), X, Y, w = _pair(specs, B, T, loss=loss)
    for step in range(2):
        _step(a, B, X, Y, fused=False)
        _step(b, B, X, Y, fused=True)
        assert np.array_equal(a.download_gradient(), b.download_gradient())
        a.Update_Parameter(B, B); b.Update_Parameter(B, B)
        assert np.array_equal(a.download_parameters(), b.download_parameters())
    with pytest.raises(mb.MyeaError):          # the error behaviour of Backward_Pass: not in the inference state
        b.set_state_propagation(mb.STATE_INFERENCE)
        b.Backward_Pass__Update_Derivative_Weight(B)


@pytest.mark.parametrize("B", [512, 500, 449])
def test_weight_gradient_rides_with_the_delta_at_batch_512(B):
    """one size down: the delta's contraction as 64 x 64 tiles beside the weight gradient's 128 x 128 ones; batches that leave
    the last row tile ragged (500) and that end a k range off the step of 32 (449, also an odd row count)"""
    specs = [dict(units=2048), dict(units=2048, activation="RELU"), dict(units=2048, activation="TANH"), dict(units=100, activation="SOFTMAX")]
    desc, (a, b), X, Y, w = _pair(specs, B, loss="CROSS_ENTROPY", Bmax=512)
    b.profile_enable(True)
    for step in range(2):
        _step(a, B, X, Y, fused=False)
        _step(b, B, X, Y, fused=True)
    pairs = b.profile_read(4)
    b.profile_enable(False)
    assert pairs[0] >= 2, "no paired launch happened: %r" % (pairs,)
    assert np.array_equal(a.download_gradient(), b.download_gradient())
    for li in range(1, desc.n_layers):
        assert np.array_equal(a.download_tensor(li, mb.TENSOR["ERRORS"]), b.download_tensor(li, mb.TENSOR["ERRORS"]))
    # and the gradient itself against float64 on a slice: dW = delta^T X over the B rows in use, accumulated twice
    l = desc.layers[2]
    delta = a.download_tensor(2, mb.TENSOR["ERRORS"]).reshape(512, 2048)[:B].astype(np.float64)
    x = a.download_tensor(1, mb.TENSOR["OUTPUTS"]).reshape(512, 2048)[:B].astype(np.float64)
    want = 2.0 * (delta[:, :48].T @ x)
    got = a.download_gradient()[l.first_connection_index:l.first_connection_index + 48 * 2048].reshape(48, 2048)
    assert_close(got, want, 1e-4, 1e-5 * float(np.abs(want).max()), what="dW rows 0..47 of layer 2")
