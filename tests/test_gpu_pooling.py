"""GPU parity of average / max pooling layers inside fully-connected stacks: the HIP library (through its C ABI) against the
CPU oracle.  Pooled values, kept positions' effect and the scattered errors involve no rounding beyond the oracle's own
order of additions (the backward gather adds in the same order), so the layer's tensors are compared bit for bit; the
contractions around them to rel 1e-4 / abs 1e-5."""
import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, one_hot, run_step
from tests.oracle_lib import OracleNetwork

pytestmark = pytest.mark.gpu
REL, ABS = 1e-4, 1e-5

avg = lambda **kw: dict(type="average_pooling", **kw)
mx = lambda **kw: dict(type="max_pooling", **kw)
CASES = [
    ("average-2-2", [dict(units=20), dict(units=64, activation="RELU"), avg(kernel=2, stride=2), dict(units=10, activation="SOFTMAX")], 1, 9, 9),
    ("average-overlap-padding-ceil", [dict(units=12), dict(units=45, activation="TANH"), avg(kernel=5, stride=3, padding=2, ceil_mode=1), dict(units=7, activation="LINEAR")], 1, 6, 8),
    ("max-3-2-padding", [dict(units=20), dict(units=63, activation="TANH"), mx(kernel=3, stride=2, padding=1), dict(units=10, activation="SOFTMAX")], 1, 9, 9),
    ("max-dilated", [dict(units=8), dict(units=40, activation="LEAKY_RELU"), mx(kernel=3, stride=2, padding=2, dilation=3), dict(units=5, activation="LINEAR")], 1, 7, 7),
    ("two-poolings-in-a-row-bn-dropout", [dict(units=16), dict(units=96, activation="RELU", normalization="BATCH_NORMALIZATION", norm_before=True, dropout="BERNOULLI_INVERTED", keep=0.7),
                                          mx(kernel=2, stride=2), avg(kernel=3, stride=1, padding=1), dict(units=24, activation="TANH"), dict(units=4, activation="SOFTMAX")], 1, 32, 32),
    ("pooling-on-the-inputs", [dict(units=30), avg(kernel=3, stride=3), dict(units=12, activation="TANH"), dict(units=3, activation="LINEAR")], 1, 5, 5),
    ("per-time-step-partial-batch", [dict(units=6), dict(units=20, activation="TANH"), mx(kernel=4, stride=2), dict(units=5, activation="LINEAR")], 3, 4, 6),
]


@pytest.mark.parametrize("name,specs,T,B,Bmax", CASES, ids=[c[0] for c in CASES])
def test_pooling_stack_parity(name, specs, T, B, Bmax):
    desc = mb.make_desc(specs, Bmax, T)
    head = specs[-1]["activation"]
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["ADAM"], type_loss_function=mb.LOSS["CROSS_ENTROPY" if head == "SOFTMAX" else "MSE"])
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h)
    w = glorot_parameters(desc, 5, bias_range=0.3)
    rng = np.random.default_rng(5)
    masks = (rng.uniform(0, 1, desc.total_mask_units) < 0.7).astype(np.uint8)
    n_in, n_out = specs[0]["units"], specs[-1]["units"]
    X = rng.normal(0, 1, (B, T * n_in)).astype(np.float32)
    Y = (one_hot(rng.integers(0, n_out, B * T), n_out).reshape(B, T * n_out) if head == "SOFTMAX" else rng.normal(0, 1, (B, T * n_out)).astype(np.float32))
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.upload_masks(masks)
        n.Clear_Training_Arrays()
    for step in range(2):
        for n in (gpu, cpu):
            n.Reset__Loss()
            run_step(n, B, X, Y, update=False)
        for li in range(1, desc.n_layers):
            l = desc.layers[li]
            W = l.n_units
            for kind in ("OUTPUTS", "ERRORS"):
                a = gpu.download_tensor(li, mb.TENSOR[kind], T * Bmax * W).reshape(T, Bmax, W)[:, :B]
                b = cpu.download_tensor(li, mb.TENSOR[kind], T * Bmax * W).reshape(T, Bmax, W)[:, :B]
                assert_close(a, b, REL, ABS, what="step %d layer %d %s" % (step, li, kind))
        assert_close(gpu.download_gradient(), cpu.download_gradient(), REL, ABS, what="gradient step %d" % step)
        for n in (gpu, cpu):
            n.Update_Parameter(B, B)
        gpu.upload_parameters(cpu.download_parameters())
    assert gpu.get_loss().loss_values == pytest.approx(cpu.get_loss().loss_values, rel=1e-4)


def test_pooling_layer_tensors_are_bit_exact_given_the_same_input():
    """identity first layer: the pooling layers see exactly the uploaded inputs on both sides"""
    In = 37
    specs = [dict(units=In), mx(kernel=3, stride=2, padding=1), avg(kernel=2, stride=1), dict(units=6, activation="LINEAR")]
    desc = mb.make_desc(specs, 11)
    h = mb.default_hyper(type_loss_function=mb.LOSS["MSE"])
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h)
    w = glorot_parameters(desc, 2)
    rng = np.random.default_rng(2)
    X = rng.normal(0, 1, (11, In)).astype(np.float32)
    X[:, 5] = X[:, 6]                         # ties: the first maximum wins
    X[3] = -np.abs(X[3])                      # all negative: the padding's zero wins at the edges
    Y = rng.normal(0, 1, (11, 6)).astype(np.float32)
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        run_step(n, 11, X, Y, update=False)
    for li in (1, 2):
        W = desc.layers[li].n_units
        assert np.array_equal(gpu.download_tensor(li, mb.TENSOR["OUTPUTS"], 11 * W), cpu.download_tensor(li, mb.TENSOR["OUTPUTS"], 11 * W)), li
    # layer 2's errors come out of a contraction (tolerance); layer 1's are layer 2's errors scattered: exact given equal inputs
    e2g, e2c = gpu.download_tensor(2, mb.TENSOR["ERRORS"], 11 * desc.layers[2].n_units), cpu.download_tensor(2, mb.TENSOR["ERRORS"], 11 * desc.layers[2].n_units)
    assert_close(e2g, e2c, REL, ABS)
    assert_close(gpu.download_tensor(1, mb.TENSOR["ERRORS"], 11 * desc.layers[1].n_units), cpu.download_tensor(1, mb.TENSOR["ERRORS"], 11 * desc.layers[1].n_units), REL, ABS)


def test_pooling_error_paths():
    with pytest.raises(ValueError):
        mb.make_desc([dict(units=6), dict(units=8, activation="TANH"), mx(kernel=2, stride=2)], 2)
    desc = mb.make_desc([dict(units=6), dict(units=8, activation="TANH"), mx(kernel=2, stride=2), dict(units=3, activation="LINEAR")], 2)
    desc.layers[2].n_units = 5                # a width that does not follow from the parameters
    with pytest.raises(mb.MyeaError) as e:
        mb.HipNetwork(desc)
    assert e.value.code == mb.E_INVALID and "pooling width" in str(e.value)
