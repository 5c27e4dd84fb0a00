"""GPU parity of ShakeDrop on residual blocks: the HIP library (through its C ABI) against the CPU oracle fed the same masks
and draws (uploaded ones, and the device generator's own read back); the generator is held to its distributions."""
import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, one_hot, run_step
from tests.oracle_lib import OracleNetwork

pytestmark = pytest.mark.gpu
REL, ABS = 1e-4, 1e-5

res = lambda depth, p, **kw: dict(type="residual", block_depth=depth, dropout="SHAKEDROP", keep=p, **kw)
CASES = [
    ("plain", [dict(units=12), dict(units=32, activation="TANH"), res(2, 0.5), dict(units=24, activation="RELU"), dict(units=32, activation="RELU"), dict(units=5, activation="LINEAR")], 9, 9),
    ("block-norm-wide-shortcut-softmax", [dict(units=20), dict(units=48, activation="RELU"), res(3, 0.4, normalization="BATCH_NORMALIZATION"),
                                          dict(units=40, activation="RELU", normalization="BATCH_NORMALIZATION"), dict(units=40, activation="TANH", dropout="BERNOULLI_INVERTED", keep=0.8),
                                          dict(units=36, activation="RELU"), dict(units=10, activation="SOFTMAX")], 30, 32),
    ("two-blocks-narrow-shortcut", [dict(units=16), dict(units=20, activation="TANH"), res(1, 0.7), dict(units=28, activation="LEAKY_RELU"),
                                    res(2, 0.2), dict(units=16, activation="RELU"), dict(units=28, activation="RELU"), dict(units=4, activation="LINEAR")], 16, 16),
]


@pytest.mark.parametrize("name,specs,B,Bmax", CASES, ids=[c[0] for c in CASES])
def test_shakedrop_stack_parity(name, specs, B, Bmax):
    desc = mb.make_desc(specs, Bmax)
    head = specs[-1]["activation"]
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["ADAM"], type_loss_function=mb.LOSS["CROSS_ENTROPY" if head == "SOFTMAX" else "MSE"])
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h)
    w = glorot_parameters(desc, 21, bias_range=0.3)
    rng = np.random.default_rng(21)
    masks = (rng.uniform(0, 1, desc.total_mask_units) < 0.8).astype(np.uint8)
    n_in, n_out = specs[0]["units"], specs[-1]["units"]
    X = rng.normal(0, 1, (B, n_in)).astype(np.float32)
    Y = one_hot(rng.integers(0, n_out, B), n_out) if head == "SOFTMAX" else rng.normal(0, 1, (B, n_out)).astype(np.float32)
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.upload_masks(masks)
        n.Clear_Training_Arrays()
    blocks = [li for li in range(desc.n_layers) if desc.layers[li].type_layer == mb.LAYER_RESIDUAL]
    width = {li: desc.layers[li + desc.layers[li].block_depth].n_units for li in blocks}
    count = {li: Bmax * (1 + 2 * width[li]) for li in blocks}

    def compare(what):
        for li in range(1, desc.n_layers):
            W = gpu.lib.myea_net_desc_number_outputs(desc, li)
            for kind in ("OUTPUTS", "ERRORS"):
                a, b = gpu.download_tensor(li, mb.TENSOR[kind], B * W), cpu.download_tensor(li, mb.TENSOR[kind], B * W)
                assert_close(a, b, REL, ABS * max(1.0, float(np.abs(b).max())), what="%s layer %d %s" % (what, li, kind))
        g, want = gpu.download_gradient(), cpu.download_gradient()
        assert_close(g, want, REL, ABS * max(1.0, float(np.abs(want).max())), what=what + " gradient")

    # (1) uploaded masks and draws
    for li in blocks:
        p = desc.layers[li].dropout_values[0]
        m = (rng.uniform(0, 1, Bmax) < p).astype(np.float32)
        m[0], m[1] = 1, 0
        draws = np.concatenate([m, rng.uniform(-1, 1, Bmax * width[li]), rng.uniform(0, 1, Bmax * width[li])]).astype(np.float32)
        gpu.upload_dropout_noise(li, draws); cpu.upload_dropout_noise(li, draws)
    for n in (gpu, cpu):
        run_step(n, B, X, Y, update=False)
    compare("uploaded draws:")
    # (2) the device generator's, read back
    for n in (gpu, cpu):
        n.Clear_Training_Arrays()
    for li in blocks:
        gpu.upload_dropout_noise(li, None)
    run_step(gpu, B, X, Y, update=False)
    for li in blocks:
        d = gpu.download_tensor(li, mb.TENSOR["DROPOUT_NOISE"], count[li])
        assert set(np.unique(d[:Bmax])) <= {0.0, 1.0}
        cpu.upload_dropout_noise(li, d)
    run_step(cpu, B, X, Y, update=False)
    compare("generated draws:")
    # (3) inference
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_INFERENCE)
        n.Forward_Pass(B, X)
    lo = desc.n_layers - 1
    assert_close(gpu.download_tensor(lo, mb.TENSOR["OUTPUTS"], B * n_out), cpu.download_tensor(lo, mb.TENSOR["OUTPUTS"], B * n_out), REL, ABS, what="inference outputs")


def test_device_generator_masks_and_ranges():
    Bmax, W, p = 4096, 64, 0.3
    specs = [dict(units=8), dict(units=W, activation="TANH"), res(1, p), dict(units=W, activation="RELU"), dict(units=2, activation="LINEAR")]
    desc = mb.make_desc(specs, Bmax)
    gpu = mb.HipNetwork(desc, mb.default_hyper(type_loss_function=mb.LOSS["MSE"]))
    gpu.set_state_propagation(mb.STATE_TRAINING)
    gpu.upload_parameters(glorot_parameters(desc, 1))
    gpu.set_dropout_seed(7)
    X = np.random.default_rng(1).normal(0, 1, (Bmax, 8)).astype(np.float32)
    gpu.Forward_Pass(Bmax, X)
    d = gpu.download_tensor(2, mb.TENSOR["DROPOUT_NOISE"], Bmax * (1 + 2 * W))
    mask, alpha, beta = d[:Bmax], d[Bmax:Bmax + Bmax * W], d[Bmax + Bmax * W:]
    assert abs(mask.mean() - p) < 5 * np.sqrt(p * (1 - p) / Bmax)
    n = alpha.size
    assert alpha.min() >= -1 and alpha.max() < 1 and abs(alpha.mean()) < 5 * np.sqrt(1 / 3 / n) and abs(alpha.var() - 1 / 3) < 5 * np.sqrt(4 / 45 / n)
    assert beta.min() >= 0 and beta.max() < 1 and abs(beta.mean() - 0.5) < 5 * np.sqrt(1 / 12 / n) and abs(beta.var() - 1 / 12) < 5 * np.sqrt(1 / 180 / n)
    assert abs(np.corrcoef(alpha.astype(np.float64), beta.astype(np.float64))[0, 1]) < 5 / np.sqrt(n)
    gpu.Forward_Pass(Bmax, X)
    d2 = gpu.download_tensor(2, mb.TENSOR["DROPOUT_NOISE"], Bmax * (1 + 2 * W))
    assert not np.array_equal(d, d2)
    gpu.set_dropout_seed(7)
    gpu.Forward_Pass(Bmax, X)
    assert np.array_equal(gpu.download_tensor(2, mb.TENSOR["DROPOUT_NOISE"], Bmax * (1 + 2 * W)), d)


def test_refusals():
    with pytest.raises(mb.MyeaError):      # ShakeDrop belongs to residual layers
        mb.HipNetwork(mb.make_desc([dict(units=6), dict(units=8, activation="TANH", dropout="SHAKEDROP", keep=0.3), dict(units=3, activation="LINEAR")], 4))
    with pytest.raises(mb.MyeaError):
        mb.HipNetwork(mb.make_desc([dict(units=6), dict(units=8, activation="TANH"), res(1, 1.5), dict(units=8, activation="RELU"), dict(units=3, activation="LINEAR")], 4))
