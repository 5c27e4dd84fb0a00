"""GPU parity of Gaussian / Uout dropout: the HIP library (through its C ABI) against the CPU oracle fed the same draws -
uploaded ones, and the device generator's own read back.  The generator's stream is its own (the reference draws from host
std::mt19937 generators inside the pass), so it is held to its distributions: moments, range, independence between passes,
reproducibility from the seed."""
import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, one_hot, run_step
from tests.oracle_lib import OracleNetwork

pytestmark = pytest.mark.gpu
REL, ABS = 1e-4, 1e-5

CASES = [
    ("gaussian", [dict(units=12), dict(units=40, activation="TANH", dropout="GAUSSIAN", keep=0.25), dict(units=5, activation="LINEAR")], 1, 9, 9),
    ("uout-softmax-head", [dict(units=20), dict(units=96, activation="RELU", dropout="UOUT", keep=0.3), dict(units=10, activation="SOFTMAX")], 1, 30, 32),
    ("both-bn-after-k-sparse", [dict(units=16), dict(units=64, activation="TANH", normalization="BATCH_NORMALIZATION", norm_before=False, dropout="GAUSSIAN", keep=0.5, k_sparsity=20),
                                dict(units=48, activation="LEAKY_RELU", dropout="UOUT", keep=0.2), dict(units=4, activation="LINEAR")], 1, 32, 32),
    ("recurrent-depth-partial-batch", [dict(units=6), dict(units=30, activation="TANH", dropout="GAUSSIAN", keep=0.3), dict(type="lstm", units=8), dict(units=8, activation="LINEAR", dropout="UOUT", keep=0.1)], 4, 5, 6),
]


def _pair(specs, T, B, Bmax, seed):
    desc = mb.make_desc(specs, Bmax, T)
    head = specs[-1]["activation"]
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["ADAM"], type_loss_function=mb.LOSS["CROSS_ENTROPY" if head == "SOFTMAX" else "MSE"])
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h)
    w = glorot_parameters(desc, seed, bias_range=0.3)
    rng = np.random.default_rng(seed)
    n_in, n_out = specs[0]["units"], specs[-1]["units"]
    X = rng.normal(0, 1, (B, T * n_in)).astype(np.float32)
    Y = (one_hot(rng.integers(0, n_out, B * T), n_out).reshape(B, T * n_out) if head == "SOFTMAX" else rng.normal(0, 1, (B, T * n_out)).astype(np.float32))
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
    return desc, gpu, cpu, X, Y, rng


def _compare(desc, gpu, cpu, T, B, Bmax, what):
    for li in range(1, desc.n_layers):
        l = desc.layers[li]
        if l.type_layer == mb.LAYER_LSTM:
            continue
        W = l.n_units
        for kind in ("OUTPUTS", "ERRORS"):
            a = gpu.download_tensor(li, mb.TENSOR[kind], T * Bmax * W).reshape(T, Bmax, W)[:, :B]
            b = cpu.download_tensor(li, mb.TENSOR[kind], T * Bmax * W).reshape(T, Bmax, W)[:, :B]
            assert_close(a, b, REL, ABS, what="%s layer %d %s" % (what, li, kind))
    assert_close(gpu.download_gradient(), cpu.download_gradient(), REL, ABS, what=what + " gradient")


@pytest.mark.parametrize("name,specs,T,B,Bmax", CASES, ids=[c[0] for c in CASES])
def test_noise_dropout_stack_parity(name, specs, T, B, Bmax):
    desc, gpu, cpu, X, Y, rng = _pair(specs, T, B, Bmax, 13)
    noisy = [li for li in range(1, desc.n_layers) if desc.layers[li].type_dropout in (mb.DROPOUT["GAUSSIAN"], mb.DROPOUT["UOUT"])]
    # (1) the caller's draws on both sides
    for li in noisy:
        l = desc.layers[li]
        v = l.dropout_values[0]
        g = (rng.normal(1, v, (T, Bmax, l.n_units)) if l.type_dropout == mb.DROPOUT["GAUSSIAN"] else rng.uniform(-v, v, (T, Bmax, l.n_units))).astype(np.float32)
        gpu.upload_dropout_noise(li, g); cpu.upload_dropout_noise(li, g)
    for n in (gpu, cpu):
        run_step(n, B, X, Y, update=False)
    for li in noisy:
        assert np.array_equal(gpu.download_tensor(li, mb.TENSOR["DROPOUT_NOISE"]), cpu.download_tensor(li, mb.TENSOR["DROPOUT_NOISE"]))
    _compare(desc, gpu, cpu, T, B, Bmax, "uploaded draws:")
    # (2) the device generator's draws, read back and handed to the oracle
    for n in (gpu, cpu):
        n.Clear_Training_Arrays()
    for li in noisy:
        gpu.upload_dropout_noise(li, None)
    run_step(gpu, B, X, Y, update=False)
    for li in noisy:
        cpu.upload_dropout_noise(li, gpu.download_tensor(li, mb.TENSOR["DROPOUT_NOISE"]))
    run_step(cpu, B, X, Y, update=False)
    _compare(desc, gpu, cpu, T, B, Bmax, "generated draws:")
    # (3) inference: no draws
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_INFERENCE)
        n.Forward_Pass(B, X)
    lo = desc.n_layers - 1
    assert_close(gpu.download_tensor(lo, mb.TENSOR["OUTPUTS"]), cpu.download_tensor(lo, mb.TENSOR["OUTPUTS"]), REL, ABS, what="inference outputs")


def test_device_generator_distributions_and_reproducibility():
    H, B = 1000, 256
    p = 0.2
    specs = [dict(units=4), dict(units=H, activation="TANH", dropout="GAUSSIAN", keep=p / (1 - p)), dict(units=H, activation="TANH", dropout="UOUT", keep=0.3), dict(units=2, activation="LINEAR")]
    desc = mb.make_desc(specs, B)
    gpu = mb.HipNetwork(desc, mb.default_hyper(type_loss_function=mb.LOSS["MSE"]))
    gpu.set_state_propagation(mb.STATE_TRAINING)
    gpu.upload_parameters(glorot_parameters(desc, 1))
    X = np.random.default_rng(1).normal(0, 1, (B, 4)).astype(np.float32)
    # neutral until a training-state pass has drawn
    assert (gpu.download_tensor(1, mb.TENSOR["DROPOUT_NOISE"]) == 1).all() and (gpu.download_tensor(2, mb.TENSOR["DROPOUT_NOISE"]) == 0).all()
    gpu.set_dropout_seed(1234)
    gpu.Forward_Pass(B, X)
    g1, u1 = gpu.download_tensor(1, mb.TENSOR["DROPOUT_NOISE"]), gpu.download_tensor(2, mb.TENSOR["DROPOUT_NOISE"])
    gpu.Forward_Pass(B, X)
    g2, u2 = gpu.download_tensor(1, mb.TENSOR["DROPOUT_NOISE"]), gpu.download_tensor(2, mb.TENSOR["DROPOUT_NOISE"])
    n = g1.size
    sd = p / (1 - p)
    # N(1, sd): mean, spread, third and fourth standardised moments, tails; tolerances are ~5 standard errors at n = 256000
    z = (g1.astype(np.float64) - 1) / sd
    assert abs(z.mean()) < 5 / np.sqrt(n) and abs(z.std() - 1) < 5 / np.sqrt(2 * n)
    assert abs((z ** 3).mean()) < 5 * np.sqrt(6 / n) and abs((z ** 4).mean() - 3) < 5 * np.sqrt(24 / n)
    assert abs((np.abs(z) > 1.959964).mean() - 0.05) < 5 * np.sqrt(0.05 * 0.95 / n) and np.isfinite(g1).all()
    # U(-0.3, 0.3)
    assert u1.min() >= -0.3 and u1.max() < 0.3
    v = (u1.astype(np.float64) + 0.3) / 0.6
    assert abs(v.mean() - 0.5) < 5 * np.sqrt(1 / 12 / n) and abs(v.var() - 1 / 12) < 5 * np.sqrt(1 / 180 / n)
    hist = np.histogram(v, bins=64, range=(0, 1))[0]
    assert ((hist - n / 64) ** 2 / (n / 64)).sum() < 63 + 5 * np.sqrt(2 * 63)          # chi-square, 63 degrees of freedom
    # passes and layers draw independently; neighbouring draws are uncorrelated
    for a, b in ((g1, g2), (u1, u2), (g1, u1)):
        assert abs(np.corrcoef(a.astype(np.float64), b.astype(np.float64))[0, 1]) < 5 / np.sqrt(n)
    assert abs(np.corrcoef(z[:-1], z[1:])[0, 1]) < 5 / np.sqrt(n) and abs(np.corrcoef(v[:-1], v[1:])[0, 1]) < 5 / np.sqrt(n)
    # the same seed replays the same sequence of passes; another seed does not
    gpu.set_dropout_seed(1234)
    gpu.Forward_Pass(B, X)
    assert np.array_equal(gpu.download_tensor(1, mb.TENSOR["DROPOUT_NOISE"]), g1) and np.array_equal(gpu.download_tensor(2, mb.TENSOR["DROPOUT_NOISE"]), u1)
    gpu.set_dropout_seed(99)
    gpu.Forward_Pass(B, X)
    assert not np.array_equal(gpu.download_tensor(1, mb.TENSOR["DROPOUT_NOISE"]), g1)
    # the inference state draws nothing
    gpu.set_state_propagation(mb.STATE_INFERENCE)
    before = gpu.download_tensor(1, mb.TENSOR["DROPOUT_NOISE"])
    gpu.Forward_Pass(B, X)
    assert np.array_equal(gpu.download_tensor(1, mb.TENSOR["DROPOUT_NOISE"]), before)


def test_refusals():
    for bad in ([dict(units=6, dropout="GAUSSIAN", keep=0.3), dict(units=8, activation="TANH"), dict(units=3, activation="LINEAR")],
                [dict(units=6), dict(type="ind_rnn", units=8, activation="TANH", dropout="UOUT", keep=0.3), dict(units=3, activation="LINEAR")]):
        with pytest.raises(mb.MyeaError):
            mb.HipNetwork(mb.make_desc(bad, 4, 3))
    net = mb.HipNetwork(mb.make_desc([dict(units=6), dict(units=8, activation="TANH", dropout="GAUSSIAN", keep=0.3), dict(units=3, activation="LINEAR")], 4))
    with pytest.raises(mb.MyeaError):
        net.upload_dropout_noise(2, np.ones(12, dtype=np.float32))        # a layer without such dropout
    with pytest.raises(mb.MyeaError):
        net.upload_dropout_noise(1, np.ones(5, dtype=np.float32))         # wrong count
