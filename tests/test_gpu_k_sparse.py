"""GPU parity of the k-sparse filter on hidden fully-connected layers: the HIP library (through its C ABI) against the CPU
oracle.  The filter itself is exact work (a selection and zeros): given identical inputs its output is compared bit for bit,
ties at the cut included; inside trained stacks the usual rel 1e-4 / abs 1e-5 applies to what surrounds it."""
import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, one_hot, run_step
from tests.oracle_lib import OracleNetwork

pytestmark = pytest.mark.gpu
REL, ABS = 1e-4, 1e-5

CASES = [
    ("tanh-k8", [dict(units=12), dict(units=40, activation="TANH", k_sparsity=8), dict(units=5, activation="LINEAR")], 1, 9, 9),
    ("relu-alpha2-softmax-head", [dict(units=20), dict(units=300, activation="RELU", k_sparsity=40, alpha_sparsity=2.0), dict(units=10, activation="SOFTMAX")], 1, 33, 40),
    ("bn-after-dropout-two-filters", [dict(units=16), dict(units=64, activation="TANH", normalization="BATCH_NORMALIZATION", norm_before=False, dropout="BERNOULLI_INVERTED", keep=0.7, k_sparsity=16),
                                      dict(units=48, activation="LEAKY_RELU", k_sparsity=5, alpha_sparsity=3.0), dict(units=4, activation="LINEAR")], 1, 32, 32),
    ("recurrent-depth-partial-batch", [dict(units=6), dict(units=70, activation="TANH", k_sparsity=7), dict(type="lstm", units=8), dict(units=8, activation="LINEAR")], 4, 5, 6),
    ("wide-row", [dict(units=32), dict(units=3000, activation="SIGMOID", k_sparsity=100, alpha_sparsity=1.5), dict(units=6, activation="LINEAR")], 1, 16, 16),
]


@pytest.mark.parametrize("name,specs,T,B,Bmax", CASES, ids=[c[0] for c in CASES])
def test_k_sparse_stack_parity(name, specs, T, B, Bmax):
    desc = mb.make_desc(specs, Bmax, T)
    head = specs[-1]["activation"]
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["ADAM"], type_loss_function=mb.LOSS["CROSS_ENTROPY" if head == "SOFTMAX" else "MSE"])
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h)
    w = glorot_parameters(desc, 8, bias_range=0.3)
    rng = np.random.default_rng(8)
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
            if l.type_layer == mb.LAYER_LSTM:
                continue
            W = l.n_units
            a = gpu.download_tensor(li, mb.TENSOR["OUTPUTS"], T * Bmax * W).reshape(T, Bmax, W)[:, :B]
            b = cpu.download_tensor(li, mb.TENSOR["OUTPUTS"], T * Bmax * W).reshape(T, Bmax, W)[:, :B]
            assert_close(a, b, REL, ABS, what="step %d layer %d outputs" % (step, li))
            if l.k_sparsity:
                assert ((a != 0).sum(-1) <= l.k_sparsity).all() and np.array_equal(a != 0, b != 0)
        assert_close(gpu.download_gradient(), cpu.download_gradient(), REL, ABS, what="gradient step %d" % step)
        for n in (gpu, cpu):
            n.Update_Parameter(B, B)
        gpu.upload_parameters(cpu.download_parameters())
    assert gpu.get_loss().loss_values == pytest.approx(cpu.get_loss().loss_values, rel=1e-4)
    for n in (gpu, cpu):           # inference: size_t(alpha k) values stay
        n.set_state_propagation(mb.STATE_INFERENCE)
        n.Forward_Pass(B, X)
    for li in range(1, desc.n_layers):
        l = desc.layers[li]
        if l.type_layer == mb.LAYER_LSTM:
            continue
        W = l.n_units
        a = gpu.download_tensor(li, mb.TENSOR["OUTPUTS"], T * Bmax * W).reshape(T, Bmax, W)[:, :B]
        b = cpu.download_tensor(li, mb.TENSOR["OUTPUTS"], T * Bmax * W).reshape(T, Bmax, W)[:, :B]
        assert_close(a, b, REL, ABS, what="inference layer %d outputs" % li)
        if l.k_sparsity:
            assert ((a != 0).sum(-1) <= int(np.float32(l.alpha_sparsity) * np.float32(l.k_sparsity))).all()


@pytest.mark.parametrize("H,k", [(8, 3), (64, 1), (257, 100), (1000, 999), (5000, 37)])
def test_filter_is_bit_exact_on_identical_inputs_with_ties(H, k):
    """a LINEAR layer with the identity as its weight matrix hands the uploaded rows to the filter unchanged on both sides;
    the rows hold many repeated values, so the cut falls inside a run of equal values in most of them"""
    B = 12
    specs = [dict(units=H), dict(units=H, activation="LINEAR", k_sparsity=k), dict(units=2, activation="LINEAR")]
    desc = mb.make_desc(specs, B)
    h = mb.default_hyper(type_loss_function=mb.LOSS["MSE"])
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h)
    w = np.zeros(desc.total_parameters, dtype=np.float32)
    w[:H * H] = np.eye(H, dtype=np.float32).ravel()
    rng = np.random.default_rng(H + k)
    X = rng.integers(-4, 5, (B, H)).astype(np.float32) * 0.5          # 9 distinct values, negative zero among them
    X[0] = 1.0                                                          # one value only
    X[1] = -np.arange(H, dtype=np.float32)                              # strictly descending: the first k stay
    X[2] = np.arange(H, dtype=np.float32)                               # strictly ascending: the last k stay
    X[3, ::2] = -0.0
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Forward_Pass(B, X)
    a = gpu.download_tensor(1, mb.TENSOR["OUTPUTS"], B * H).reshape(B, H)
    b = cpu.download_tensor(1, mb.TENSOR["OUTPUTS"], B * H).reshape(B, H)
    assert np.array_equal(a, b)
    assert np.array_equal(np.nonzero(a[1])[0], np.arange(1 if k > 1 else 0, k)) or k == 1      # -0 at index 0 is a zero either way
    assert np.array_equal(np.nonzero(a[2])[0], np.arange(H - k, H))
    assert (a[0] != 0).sum() == k and (a[0][:k] == 1).all()


def test_refusals():
    for bad in ([dict(units=6), dict(type="ind_rnn", units=8, activation="TANH", k_sparsity=3), dict(units=3, activation="LINEAR")],
                [dict(units=6), dict(type="lstm", units=8, k_sparsity=3), dict(units=8, activation="LINEAR")]):
        with pytest.raises(ValueError):
            mb.make_desc(bad, 4, 3)
