"""GPU parity, through the C ABI against the CPU oracle, of the stacks that mix residual blocks with a recurrent depth:
independently recurrent and LSTM layers as members of a block, residual and pooling layers beside LSTM layers, noise dropout,
the k-sparse filter and Bernoulli dropout on members, ShakeDrop with a mask per (time step, example).  The oracle's side of
these is pinned by float64 autograd through time in tests/test_oracle_recurrent_residual.py.  Tolerance rel 1e-4 / abs 1e-5 of
the tensor's largest magnitude (fp32); normalised stacks: up to 1 % of the entries may be off by up to 1 %."""
import numpy as np
import pytest

from myea_amd import binding as mb
from myea_amd.synthetic import simple_debug_layers
from tests.common import assert_close, glorot_parameters, run_step
from tests.oracle_lib import OracleNetwork
from tests.test_oracle_recurrent_residual import CASES, _self_weights, avg, fc, ind, lstm, mx, res

pytestmark = pytest.mark.gpu
REL, ABS = 1e-4, 1e-5

EXTRA = {
    # the reference's example network (Neural_Network_Launcher_Windows/Source_Files/debug.cpp:36-1555) at a short depth and a small batch
    "example_network_short": (simple_debug_layers(), 5, 12),
    # widths the tiled contraction and the wide element-wise kernels see
    "ind_rnn_members_wide": ([fc(40), fc(96, "RELU"), res(3), ind(96, "TANH"), ind(96, "ISRLU"), ind(96, "TANH"), mx(2, 2),
                              res(2), ind(64, "TANH"), ind(64, "SIGMOID"), fc(10, "SOFTMAX")], 6, 40),
    "lstm_members_wide": ([fc(24), fc(64, "TANH"), res(3), fc(48, "TANH"), lstm(64), fc(64, "TANH"), res(2), lstm(16, cells_per_block=3), ind(48, "TANH"),
                           fc(48, "LINEAR")], 5, 24),
    "two_directions_member_then_pooling": ([fc(16), lstm(32, bidirectional=True), res(2), fc(40, "TANH"), lstm(32, bidirectional=True), avg(2, 2),
                                            lstm(24), fc(24, "LINEAR")], 4, 16),
    # Bernoulli dropout and renormalisation on members of both recurrent kinds
    "members_with_dropout_and_renormalisation": ([fc(12), fc(20, "TANH"), res(3, normalization="BATCH_RENORMALIZATION"),
                                                  fc(20, "TANH", normalization="BATCH_NORMALIZATION"), ind(20, "TANH", dropout="BERNOULLI", keep=0.7),
                                                  ind(20, "SIGMOID", normalization="BATCH_RENORMALIZATION", dropout="BERNOULLI_INVERTED", keep=0.6),
                                                  fc(5, "LINEAR")], 4, 32),
}
# the small stacks the float64 model pins the oracle on, at four times their batch (a normalisation over three examples amplifies
# fp32 rounding beyond any tolerance worth stating)
ALL = dict({name: (specs, T, 4 * B) for name, (specs, T, B) in CASES.items()}, **EXTRA)


def _mostly_close(a, b, what, fraction=0.01):
    """rel 1e-4 / abs 1e-5 of the largest magnitude, except that up to 1 % of the entries (one entry of a small tensor) may be off
    by up to 1 %: a batch normalisation over a few dozen examples subtracts nearly equal terms on its way back and amplifies the
    fp32 rounding of its statistics on either side."""
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    scale = max(1.0, float(np.abs(b).max()))
    err = np.abs(a - b)
    bad = err > REL * np.abs(b) + ABS * scale
    assert bad.sum() <= max(1, int(fraction * a.size)), "%s: %d / %d out of tolerance" % (what, int(bad.sum()), a.size)
    assert np.all(err[bad] <= 1e-2 * np.abs(b[bad]) + 1e-4 * scale), "%s: an entry is off by more than rounding can explain" % what


def _normalised(specs):
    return any(s.get("normalization", "NONE") != "NONE" for s in specs)


def _setup(specs, T, Bmax, seed, optimizer="GD", **hyper):
    desc = mb.make_desc(specs, Bmax, T)
    softmax = specs[-1]["activation"] == "SOFTMAX"
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER[optimizer], type_loss_function=mb.LOSS["CROSS_ENTROPY" if softmax else "MSE"],
                         batch_renormalization_r_correction_maximum=1.5, batch_renormalization_d_correction_maximum=0.5, **hyper)
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h)
    rng = np.random.default_rng(seed)
    w = _self_weights(desc, specs, glorot_parameters(desc, seed, bias_range=0.3), seed)
    masks = (rng.uniform(0, 1, max(1, desc.total_mask_units)) < 0.6).astype(np.uint8)[:desc.total_mask_units]
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
        if desc.total_mask_units:
            n.upload_masks(masks)
    return desc, gpu, cpu, rng


def _data(rng, specs, T, B):
    n_in, n_out = specs[0]["units"], specs[-1]["units"]
    X = rng.normal(0, 1, (B, T * n_in)).astype(np.float32)
    if specs[-1]["activation"] == "SOFTMAX":
        Y = np.zeros((B, T, n_out), np.float32)
        np.put_along_axis(Y, rng.integers(0, n_out, (B, T))[..., None], 1.0, axis=2)
        return X, Y.reshape(B, -1)
    return X, rng.normal(0, 1, (B, T * n_out)).astype(np.float32)


def _rows(a, T, Bmax, B, width):
    """the rows of the first B examples of a [T][Bmax][width] tensor"""
    return a.reshape(T, Bmax, width)[:, :B]


def _compare(desc, gpu, cpu, specs, T, B, what):
    Bmax = desc.batch_size
    close = _mostly_close if _normalised(specs) else (lambda a, b, w: assert_close(a, b, REL, ABS * max(1.0, float(np.abs(b).max())), w))
    for li in range(1, desc.n_layers):
        width = gpu.lib.myea_net_desc_number_outputs(desc, li)
        for kind in ("OUTPUTS", "ERRORS"):
            a, b = gpu.download_tensor(li, mb.TENSOR[kind]), cpu.download_tensor(li, mb.TENSOR[kind])
            close(_rows(a, T, Bmax, B, width), _rows(b, T, Bmax, B, width), "%s layer %d %s" % (what, li, kind))
    close(gpu.download_gradient(), cpu.download_gradient(), what + " gradient")
    assert gpu.get_loss().loss_values == pytest.approx(cpu.get_loss().loss_values, rel=1e-4)


@pytest.mark.parametrize("batch", ["whole", "partial"])
@pytest.mark.parametrize("name", sorted(ALL))
def test_recurrent_residual_step_matches_oracle(name, batch):
    specs, T, Bmax = ALL[name]
    B = Bmax if batch == "whole" else Bmax - 1
    desc, gpu, cpu, rng = _setup(specs, T, Bmax, 31, "GD", learning_rate=0.01, learning_momentum=0.9, use_Nesterov=1)
    X, Y = _data(rng, specs, T, B)
    for step in range(2):
        for n in (gpu, cpu):
            n.Reset__Loss()
            run_step(n, B, X, Y, update=False)
        _compare(desc, gpu, cpu, specs, T, B, "%s step %d" % (name, step))
        for n in (gpu, cpu):
            n.Update_Parameter(B, B)
        pc = cpu.download_parameters()
        if _normalised(specs):
            _mostly_close(gpu.download_parameters(), pc, "parameters step %d" % step)
        else:
            assert_close(gpu.download_parameters(), pc, REL, 2 * ABS, "parameters step %d" % step)
        gpu.upload_parameters(pc)          # both sides start the next step from the same point
        for k in (1,):
            gpu.upload_optimizer_state(k, cpu.download_optimizer_state(k))


def test_example_network_trains_with_amsgrad_and_its_constraint():
    """The example's optimizer settings (debug.cpp:96-117): AMSGrad at 1e-3, max-norm constraint 8, cross-entropy; three steps,
    the loss of each held against the oracle's and the parameters after the last."""
    specs, T, Bmax = simple_debug_layers(), 4, 16
    desc, gpu, cpu, rng = _setup(specs, T, Bmax, 5, "AMSGRAD", learning_rate=1e-3, regularization__max_norm_constraints=8.0,
                                 normalization_momentum_average=1.0, normalization_epsilon=0.1)
    X, Y = _data(rng, specs, T, Bmax)
    for step in range(3):
        for n in (gpu, cpu):
            n.Reset__Loss()
            run_step(n, Bmax, X, Y, update=False)
        assert gpu.get_loss().loss_values == pytest.approx(cpu.get_loss().loss_values, rel=1e-4)
        _mostly_close(gpu.download_gradient(), cpu.download_gradient(), "gradient step %d" % step)
        for n in (gpu, cpu):
            n.Update_Parameter(Bmax, Bmax)
        # an AMSGrad step is lr * m / sqrt(v): where the gradient is rounding noise the step is ill-conditioned, bounded by 2.1 lr
        assert np.max(np.abs(gpu.download_parameters().astype(np.float64) - cpu.download_parameters())) <= 2.1e-3
        gpu.upload_parameters(cpu.download_parameters())
        for k in (1, 2, 3):
            gpu.upload_optimizer_state(k, cpu.download_optimizer_state(k))


@pytest.mark.parametrize("kind", ["GAUSSIAN", "UOUT"])
def test_noise_dropout_and_k_sparse_filter_on_members(kind):
    """Uploaded draws ([T][batch][fan-in] per member), then the device generator's own read back and handed to the oracle."""
    T, Bmax, B = 3, 12, 11
    specs = [fc(10), fc(24, "TANH"), res(3), fc(20, "TANH"), fc(24, "TANH", dropout=kind, keep=0.3, k_sparsity=9),
             fc(24, "SIGMOID", k_sparsity=14, alpha_sparsity=1.5), fc(6, "LINEAR")]
    desc, gpu, cpu, rng = _setup(specs, T, Bmax, 41)
    X, Y = _data(rng, specs, T, B)
    draws = (rng.normal(1, 1, T * Bmax * 20) if kind == "GAUSSIAN" else rng.uniform(-0.3, 0.3, T * Bmax * 20)).astype(np.float32)
    for n in (gpu, cpu):
        n.upload_dropout_noise(4, draws)
        run_step(n, B, X, Y, update=False)
    _compare(desc, gpu, cpu, specs, T, B, "uploaded draws:")
    for n in (gpu, cpu):
        n.Clear_Training_Arrays()
    gpu.upload_dropout_noise(4, None)
    run_step(gpu, B, X, Y, update=False)
    d = gpu.download_tensor(4, mb.TENSOR["DROPOUT_NOISE"], T * Bmax * 20)
    assert not np.array_equal(d, draws) and np.isfinite(d).all() and d.std() > 0.05
    cpu.upload_dropout_noise(4, d)
    run_step(cpu, B, X, Y, update=False)
    _compare(desc, gpu, cpu, specs, T, B, "generated draws:")
    # outside the training state: no noise; the filter keeps alpha * k values
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_INFERENCE)
        n.Forward_Pass(B, X)
    last = desc.n_layers - 1
    assert_close(_rows(gpu.download_tensor(last, mb.TENSOR["OUTPUTS"]), T, Bmax, B, 6), _rows(cpu.download_tensor(last, mb.TENSOR["OUTPUTS"]), T, Bmax, B, 6), REL, ABS, "inference")


def test_bernoulli_members_scale_at_inference():
    T, Bmax = 3, 8
    specs = [fc(6), fc(12, "TANH"), res(2), fc(10, "TANH"), ind(10, "TANH", dropout="BERNOULLI", keep=0.6), fc(4, "LINEAR")]
    desc, gpu, cpu, rng = _setup(specs, T, Bmax, 43)
    X, _ = _data(rng, specs, T, Bmax)
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_INFERENCE)
        n.Forward_Pass(Bmax, X)
    for li in range(1, desc.n_layers):
        assert_close(gpu.download_tensor(li, mb.TENSOR["OUTPUTS"]), cpu.download_tensor(li, mb.TENSOR["OUTPUTS"]), REL, ABS, "layer %d" % li)


@pytest.mark.parametrize("last", ["dense", "lstm", "pooling"])
def test_shakedrop_with_a_recurrent_depth(last):
    """[T][batch] masks, [T][batch][width] forward draws, [T][batch][width] backward draws: uploaded, then generated and read back."""
    T, Bmax, B = 4, 10, 9
    tail = dict(dense=[fc(14, "TANH"), fc(12, "TANH")], lstm=[fc(14, "TANH"), lstm(12)], pooling=[ind(12, "TANH"), avg(2, 1, padding=1)])[last]
    specs = [fc(8), fc(12, "TANH"), res(2, dropout="SHAKEDROP", keep=0.5, normalization="BATCH_NORMALIZATION" if last == "dense" else "NONE")] + tail + [fc(12, "LINEAR")]
    desc, gpu, cpu, rng = _setup(specs, T, Bmax, 47)
    W = gpu.lib.myea_net_desc_number_outputs(desc, 4)
    X, Y = _data(rng, specs, T, B)
    mask = (rng.uniform(0, 1, (T, Bmax)) < 0.5).astype(np.float32)
    mask[0, 0], mask[0, 1] = 1, 0
    draws = np.concatenate([mask.ravel(), rng.uniform(-1, 1, T * Bmax * W), rng.uniform(0, 1, T * Bmax * W)]).astype(np.float32)
    for n in (gpu, cpu):
        n.upload_dropout_noise(2, draws)
        run_step(n, B, X, Y, update=False)
    _compare(desc, gpu, cpu, specs, T, B, "uploaded draws:")
    for n in (gpu, cpu):
        n.Clear_Training_Arrays()
    gpu.upload_dropout_noise(2, None)
    run_step(gpu, B, X, Y, update=False)
    d = gpu.download_tensor(2, mb.TENSOR["DROPOUT_NOISE"], T * Bmax * (1 + 2 * W))
    assert set(np.unique(d[:T * Bmax])) <= {0.0, 1.0} and 0 < d[:T * Bmax].sum() < T * Bmax
    alpha, beta = d[T * Bmax:T * Bmax * (1 + W)], d[T * Bmax * (1 + W):]
    assert alpha.min() >= -1 and alpha.max() < 1 and alpha.min() < -0.5 and beta.min() >= 0 and beta.max() < 1
    cpu.upload_dropout_noise(2, d)
    run_step(cpu, B, X, Y, update=False)
    _compare(desc, gpu, cpu, specs, T, B, "generated draws:")
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_INFERENCE)
        n.Forward_Pass(B, X)
    lo = desc.n_layers - 1
    assert_close(_rows(gpu.download_tensor(lo, mb.TENSOR["OUTPUTS"]), T, Bmax, B, 12), _rows(cpu.download_tensor(lo, mb.TENSOR["OUTPUTS"]), T, Bmax, B, 12), REL, ABS, "inference")


def test_an_independently_recurrent_member_narrower_than_its_input_is_refused():
    with pytest.raises(mb.MyeaError) as e:
        mb.HipNetwork(mb.make_desc([fc(5), fc(7), res(2), fc(6), ind(4), fc(3, "LINEAR")], 2, 3))
    assert e.value.code == mb.E_UNSUPPORTED
