"""GPU parity of the residual-block family (pre-activation members, block-level normalisation, zero-padded identity
shortcut and its gradient) through the C ABI against the CPU oracle.  Tolerance rel 1e-4 / abs 1e-5 (fp32)."""
import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import assert_close, assert_close_or_nearer_truth, glorot_parameters, one_hot, run_step
from tests.oracle_lib import OracleNetwork
from tests.test_oracle_residual import CASES, TorchResidualNet, fc, res

pytestmark = pytest.mark.gpu
REL, ABS = 1e-4, 1e-5

EXTRA = {
    # activations the contraction epilogues cannot apply (separate act / act' kernels), renormalisation, dropout on members
    "unfused_brn_dropout": ([fc(24), fc(40, "ELLIOT_SYMMETRIC"), res(3, normalization="BATCH_RENORMALIZATION"),
                             fc(33, "SINE_SYMMETRIC", normalization="BATCH_RENORMALIZATION"), fc(48, "GAUSSIAN", dropout="BERNOULLI", keep=0.7),
                             fc(29, "ISRU", normalization="BATCH_NORMALIZATION", dropout="BERNOULLI_INVERTED", keep=0.5), fc(10, "SOFTMAX")], 32),
    # the stack BASELINE config 4 describes, as residual blocks: [BN -> ReLU -> inverted dropout -> FC] members
    "relu_bn_dropout_blocks": ([fc(64), fc(96, "RELU")] + sum(([res(2), fc(96, "RELU", normalization="BATCH_NORMALIZATION"),
                                fc(96, "RELU", normalization="BATCH_NORMALIZATION", dropout="BERNOULLI_INVERTED", keep=0.5)] for _ in range(4)), [])
                               + [fc(20, "SOFTMAX")], 64),
    # pooling members at a width the tiled kernels see: a dilated max pooling (96 -> 47) between normalised dense members, dropout behind it
    "pooling_member_wide": ([fc(48), fc(64, "RELU"), res(3, normalization="BATCH_NORMALIZATION"), fc(96, "RELU", normalization="BATCH_NORMALIZATION"),
                             dict(type="max_pooling", kernel=3, stride=2, padding=1, dilation=2), fc(64, "TANH", dropout="BERNOULLI_INVERTED", keep=0.5),
                             fc(10, "SOFTMAX")], 32),
    # odd widths: guarded scalar-load contraction path, shortcut wider and narrower in consecutive blocks
    "odd_widths": ([fc(19), res(2), fc(31, "TANH"), fc(27, "LEAKY_RELU"), res(1), fc(13, "SIGMOID"), fc(7, "LINEAR")], 11),
}
ALL = dict(CASES, **EXTRA)


@pytest.mark.parametrize("name", sorted(ALL))
@pytest.mark.parametrize("optimizer", ["GD", "ADAM"])
def test_residual_step_matches_oracle(name, optimizer):
    specs, B = ALL[name]
    desc = mb.make_desc(specs, B)
    softmax = specs[-1]["activation"] == "SOFTMAX"
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER[optimizer], type_loss_function=mb.LOSS["CROSS_ENTROPY" if softmax else "MSE"],
                         use_Nesterov=1, batch_renormalization_r_correction_maximum=1.5, batch_renormalization_d_correction_maximum=0.5)
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h)
    w = glorot_parameters(desc, 21, bias_range=0.3)
    rng = np.random.default_rng(22)
    masks = (rng.uniform(0, 1, max(1, desc.total_mask_units)) < 0.6).astype(np.uint8)[:desc.total_mask_units]
    n_in, n_out = specs[0]["units"], specs[-1]["units"]
    X = rng.normal(0, 1, (B, n_in)).astype(np.float32)
    Y = one_hot(rng.integers(0, n_out, B), n_out) if softmax else rng.normal(0, 1, (B, n_out)).astype(np.float32)
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
        if desc.total_mask_units:
            n.upload_masks(masks)
    lib = mb.load_library()
    normed = [li for li in range(1, desc.n_layers) if specs[li].get("normalization", "NONE") != "NONE"]
    for step in range(2):
        # float64 arbiter for the few entries where fp32 rounding inside the normalisation statistics is amplified
        running = {li: (cpu.download_tensor(li, mb.TENSOR["NORM_MEANS_AVERAGES"]), cpu.download_tensor(li, mb.TENSOR["NORM_VARIANCES_AVERAGES"])) for li in normed}
        model = TorchResidualNet(desc, specs, cpu.download_parameters(), r_max=1.5, d_max=0.5, running=running)
        model.loss(model.forward(X, masks=masks if desc.total_mask_units else None), Y).backward()
        for n in (gpu, cpu):
            n.Reset__Loss()
            run_step(n, B, X, Y, update=False)
        for li in range(1, desc.n_layers):
            width = lib.myea_net_desc_number_outputs(desc, li)
            for kind in ("OUTPUTS", "ERRORS"):
                assert_close(gpu.download_tensor(li, mb.TENSOR[kind], B * width), cpu.download_tensor(li, mb.TENSOR[kind], B * width),
                             REL, ABS, "step %d layer %d %s" % (step, li, kind))
        assert_close_or_nearer_truth(gpu.download_gradient(), cpu.download_gradient(), model.flat.grad.numpy(), REL, ABS, "gradient step %d" % step, require_nearer=False)
        assert gpu.get_loss().loss_values == pytest.approx(cpu.get_loss().loss_values, rel=1e-4)
        for n in (gpu, cpu):
            n.Update_Parameter(B, B)
        if optimizer == "ADAM":
            # entries whose gradient is rounding noise take an ill-conditioned Adam step: hold them to the step bound, then resynchronise
            g = cpu.download_gradient()
            pg, pc = gpu.download_parameters(), cpu.download_parameters()
            assert np.max(np.abs(pg.astype(np.float64) - pc)) <= 2.1e-3
            cpu_state = [cpu.download_optimizer_state(k) for k in (1, 2)]
            gpu.upload_parameters(pc)
            for k, v in zip((1, 2), cpu_state):
                gpu.upload_optimizer_state(k, v)
        else:
            assert_close(gpu.download_parameters(), cpu.download_parameters(), REL, 2 * ABS, "parameters step %d" % step)
            gpu.upload_parameters(cpu.download_parameters())


def test_residual_inference_forward_matches_oracle():
    specs, B = EXTRA["relu_bn_dropout_blocks"]
    desc = mb.make_desc(specs, B)
    h = mb.default_hyper()
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h)
    w = glorot_parameters(desc, 23, bias_range=0.3)
    rng = np.random.default_rng(24)
    X = rng.normal(0, 1, (B, 64)).astype(np.float32)
    Y = one_hot(rng.integers(0, 20, B), 20)
    for n in (gpu, cpu):
        n.upload_parameters(w)
        n.set_state_propagation(mb.STATE_TRAINING)
        run_step(n, B, X, Y, update=False)       # one training pass moves the running averages
        n.set_state_propagation(mb.STATE_INFERENCE)
        n.Forward_Pass(B - 3, X[:B - 3])
    last = desc.n_layers - 1
    assert_close(gpu.download_tensor(last, mb.TENSOR["OUTPUTS"], (B - 3) * 20), cpu.download_tensor(last, mb.TENSOR["OUTPUTS"], (B - 3) * 20), REL, ABS)


def test_unsupported_residual_shapes_are_refused():
    B = 4
    for specs, T in (([fc(4), res(1, dropout="BERNOULLI", keep=0.5), fc(4), fc(2)], 1),                  # block-level dropout
                     ([fc(4), res(2), fc(4), fc(4, "SOFTMAX"), fc(2)], 1)):                              # softmax inside a block
        desc = mb.make_desc(specs, B, T, network=mb.NETWORK_FEEDFORWARD)
        with pytest.raises(mb.MyeaError):
            mb.HipNetwork(desc)


def _mostly_close(a, b, what, fraction=0.01):
    """rel 1e-4 / abs 1e-5, except that up to 1 % of the entries may be off by up to 1 %: a batch normalisation over a few
    dozen examples subtracts nearly equal terms on its way back and amplifies the fp32 rounding of its statistics on either
    side.  (The feed-forward cases above have a float64 arbiter for such entries; the time-step-by-time-step check against the
    library's own feed-forward path holds every entry to 1e-4.)"""
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    err = np.abs(a - b)
    bad = err > REL * np.abs(b) + ABS
    assert bad.mean() <= fraction, "%s: %d / %d out of tolerance" % (what, int(bad.sum()), a.size)
    assert np.all(err[bad] <= 1e-2 * np.abs(b[bad]) + 1e-4), "%s: an entry is off by more than rounding can explain" % what


def test_recurrent_depth_is_the_block_time_step_by_time_step_on_the_gpu():
    """residual blocks with a recurrent depth: against T feed-forward runs of the same library, then against the oracle"""
    from tests.test_oracle_residual import RECURRENT_POOLING_SPECS, RECURRENT_SPECS, check_recurrent_depth_is_the_block_time_step_by_time_step
    for specs in (None, RECURRENT_POOLING_SPECS):   # the normalised stack, then one with pooling members
        check_recurrent_depth_is_the_block_time_step_by_time_step(
            lambda desc: mb.HipNetwork(desc, mb.default_hyper(type_loss_function=mb.LOSS["MSE"])), lambda specs, B, T: mb.make_desc(specs, B, T), rel=1e-4, abs_=1e-5,
            specs=specs)
    T, B, Bmax = 4, 29, 32   # enough examples for well-conditioned batch statistics
    desc = mb.make_desc(RECURRENT_SPECS, Bmax, T)
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["ADAM"], type_loss_function=mb.LOSS["MSE"])
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h)
    w = glorot_parameters(desc, 23, bias_range=0.3)
    rng = np.random.default_rng(23)
    masks = (rng.uniform(0, 1, desc.total_mask_units) < 0.6).astype(np.uint8)
    X = rng.normal(0, 1, (B, T * 5)).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * 3)).astype(np.float32)
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
            for kind in ("OUTPUTS", "ERRORS"):
                a, b = gpu.download_tensor(li, mb.TENSOR[kind]), cpu.download_tensor(li, mb.TENSOR[kind])
                W = len(a) // (T * Bmax)
                _mostly_close(np.asarray(a).reshape(T, Bmax, W)[:, :B], np.asarray(b).reshape(T, Bmax, W)[:, :B], "step %d layer %d %s" % (step, li, kind))
        # The bias of block 1's last member feeds the block's normalisation, which removes any constant: its gradient is zero
        # in exact arithmetic, and what either side holds there is the rounding of a sum that cancels.
        gg, gc = gpu.download_gradient(), cpu.download_gradient()
        b4 = desc.layers[4].first_bias_connection_index
        assert np.all(np.abs(gg[b4:b4 + 8]) < 5e-3) and np.all(np.abs(gc[b4:b4 + 8]) < 5e-3)
        keep = np.ones(len(gg), dtype=bool)
        keep[b4:b4 + 8] = False
        _mostly_close(gg[keep], gc[keep], "gradient step %d" % step, fraction=0.02)   # sums of T x B terms of either sign
        for n in (gpu, cpu):
            n.Update_Parameter(B, B)
        gpu.upload_parameters(cpu.download_parameters())
    # inference: the running averages of each time step
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_INFERENCE)
        n.Forward_Pass(B, X)
    last = desc.n_layers - 1
    assert_close(np.asarray(gpu.download_tensor(last, mb.TENSOR["OUTPUTS"])).reshape(T, Bmax, 3)[:, :B],
                 np.asarray(cpu.download_tensor(last, mb.TENSOR["OUTPUTS"])).reshape(T, Bmax, 3)[:, :B], 1e-4, 1e-5, what="inference")
