"""GPU parity of the evaluation side and the epoch loops: Compute__Loss, the R accuracy, device-side mini-batch
gathering and whole training / testing epochs over a dataset resident in HBM - the HIP library (through its C ABI)
against the CPU oracle driven by the same host loops.  Tolerance rel 1e-4 / abs 1e-5 (fp32); gathered rows and
integer counters bit-exact."""
import numpy as np
import pytest
import torch

from myea_amd import binding as mb
from myea_amd.dataset import Dataset, Dataset_Mini_Batch
from tests.common import assert_close, glorot_parameters, one_hot
from tests.oracle_lib import OracleNetwork

pytestmark = pytest.mark.gpu
REL, ABS = 1e-4, 1e-5


def _pair(specs, bmax, hyper_kw, T=1, seed=0):
    desc = mb.make_desc(specs, bmax, T)
    h = mb.default_hyper(**hyper_kw)
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h)
    w = glorot_parameters(desc, seed)
    for n in (gpu, cpu):
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
    return desc, gpu, cpu


def _same_counters(a, b, what):
    assert a.number_loss == b.number_loss and a.number_bit_fail == b.number_bit_fail, what
    assert a.loss_values == pytest.approx(b.loss_values, rel=REL, abs=ABS), what
    assert a.accuracy_value == pytest.approx(b.accuracy_value, rel=REL, abs=ABS), what
    for k in range(4):
        assert a.accuracy_r[k] == pytest.approx(b.accuracy_r[k], rel=REL, abs=1e-4), "%s accuracy_r[%d]" % (what, k)


LOSSES = ["MSE", "RMSE", "MAE", "ME", "L1", "L2", "MAPE", "SMAPE", "BIT", "CROSS_ENTROPY"]
ACCURACIES = ["DISTANCE", "DIRECTIONAL", "SIGN", "R", "CROSS_ENTROPY"]


@pytest.mark.parametrize("T,delays", [(1, 0), (5, 0), (5, 2)])
def test_compute_loss_every_loss_and_accuracy_kind(T, delays):
    specs = [dict(units=6), dict(type="lstm", units=7) if T > 1 else dict(units=7, activation="TANH"), dict(units=70, activation="SIGMOID")]
    desc, gpu, cpu = _pair(specs, 9, dict(number_time_delays=delays), T=T)
    rng = np.random.default_rng(T)
    B = 7
    X = rng.normal(0, 1, (B, T * 6)).astype(np.float32)
    Y = rng.uniform(0, 1, (B, T, 70)).astype(np.float32)
    Y[:, :, 3] = 1.0                                            # a target class for the cross-entropy accuracy
    Y[0, :, 5] = 0.0                                            # an exact zero for the sign accuracy
    Y = Y.reshape(B, -1)
    for n in (gpu, cpu):
        n.Forward_Pass(B, X)
        n.Compute__Error(B, Y)
    delta = gpu.download_tensor(2, mb.TENSOR["ERRORS"], T * 9 * 70)
    for loss in LOSSES:
        for acc in ACCURACIES:
            for n in (gpu, cpu):
                h = n.get_hyper(); h.type_loss_function = mb.LOSS[loss]; h.type_accuracy_function = mb.ACCURACY[acc]; n.set_hyper(h)
                n.Reset__Loss()
                n.Compute__Loss(B, Y)
                n.Compute__Loss(B - 2, Y)                           # counters accumulate over calls, ragged second batch
            _same_counters(gpu.get_loss(), cpu.get_loss(), "%s / %s" % (loss, acc))
    assert np.array_equal(gpu.download_tensor(2, mb.TENSOR["ERRORS"], T * 9 * 70), delta)     # Compute__Loss writes no delta
    Yd = torch.tensor(Y, device="cuda")
    gpu.Reset__Loss(); gpu.Compute__Loss(B, Yd, on_device=True); gpu.Compute__Loss(B - 2, Yd, on_device=True)
    _same_counters(gpu.get_loss(), cpu.get_loss(), "device-resident targets")


@pytest.mark.parametrize("T,delays", [(1, 0), (4, 1)])
def test_testing_epoch_with_r_accuracy_over_a_resident_dataset(T, delays):
    specs = [dict(units=6), dict(type="lstm", units=8) if T > 1 else dict(units=8, activation="TANH"), dict(units=8, activation="LINEAR")]
    desc, gpu, cpu = _pair(specs, 16, dict(type_loss_function=mb.LOSS["RMSE"], type_accuracy_function=mb.ACCURACY["R"], number_time_delays=delays), T=T)
    rng = np.random.default_rng(7)
    N = 50                                                       # 16 + 16 + 16 + 2
    X = rng.normal(0, 1, (N, T * 6)).astype(np.float32)
    cpu_data = Dataset(X, np.zeros((N, T * 8), dtype=np.float32), T)
    ys = []
    for first in range(0, N, 16):
        b = min(16, N - first)
        cpu.Forward_Pass(b, X[first:first + b])
        ys.append(cpu.download_tensor(2, mb.TENSOR["OUTPUTS"], T * 16 * 8).reshape(T, 16, 8)[:, :b].transpose(1, 0, 2))
    Y = (0.5 * np.concatenate(ys) + rng.normal(0, 0.3, (N, T, 8))).astype(np.float32).reshape(N, -1)
    cpu_data = Dataset(X, Y, T)
    gpu_data = Dataset(torch.tensor(X, device="cuda"), torch.tensor(Y, device="cuda"), T)
    want, got = cpu_data.Testing(cpu), gpu_data.Testing(gpu)
    assert got == pytest.approx(want, rel=REL)
    assert 0.2 < cpu_data.accuracy_testing < 0.999
    assert gpu_data.accuracy_testing == pytest.approx(cpu_data.accuracy_testing, rel=REL)
    _same_counters(gpu.get_loss(), cpu.get_loss(), "after Testing")


@pytest.mark.parametrize("row_floats", [64, 37, 1])
def test_gather_examples_is_bit_exact(row_floats):
    desc, gpu, _ = _pair([dict(units=4), dict(units=4, activation="LINEAR")], 32, {})
    rng = np.random.default_rng(row_floats)
    data = rng.normal(0, 1, (200, row_floats)).astype(np.float32)
    src = torch.tensor(data, device="cuda")
    dst = torch.full((40, row_floats), -1.0, device="cuda")
    index = rng.integers(0, 200, 32).astype(np.uint64)
    index[:3] = (199, 0, 199)                                    # repeats and both ends
    gpu.gather_examples(dst, src, 200, row_floats, index, 32)
    gpu.synchronize()
    out = dst.cpu().numpy()
    assert np.array_equal(out[:32], data[index.astype(np.int64)]) and np.all(out[32:] == -1.0)
    # a whole epoch's permutation uploaded once, batches taken at an offset (unaligned destination rows for odd widths)
    perm = torch.tensor(rng.permutation(200).astype(np.int64), device="cuda")
    big = torch.empty((200, row_floats), device="cuda")
    for first in range(0, 200, 24):
        b = min(24, 200 - first)
        gpu.gather_examples(big[first:], src, 200, row_floats, perm[first:], b, index_on_device=True)
    gpu.synchronize()
    assert np.array_equal(big.cpu().numpy(), data[perm.cpu().numpy()])
    with pytest.raises(mb.MyeaError) as e:
        gpu.gather_examples(dst, src, 200, row_floats, np.array([0, 200], dtype=np.uint64), 2)
    assert e.value.code == mb.E_INVALID
    with pytest.raises(mb.MyeaError) as e:
        gpu.gather_examples(dst, src, 200, row_floats, np.zeros(33, dtype=np.uint64), 33)
    assert e.value.code == mb.E_BATCH


def test_mini_batch_epochs_on_a_resident_dataset_match_the_oracle():
    """BN + inverted dropout MLP, AMSBound with normalized decay, shuffled mini-batches of 48 out of 200 examples gathered in HBM
    (allocated batch 32: every mini-batch runs as 32 + 16 / the last one 32 + 24), then Testing in the inference state."""
    specs = [dict(units=12), dict(units=24, activation="RELU", normalization="BATCH_NORMALIZATION", norm_before=True, dropout="BERNOULLI_INVERTED", keep=0.8),
             dict(units=16, activation="TANH"), dict(units=5, activation="SOFTMAX")]
    kw = dict(type_optimizer_function=mb.OPTIMIZER["AMSBOUND"], regularization__weight_decay=0.01, type_loss_function=mb.LOSS["CROSS_ENTROPY"],
              type_accuracy_function=mb.ACCURACY["CROSS_ENTROPY"])
    desc, gpu, cpu = _pair(specs, 32, kw, seed=3)
    rng = np.random.default_rng(3)
    N = 200
    X = rng.normal(0, 1, (N, 12)).astype(np.float32)
    labels = rng.integers(0, 5, N)
    Y = one_hot(labels, 5)
    masks = (rng.uniform(0, 1, desc.total_mask_units) < 0.8).astype(np.uint8)
    for n in (gpu, cpu):
        n.upload_masks(masks)
    cpu_data = Dataset_Mini_Batch(X, Y, True, 48, rng=np.random.default_rng(11))
    gpu_data = Dataset_Mini_Batch(torch.tensor(X, device="cuda"), torch.tensor(Y, device="cuda"), True, 48, rng=np.random.default_rng(11))
    assert (gpu_data.number_mini_batch, gpu_data.number_examples_last_iteration) == (4, 56)
    for epoch in range(2):
        want, got = cpu_data.Training(cpu), gpu_data.Training(gpu)
        assert np.array_equal(cpu_data.stochastic_index, gpu_data.stochastic_index)
        assert got == pytest.approx(want, rel=REL), "epoch %d" % epoch
        assert gpu_data.accuracy_training == pytest.approx(cpu_data.accuracy_training, abs=1e-9)
    assert gpu.get_hyper().optimizer_time_step == 8 and gpu.get_hyper().epoch_time_step == 3
    assert_close(gpu.download_parameters(), cpu.download_parameters(), REL, ABS, what="parameters after two epochs")
    assert_close(gpu.download_tensor(1, mb.TENSOR["NORM_MEANS_AVERAGES"], 24), cpu.download_tensor(1, mb.TENSOR["NORM_MEANS_AVERAGES"], 24), REL, ABS)
    want, got = cpu_data.Testing(cpu), gpu_data.Testing(gpu)
    assert got == pytest.approx(want, rel=REL)
    assert gpu_data.accuracy_testing == pytest.approx(cpu_data.accuracy_testing, abs=1e-9)
    assert gpu.get_loss().number_loss == N * 5


def test_batch_training_epoch_with_irprop_plus_on_a_resident_dataset():
    specs = [dict(units=10), dict(units=20, activation="TANH"), dict(units=4, activation="LINEAR")]
    kw = dict(type_optimizer_function=mb.OPTIMIZER["IRPROP_PLUS"], rprop_delta_zero=0.01, type_loss_function=mb.LOSS["MSE"], type_accuracy_function=mb.ACCURACY["DISTANCE"])
    desc, gpu, cpu = _pair(specs, 64, kw, seed=4)
    rng = np.random.default_rng(4)
    X, Y = rng.normal(0, 1, (150, 10)).astype(np.float32), rng.normal(0, 1, (150, 4)).astype(np.float32)
    cpu_data, gpu_data = Dataset(X, Y), Dataset(torch.tensor(X, device="cuda"), torch.tensor(Y, device="cuda"))
    for epoch in range(4):
        want, got = cpu_data.Training(cpu), gpu_data.Training(gpu)
        assert got == pytest.approx(want, rel=REL), "epoch %d" % epoch
        assert gpu_data.accuracy_training == pytest.approx(cpu_data.accuracy_training, abs=0.7)      # one borderline hit of 600 = 0.17 %
    hg, hc = gpu.get_hyper(), cpu.get_hyper()
    assert hg.loss_rprop == pytest.approx(hc.loss_rprop, rel=REL) and hg.previous_loss_rprop == pytest.approx(hc.previous_loss_rprop, rel=REL)
    # sign-driven steps: a gradient entry whose sign differs between two summation orders would move a weight by a whole step
    a, b = gpu.download_parameters(), cpu.download_parameters()
    assert (np.abs(a - b) <= ABS + REL * np.abs(b)).mean() > 0.995
