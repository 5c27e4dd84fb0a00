"""Pins the evaluation side of the oracle (Compute__Loss, the R accuracy) and the host-side epoch drivers
(myea_amd/dataset.py: Training / Testing / Measure_Accuracy, mini-batches) with library routines and invariants:
scipy's Pearson r, torch's cross-entropy and SGD over the same mini-batch order, batch-split invariance.  CPU only."""
import math

import numpy as np
import pytest
import scipy.stats
import torch

from myea_amd import binding as mb
from myea_amd.dataset import Dataset, Dataset_Mini_Batch, get_loss
from tests.common import assert_close, glorot_parameters, one_hot, oracle_desc, oracle_hyper
from tests.oracle_lib import OracleNetwork

MLP = [dict(units=7), dict(units=9, activation="TANH"), dict(units=4, activation="SOFTMAX")]
REG = [dict(units=5), dict(units=8, activation="TANH"), dict(units=3, activation="LINEAR")]
RNN = [dict(units=4), dict(type="lstm", units=5), dict(units=5, activation="LINEAR")]


def _net(specs, bmax, T=1, seed=0, **kw):
    desc = oracle_desc(specs, bmax, T)
    net = OracleNetwork(desc, oracle_hyper(**kw))
    w = glorot_parameters(desc, seed)
    net.upload_parameters(w)
    net.Clear_Training_Arrays()
    return desc, net, w


def _outputs(net, desc, B, T=1):
    H = desc.layers[desc.n_layers - 1].n_units
    full = net.download_tensor(desc.n_layers - 1, mb.TENSOR["OUTPUTS"], T * desc.batch_size * H).reshape(T, desc.batch_size, H)
    return full[:, :B, :].transpose(1, 0, 2)     # [B][T][H]


def test_compute_loss_accumulates_like_compute_error_and_writes_no_delta():
    desc, net, _ = _net(REG, 6, type_loss_function=mb.LOSS["MSE"], type_accuracy_function=mb.ACCURACY["DISTANCE"], accuracy_variance=0.3)
    rng = np.random.default_rng(0)
    X, Y = rng.normal(0, 1, (6, 5)).astype(np.float32), rng.normal(0, 1, (6, 3)).astype(np.float32)
    net.Forward_Pass(6, X)
    net.Compute__Error(6, Y)
    want = net.get_loss()
    delta = net.download_tensor(2, mb.TENSOR["ERRORS"], 18)
    net.Reset__Loss()
    net.Forward_Pass(6, X + 1)                    # different values: a delta written now would differ
    net.Forward_Pass(6, X)
    net.Compute__Loss(6, Y)
    got = net.get_loss()
    assert (got.loss_values, got.number_loss, got.accuracy_value) == (want.loss_values, want.number_loss, want.accuracy_value)
    assert np.array_equal(net.download_tensor(2, mb.TENSOR["ERRORS"], 18), delta)
    y = _outputs(net, desc, 6)[:, 0, :].astype(np.float64)
    assert got.number_loss == 18 and abs(got.loss_values - ((y - Y) ** 2).sum()) < 1e-5
    assert got.accuracy_value == (np.abs(y - Y) <= np.float32(0.3)).sum()


@pytest.mark.parametrize("kind,fn", [
    ("MSE", lambda y, d: ((y - d) ** 2).mean()), ("RMSE", lambda y, d: math.sqrt(((y - d) ** 2).mean())),
    ("MAE", lambda y, d: np.abs(y - d).mean()), ("ME", lambda y, d: (y - d).mean()),
    ("L1", lambda y, d: (y - d).sum()), ("L2", lambda y, d: ((y - d) ** 2).sum()),
    ("SMAPE", lambda y, d: (np.abs(y - d) / (np.abs(y) + np.abs(d))).mean()),
])
def test_loss_read_outs_match_their_textbook_definitions(kind, fn):
    desc, net, _ = _net(REG, 4, type_loss_function=mb.LOSS[kind])
    rng = np.random.default_rng(1)
    X, Y = rng.normal(0, 1, (10, 5)).astype(np.float32), rng.normal(0, 1, (10, 3)).astype(np.float32)
    data = Dataset(X, Y)
    got = data.Testing(net)                        # 10 examples through a batch of 4: 4 + 4 + 2
    ys = []
    for first in range(0, 10, 4):
        b = min(4, 10 - first)
        net.Forward_Pass(b, X[first:first + b])
        ys.append(_outputs(net, desc, b)[:, 0, :])
    y = np.concatenate(ys).astype(np.float64)
    assert got == pytest.approx(fn(y, Y.astype(np.float64)), rel=2e-5, abs=1e-6)


def test_cross_entropy_read_out_is_torch_cross_entropy_per_example():
    desc, net, _ = _net(MLP, 5, type_loss_function=mb.LOSS["CROSS_ENTROPY"], type_accuracy_function=mb.ACCURACY["CROSS_ENTROPY"])
    rng = np.random.default_rng(2)
    X = rng.normal(0, 1, (12, 7)).astype(np.float32)
    labels = rng.integers(0, 4, 12)
    data = Dataset(X, one_hot(labels, 4))
    got = data.Testing(net)
    logits = []
    for first in range(0, 12, 5):
        b = min(5, 12 - first)
        net.Forward_Pass(b, X[first:first + b])
        logits.append(net.download_tensor(2, mb.TENSOR["SUMMATIONS"], 5 * 4).reshape(5, 4)[:b])
    logits = torch.tensor(np.concatenate(logits).astype(np.float64))
    want = torch.nn.functional.cross_entropy(logits, torch.tensor(labels), reduction="mean").item()
    assert got == pytest.approx(want, rel=2e-5)
    assert data.accuracy_testing == pytest.approx(100.0 * (logits.argmax(1).numpy() == labels).mean(), abs=1e-9)
    assert data.loss_testing == got


@pytest.mark.parametrize("specs,T,delays", [(REG, 1, 0), (RNN, 6, 0), (RNN, 6, 2)])
def test_r_accuracy_is_pearson_correlation_over_all_counted_entries(specs, T, delays):
    desc, net, _ = _net(specs, 4, T=T, type_loss_function=mb.LOSS["MSE"], type_accuracy_function=mb.ACCURACY["R"], number_time_delays=delays)
    n_in, n_out = specs[0]["units"], specs[-1]["units"]
    rng = np.random.default_rng(3)
    X = rng.normal(0, 1, (11, T * n_in)).astype(np.float32)
    ys = []
    for first in range(0, 11, 4):
        b = min(4, 11 - first)
        net.Forward_Pass(b, X[first:first + b])
        ys.append(_outputs(net, desc, b, T))
    y = np.concatenate(ys)                                                       # [11][T][out]
    Y = (0.6 * y + rng.normal(0, 0.2, y.shape) + 0.3).astype(np.float32)           # correlated targets
    data = Dataset(X, Y.reshape(11, -1), recurrent_depth=T)
    data.Testing(net)
    want = scipy.stats.pearsonr(y[:, delays:, :].ravel().astype(np.float64), Y[:, delays:, :].ravel().astype(np.float64))[0]
    assert 0.3 < want < 0.999
    assert data.accuracy_testing == pytest.approx(want, rel=1e-5)
    s = net.get_loss()
    assert s.number_loss == 11 * (T - delays) * n_out


def test_r_accuracy_of_constant_predictions_is_zero():
    desc, net, _ = _net(REG, 4, type_loss_function=mb.LOSS["MSE"], type_accuracy_function=mb.ACCURACY["R"])
    net.upload_parameters(np.zeros(desc.total_parameters, dtype=np.float32))        # every output is 0
    rng = np.random.default_rng(4)
    data = Dataset(rng.normal(0, 1, (8, 5)).astype(np.float32), rng.normal(0, 1, (8, 3)).astype(np.float32))
    data.Testing(net)
    assert data.accuracy_testing == 0.0


def test_batch_training_accumulates_over_sub_batches_and_updates_once():
    """Dataset::Training: the gradient of the whole set, summed over sub-batches of the allocated size, then ONE update with
    (N, N) - so the allocated batch size must not change the result (no batch statistics in this net)."""
    kw = dict(type_optimizer_function=mb.OPTIMIZER["ADAM"], type_loss_function=mb.LOSS["MSE"], regularization__weight_decay=0.01)
    rng = np.random.default_rng(5)
    X, Y = rng.normal(0, 1, (10, 5)).astype(np.float32), rng.normal(0, 1, (10, 3)).astype(np.float32)
    results = []
    for bmax in (10, 4, 3):
        desc, net, _ = _net(REG, bmax, **kw)
        data = Dataset(X, Y)
        losses = [data.Training(net) for _ in range(3)]
        h = net.get_hyper()
        assert h.optimizer_time_step == 3 and h.epoch_time_step == 4
        results.append((net.download_parameters(), losses, data.accuracy_training))
    for w, losses, _ in results[1:]:
        assert_close(w, results[0][0], rel=2e-5, abs_=2e-6)
        assert losses == pytest.approx(results[0][1], rel=1e-5)


class _TorchMLP(torch.nn.Module):
    def __init__(self, desc, w):
        super().__init__()
        self.l1, self.l2 = torch.nn.Linear(7, 9), torch.nn.Linear(9, 4)
        w = torch.tensor(w.astype(np.float64))
        a, b = desc.layers[1], desc.layers[2]
        bias = desc.total_weights
        with torch.no_grad():
            self.l1.weight.copy_(w[a.first_connection_index:a.last_connection_index].reshape(9, 7))
            self.l2.weight.copy_(w[b.first_connection_index:b.last_connection_index].reshape(4, 9))
            self.l1.bias.copy_(w[bias:bias + 9]); self.l2.bias.copy_(w[bias + 9:bias + 13])

    def forward(self, x):
        return self.l2(torch.tanh(self.l1(x)))


def test_mini_batch_epochs_match_torch_sgd_over_the_same_shuffled_batches():
    """23 examples, mini-batches of 5, allocated batch 3 (sub-batches accumulate), momentum SGD.  The last mini-batch takes the
    remainder as the reference computes it - 5 + size_t((23.0 / 5.0 - 4) * 5.0) = 5 + size_t(2.999...) = 7, so one example of the
    23 is left out of every epoch (Set__Desired_Data_Per_Batch, Dataset__Mini_Batch.cpp:208-209, in double arithmetic).
    torch: summed cross-entropy per mini-batch (the reference's gradient carries no 1/B)."""
    torch.set_default_dtype(torch.float64)
    try:
        kw = dict(type_optimizer_function=mb.OPTIMIZER["GD"], learning_rate=0.02, learning_momentum=0.9,
                  type_loss_function=mb.LOSS["CROSS_ENTROPY"], type_accuracy_function=mb.ACCURACY["CROSS_ENTROPY"])
        desc, net, w0 = _net(MLP, 3, seed=6, **kw)
        rng = np.random.default_rng(6)
        X = rng.normal(0, 1, (23, 7)).astype(np.float32)
        labels = rng.integers(0, 4, 23)
        data = Dataset_Mini_Batch(X, one_hot(labels, 4), True, 5, rng=np.random.default_rng(99))
        assert (data.number_mini_batch, data.number_examples_last_iteration) == (4, 7)
        model = _TorchMLP(desc, w0)
        opt = torch.optim.SGD(model.parameters(), lr=0.02, momentum=0.9)
        replay = np.random.default_rng(99)
        order = np.arange(23)
        for epoch in range(3):
            loss = data.Training(net)
            for i in range(22, -1, -1):                       # the same Fisher-Yates draws
                j = int(replay.integers(0, i + 1)); order[i], order[j] = order[j], order[i]
            assert np.array_equal(order, data.stochastic_index.astype(np.int64))
            want_loss = want_acc = 0.0
            for it in range(4):
                sel = order[it * 5: it * 5 + (5 if it < 3 else 7)]
                logits = model(torch.tensor(X[sel].astype(np.float64)))
                ce = torch.nn.functional.cross_entropy(logits, torch.tensor(labels[sel]), reduction="sum")
                want_loss += ce.item() / len(sel)
                want_acc += 100.0 * (logits.argmax(1).numpy() == labels[sel]).mean()
                opt.zero_grad(); ce.backward(); opt.step()
            assert loss == pytest.approx(want_loss / 4, rel=3e-5)
            assert data.accuracy_training == pytest.approx(want_acc / 4, abs=1e-6)
        h = net.get_hyper()
        assert h.optimizer_time_step == 12 and h.epoch_time_step == 4
        got = net.download_parameters().astype(np.float64)
        a, b = desc.layers[1], desc.layers[2]
        assert_close(got[a.first_connection_index:a.last_connection_index], model.l1.weight.detach().numpy().ravel(), rel=1e-4, abs_=1e-5)
        assert_close(got[b.first_connection_index:b.last_connection_index], model.l2.weight.detach().numpy().ravel(), rel=1e-4, abs_=1e-5)
        assert_close(got[desc.total_weights:desc.total_weights + 9], model.l1.bias.detach().numpy(), rel=1e-4, abs_=1e-5)
    finally:
        torch.set_default_dtype(torch.float32)


def test_mini_batch_update_passes_the_whole_set_as_training_size():
    """Update_Parameter(mini-batch size, Dataset<T>::Get__Number_Examples()): visible through the normalized weight decay"""
    rng = np.random.default_rng(7)
    X, Y = rng.normal(0, 1, (12, 5)).astype(np.float32), rng.normal(0, 1, (12, 3)).astype(np.float32)
    kw = dict(type_optimizer_function=mb.OPTIMIZER["GD"], learning_rate=0.0, learning_momentum=0.0, type_loss_function=mb.LOSS["MSE"])
    desc, net, w0 = _net(REG, 6, regularization__weight_decay=0.1, **kw)
    Dataset_Mini_Batch(X, Y, False, 6).Training(net)                                # two updates of 6 out of 12 at epoch 1
    shrink = 1 - 0.1 * math.sqrt(6 / (12 * 1.0))
    w = net.download_parameters()
    assert_close(w[:desc.total_weights], w0[:desc.total_weights].astype(np.float64) * shrink ** 2, rel=1e-5, abs_=1e-8)
    assert np.array_equal(w[desc.total_weights:], w0[desc.total_weights:])


def test_irprop_plus_losses_are_maintained_by_the_epoch_loop():
    desc, net, _ = _net(REG, 8, type_optimizer_function=mb.OPTIMIZER["IRPROP_PLUS"], type_loss_function=mb.LOSS["MSE"], rprop_delta_zero=0.01)
    rng = np.random.default_rng(8)
    data = Dataset(rng.normal(0, 1, (8, 5)).astype(np.float32), rng.normal(0, 1, (8, 3)).astype(np.float32))
    first = data.Training(net)
    h = net.get_hyper()
    assert h.loss_rprop == pytest.approx(first, rel=1e-6) and h.previous_loss_rprop == np.finfo(np.float32).max
    second = data.Training(net)
    h = net.get_hyper()
    assert h.previous_loss_rprop == pytest.approx(first, rel=1e-6) and h.loss_rprop == pytest.approx(second, rel=1e-6)
    assert second < first
