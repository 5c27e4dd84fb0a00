"""Host-side epoch drivers over a network handle: the reference's `Dataset<T>` / `Dataset_Mini_Batch<T>` training and
testing loops (Neural_Network/Dataset.cpp:549-700, 7574-7870; Neural_Network/Dataset__Mini_Batch.cpp:45-420) and the
loss / accuracy read-outs of `Neural_Network` (Neural_Network__Loss.cpp:103-214, Neural_Network__Accuracy.cpp:88-113),
written against the step entry points only.  The same code drives `binding.HipNetwork` (where the examples may live
in HBM as torch tensors and shuffled mini-batches are gathered on the device) and any object with the same methods."""
import math

import numpy as np

from . import binding as mb

FLT_MAX = float(np.finfo(np.float32).max)


def get_loss(net, output_size):
    """Neural_Network::Get__Loss(TYPE_DATASET_NONE), Neural_Network__Loss.cpp:103-214"""
    s = net.get_loss()
    kind = net.get_hyper().type_loss_function
    L = mb.LOSS
    if kind in (L["L1"], L["L2"]):
        return s.loss_values
    if kind == L["BIT"]:
        return float(s.number_bit_fail)
    if kind == L["CROSS_ENTROPY"]:   # per example (and time step), not per output
        return s.loss_values / (s.number_loss // output_size) if s.number_loss else FLT_MAX
    if kind in (L["ME"], L["MAE"], L["MSE"], L["MAPE"], L["SMAPE"]):
        return s.loss_values / s.number_loss if s.number_loss else 1.0
    if kind == L["RMSE"]:
        return math.sqrt(s.loss_values / s.number_loss) if s.number_loss else 1.0
    return 1.0


def number_accuracy_trial(net, examples, recurrent_depth, output_size):
    """Dataset::Train_Batch_BP_* / Testing_*: examples x (T - delays) x (1 for the cross-entropy accuracy, else outputs)"""
    h = net.get_hyper()
    per = 1 if h.type_accuracy_function == mb.ACCURACY["CROSS_ENTROPY"] else output_size
    return examples * (recurrent_depth - (h.number_time_delays if recurrent_depth > 1 else 0)) * per


class Dataset:
    """Examples as two 2-D arrays [N][T*inputs], [N][T*outputs]: numpy arrays, or torch tensors resident in HBM
    (then every batch is handed over with on_device = 1)."""

    def __init__(self, inputs, outputs, recurrent_depth=1):
        self.inputs, self.outputs = inputs, outputs
        self.on_device = not isinstance(inputs, np.ndarray)
        self.recurrent_depth = recurrent_depth
        self.output_size = outputs.shape[1] // recurrent_depth
        self.loss_training = self.loss_testing = FLT_MAX
        self.accuracy_training = self.accuracy_testing = 0.0

    def Get__Number_Examples(self):
        return self.inputs.shape[0]

    # the examples one pass works on: the whole set here, the current mini-batch in the subclass
    def _current(self):
        return self.inputs, self.outputs

    def _batches(self, net, n):
        bmax = net.desc.batch_size
        for first in range(0, n, bmax):
            yield first, min(bmax, n - first)

    def Train_Epoch(self, net):
        """Train_Epoch_Loop + Train_Batch_BP_Loop (Dataset.cpp:593-700); the caller draws the dropout masks"""
        X, Y = self._current()
        n = X.shape[0]
        h = net.get_hyper()
        rprop = h.type_optimizer_function == mb.OPTIMIZER["IRPROP_PLUS"]
        net.Reset__Loss()
        if rprop:
            h.previous_loss_rprop = h.loss_rprop
            net.set_hyper(h)
        for first, b in self._batches(net, n):
            net.Forward_Pass(b, X[first:first + b], self.on_device)
            net.Compute__Error(b, Y[first:first + b], self.on_device)
            net.Backward_Pass(b)
            net.Update_Derivative_Weight(b)
        self.number_accuracy_trial = number_accuracy_trial(net, n, self.recurrent_depth, self.output_size)
        if rprop:
            h = net.get_hyper()
            h.loss_rprop = abs(get_loss(net, self.output_size))
            net.set_hyper(h)

    def Measure_Accuracy(self, net, examples=None):
        """Dataset::Measure_Accuracy (Dataset.cpp:7690-7756) on the current examples, after the counters were filled"""
        X, Y = examples or self._current()
        n = X.shape[0]
        h = net.get_hyper()
        if h.type_accuracy_function == mb.ACCURACY["R"]:
            s = net.get_loss()
            entries = n * (self.recurrent_depth - (h.number_time_delays if self.recurrent_depth > 1 else 0)) * self.output_size
            mean_d, mean_y = s.accuracy_value / entries, s.accuracy_r[0] / entries
            for first, b in self._batches(net, n):
                net.Forward_Pass(b, X[first:first + b], self.on_device)
                net.Compute__Accuracy__R(b, Y[first:first + b], mean_d, mean_y, self.on_device)
            s = net.get_loss()
            num, dd, dy = s.accuracy_r[1], s.accuracy_r[2], s.accuracy_r[3]
            r = 0.0 if dd * dy == 0 else num / (math.sqrt(dd) * math.sqrt(dy))
            return min(1.0, max(-1.0, r))
        trial = self.number_accuracy_trial
        return 0.0 if trial == 0 else net.get_loss().accuracy_value / trial * 100.0

    def Training(self, net):
        """Dataset::Training + Training_Loop (Dataset.cpp:7574-7688): one pass over all examples, ONE update"""
        net.set_state_propagation(mb.STATE_TRAINING)
        self.Train_Epoch(net)
        n = self.Get__Number_Examples()
        net.Update_Parameter(n, n)
        h = net.get_hyper()
        h.epoch_time_step += 1.0
        net.set_hyper(h)
        self.loss_training = get_loss(net, self.output_size)
        self.accuracy_training = self.Measure_Accuracy(net)
        net.set_state_propagation(mb.STATE_INFERENCE)
        return self.loss_training

    def Testing(self, net):
        """Dataset::Testing + Testing_Loop (Dataset.cpp:7758-7860, 8023-8050): inference forward + Compute__Loss"""
        net.set_state_propagation(mb.STATE_INFERENCE)
        net.Reset__Loss()
        n = self.Get__Number_Examples()
        for first, b in self._batches(net, n):
            net.Forward_Pass(b, self.inputs[first:first + b], self.on_device)
            net.Compute__Loss(b, self.outputs[first:first + b], self.on_device)
        self.number_accuracy_trial = number_accuracy_trial(net, n, self.recurrent_depth, self.output_size)
        self.loss_testing = get_loss(net, self.output_size)
        self.accuracy_testing = self.Measure_Accuracy(net, (self.inputs, self.outputs))   # always the whole set (Dataset<T>:: calls)
        return self.loss_testing


class Dataset_Mini_Batch(Dataset):
    """Dataset_Mini_Batch<T> (Dataset__Mini_Batch.cpp): shuffled index, one update per mini-batch; the last mini-batch
    takes the remainder.  `rng` stands in for the reference's clock-seeded generator (an `integers(low, high)` source)."""

    def __init__(self, inputs, outputs, use_shuffle, desired_examples_per_mini_batch, number_mini_batch_maximum=0, recurrent_depth=1, rng=None):
        super().__init__(inputs, outputs, recurrent_depth)
        n = inputs.shape[0]
        real = n / desired_examples_per_mini_batch
        count = int(real)
        if number_mini_batch_maximum:
            count = min(count, number_mini_batch_maximum)
        if desired_examples_per_mini_batch == 0 or desired_examples_per_mini_batch > n or count <= 1:
            raise ValueError("Set__Desired_Data_Per_Batch: invalid number of mini-batch")
        self.number_mini_batch = count
        self.number_examples_per_iteration = desired_examples_per_mini_batch
        self.number_examples_last_iteration = desired_examples_per_mini_batch + int((real - count) * desired_examples_per_mini_batch)
        self.use_shuffle = use_shuffle
        self.stochastic_index = np.arange(n, dtype=np.uint64)
        self.rng = rng or np.random.default_rng()
        self._batch = None
        self._stage = None

    def Shuffle(self):
        """Fisher-Yates from the top, as Dataset_Mini_Batch::Shuffle (:45-66)"""
        idx = self.stochastic_index
        for i in range(len(idx) - 1, -1, -1):
            j = int(self.rng.integers(0, i + 1))
            idx[i], idx[j] = idx[j], idx[i]

    def Increment_Mini_Batch(self, net, iteration):
        """:290-314; device-resident examples are gathered in HBM instead of re-pointing row pointers"""
        size = self.number_examples_per_iteration if iteration + 1 != self.number_mini_batch else self.number_examples_last_iteration
        first = iteration * self.number_examples_per_iteration
        index = self.stochastic_index[first:first + size]
        if not self.on_device:
            sel = index.astype(np.int64)
            self._batch = (self.inputs[sel], self.outputs[sel])
            return
        import torch
        if self._stage is None:
            big = max(self.number_examples_per_iteration, self.number_examples_last_iteration)
            self._stage = (torch.empty((big, self.inputs.shape[1]), dtype=torch.float32, device=self.inputs.device),
                           torch.empty((big, self.outputs.shape[1]), dtype=torch.float32, device=self.outputs.device))
        bmax = net.desc.batch_size
        for off in range(0, size, bmax):   # host index arrays go through a staging buffer of one maximum batch
            b = min(bmax, size - off)
            for stage, src in zip(self._stage, (self.inputs, self.outputs)):
                net.gather_examples(stage[off:], src, src.shape[0], src.shape[1], index[off:off + b], b)
        self._batch = (self._stage[0][:size], self._stage[1][:size])

    def _current(self):
        return self._batch

    def Training(self, net):
        """Dataset_Mini_Batch::Training_Loop (:381-420): per mini-batch train, read loss / accuracy, update with (batch, whole set)"""
        net.set_state_propagation(mb.STATE_TRAINING)
        if self.use_shuffle:
            self.Shuffle()
        loss = acc = 0.0
        for it in range(self.number_mini_batch):
            self.Increment_Mini_Batch(net, it)
            self.Train_Epoch(net)
            loss += get_loss(net, self.output_size)
            acc += self.Measure_Accuracy(net)
            net.Update_Parameter(self._batch[0].shape[0], self.Get__Number_Examples())
        h = net.get_hyper()
        h.epoch_time_step += 1.0
        net.set_hyper(h)
        self.loss_training = loss / self.number_mini_batch
        self.accuracy_training = acc / self.number_mini_batch
        net.set_state_propagation(mb.STATE_INFERENCE)
        return self.loss_training
