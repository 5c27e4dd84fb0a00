"""Gradients accumulated over sub-batches of different sizes before one update - the pattern of the reference's
Dataset::Training (Neural_Network/Dataset.cpp:549-691: every sub-batch runs forward, error, backward and
Update_Derivative_Weight, one Update_Parameter follows).  The library may run a layer's weight contraction in several
forms depending on the rows it sums over: split along k into slabs that a second kernel adds onto the gradient (long
batches in front of narrow layers), one launch adding at the L2, or - when the layer's slice of the gradient is known to be
zero - one launch that stores.  A full sub-batch followed by a short one takes the first form and then the second or
third on the same slice: the second must add to what the first left.  Held against the CPU oracle (rel 1e-4 / abs 1e-5 of
the gradient's scale), through the separate calls and through the combined backward + weight-gradient call."""
import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, one_hot
from tests.oracle_lib import OracleNetwork

pytestmark = pytest.mark.gpu


def _step(net, B, X, Y, combined):
    net.Forward_Pass(B, X[:B])
    net.Compute__Error(B, Y[:B])
    if combined and hasattr(net, "Backward_Pass__Update_Derivative_Weight"):
        net.Backward_Pass__Update_Derivative_Weight(B)
    else:
        net.Backward_Pass(B)
        net.Update_Derivative_Weight(B)


@pytest.mark.parametrize("combined", [False, True], ids=["separate-calls", "combined-call"])
@pytest.mark.parametrize("sizes", [(1024, 100), (100, 1024), (1024, 1024, 37), (640, 1024)], ids=lambda s: "-".join(map(str, s)))
def test_sub_batches_of_different_sizes_accumulate(sizes, combined):
    Bmax = 1024
    specs = [dict(units=512), dict(units=512, activation="TANH"), dict(units=512, activation="SIGMOID"), dict(units=512, activation="TANH"), dict(units=16, activation="SOFTMAX")]
    desc = mb.make_desc(specs, Bmax)
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["GD"], learning_rate=0.01, type_loss_function=mb.LOSS["CROSS_ENTROPY"])
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h, threads=8)
    w = glorot_parameters(desc, 43, bias_range=0.2)
    rng = np.random.default_rng(43)
    X = rng.normal(0, 1, (Bmax, 512)).astype(np.float32)
    Y = one_hot(rng.integers(0, 16, Bmax), 16)
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.Clear_Training_Arrays()
    for round_ in range(2):          # the second round starts from the zeros the update left, not from Clear_Training_Arrays
        for B in sizes:
            perm = rng.permutation(Bmax)
            for n in (gpu, cpu):
                _step(n, B, np.ascontiguousarray(X[perm]), np.ascontiguousarray(Y[perm]), combined)
        g = cpu.download_gradient()
        assert_close(gpu.download_gradient(), g, 1e-4, 1e-5 * max(1.0, float(np.abs(g).max())), what="gradient over sub-batches %r, round %d" % (sizes, round_))
        for n in (gpu, cpu):
            n.Update_Parameter(sum(sizes), sum(sizes))
        # plain gradient descent, w -= lr g: the gradient's absolute tolerance reaches the parameters times lr
        wc = cpu.download_parameters()
        assert_close(gpu.download_parameters(), wc, 1e-4, 1e-5 + 0.01 * 1e-5 * max(1.0, float(np.abs(g).max())), what="parameters, round %d" % round_)
        assert not gpu.download_gradient().any()
        gpu.upload_parameters(wc)    # identical parameters for the next round
