"""Pins the oracle's k-sparse filter (the k largest values of an example's row stay, the rest become 0): against a sort
(numpy / torch.topk) on the unfiltered network's outputs, the inference variant size_t(alpha k), ties at the cut, and the
backward pass - which does not look at the filter - against float64 autograd of a straight-through model.  CPU only."""
import numpy as np
import pytest
import torch

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, oracle_desc, oracle_hyper
from tests.oracle_lib import OracleNetwork


def _net(specs, B, T=1, seed=1, state=mb.STATE_TRAINING, masks=None):
    desc = oracle_desc(specs, B, T)
    net = OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS["MSE"]))
    w = glorot_parameters(desc, seed, bias_range=0.3)
    net.set_state_propagation(state)
    net.upload_parameters(w)
    if masks is not None:
        net.upload_masks(masks)
    net.Clear_Training_Arrays()
    return desc, net, w


def _topk_rows(a, k):
    """keep the k largest per row (ties: the lower index), zero the rest"""
    out = np.zeros_like(a)
    for r in range(a.shape[0]):
        order = sorted(range(a.shape[1]), key=lambda j: (-a[r, j], j))[:k]
        out[r, order] = a[r, order]
    return out


@pytest.mark.parametrize("act,k,alpha,dropout", [("TANH", 5, 1.0, None), ("RELU", 9, 2.0, None), ("SIGMOID", 1, 3.5, "BERNOULLI_INVERTED"), ("LINEAR", 23, 1.0, None), ("TANH", 24, 1.0, None)])
def test_filter_keeps_the_k_largest_of_each_row(act, k, alpha, dropout):
    B, T, H = 7, 3, 24
    hid = dict(units=H, activation=act)
    if dropout:
        hid.update(dropout=dropout, keep=0.7)
    plain = [dict(units=6), dict(hid), dict(units=4, activation="LINEAR")]
    sparse = [dict(units=6), dict(hid, k_sparsity=k, alpha_sparsity=alpha), dict(units=4, activation="LINEAR")]
    d0 = oracle_desc(plain, B, T)
    masks = (np.random.default_rng(2).uniform(0, 1, d0.total_mask_units) < 0.7).astype(np.uint8)
    X = np.random.default_rng(3).normal(0, 1, (B, T * 6)).astype(np.float32)
    for state, keep in ((mb.STATE_TRAINING, k), (mb.STATE_INFERENCE, int(np.float32(alpha) * np.float32(k)))):
        _, a, _ = _net(plain, B, T, state=state, masks=masks)
        _, b, _ = _net(sparse, B, T, state=state, masks=masks)
        a.Forward_Pass(B, X); b.Forward_Pass(B, X)
        dense = a.download_tensor(1, mb.TENSOR["OUTPUTS"], T * B * H).reshape(T * B, H)
        got = b.download_tensor(1, mb.TENSOR["OUTPUTS"], T * B * H).reshape(T * B, H)
        want = _topk_rows(dense, min(keep, H))
        assert np.array_equal(got, want)
        if act != "RELU" and not dropout:      # no zeros among the activations: exactly `keep` survivors per row
            assert ((got != 0).sum(1) == min(keep, H)).all()
        vals, idx = torch.topk(torch.tensor(dense), min(keep, H), dim=1)      # a library routine's word for the same thing
        assert np.array_equal(got, torch.zeros(T * B, H).scatter(1, idx, vals).numpy())


def test_ties_at_the_cut_keep_the_lower_indices():
    """identity-like layer: LINEAR activation of inputs routed one to one, with repeated values"""
    H, B = 8, 3
    specs = [dict(units=H), dict(units=H, activation="LINEAR", k_sparsity=3), dict(units=2, activation="LINEAR")]
    desc, net, w = _net(specs, B)
    w[:] = 0
    w[:H * H] = np.eye(H, dtype=np.float32).ravel()
    net.upload_parameters(w)
    X = np.array([[1, 5, 5, 5, 5, 0, -1, 2], [3, 3, 3, 3, 3, 3, 3, 3], [0, 0, 0, -2, 0, 7, 0, 0]], dtype=np.float32)
    net.Forward_Pass(B, X)
    got = net.download_tensor(1, mb.TENSOR["OUTPUTS"], B * H).reshape(B, H)
    assert np.array_equal(got, np.array([[0, 5, 5, 5, 0, 0, 0, 0], [3, 3, 3, 0, 0, 0, 0, 0], [0, 0, 0, 0, 0, 7, 0, 0]], dtype=np.float32))


def test_backward_ignores_the_filter():
    """the deltas pass the filter unchanged (no branch for it in the reference's backward pass); with an activation whose
    derivative reads the pre-activation only, the gradient is that of a straight-through filter"""
    B, H, k = 6, 16, 5
    specs = [dict(units=7), dict(units=H, activation="LEAKY_RELU", k_sparsity=k), dict(units=3, activation="LINEAR")]
    desc, net, w = _net(specs, B, seed=4)
    rng = np.random.default_rng(4)
    X, Y = rng.normal(0, 1, (B, 7)).astype(np.float32), rng.normal(0, 1, (B, 3)).astype(np.float32)
    net.Forward_Pass(B, X); net.Compute__Error(B, Y); net.Backward_Pass(B); net.Update_Derivative_Weight(B)
    W = torch.tensor(w.astype(np.float64), requires_grad=True)
    l1, l2 = desc.layers[1], desc.layers[2]
    W1 = W[l1.first_connection_index:l1.last_connection_index].reshape(H, 7)
    W2 = W[l2.first_connection_index:l2.last_connection_index].reshape(3, H)
    b1 = W[l1.first_bias_connection_index:l1.first_bias_connection_index + H]
    b2 = W[l2.first_bias_connection_index:l2.first_bias_connection_index + 3]
    s = torch.tensor(X.astype(np.float64)) @ W1.T + b1
    a = torch.where(s < 0, 0.01 * s, s)
    thr = torch.topk(a.detach(), k, dim=1).values[:, -1:]
    filtered = torch.where(a.detach() >= thr, a.detach(), torch.zeros_like(a))
    h = a + (filtered - a).detach()                    # forward: filtered; backward: identity
    y = h @ W2.T + b2
    (0.5 * ((y - torch.tensor(Y.astype(np.float64))) ** 2).sum()).backward()
    assert_close(net.download_tensor(2, mb.TENSOR["OUTPUTS"], B * 3), y.detach().numpy().ravel(), rel=1e-5, abs_=2e-6, what="outputs")
    assert_close(net.download_gradient(), W.grad.numpy(), rel=3e-4, abs_=3e-6, what="gradient")


def test_refusals():
    mk = lambda **kw: oracle_desc([dict(units=6), dict(units=8, activation="TANH", **kw), dict(units=3, activation="LINEAR")], 4)
    for bad in (dict(k_sparsity=9), dict(k_sparsity=4, alpha_sparsity=2.5), dict(k_sparsity=4, alpha_sparsity=0.1), dict(k_sparsity=4, alpha_sparsity=-1.0)):
        with pytest.raises(ValueError):
            mk(**bad)
    with pytest.raises(ValueError):      # not on the output layer
        oracle_desc([dict(units=6), dict(units=8, activation="TANH"), dict(units=3, activation="LINEAR", k_sparsity=2)], 4)
    mk(k_sparsity=8)                     # k == width: no filter
